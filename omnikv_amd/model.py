"""A Llama-3-shaped decoder whose decode attention and token selection run on the
HIP kernels: the counterpart of the reference's OmniKVMulLM / OmniKVMulModel /
OmniKVMulLayer (modeling/omnikv.py:113-394) without the transformers dependency.

GEMMs, norms, RoPE and the prefill attention are PyTorch-ROCm ops; the decode path
(filter-layer scoring + top-k, dense and sparse attention, KV tiering) goes through
omnikv_amd.cache.OmniKVMultiStageCache.  Weights are whatever the caller loads; the
benchmark uses seeded N(0, 0.02) initialisation.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops, trace
from .cache import OmniKVMultiStageCache, get_cache_cls
from .config import OmniKVConfig
from .selector import apply_rotary_pos_emb, select_from_query


@dataclass
class LlamaShape:
    hidden_size: int = 4096
    intermediate_size: int = 14336
    vocab_size: int = 128256
    num_hidden_layers: int = 32
    num_attention_heads: int = 32
    num_key_value_heads: int = 8
    head_dim: int = 128
    rope_theta: float = 500000.0
    rms_norm_eps: float = 1e-5


# The per-token operations of a decode step (RMSNorm with the residual add in front of it, rotary
# embedding, SiLU(gate) * up) as one HIP launch each instead of torch's op-by-op chains; prefill and
# CPU tensors take the torch path.  Off: every op as the reference's modules issue it.
FUSED_LAYER_OPS = True


def _fusable(x: torch.Tensor, *others: torch.Tensor) -> bool:
    return (FUSED_LAYER_OPS and x.is_cuda and x.shape[-2] == 1 and x.is_contiguous()
            and all(o.dtype == x.dtype and o.is_contiguous() for o in others))


class RMSNorm(nn.Module):
    def __init__(self, dim: int, eps: float):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim))
        self.eps = eps

    def forward(self, x, residual=None):
        """Normalised x, or with `residual`: (normalised (x + residual), x + residual)."""
        if _fusable(x, self.weight, *([residual] if residual is not None else [])):
            return ops.rmsnorm(x, self.weight, self.eps, residual)
        total = None
        if residual is not None:
            x = total = residual + x
        dt = x.dtype
        x = x.float()
        x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + self.eps)
        x = self.weight * x.to(dt)
        return x if residual is None else (x, total)


class RotaryEmbedding(nn.Module):
    def __init__(self, dim: int, theta: float):
        super().__init__()
        self.register_buffer("inv_freq", 1.0 / (theta ** (torch.arange(0, dim, 2, dtype=torch.float32) / dim)),
                             persistent=False)

    @torch.no_grad()
    def forward(self, x, position_ids):
        ang = position_ids[:, :, None].float() * self.inv_freq[None, None, :].to(position_ids.device)
        emb = torch.cat([ang, ang], dim=-1)
        return emb.cos().to(x.dtype), emb.sin().to(x.dtype)


class _Rows:
    """A block of output rows of a merged projection, usable like the nn.Linear it stands for: `.weight` is a
    view of the merged weight, calling it multiplies by those rows only.  The merged module owns the parameter
    (q/k/v share one GEMM per token, gate/up another: at batch 1 a projection is a memory-bound GEMV and the
    small ones are pure launch latency); code written against q_proj / k_proj / ... keeps working."""

    def __init__(self, linear: nn.Linear, lo: int, hi: int):
        self.linear, self.lo, self.hi = linear, lo, hi

    @property
    def weight(self):
        return self.linear.weight[self.lo: self.hi]

    def __call__(self, x):
        return F.linear(x, self.weight)


class MLP(nn.Module):
    def __init__(self, s: LlamaShape):
        super().__init__()
        self.inter = s.intermediate_size
        self.gate_up_proj = nn.Linear(s.hidden_size, 2 * s.intermediate_size, bias=False)  # rows: gate, then up
        self.gate_proj = _Rows(self.gate_up_proj, 0, self.inter)
        self.up_proj = _Rows(self.gate_up_proj, self.inter, 2 * self.inter)
        self.down_proj = nn.Linear(s.intermediate_size, s.hidden_size, bias=False)

    def forward(self, x):
        gu = self.gate_up_proj(x)
        gate, up = gu[..., : self.inter], gu[..., self.inter:]
        if _fusable(gate, up):
            return self.down_proj(ops.silu_mul(gate, up))
        return self.down_proj(F.silu(gate) * up)


class OmniKVAttention(nn.Module):
    """q/k/v/o projections + RoPE; the attributes select_tokens_by_attn_universal reads."""

    def __init__(self, s: LlamaShape, config: OmniKVConfig, layer_idx: int):
        super().__init__()
        self.config = config
        self.layer_idx = layer_idx
        self.num_heads = s.num_attention_heads
        self.num_key_value_heads = s.num_key_value_heads
        self.num_key_value_groups = self.num_heads // self.num_key_value_heads
        self.head_dim = s.head_dim
        nq, nkv = self.num_heads * self.head_dim, self.num_key_value_heads * self.head_dim
        self.qkv_proj = nn.Linear(s.hidden_size, nq + 2 * nkv, bias=False)  # rows: q, then k, then v
        self.q_proj = _Rows(self.qkv_proj, 0, nq)
        self.k_proj = _Rows(self.qkv_proj, nq, nq + nkv)
        self.v_proj = _Rows(self.qkv_proj, nq + nkv, nq + 2 * nkv)
        self.o_proj = nn.Linear(self.num_heads * self.head_dim, s.hidden_size, bias=False)
        self.rotary_emb = RotaryEmbedding(self.head_dim, s.rope_theta)

    def _project(self, hidden_states):
        """q, k, v of one merged GEMM, as views (bsz, n, heads * D) of its output."""
        nq, nkv = self.num_heads * self.head_dim, self.num_key_value_heads * self.head_dim
        qkv = self.qkv_proj(hidden_states)
        return qkv[..., :nq], qkv[..., nq: nq + nkv], qkv[..., nq + nkv:]

    def qkv(self, hidden_states, position_ids, rope=None):
        """Rotated q, k and v as (bsz, heads, n, D).  rope: (cos, sin) of these positions when the
        caller has them already (they are the same for every layer of a step)."""
        b, n, _ = hidden_states.shape
        q, k, v = self._project(hidden_states)
        v = v.view(b, n, self.num_key_value_heads, self.head_dim).transpose(1, 2)
        cos, sin = rope if rope is not None else self.rotary_emb(v, position_ids)
        if n == 1 and self.head_dim == 128 and _fusable(q, k, cos, sin):
            q, k = ops.rope(q, k, cos, sin, self.num_heads, self.num_key_value_heads)
            return q, k, v
        q = q.view(b, n, self.num_heads, self.head_dim).transpose(1, 2)
        k = k.view(b, n, self.num_key_value_heads, self.head_dim).transpose(1, 2)
        q, k = apply_rotary_pos_emb(q, k, cos, sin)
        return q, k, v


    def q_and_append(self, hidden_states, position_ids, rope, cache):
        """One new token: the rotated q (bsz, Hq, 1, D), with the rotated k and the v appended to the cache."""
        if getattr(cache, "_static", False) and self.head_dim == 128 and rope is not None:
            q, k, v = self._project(hidden_states)
            if _fusable(q, k, v, rope[0], rope[1]):  # rotation and append in one launch
                return cache.append_projected(q, k, v, rope[0], rope[1], self.layer_idx, self.num_heads)
        q, k, v = self.qkv(hidden_states, position_ids, rope)
        cache.append(k, v, self.layer_idx)
        return q


class OmniKVMulLayer(nn.Module):
    """modeling/omnikv.py:113-246."""

    def __init__(self, s: LlamaShape, config: OmniKVConfig, layer_idx: int):
        super().__init__()
        self.config = config
        self.layer_idx = layer_idx
        self.self_attn = OmniKVAttention(s, config, layer_idx)
        self.mlp = MLP(s)
        self.input_layernorm = RMSNorm(s.hidden_size, s.rms_norm_eps)
        self.post_attention_layernorm = RMSNorm(s.hidden_size, s.rms_norm_eps)
        self.prefill_len = None
        self.cache_cls = get_cache_cls(config)
        self.do_select_layers = [int(i) for i in config.get("do_select_layers").split(",")]
        self.hidden_state_window = None
        self.selector_cls = config.get("selector_cls", "softmax_before_last")
        self.window_size = config.get("window_size", 16)
        self.decode_step = 0

    def forward(self, hidden_states, position_ids, past_key_value: OmniKVMultiStageCache, delta=None, rope=None,
                defer_add: bool = False):
        """delta: what the previous layer left to be added to hidden_states (its MLP output), folded
        into this layer's first norm; defer_add: return (hidden_states, mlp output) instead of their sum."""
        if delta is not None:
            hidden_states, residual = self.input_layernorm(delta, residual=hidden_states)
        else:
            residual = hidden_states
            hidden_states = self.input_layernorm(hidden_states)
        q_len = hidden_states.shape[1]
        if q_len > 1:
            self.prefill_len = q_len
            if "last" not in self.selector_cls and self.layer_idx in self.do_select_layers:
                self.hidden_state_window = hidden_states[:, -self.window_size:]
                self.decode_step = 1
        assert isinstance(past_key_value, self.cache_cls)
        attn = self.self_attn
        if q_len > 1:
            q, k, v = attn.qkv(hidden_states, position_ids, rope)
            # prefill: store K/V (tiered by the cache), causal attention over the prompt
            past_key_value.append(k, v, self.layer_idx)
            out = F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)
            out = out.transpose(1, 2).reshape(hidden_states.shape[0], q_len, -1)
        else:
            consider_len = self.prefill_len
            num_selected_tokens = self.config.get("num_of_selected_tokens", 4096)
            if isinstance(num_selected_tokens, float):
                num_selected_tokens = int(num_selected_tokens * consider_len)
            q = attn.q_and_append(hidden_states, position_ids, rope, past_key_value)
            if trace.idx_tracer is not None:
                # every layer reports what it would select (modeling/offload_select_once.py:170-174)
                trace.idx_tracer.observe(self.layer_idx, q, past_key_value.key_cache[self.layer_idx], consider_len)
            if self.layer_idx in self.do_select_layers:
                if not self.config.get("dense_more", False):
                    raise ValueError("dense_more=False is not supported")
                if "last" in self.selector_cls:
                    # scores and this layer's attention share one pass over K
                    o, _ = past_key_value.attend_and_select(q, self.layer_idx, num_selected_tokens, consider_len,
                                                            self.selector_cls)
                else:
                    forced = max(0, self.window_size - self.decode_step)
                    if getattr(past_key_value, "_static", False):
                        # in place (one fixed buffer per layer), so that a captured step finds on replay
                        # what the previous replay left
                        self.hidden_state_window.copy_(torch.cat([self.hidden_state_window[:, 1:], hidden_states], dim=1))
                    else:
                        self.hidden_state_window = torch.cat([self.hidden_state_window, hidden_states], dim=1)[
                            :, -self.window_size:].contiguous()
                    win = self.hidden_state_window
                    # every window row is rotated with the CURRENT position (modeling/omnikv.py:34-35)
                    wq = attn.q_proj(win).view(win.shape[0], win.shape[1], attn.num_heads, attn.head_dim).transpose(1, 2)
                    cos, sin = attn.rotary_emb(wq, position_ids)
                    wq, _ = apply_rotary_pos_emb(wq, wq, cos, sin)
                    # the first of the two scoring passes over K rides on the layer's own attention
                    o, _ = past_key_value.attend_and_select_window(q, wq.contiguous(), self.layer_idx,
                                                                   max(1, num_selected_tokens - forced),
                                                                   consider_len - forced, self.selector_cls,
                                                                   forced_tail=forced)
                past_key_value.stage = "decoding"
                self.decode_step += 1
            else:
                o = past_key_value.attend(q, self.layer_idx)
            out = o.reshape(hidden_states.shape[0], 1, -1)
        hidden_states, residual = self.post_attention_layernorm(attn.o_proj(out), residual=residual)
        if hidden_states.shape[1] <= 4000:
            hidden_states = self.mlp(hidden_states)
        else:  # modeling/omnikv.py:233-235: long prompts go through the MLP in pieces
            hidden_states = torch.cat([self.mlp(hs) for hs in torch.split(hidden_states, 4000, dim=1)], dim=1)
        if defer_add:
            return residual, hidden_states
        return residual + hidden_states


class OmniKVMulModel(nn.Module):
    def __init__(self, s: LlamaShape, config: OmniKVConfig):
        super().__init__()
        self.embed_tokens = nn.Embedding(s.vocab_size, s.hidden_size)
        self.layers = nn.ModuleList([OmniKVMulLayer(s, config, i) for i in range(s.num_hidden_layers)])
        self.norm = RMSNorm(s.hidden_size, s.rms_norm_eps)

    def forward(self, input_ids, position_ids, past_key_values):
        h = self.embed_tokens(input_ids)
        if input_ids.shape[1] > 1 or not FUSED_LAYER_OPS or not h.is_cuda:
            for layer in self.layers:
                h = layer(h, position_ids, past_key_values)
            return self.norm(h)
        # decode: cos / sin of the position once for all layers; every layer's closing residual add is
        # folded into the norm that follows it
        attn0 = self.layers[0].self_attn
        rope = attn0.rotary_emb(h, position_ids)
        delta = None
        for layer in self.layers:
            h, delta = layer(h, position_ids, past_key_values, delta=delta, rope=rope, defer_add=True)
        return self.norm(delta, residual=h)[0]


class StaticDecodeGraph:
    """A captured decode step plus the host-side count of its replays: every replay appends one
    row at a device position, so the replay that would run past the preallocated buffers raises
    instead (the captured kernels themselves check nothing)."""

    def __init__(self, graph: torch.cuda.CUDAGraph, cache: OmniKVMultiStageCache):
        self.graph = graph
        self.cache = cache

    def replay(self) -> None:
        self.cache.note_static_step()
        self.graph.replay()


class OmniKVMulLM(nn.Module):
    """modeling/omnikv.py:271-394: builds the cache on first use, keeps `stage`,
    runs the model, applies lm_head to the LAST position only, returns fp32 logits."""

    def __init__(self, s: LlamaShape, config: OmniKVConfig):
        super().__init__()
        self.shape = s
        self.config = config
        self.model = OmniKVMulModel(s, config)
        self.lm_head = nn.Linear(s.hidden_size, s.vocab_size, bias=False)
        self.cache_cls = get_cache_cls(config)

    @torch.no_grad()
    def init_weights(self, seed: int = 0, std: float = 0.02):
        g = torch.Generator(device=self.lm_head.weight.device).manual_seed(seed)
        for name, p in self.named_parameters():
            if p.dim() >= 2:
                p.normal_(0.0, std, generator=g)
        return self

    @torch.no_grad()
    def load_llama_state_dict(self, state_dict) -> None:
        """Weights under the names a Llama checkpoint uses (the reference loads one with from_pretrained,
        infer.py): `...self_attn.{q,k,v}_proj.weight` go into the rows of the merged `qkv_proj.weight`,
        `...mlp.{gate,up}_proj.weight` into `gate_up_proj.weight`, everything else by its own name."""
        own = dict(self.named_parameters())
        seen = set()
        for name, w in state_dict.items():
            parts = name.rsplit(".", 2)
            if len(parts) == 3 and parts[2] == "weight" and parts[1] in ("q_proj", "k_proj", "v_proj", "gate_proj", "up_proj"):
                merged = "qkv_proj" if parts[1][0] in "qkv" else "gate_up_proj"
                mod = self.get_submodule(parts[0])
                rows = getattr(mod, parts[1])
                dst = own[f"{parts[0]}.{merged}.weight"][rows.lo: rows.hi]
                if dst.shape != w.shape:
                    raise ValueError(f"{name}: shape {tuple(w.shape)}, expected {tuple(dst.shape)}")
                dst.copy_(w)
                seen.add((parts[0], parts[1]))
            elif name in own:
                if own[name].shape != w.shape:
                    raise ValueError(f"{name}: shape {tuple(w.shape)}, expected {tuple(own[name].shape)}")
                own[name].copy_(w)
                seen.add(name)
            elif not name.endswith("rotary_emb.inv_freq"):
                raise KeyError(f"unexpected key {name}")
        missing = [n for n in own if n not in seen and not n.endswith(("qkv_proj.weight", "gate_up_proj.weight"))]
        for li in range(self.shape.num_hidden_layers):
            for mod, names in ((f"model.layers.{li}.self_attn", ("q_proj", "k_proj", "v_proj")),
                               (f"model.layers.{li}.mlp", ("gate_proj", "up_proj"))):
                missing += [f"{mod}.{n}.weight" for n in names if (mod, n) not in seen]
        if missing:
            raise KeyError(f"missing keys: {missing[:5]}{' ...' if len(missing) > 5 else ''}")

    def new_cache(self, **kwargs) -> OmniKVMultiStageCache:
        sel = [int(i) for i in self.config.get("do_select_layers").split(",")]
        full = list(range(0, sel[0])) + sel + [self.shape.num_hidden_layers]  # modeling/omnikv.py:322-331
        if hasattr(self.config, "skip_threshold"):
            kwargs.setdefault("skip_threshold", self.config.get("skip_threshold"))
        return self.cache_cls(full, self.shape.num_hidden_layers,
                              self.config.get("num_wait_load_layers", 2), self.config.get("real_offload", True), **kwargs)

    @torch.no_grad()
    def forward(self, input_ids, past_key_values: Optional[OmniKVMultiStageCache] = None, position_ids=None,
                **cache_kwargs):
        n = input_ids.shape[1]
        if not isinstance(past_key_values, self.cache_cls):
            past_key_values = self.new_cache(**cache_kwargs)
        past_key_values.stage = "decoding" if n == 1 else "prefill"
        static = n == 1 and getattr(past_key_values, "_static", False)
        if static:
            if not torch.cuda.is_current_stream_capturing():  # replays are counted by StaticDecodeGraph
                past_key_values.note_static_step()
            position_ids = past_key_values._pos.view(1, 1).expand(input_ids.shape[0], -1)
        elif position_ids is None:
            start = past_key_values.get_seq_length()
            position_ids = torch.arange(start, start + n, device=input_ids.device)[None].expand(input_ids.shape[0], -1)
        h = self.model(input_ids, position_ids, past_key_values)
        logits = self.lm_head(h[:, -1:]).float()
        if trace.idx_tracer is not None and n == 1:
            trace.idx_tracer.end_step(self.shape.num_hidden_layers)
        if static:
            past_key_values.advance_static()
        return logits, past_key_values

    @torch.no_grad()
    def capture_decode(self, cache: OmniKVMultiStageCache, first_token: torch.Tensor, warmup: int = 2):
        """Capture one greedy decode step in a HIP graph.  Returns (graph, token, logits):
        each graph.replay() consumes `token` (1, 1), writes the step's fp32 logits into
        `logits` and the argmax back into `token`, and moves every length on the device
        by one -- a generation loop with no host work per token besides the replay.
        Before the capture `warmup` eager steps run (after, for the window selectors, as many
        as the query window needs to leave the prompt): `token` is the one they ended on."""
        if trace.idx_tracer is not None:
            raise RuntimeError("selection tracing keeps per-step host state; trace an eager run")
        token = first_token.clone().view(1, 1)
        if "last" not in self.config.get("selector_cls", "softmax_before_last"):
            # the window selectors force-keep the last prompt positions until the query window has left
            # the prompt (modeling/omnikv.py:177-210): those steps change shape and run eagerly first
            sel_layers = [l for l in self.model.layers if l.layer_idx in l.do_select_layers]
            if any(l.hidden_state_window is None or l.hidden_state_window.shape[1] < l.window_size for l in sel_layers):
                raise NotImplementedError("a captured step needs a full query window: the prompt is shorter than window_size")
            for _ in range(max([0] + [l.window_size - l.decode_step for l in sel_layers])):
                logits, _ = self.forward(token, cache)
                token.copy_(logits[:, -1].argmax(-1, keepdim=True))
        cache.enable_static_decode()
        stream = torch.cuda.Stream(device=token.device)
        stream.wait_stream(torch.cuda.current_stream(token.device))
        with torch.cuda.stream(stream):
            for _ in range(warmup):  # eager steps on the capture stream: workspaces, first selection
                logits, _ = self.forward(token, cache)
                token.copy_(logits[:, -1].argmax(-1, keepdim=True))
            stream.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                logits, _ = self.forward(token, cache)
                token.copy_(logits[:, -1].argmax(-1, keepdim=True))
        torch.cuda.current_stream(token.device).wait_stream(stream)
        return StaticDecodeGraph(graph, cache), token, logits

    @torch.no_grad()
    def generate_greedy(self, input_ids, num_tokens: int, **cache_kwargs) -> Tuple[torch.Tensor, List[torch.Tensor]]:
        """num_tokens greedy tokens after the prompt; returns (tokens, per-step fp32 logits)."""
        cache_kwargs.setdefault("max_new_tokens", num_tokens + 1)
        logits, cache = self.forward(input_ids, None, **cache_kwargs)
        out, all_logits = [], [logits]
        tok = logits[:, -1].argmax(-1, keepdim=True)
        out.append(tok)
        for _ in range(num_tokens - 1):
            logits, cache = self.forward(tok, cache)
            all_logits.append(logits)
            tok = logits[:, -1].argmax(-1, keepdim=True)
            out.append(tok)
        return torch.cat(out, dim=1), all_logits
