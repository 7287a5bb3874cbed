"""End-to-end greedy decode of a small random-init Llama-shaped model: the HIP path
(omnikv_amd.model) against the same weights run on the CPU with the oracle's
selection, cache tiering and attention wired exactly as the reference's layer forward
(modeling/omnikv.py:143-246, 287-394)."""
import copy

import pytest
import torch
import torch.nn.functional as F

from omnikv_amd.config import OmniKVConfig
from omnikv_amd.model import LlamaShape, OmniKVMulLM
from omnikv_amd.selector import apply_rotary_pos_emb
from oracle import okv_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

SHAPE = LlamaShape(hidden_size=256, intermediate_size=512, vocab_size=1000, num_hidden_layers=7,
                   num_attention_heads=32, num_key_value_heads=8, head_dim=128)


def _config(selector_cls, real_offload, ratio=0.1):
    return OmniKVConfig(model_cls="multi", cache_cls="multi", do_select_layers="1,4", num_wait_load_layers=1,
                        real_offload=real_offload, dense_more=True, num_of_selected_tokens=ratio,
                        selector_cls=selector_cls, window_size=4)


class _OracleRunner:
    """The reference's forward on the CPU: select -> set_idx_on_gpu -> update -> attention."""

    def __init__(self, lm: OmniKVMulLM, cfg):
        self.lm = lm
        self.cfg = cfg
        L = lm.shape.num_hidden_layers
        sel = [int(i) for i in cfg.get("do_select_layers").split(",")]
        self.sel = sel
        self.cache = orc.OracleMultiStageCache(orc.full_attn_layers_from_select_layers(sel, L), L,
                                               cfg.get("num_wait_load_layers", 2), cfg.get("real_offload", True))
        self.state = [dict(prefill_len=None, decode_step=0, window=None) for _ in range(L)]
        self.seen = 0

    @torch.no_grad()
    def forward(self, input_ids):
        lm, cfg = self.lm, self.cfg
        n = input_ids.shape[1]
        self.cache.stage = "decoding" if n == 1 else "prefill"
        pos = torch.arange(self.seen, self.seen + n)[None]
        self.seen += n
        h = lm.model.embed_tokens(input_ids)
        selector_cls, W = cfg.get("selector_cls"), cfg.get("window_size")
        for li, layer in enumerate(lm.model.layers):
            st = self.state[li]
            attn = layer.self_attn
            residual = h
            x = layer.input_layernorm(h)
            if n > 1:
                st["prefill_len"] = n
                if "last" not in selector_cls and li in self.sel:
                    st["window"] = x[:, -W:]
                    st["decode_step"] = 1
            consider_len = st["prefill_len"]
            k_sel = orc.num_selected_tokens(cfg.get("num_of_selected_tokens"), consider_len)
            if n == 1 and li in self.sel:
                window_hs = x
                forced = 0
                if "last" not in selector_cls:
                    st["window"] = torch.cat([st["window"], x], dim=1)[:, -W:]
                    window_hs = st["window"]
                    k_sel, consider_len, forced = orc.window_adjust(k_sel, consider_len, W, st["decode_step"])
                wq = attn.q_proj(window_hs).view(1, window_hs.shape[1], attn.num_heads, attn.head_dim).transpose(1, 2)
                cos, sin = attn.rotary_emb(wq, pos)
                wq, _ = apply_rotary_pos_emb(wq, wq, cos, sin)
                scores = orc.score_tokens(wq, self.cache.key_cache[li], consider_len, selector_cls)
                idx = orc.select_topk(scores, k_sel)
                if "last" not in selector_cls:
                    idx = torch.cat([idx, torch.arange(st["prefill_len"] - forced, st["prefill_len"])[None]], dim=1)
                self.cache.set_idx_on_gpu(idx, li)
                self.cache.stage = "decoding"
                st["decode_step"] += 1
            q, k, v = attn.qkv(x, pos)
            K, V = self.cache.update(k, v, li)
            if n > 1:
                o = F.scaled_dot_product_attention(q, K, V, is_causal=True, enable_gqa=True)
            else:
                o = orc.gqa_attention(q, K, V)
            o = o.transpose(1, 2).reshape(1, n, -1)
            h = residual + attn.o_proj(o)
            h = h + layer.mlp(layer.post_attention_layernorm(h))
        return lm.lm_head(lm.model.norm(h)[:, -1:]).float()


@pytest.mark.parametrize("selector_cls", ["last", "softmax_before_last", "uniform", "exp"])
@pytest.mark.parametrize("real_offload", [False, True, "incremental", "memcpy"])
def test_greedy_decode_matches_oracle(selector_cls, real_offload):
    torch.manual_seed(0)
    mode = {"offload_mode": real_offload} if isinstance(real_offload, str) else {}  # a string names the tier's staging mode
    real_offload = bool(real_offload)
    cfg = _config(selector_cls, real_offload)
    lm = OmniKVMulLM(SHAPE, cfg).float()
    lm.init_weights(seed=3, std=0.08)
    ref = _OracleRunner(copy.deepcopy(lm), _config(selector_cls, real_offload))
    dut = lm.to(DEV)
    n, steps = 500, 6
    ids = torch.randint(0, SHAPE.vocab_size, (1, n), generator=torch.Generator().manual_seed(1))
    want = ref.forward(ids)
    got, cache = dut.forward(ids.to(DEV), None, max_new_tokens=16, cpu_num_threads=2, **mode)
    assert got.shape == (1, 1, SHAPE.vocab_size) and got.dtype == torch.float32
    assert (got.cpu() - want).abs().max() < 2e-3
    dense = sorted(i for i, s in cache.layer_state.items() if not s[0])
    assert dense == [0, 1, 2, 4, 5]
    agree = 0
    for t in range(steps):
        tok = want[:, -1].argmax(-1, keepdim=True)  # teacher forcing with the oracle's token
        want = ref.forward(tok)
        got, cache = dut.forward(tok.to(DEV), cache)
        assert (got.cpu() - want).abs().max() < 3e-3, (selector_cls, real_offload, t)
        top2 = want[0, 0].topk(2).values
        if float(top2[0] - top2[1]) > 1e-2:
            assert int(got[0, 0].argmax()) == int(want[0, 0].argmax())
            agree += 1
    assert agree >= steps - 1  # at most one step's top two logits were too close to call
    assert cache.get_seq_length() == n + steps
    if real_offload:
        cache._join_worker()


class _CallCounter:
    """Wraps a function of the ops module and counts its calls."""

    def __init__(self, monkeypatch, name):
        from omnikv_amd import ops
        self.calls = 0
        inner = getattr(ops, name)

        def wrapped(*a, **kw):
            self.calls += 1
            return inner(*a, **kw)

        monkeypatch.setattr(ops, name, wrapped)


@pytest.mark.parametrize("selector_cls", ["uniform", "exp"])
@pytest.mark.parametrize("real_offload", [False, True])
def test_greedy_decode_bf16_window_selectors_take_the_fused_filter_layer(selector_cls, real_offload, monkeypatch):
    """The 16-bit model path of the window selectors: the filter layer's attention and its first scoring
    pass are one call (okv_dense_attn_window), through the steps in which the window still overlaps the
    prompt (forced positions appended) and beyond.  Two references, teacher-forced with the first one's tokens:
    the same bf16 model with the fused call switched off (selection and attention as separate calls: the same
    bf16 roundings everywhere, only partial sums grouped differently -- tight), and the oracle runner in fp32
    on the same bf16-rounded weights (bf16 activations against fp32 ones through seven layers -- loose)."""
    from omnikv_amd import ops
    torch.manual_seed(0)

    def fresh():
        lm = OmniKVMulLM(SHAPE, _config(selector_cls, real_offload)).float()
        lm.init_weights(seed=3, std=0.08)
        return lm.to(torch.bfloat16)

    ref = _OracleRunner(copy.deepcopy(fresh()).float(), _config(selector_cls, real_offload))
    n, steps = 500, 7  # window_size 4: steps 1..3 append forced prompt positions, 4.. do not
    ids = torch.randint(0, SHAPE.vocab_size, (1, n), generator=torch.Generator().manual_seed(1))

    # the separate path first: window_supported() says no, select_with_query + attend run
    with monkeypatch.context() as mp:
        mp.setattr(ops, "window_supported", lambda q, k: False)
        fused_off = _CallCounter(mp, "dense_attn_window")
        plain = fresh().to(DEV)
        logits, cache = plain.forward(ids.to(DEV), None, max_new_tokens=16)
        separate = [logits.clone()]
        toks = []
        for t in range(steps):
            toks.append(separate[-1][:, -1].argmax(-1, keepdim=True))
            logits, cache = plain.forward(toks[-1], cache)
            separate.append(logits.clone())
        assert fused_off.calls == 0
        if real_offload:
            cache._join_worker()

    fused = _CallCounter(monkeypatch, "dense_attn_window")
    dut = fresh().to(DEV)
    want = ref.forward(ids)
    got, cache = dut.forward(ids.to(DEV), None, max_new_tokens=16)
    scale = float(want.abs().max())
    assert torch.equal(got, separate[0])  # the prefill does not select
    assert (got.cpu() - want).abs().max() < 0.1 * scale
    for t in range(steps):
        want = ref.forward(toks[t].cpu())
        got, cache = dut.forward(toks[t], cache)
        # fused against separate: the window scores agree to ~2e-5 (other split grouping), so the selections
        # are the same up to near-ties and the logits to bf16 rounding of a few attention outputs
        assert (got - separate[t + 1]).abs().max() < 0.02 * scale, (selector_cls, real_offload, t)
        assert int(got[0, 0].argmax()) == int(separate[t + 1][0, 0].argmax()) or \
            float(separate[t + 1][0, 0].topk(2).values.diff().abs()) < 0.04 * scale
        assert (got.cpu() - want).abs().max() < 0.1 * scale, (selector_cls, real_offload, t)
        top2 = want[0, 0].topk(2).values
        if float(top2[0] - top2[1]) > 0.2 * scale:
            assert int(got[0, 0].argmax()) == int(want[0, 0].argmax())
    assert fused.calls == 2 * steps  # both filter layers, every decode step
    sel = cache._idx[1]
    assert sel.dtype == torch.int32 and sel.shape[1] == int(0.1 * n)  # forced window gone: k rows again
    if real_offload:
        cache._join_worker()


def test_generate_greedy_and_error_paths():
    cfg = _config("last", False)
    lm = OmniKVMulLM(SHAPE, cfg).to(torch.bfloat16).to(DEV)
    lm.init_weights(seed=5, std=0.08)
    ids = torch.randint(0, SHAPE.vocab_size, (1, 300), generator=torch.Generator().manual_seed(2)).to(DEV)
    toks, logits = lm.generate_greedy(ids, 5)
    assert toks.shape == (1, 5) and len(logits) == 5 and logits[0].dtype == torch.float32
    toks2, _ = lm.generate_greedy(ids, 5)
    assert torch.equal(toks, toks2)  # deterministic: fixed split order, no float atomics
    bad = _config("last", False)
    bad.dense_more = False
    lm2 = OmniKVMulLM(SHAPE, bad).to(torch.bfloat16).to(DEV)
    lm2.init_weights(seed=5, std=0.08)
    _, cache = lm2.forward(ids, None)
    with pytest.raises(ValueError):  # modeling/omnikv.py:213-214
        lm2.forward(ids[:, :1], cache)


@pytest.mark.parametrize("selector_cls,offload", [("uniform", True), ("exp", "incremental"), ("uniform", False)])
def test_graph_replayed_bf16_window_decode_takes_the_fused_branch(selector_cls, offload, monkeypatch):
    """Static decode of a 16-bit model with a window selector, eager static steps and graph replays, with
    and without the host tier: the captured step holds okv_dense_attn_window (the fused filter layer writing
    into the fixed index buffer, the copy stream staging behind it), and every replay reproduces what the
    same number of eager STATIC steps of a second, identically initialised model produce -- the same
    kernels on the same shapes, so bit for bit."""
    ids = torch.randint(0, SHAPE.vocab_size, (1, 400), generator=torch.Generator().manual_seed(4)).to(DEV)
    kw = {"offload_mode": offload} if isinstance(offload, str) else {}
    steps = 6

    def fresh():
        lm = OmniKVMulLM(SHAPE, _config(selector_cls, bool(offload))).float()
        lm.init_weights(seed=11, std=0.08)
        return lm.to(torch.bfloat16).to(DEV)

    def prime(lm):
        """Prefill, then the three non-static steps in which the window still overlaps the prompt."""
        logits, cache = lm.forward(ids, None, max_new_tokens=32, **kw)
        tok = logits[:, -1].argmax(-1, keepdim=True)
        for _ in range(3):
            logits, cache = lm.forward(tok, cache)
            tok = logits[:, -1].argmax(-1, keepdim=True)
        return cache, tok

    # eager static steps
    lm = fresh()
    cache, tok = prime(lm)
    cache.enable_static_decode()
    fused = _CallCounter(monkeypatch, "dense_attn_window")
    eager = []
    for _ in range(steps + 2):
        logits, cache = lm.forward(tok, cache)
        tok = logits[:, -1].argmax(-1, keepdim=True)
        eager.append((logits.clone(), int(tok)))
    assert fused.calls == 2 * (steps + 2)
    # the same steps: two eager static ones (capture_decode's warm-up), then replays
    lm2 = fresh()
    cache2, tok2 = prime(lm2)
    graph, token, glogits = lm2.capture_decode(cache2, tok2, warmup=2)
    after_capture = 2 * (steps + 2) + 2 * 3 + 2 * 3  # + the second model's three priming steps, two warm-up steps and the captured one
    assert fused.calls == after_capture
    assert int(token) == eager[1][1]
    for t in range(steps):
        graph.replay()
        torch.cuda.synchronize()
        _ = (glogits.clone() * 2).sum().item()
        assert torch.equal(glogits, eager[2 + t][0]), t
        assert int(token) == eager[2 + t][1], t
    assert fused.calls == after_capture  # replays run the captured launches, not Python


@pytest.mark.parametrize("selector_cls,offload", [("last", False), ("softmax_before_last", False), ("last", True),
                                                  ("last", "incremental"), ("uniform", False), ("exp", True)])
def test_graph_replayed_decode_matches_eager(selector_cls, offload):
    """A decode step captured in a HIP graph (device-side lengths and positions; with the
    host tier also the copy stream's zero-copy gathers) must reproduce the eager path
    token for token and logit for logit on every replay."""
    ids = torch.randint(0, SHAPE.vocab_size, (1, 400), generator=torch.Generator().manual_seed(4)).to(DEV)
    steps = 7
    kw = {"offload_mode": offload} if isinstance(offload, str) else {}  # a string names the staging mode of the tier

    def fresh():
        lm = OmniKVMulLM(SHAPE, _config(selector_cls, bool(offload))).float().to(DEV)
        lm.init_weights(seed=11, std=0.08)
        return lm

    # the window selectors first run the steps in which the query window still overlaps the prompt
    # (window_size 4: decode steps 1..3 force-keep prompt positions and change shape)
    extra = 3 if selector_cls in ("uniform", "exp") else 0
    lm = fresh()
    eager_toks, eager_logits = lm.generate_greedy(ids, steps + 4 + extra, max_new_tokens=32, **kw)
    lm2 = fresh()
    logits, cache = lm2.forward(ids, None, max_new_tokens=32, **kw)
    assert torch.equal(logits, eager_logits[0])
    tok = logits[:, -1].argmax(-1, keepdim=True)
    graph, token, glogits = lm2.capture_decode(cache, tok, warmup=2)  # two eager static steps, then capture
    first = 2 + extra
    assert int(token) == int(eager_toks[0, first])
    for t in range(steps):
        graph.replay()
        torch.cuda.synchronize()
        # other work between replays, as a real loop would have
        _ = (glogits.clone() * 2).sum().item()
        assert (glogits - eager_logits[first + 1 + t]).abs().max() < 1e-4, t
        assert int(token) == int(eager_toks[0, first + 1 + t]), t
    assert int(cache._len32) == 400 + 1 + first + steps  # capture itself executes nothing
    if offload and "last" in selector_cls:  # rows packed by host threads cannot be part of a graph
        lm3 = fresh()
        _, c3 = lm3.forward(ids, None, max_new_tokens=32, offload_mode="memcpy")
        with pytest.raises(NotImplementedError):
            lm3.capture_decode(c3, tok)


def test_static_decode_refuses_to_run_past_its_buffers():
    """max_new_tokens rows are preallocated; the step that would write row max_new_tokens + 1
    raises on the host (eager static steps and graph replays alike) and launches nothing."""
    ids = torch.randint(0, SHAPE.vocab_size, (1, 200), generator=torch.Generator().manual_seed(6)).to(DEV)
    lm = OmniKVMulLM(SHAPE, _config("last", False)).float().to(DEV)
    lm.init_weights(seed=3, std=0.08)
    budget = 6
    logits, cache = lm.forward(ids, None, max_new_tokens=budget)
    tok = logits[:, -1].argmax(-1, keepdim=True)
    graph, token, _ = lm.capture_decode(cache, tok, warmup=2)
    assert cache.static_steps_left == budget - 2
    for _ in range(budget - 2):
        graph.replay()
    torch.cuda.synchronize()
    assert cache.static_steps_left == 0
    assert int(cache._pos) == 200 + budget - 1 and int(cache._len32) == 200 + budget  # clamped at the last row
    with pytest.raises(RuntimeError, match="max_new_tokens"):
        graph.replay()
    with pytest.raises(RuntimeError, match="max_new_tokens"):
        lm.forward(token, cache)


def test_selection_tracing_compares_layers_and_leaves_decode_untouched(tmp_path):
    """Every layer reports what it would select (the reference's SAVE_SELECTED_IDX runs):
    the matrices are checked against the oracle's scores and stable top-k of the same
    queries and keys, and a traced run generates what an untraced one does."""
    from omnikv_amd import trace

    cfg = _config("last", False)
    lm = OmniKVMulLM(SHAPE, cfg).float().to(DEV)
    lm.init_weights(seed=9, std=0.08)
    n, steps, L = 400, 3, SHAPE.num_hidden_layers
    ids = torch.randint(0, SHAPE.vocab_size, (1, n), generator=torch.Generator().manual_seed(4)).to(DEV)
    plain, _ = lm.generate_greedy(ids, steps + 1)

    seen = []  # (layer, q, K, consider_len) as the hook receives them

    class Spy(trace.SelectedIndexTracer):
        def observe(self, layer_idx, q, kview, consider_len):
            seen.append((layer_idx, q.detach().cpu().clone(), kview[:, :, :consider_len].detach().cpu().clone()))
            super().observe(layer_idx, q, kview, consider_len)

    tr = Spy(desc="unit", num_selected_tokens=0.1, keep=5, save_dir=str(tmp_path))
    assert trace.set_tracer(tr) is None
    try:
        traced, _ = lm.generate_greedy(ids, steps + 1)
        with pytest.raises(RuntimeError):
            lm.capture_decode(lm.new_cache(), plain[:, :1])
    finally:
        trace.set_tracer(None)
    assert torch.equal(plain, traced)
    assert tr.steps == steps and len(seen) == steps * L

    k = int(0.1 * n)
    mass = torch.zeros((L, L), dtype=torch.float64)
    overlap = torch.zeros_like(mass)
    for t in range(steps):
        p, sel = [], []
        for li, q, K in seen[t * L:(t + 1) * L]:
            s = orc.score_tokens(q, K, n, "last")
            p.append(torch.softmax(s[0].double(), -1))
            sel.append(orc.select_topk_stable(s, k)[0])
        for i in range(L):
            for j in range(L):
                mass[i, j] += p[j][sel[i]].sum()
                overlap[i, j] += len(set(sel[i].tolist()) & set(sel[j].tolist())) / k
    got_mass, got_overlap = tr.matrices()
    assert (got_mass - mass / steps).abs().max() < 1e-4
    assert (got_overlap - overlap / steps).abs().max() < 2.0 / k   # a near-tie may swap one index
    assert torch.allclose(got_overlap.diagonal(), torch.ones(L, dtype=torch.float64))
    # no other layer's choice keeps more of layer j's attention than layer j's own
    assert (got_mass <= got_mass.diagonal()[None, :] + 1e-6).all()

    path = tr.save_idx()
    blob = trace.read_idx_tracer(path)
    assert blob["steps"] == steps and torch.equal(blob["mass"], got_mass)
    rec = blob["layers_idx"][0][2]
    assert len(rec) == steps and rec[0]["idx"].shape == (1, 5) and rec[0]["prefill_len"] == n
    assert (rec[0]["value"][0, :-1] >= rec[0]["value"][0, 1:]).all()
    layers, quality = trace.suggest_filter_layers(got_mass, num_filters=2, num_wait_load_layers=1, max_dense_layers=5)
    assert len(layers) == 2 and 0 < quality <= 1
    assert quality == pytest.approx(trace.schedule_quality(got_mass, layers, 1)[0])
