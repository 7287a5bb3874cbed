"""Which layers make good filters: per-layer selection tracing for a decode run.

The reference answers this with an environment switch, SAVE_SELECTED_IDX: every
decoder layer of a decode step scores the prompt with the `last` selector, turns the
head-max scores into a softmax over tokens, sorts them and hands (indices, values,
prefill_len, layer) to a process-wide `idx_tracer`, which pickles everything at exit
(tiny_tools/tensor_tools.py:38-99, modeling/offload_select_once.py:112-122,170-174).
The recorded lists are then compared offline, layer against layer.

Here the same hook runs on the HIP kernels -- one scoring pass over the layer's resident
K and one top-k per layer and step -- and the layer-against-layer comparison is done on
the GPU as the steps go by, so a 128K-token run keeps two small matrices instead of
32 sorted copies of the context per token:

  mass[i, j]     the share of layer j's own token distribution that falls on the k tokens
                 layer i would select (1.0 on the diagonal only if k covers everything);
  overlap[i, j]  |top-k of layer i  intersected with  top-k of layer j| / k.

`suggest_filter_layers` turns `mass` into a choice of filter layers for a model the
reference ships no configuration for.  Sorted per-layer lists in the reference's own
format are still available (`keep=`), written with torch.save as plain tensors.
"""
from __future__ import annotations

import itertools
import os
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from . import ops

__all__ = ["SelectedIndexTracer", "read_idx_tracer", "idx_tracer", "set_tracer", "suggest_filter_layers",
           "schedule_quality"]


class SelectedIndexTracer:
    """tiny_tools/tensor_tools.py:38-85, without the pickle.

    `observe()` is what a decoder layer calls at decode time; `end_step()` closes a
    token.  `keep` > 0 also records, per layer and step, the `keep` best (index, value)
    pairs in descending order of value like the reference's append_spec_layer."""

    def __init__(self, desc: Optional[str] = None, num_selected_tokens=0.067, keep: int = 0,
                 save_dir: str = "debug_logs"):
        self.desc = desc if desc is not None else os.environ.get("SAVE_SELECTED_IDX", "trace")
        self.save_path = os.path.join(save_dir, f"selected_index_{self.desc}.pt")
        self.num_selected_tokens = num_selected_tokens
        self.keep = keep
        self.num_samples = 0
        self.layers_idx: Dict[int, Dict[int, List[dict]]] = {}
        self.outs: List = []
        self._step: Dict[int, Tuple[torch.Tensor, torch.Tensor]] = {}
        self.steps = 0
        self.mass: Optional[torch.Tensor] = None      # [L, L] running sums, fp64 on the GPU
        self.overlap: Optional[torch.Tensor] = None
        self.seen: Optional[torch.Tensor] = None      # how many steps saw both layers

    # ---------------------------------------------------------------- the reference's recorder
    def append_out(self, out) -> None:
        self.outs.append(out)

    def append_spec_layer(self, idx: torch.Tensor, v: torch.Tensor, prefill_len: int, layer_idx: int) -> None:
        assert idx.dim() == 2 and v.dim() == 2
        per_layer = self.layers_idx.setdefault(self.num_samples, {}).setdefault(int(layer_idx), [])
        per_layer.append({"idx": idx.to("cpu"), "value": v.to("cpu"), "prefill_len": int(prefill_len)})

    # ---------------------------------------------------------------- the per-layer hook
    def _k(self, consider_len: int) -> int:
        k = self.num_selected_tokens
        if isinstance(k, float):
            k = int(k * consider_len)
        return max(1, min(int(k), consider_len))

    @torch.no_grad()
    def observe(self, layer_idx: int, query_states: torch.Tensor, key_states, consider_len: int) -> None:
        """query_states (bsz, Hq, 1, D) rotated; key_states the layer's resident K
        (bsz, Hkv, >=consider_len, D) or an ops.PagedKV.  Request 0 is traced."""
        if not getattr(key_states, "is_cuda", True):
            raise ValueError(f"layer {layer_idx}: tracing needs the layer's keys on the GPU "
                             "(trace with real_offload off, or with every layer dense)")
        s = ops.score(query_states, key_states, score_len=consider_len, selector="last")
        idx = ops.topk(s, self._k(consider_len))
        p = torch.softmax(s[0].float(), dim=-1)
        self._step[int(layer_idx)] = (p, idx[0].long())
        if self.keep > 0:
            v, order = torch.topk(p, min(self.keep, p.numel()), sorted=True)
            self.append_spec_layer(order[None], v[None], consider_len, layer_idx)

    @torch.no_grad()
    def end_step(self, num_layers: int) -> None:
        """Fold the layers seen since the last call into `mass` and `overlap`."""
        if not self._step:
            return
        dev = next(iter(self._step.values()))[0].device
        if self.mass is None:
            self.mass = torch.zeros((num_layers, num_layers), dtype=torch.float64, device=dev)
            self.overlap = torch.zeros_like(self.mass)
            self.seen = torch.zeros_like(self.mass)
        layers = sorted(self._step)
        n = self._step[layers[0]][0].numel()
        member = torch.zeros((len(layers), n), dtype=torch.float32, device=dev)
        probs = torch.stack([self._step[l][0] for l in layers])
        for r, l in enumerate(layers):
            member[r, self._step[l][1]] = 1.0
        ksel = member.sum(dim=1, keepdim=True)
        m = (member @ probs.t()).double()                   # [i, j] = sum of p_j over layer i's choice
        o = ((member @ member.t()) / ksel).double()
        li = torch.tensor(layers, device=dev)
        self.mass[li[:, None], li[None, :]] += m
        self.overlap[li[:, None], li[None, :]] += o
        self.seen[li[:, None], li[None, :]] += 1
        self._step.clear()
        self.steps += 1

    def matrices(self) -> Tuple[torch.Tensor, torch.Tensor]:
        """(mass, overlap) averaged over the traced steps, on the CPU; NaN where never seen."""
        if self.mass is None:
            raise RuntimeError("nothing traced yet")
        seen = self.seen.cpu()
        nan = torch.full_like(seen, float("nan"))
        return (torch.where(seen > 0, self.mass.cpu() / seen.clamp(min=1), nan),
                torch.where(seen > 0, self.overlap.cpu() / seen.clamp(min=1), nan))

    # ---------------------------------------------------------------- persistence
    def save_idx(self) -> str:
        if torch.cuda.is_available():
            torch.cuda.synchronize()
        os.makedirs(os.path.dirname(self.save_path) or ".", exist_ok=True)
        blob = {"out": self.outs, "layers_idx": self.layers_idx, "steps": self.steps}
        if self.mass is not None:
            blob["mass"], blob["overlap"] = self.matrices()
        torch.save(blob, self.save_path)
        self.num_samples += 1
        return self.save_path


def read_idx_tracer(path: str) -> dict:
    """Load a file written by SelectedIndexTracer.save_idx (tensors and plain containers only)."""
    return torch.load(path, weights_only=True)


# Process-wide tracer, like the reference's tiny_tools.tensor_tools.idx_tracer: created at import
# when SAVE_SELECTED_IDX is set, or installed with set_tracer().
idx_tracer: Optional[SelectedIndexTracer] = None
if os.environ.get("SAVE_SELECTED_IDX", False):
    idx_tracer = SelectedIndexTracer()


def set_tracer(tracer: Optional[SelectedIndexTracer]) -> Optional[SelectedIndexTracer]:
    global idx_tracer
    previous, idx_tracer = idx_tracer, tracer
    return previous


# -------------------------------------------------------------------- choosing filter layers
def _schedule(filters: Sequence[int], num_layers: int, wait: int):
    """layer -> filter whose selection it reads, for the layers that read one
    (modeling/spec_cache.py:271-281 with full_attn_layers = range(0, f0) + filters + [L])."""
    reads = {}
    for n, f in enumerate(filters):
        hi = filters[n + 1] if n + 1 < len(filters) else num_layers
        for j in range(min(hi, f + wait + 1), hi):
            reads[j] = f
    return reads


def schedule_quality(mass: torch.Tensor, filters: Sequence[int], num_wait_load_layers: int = 1) -> Tuple[float, int]:
    """(mean share of their own attention the sparse layers keep under this choice of
    filters, number of layers left dense)."""
    L = mass.shape[0]
    reads = _schedule(sorted(filters), L, num_wait_load_layers)
    if not reads:
        return float("nan"), L
    q = sum(float(mass[f, j]) for j, f in reads.items()) / len(reads)
    return q, L - len(reads)


def suggest_filter_layers(mass: torch.Tensor, num_filters: int = 3, num_wait_load_layers: int = 1,
                          max_dense_layers: Optional[int] = None) -> Tuple[List[int], float]:
    """The `do_select_layers` that keep the most attention mass in the sparse layers,
    among all choices of `num_filters` layers that leave at most `max_dense_layers`
    layers dense (default: a quarter of the model, the reference's 8 of 32).
    Exhaustive: C(32, 3) = 4960 schedules.  Returns (layers, quality)."""
    L = mass.shape[0]
    if max_dense_layers is None:
        max_dense_layers = max(num_filters * (1 + num_wait_load_layers) + 1, L // 4)
    best, best_q = None, -1.0
    count = 0
    for filters in itertools.combinations(range(L), num_filters):
        count += 1
        if count > 2_000_000:
            raise ValueError("too many schedules to enumerate; lower num_filters")
        q, dense = schedule_quality(mass, filters, num_wait_load_layers)
        if dense > max_dense_layers or q != q:
            continue
        if q > best_q:
            best, best_q = list(filters), q
    if best is None:
        raise ValueError(f"no schedule of {num_filters} filters leaves <= {max_dense_layers} layers dense")
    return best, best_q
