"""CPU oracle for the OmniKV dynamic-context-selection decode path.

TEST INFRASTRUCTURE ONLY.  This module restates, in plain torch on the CPU, the
arithmetic of the reference's filter-layer scoring, top-k selection, KV-cache
tiering and sparse / dense GQA decode attention.  It is the checker for the HIP
kernels: only tests, the smoke check and the bench's CPU-baseline leg may import
it.  Nothing in the product package imports this file, and the product never
falls back to it.

Each function cites the reference lines it follows (paths relative to the
reference checkout).  The attention arithmetic itself lives in a third-party
dependency of the reference (transformers==4.41.2, pinned in README.md:25; not
vendored): `repeat_kv`, `apply_rotary_pos_emb` and the Llama attention forward.
Those are restated here from their published textbook form (GQA softmax
attention with an fp32 softmax).

How each function is pinned (tests/test_oracle_*.py):
  * attn_logits / score_tokens  - pure-Python triple loops at tiny sizes, token
    permutation equivariance, positive-scale equivariance, per-head softmax
    mass (sum of the head-summed softmax score == number of q heads).
  * select_topk                 - brute-force rank on tiny inputs, the stable
    sort formulation, special cases k=N / k=1 / all-equal / +-inf / +-0 / NaN,
    hypothesis-driven set properties.
  * num_selected_tokens, layer_schedule, full_attn_layers_from_select_layers -
    closed-form integer tables written out by hand from the reference loops.
  * gqa_attention               - torch scaled_dot_product_attention (library
    routine), fp64 explicit loops at tiny sizes, idx=all reduces to dense.
  * score_tokens_by_kv_head, gqa_attention_by_kv_head - equal to the whole-tensor
    functions to fp32 rounding (the matrix products see other shapes).
  * paged_rows                  - scatter / gather round trip written with loops.
  * lightllm_raw_head_max_score - sqrt(D) times the `last` score.
  * lse_merge                   - joint softmax over the concatenation.
  * OracleMultiStageCache       - element-wise comparison with index_select +
    cat written independently in the test.
  * window selectors (uniform / exp) - explicit per-position Python loops.
No function here is "parity unpinned".
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence, Tuple

import torch

# --------------------------------------------------------------------------
# scoring (modeling/omnikv.py:8-110)
# --------------------------------------------------------------------------


def repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    """(b, Hkv, N, D) -> (b, Hkv*n_rep, N, D); q head h reads kv head h // n_rep.

    Third-party (transformers 4.41.2 `repeat_kv`, used at modeling/omnikv.py:38).
    """
    b, hkv, n, d = x.shape
    if n_rep == 1:
        return x
    return x[:, :, None, :, :].expand(b, hkv, n_rep, n, d).reshape(b, hkv * n_rep, n, d)


def attn_logits(q: torch.Tensor, k: torch.Tensor) -> torch.Tensor:
    """q (b,Hq,Lq,D) rotated, k (b,Hkv,N,D) -> (b,Hq,Lq,N) = q k^T / sqrt(D).

    modeling/omnikv.py:38-43 (repeat_kv, matmul, division by sqrt(head_dim)).
    """
    hq, hkv, d = q.shape[1], k.shape[1], q.shape[-1]
    kk = repeat_kv(k, hq // hkv)
    return torch.matmul(q, kk.transpose(2, 3)) / math.sqrt(d)


SELECTORS = ("last", "softmax_before_last", "softmax_sum_last", "uniform", "exp")


def score_tokens(
    q: torch.Tensor, k: torch.Tensor, consider_len: int, selector_cls: str = "last"
) -> torch.Tensor:
    """Per-token importance score (b, consider_len) before top-k.

    q: (b, Hq, Lq, D) query states of the window (Lq == 1 for the `last`
    family), already rotated.  k: (b, Hkv, N, D) cached keys of the filter
    layer; only the first `consider_len` tokens are scored
    (modeling/omnikv.py:37).

      last                 raw scaled logits of the last query row, max over q
                           heads (omnikv.py:40-46)
      softmax_before_last  softmax over the context per head, then max over
                           heads (omnikv.py:49-56)
      softmax_sum_last     softmax over the context per head, then SUM over
                           heads.  Not in the reference: the benchmark
                           configuration's variant.
      uniform              per window position: softmax, head max; summed over
                           the window (omnikv.py:59-80)
      exp                  same with weight 2^(t-W+1) for window position t
                           (omnikv.py:81-103; with one-row splits the recurrence
                           `attn_sum * 2**-1 + score` yields exactly that)
    """
    k = k[:, :, :consider_len]
    if selector_cls == "last":
        s = attn_logits(q, k)
        return torch.max(s[..., -1, :], dim=1).values
    if selector_cls == "softmax_before_last":
        s = torch.nn.functional.softmax(attn_logits(q, k), dim=-1)
        return torch.max(s[..., -1, :], dim=1).values
    if selector_cls == "softmax_sum_last":
        s = torch.nn.functional.softmax(attn_logits(q, k), dim=-1)
        return torch.sum(s[..., -1, :], dim=1)
    if selector_cls in ("uniform", "exp"):
        attn_sum = None
        for qi in torch.split(q, 1, dim=2):
            s = torch.nn.functional.softmax(attn_logits(qi, k), dim=-1)
            s = torch.max(s, dim=1).values  # (b, 1, N)
            if selector_cls == "uniform":
                s = torch.sum(s, dim=-2)
                attn_sum = s if attn_sum is None else attn_sum + s
            else:
                ql = s.shape[-2]
                alpha = 2.0 ** torch.arange(-ql + 1, 1)[None, :, None]
                s = torch.sum(s * alpha, dim=-2)
                attn_sum = s if attn_sum is None else attn_sum * (2.0**-ql) + s
        return attn_sum
    raise NotImplementedError(selector_cls)


def score_tokens_by_kv_head(
    q: torch.Tensor, k: torch.Tensor, consider_len: int, selector_cls: str = "last"
) -> torch.Tensor:
    """`score_tokens` of the `last` family evaluated one kv head at a time (the head
    reduction is then max of maxes / sum of sums): the same arithmetic without the
    4x repeated K of modeling/omnikv.py:38 held in memory at once, for the long
    contexts.  Softmax is per q head, so splitting by head changes no per-head value;
    only the order of the final additions over heads differs for the sum variant."""
    hq, hkv = q.shape[1], k.shape[1]
    g = hq // hkv
    parts = [
        score_tokens(q[:, g * i: g * (i + 1)], k[:, i: i + 1], consider_len, selector_cls)
        for i in range(hkv)
    ]
    stack = torch.stack(parts, dim=0)
    if selector_cls == "softmax_sum_last":
        return stack.sum(dim=0)
    if selector_cls in ("last", "softmax_before_last"):
        return stack.max(dim=0).values
    raise NotImplementedError(selector_cls)


def score_window_by_kv_head(
    q: torch.Tensor, k: torch.Tensor, consider_len: int, selector_cls: str = "uniform"
) -> torch.Tensor:
    """`score_tokens` of the window selectors (`uniform`, `exp`; modeling/omnikv.py:59-105)
    evaluated one kv head at a time for the long contexts: per window position the softmax is
    per q head and the head reduction a max, so the max over all q heads is the max over kv
    heads of the max over each group; the positions are then added up in the reference's
    order (`attn_sum + s`, or `attn_sum * 2**-1 + s` for `exp`).  Holds (group, W, N) logits of
    one kv head at a time instead of the (Hq, N) of every position over a 4x repeated K."""
    if selector_cls not in ("uniform", "exp"):
        raise NotImplementedError(selector_cls)
    hq, hkv = q.shape[1], k.shape[1]
    g = hq // hkv
    k = k[:, :, :consider_len]
    per_pos = None  # (b, W, N): max over the q heads seen so far of their softmax probabilities
    for i in range(hkv):
        p = torch.nn.functional.softmax(attn_logits(q[:, g * i: g * (i + 1)], k[:, i: i + 1]), dim=-1)
        p = torch.max(p, dim=1).values
        per_pos = p if per_pos is None else torch.maximum(per_pos, p)
    attn_sum = None
    for w in range(per_pos.shape[1]):
        s = per_pos[:, w]
        if attn_sum is None:
            attn_sum = s
        elif selector_cls == "uniform":
            attn_sum = attn_sum + s
        else:
            attn_sum = attn_sum * (2.0 ** -1) + s
    return attn_sum


# --------------------------------------------------------------------------
# top-k (modeling/omnikv.py:47-48,109-110)
# --------------------------------------------------------------------------


def select_topk(scores: torch.Tensor, k: int) -> torch.Tensor:
    """(b, N) scores -> (b, min(k,N)) int64 indices, ascending.

    modeling/omnikv.py:47-48 (`min`, `torch.topk(sorted=True)`) then :109
    (`torch.sort(idx)`).  torch.topk does not define which of several equal
    values at the k-th boundary it keeps; use `select_topk_stable` for the
    deterministic refinement.
    """
    k = min(k, scores.shape[-1])
    _, idx = torch.topk(scores, k=k, dim=-1, sorted=True)
    return torch.sort(idx, descending=False).values


def canonical_key(scores: torch.Tensor) -> torch.Tensor:
    """Order-preserving int64 key of an fp32 score: -0.0 == +0.0, every NaN is
    the single largest key (torch.topk ranks NaN above +inf)."""
    s = scores.to(torch.float32).contiguous()
    u = s.view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    u = torch.where(u == 0x80000000, torch.zeros_like(u), u)
    key = torch.where(u >= 0x80000000, 0xFFFFFFFF - u, u + 0x80000000)
    return torch.where(torch.isnan(s), torch.full_like(key, 0xFFFFFFFF), key)


def select_topk_stable(scores: torch.Tensor, k: int) -> torch.Tensor:
    """Same set as `select_topk` whenever the k-th and (k+1)-th largest values
    differ; among values equal to the k-th it keeps the lowest indices."""
    k = min(k, scores.shape[-1])
    key = canonical_key(scores)
    order = torch.sort(key, dim=-1, descending=True, stable=True).indices[..., :k]
    return torch.sort(order, dim=-1).values


def has_boundary_tie(scores: torch.Tensor, k: int) -> bool:
    """True when the k-th and (k+1)-th largest keys of any row are equal."""
    n = scores.shape[-1]
    if k >= n or k < 1:
        return False
    key = torch.sort(canonical_key(scores), dim=-1, descending=True).values
    return bool((key[..., k - 1] == key[..., k]).any())


# --------------------------------------------------------------------------
# integer host logic
# --------------------------------------------------------------------------


def num_selected_tokens(num_of_selected_tokens, prefill_len: int) -> int:
    """modeling/omnikv.py:168-171: a float is a ratio of the prefill length and
    is truncated with int(); an int passes through."""
    if isinstance(num_of_selected_tokens, float):
        return int(num_of_selected_tokens * prefill_len)
    return num_of_selected_tokens


def window_adjust(
    num_selected: int, consider_len: int, window_size: int, decode_step: int
) -> Tuple[int, int, int]:
    """modeling/omnikv.py:177-188 for the window selectors: the last
    `window_size - decode_step` prefill tokens are force-kept, so they leave
    both the scored range and the budget.  Returns (k, consider_len, forced)."""
    forced = max(0, window_size - decode_step)
    return max(1, num_selected - forced), consider_len - forced, forced


def full_attn_layers_from_select_layers(
    do_select_layers: Sequence[int], num_hidden_layers: int
) -> List[int]:
    """modeling/omnikv.py:322-331."""
    sel = list(do_select_layers)
    return list(range(0, sel[0])) + sel + [num_hidden_layers]


def layer_schedule(
    full_attn_layers: Sequence[int], num_hidden_layers: int, num_wait_load_layers: int
) -> Dict[int, Tuple[bool, int, int]]:
    """layer -> (reads only selected rows, its filter layer, next full layer).

    modeling/spec_cache.py:271-281.
    """
    state: Dict[int, Tuple[bool, int, int]] = {}
    for lo in full_attn_layers:
        hi = num_hidden_layers
        for i in range(lo + 1, num_hidden_layers):
            if i in full_attn_layers:
                hi = i
                break
        for i in range(lo, min(hi, lo + num_wait_load_layers + 1)):
            state[i] = (False, lo, hi)
        for i in range(min(hi, lo + num_wait_load_layers + 1), hi):
            state[i] = (True, lo, hi)
    return state


# --------------------------------------------------------------------------
# attention (third-party transformers 4.41.2 Llama attention, called at
# modeling/omnikv.py:219-227; textbook GQA softmax attention, fp32 softmax)
# --------------------------------------------------------------------------


def gqa_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """q (b,Hq,Lq,D), k/v (b,Hkv,L,D) -> (b,Hq,Lq,D) in q's dtype.

    No mask: a decode query attends to every cached row it is given.
    """
    n_rep = q.shape[1] // k.shape[1]
    w = attn_logits(q, k)
    w = torch.nn.functional.softmax(w, dim=-1, dtype=torch.float32).to(q.dtype)
    return torch.matmul(w, repeat_kv(v, n_rep))


def gqa_attention_by_kv_head(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """`gqa_attention` one kv head at a time (heads are independent: same values), so
    that the repeated K and V of a 450K-token context are never held whole."""
    g = q.shape[1] // k.shape[1]
    return torch.cat(
        [gqa_attention(q[:, g * i: g * (i + 1)], k[:, i: i + 1], v[:, i: i + 1]) for i in range(k.shape[1])],
        dim=1,
    )


def attention_partial(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Normalised attention over one segment and its log-sum-exp, both fp32.

    The form split-context flash decoding stores per split
    (omnikv-lightllm/.../flash_decoding_stage1.py:222-237: acc/sum_exp and
    max + log(sum_exp))."""
    n_rep = q.shape[1] // k.shape[1]
    w = attn_logits(q.float(), k.float())
    lse = torch.logsumexp(w, dim=-1)
    o = torch.matmul(torch.exp(w - lse[..., None]), repeat_kv(v.float(), n_rep))
    return o, lse


def lse_merge(parts: Sequence[Tuple[torch.Tensor, torch.Tensor]]) -> torch.Tensor:
    """Merge per-segment (o, lse) pairs into the joint softmax attention.

    omnikv-lightllm/.../flash_decoding_stage2.py:24-43."""
    lse = torch.stack([p[1] for p in parts], dim=0)
    o = torch.stack([p[0] for p in parts], dim=0)
    m = lse.max(dim=0).values
    w = torch.exp(lse - m[None])
    return (o * w[..., None]).sum(0) / w.sum(0)[..., None]


# --------------------------------------------------------------------------
# cache tiering (modeling/spec_cache.py:253-385)
# --------------------------------------------------------------------------


def gather_rows(cache: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
    """(b,Hkv,N,D), (k,) -> (b,Hkv,k,D).  modeling/spec_cache.py:298-303."""
    return torch.index_select(cache, 2, idx.view(-1))


def idx_overlap_score(new_idx: torch.Tensor, old_idx: torch.Tensor) -> float:
    """get_idx_iou_score (modeling/spec_cache.py:10-32): the count of indices the two
    1-D tensors share, divided by the length of the NEW one (the reference's comment
    says so too: the union is deliberately not used)."""
    assert new_idx.dim() == 1 and old_idx.dim() == 1
    un = torch.cat([new_idx, old_idx], dim=0).unique().shape[0]
    return (new_idx.shape[0] + old_idx.shape[0] - un) / new_idx.shape[0]


class OracleMultiStageCache:
    """Plain-torch restatement of OmniKVMultiStageCache
    (modeling/spec_cache.py:253-385), all tensors on the CPU.

    Same attribute names and the same update / set_idx_on_gpu behaviour; the
    only thing left out is device placement, which does not change values.
    """

    def __init__(
        self,
        full_attn_layers: List[int],
        num_hidden_layers: int,
        num_wait_load_layers: int = 2,
        real_offload: bool = True,
    ):
        self.stage = "prefill"
        self.full_attn_layers = full_attn_layers
        self.num_hidden_layers = num_hidden_layers
        self.num_wait_layers = num_wait_load_layers
        self.real_offload = real_offload
        self.layer_state = layer_schedule(
            full_attn_layers, num_hidden_layers, num_wait_load_layers
        )
        self.key_cache: List[torch.Tensor] = []
        self.value_cache: List[torch.Tensor] = []
        self._seen_tokens = 0
        self.part_key: Dict[int, torch.Tensor] = {}
        self.part_value: Dict[int, torch.Tensor] = {}
        self.tail_k: Dict[int, torch.Tensor] = {}
        self.tail_v: Dict[int, torch.Tensor] = {}

    def set_idx_on_gpu(self, idx: torch.Tensor, sel_layer_idx: int) -> None:
        """spec_cache.py:290-306."""
        _idx = idx.view(-1)
        hi = self.layer_state[sel_layer_idx][2]
        for i in range(sel_layer_idx + self.num_wait_layers + 1, hi):
            self.part_key[i] = gather_rows(self.key_cache[i], _idx)
            self.part_value[i] = gather_rows(self.value_cache[i], _idx)

    def update(
        self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int
    ) -> Tuple[torch.Tensor, torch.Tensor]:
        """spec_cache.py:308-369."""
        if layer_idx == 0:
            self._seen_tokens += key_states.shape[-2]
        if self.layer_state[layer_idx][0]:
            if self.stage == "prefill":
                self.key_cache.append(key_states)
                self.value_cache.append(value_states)
                return key_states, value_states
            if layer_idx not in self.tail_k:
                self.tail_k[layer_idx] = key_states
                self.tail_v[layer_idx] = value_states
            else:
                self.tail_k[layer_idx] = torch.cat(
                    [self.tail_k[layer_idx], key_states], dim=-2
                )
                self.tail_v[layer_idx] = torch.cat(
                    [self.tail_v[layer_idx], value_states], dim=-2
                )
            return (
                torch.cat([self.part_key[layer_idx], self.tail_k[layer_idx]], dim=-2),
                torch.cat([self.part_value[layer_idx], self.tail_v[layer_idx]], dim=-2),
            )
        if len(self.key_cache) <= layer_idx:
            self.key_cache.append(key_states)
            self.value_cache.append(value_states)
        else:
            self.key_cache[layer_idx] = torch.cat(
                [self.key_cache[layer_idx], key_states], dim=-2
            )
            self.value_cache[layer_idx] = torch.cat(
                [self.value_cache[layer_idx], value_states], dim=-2
            )
        return self.key_cache[layer_idx], self.value_cache[layer_idx]


# --------------------------------------------------------------------------
# one filter-layer op end to end (the CPU-runnable benchmark configuration)
# --------------------------------------------------------------------------


def filter_layer_op(
    q: torch.Tensor,
    k: torch.Tensor,
    v_next: torch.Tensor,
    k_next: torch.Tensor,
    q_next: torch.Tensor,
    num_selected: int,
    selector_cls: str = "last",
    tail_k: Optional[torch.Tensor] = None,
    tail_v: Optional[torch.Tensor] = None,
):
    """score -> top-k -> gather -> sparse attention of one downstream layer.

    Follows omnikv.py:189-212 (select + set_idx_on_gpu) and
    spec_cache.py:337-356 (part ++ tail) with the attention of
    `gqa_attention`.  Returns (idx, scores, attention output)."""
    n = k.shape[2]
    scores = score_tokens(q, k, n, selector_cls)
    idx = select_topk(scores, num_selected)
    pk = gather_rows(k_next, idx[0])
    pv = gather_rows(v_next, idx[0])
    if tail_k is not None:
        pk = torch.cat([pk, tail_k], dim=-2)
        pv = torch.cat([pv, tail_v], dim=-2)
    return idx, scores, gqa_attention(q_next, pk, pv)


# --------------------------------------------------------------------------
# paged / token-indirected variant
# (omnikv-lightllm/lightllm/models/llama_omnikv/triton_kernel/flash_decoding.py:33-112,
#  flash_decoding_stage1.py:117-238, common/req_manager.py:12-17,
#  common/mem_manager.py:101-105)
# --------------------------------------------------------------------------


def paged_rows(
    pool: torch.Tensor, page_table: torch.Tensor, seq_len: int, page_size: int
) -> torch.Tensor:
    """pool (num_pages, page_size, Hkv, D), page_table (max_pages,) int ->
    (1, Hkv, seq_len, D): logical token t lives in page page_table[t // page_size],
    slot t % page_size.  page_size == 1 is the reference's token-slot table
    (req_to_token_indexs)."""
    t = torch.arange(seq_len)
    rows = pool[page_table[t // page_size].long(), t % page_size]  # (seq, Hkv, D)
    return rows.permute(1, 0, 2)[None]


def lightllm_raw_head_max_score(q: torch.Tensor, k: torch.Tensor) -> torch.Tensor:
    """The serving path's score: UNSCALED q.k per head (the kernel stores the
    dot product before applying sm_scale, flash_decoding_stage1.py:198-208),
    then max over heads (flash_decoding.py:76).  Rank-equivalent to `last`."""
    hq, hkv = q.shape[1], k.shape[1]
    s = torch.matmul(q, repeat_kv(k, hq // hkv).transpose(2, 3))
    return s[..., -1, :].max(dim=1).values
