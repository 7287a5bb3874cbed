"""Filter-layer token selection with the reference's signature.

`select_tokens_by_attn_universal` mirrors modeling/omnikv.py:8-110: same
arguments, same selector names, same return value (ascending int64 indices,
shape (bsz, k), on the scores' device).  The matmul / softmax / head reduction and
the top-k + sort run in the HIP kernels; the q projection and RoPE stay torch ops.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import ops


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    x1, x2 = x[..., : x.shape[-1] // 2], x[..., x.shape[-1] // 2:]
    return torch.cat((-x2, x1), dim=-1)


def apply_rotary_pos_emb(q, k, cos, sin, unsqueeze_dim: int = 1):
    """Llama rotary embedding (third-party transformers 4.41.2, called at
    modeling/omnikv.py:34-35): x*cos + rotate_half(x)*sin, cos/sin (bsz, L, D)."""
    cos = cos.unsqueeze(unsqueeze_dim)
    sin = sin.unsqueeze(unsqueeze_dim)
    return q * cos + rotate_half(q) * sin, k * cos + rotate_half(k) * sin


def score_from_query(query_states: torch.Tensor, key_cache: torch.Tensor, consider_len: int,
                     selector_cls: str = "last") -> torch.Tensor:
    """(bsz, consider_len) fp32 scores of the first consider_len cached tokens: the part of
    modeling/omnikv.py:37-105 between the rotated query and the top-k."""
    if selector_cls in ops.SELECTOR_MODES:
        scores = ops.score(query_states[:, :, -1:, :], key_cache, score_len=consider_len, selector=selector_cls)
    elif selector_cls in ("uniform", "exp"):
        # modeling/omnikv.py:59-103: per window position softmax, head max; summed
        # (uniform) or folded with weight 1/2 per step of age (exp)
        scores = None
        if ops.window_supported(query_states, key_cache):  # all positions in two passes over K
            scores = ops.score_window(query_states, key_cache, score_len=consider_len, selector=selector_cls)
        for t in range(query_states.shape[2] if scores is None else 0):
            s = ops.score(query_states[:, :, t: t + 1, :], key_cache, score_len=consider_len,
                          selector="softmax_before_last")
            if scores is None:
                scores = s
            elif selector_cls == "uniform":
                scores += s
            else:
                scores = scores * 0.5 + s
    else:
        raise NotImplementedError(selector_cls)
    return scores


def select_from_query(query_states: torch.Tensor, key_cache: torch.Tensor, num_selected_tokens: int,
                      consider_len: int, selector_cls: str = "last") -> torch.Tensor:
    """query_states (bsz, Hq, Lq, D) already rotated; key_cache (bsz, Hkv, N, D) or an
    ops.PagedKV.  Returns ascending int64 indices (bsz, min(k, consider_len))."""
    scores = score_from_query(query_states, key_cache, consider_len, selector_cls)
    k = min(num_selected_tokens, scores.shape[-1])
    return ops.topk(scores, k).to(torch.int64)


def select_tokens_by_attn_universal(raw_attn, hidden_states, position_ids, past_key_value, num_selected_tokens,
                                    consider_len, layer_idx: Optional[int] = None, selector_cls: str = "last"):
    """modeling/omnikv.py:8-110.  raw_attn needs q_proj, num_heads, head_dim,
    rotary_emb(x, position_ids) -> (cos, sin), layer_idx and config.get()."""
    bsz, q_len, _ = hidden_states.size()
    assert past_key_value
    if raw_attn.config.get("pretraining_tp", -1) > 1:
        raise NotImplementedError
    query_states = raw_attn.q_proj(hidden_states)
    query_states = query_states.view(bsz, q_len, raw_attn.num_heads, raw_attn.head_dim).transpose(1, 2)
    cos, sin = raw_attn.rotary_emb(query_states, position_ids)
    query_states, _ = apply_rotary_pos_emb(query_states, query_states, cos, sin)
    key_states = past_key_value.key_cache[raw_attn.layer_idx]
    if not key_states.is_cuda:
        raise ValueError("the filter layer's keys must be GPU resident (filter layers are never offloaded)")
    return select_from_query(query_states.contiguous(), key_states, num_selected_tokens, consider_len, selector_cls)
