"""Torch-tensor front end of the HIP kernels (one function per C entry point).

Tensors stay torch tensors; this module only extracts pointers, strides and the
current stream and calls libomnikv_hip.so.  K / V are accepted in the reference's
shape (bsz, num_kv_heads, tokens, head_dim) with ANY strides whose last dimension
is contiguous, so both the reference's contiguous cache tensors and views of a
token-major store are read in place.
"""
from __future__ import annotations

import ctypes as C
import math
from dataclasses import dataclass
from typing import Dict, Optional, Tuple

import torch

from . import _lib
from ._lib import KVLayout, Shape, check, lib

_DTYPES = {torch.float32: _lib.OKV_F32, torch.bfloat16: _lib.OKV_BF16, torch.float16: _lib.OKV_F16}
_REDUCE = {"max": _lib.OKV_REDUCE_MAX, "sum": _lib.OKV_REDUCE_SUM}
_NORM = {"raw": _lib.OKV_NORM_RAW, "softmax": _lib.OKV_NORM_SOFTMAX}

# selector name -> (normalise, head_reduce); modeling/omnikv.py:40-58 plus the
# benchmark's softmax-sum variant.
SELECTOR_MODES = {
    "last": ("raw", "max"),
    "softmax_before_last": ("softmax", "max"),
    "softmax_sum_last": ("softmax", "sum"),
}


@dataclass
class PagedKV:
    """A paged K/V pool: pool_k / pool_v (num_pages, page_size, Hkv, D) and
    page_table (bsz, max_pages) int32.  page_size == 1 is a token-slot table."""

    pool_k: torch.Tensor
    pool_v: torch.Tensor
    page_table: torch.Tensor
    page_size: int

    def slot_index(self, idx: torch.Tensor) -> torch.Tensor:
        """Token positions (bsz, k) int32 -> rows of the pool seen as one flat array of token
        slots: page_table[b, t // page_size] * page_size + t % page_size.  Composed once per
        selection (the reference's serving stack keeps exactly such a table per request,
        req_to_imp_token_indexs, common/req_manager.py:12-17), every sparse layer of the
        group then reads its rows with one lookup instead of two.  Padding entries (< 0)
        stay padding."""
        if self.pool_k.stride(0) != self.page_size * self.pool_k.stride(1):
            raise ValueError("the pool's pages must lie back to back")
        t = idx.clamp(min=0).to(torch.int64)
        page = (t // self.page_size).clamp(max=self.page_table.shape[1] - 1)  # a stray entry never reads outside the table
        slots = self.page_table.gather(1, page).to(torch.int64) * self.page_size + t % self.page_size
        return torch.where(idx < 0, idx, slots.to(torch.int32))


_workspaces: Dict[Tuple[int, int], torch.Tensor] = {}


def _stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


_retired: list = []  # outgrown scratch buffers: captured graphs may still hold their addresses


def _workspace(device, nbytes: int) -> torch.Tensor:
    """One growing scratch buffer per (device, stream).  It at least doubles when it grows and
    the buffer it replaces stays allocated (a HIP graph captured earlier keeps launching with
    the old address), so what is held in total is bounded by twice the largest request."""
    key = (device.index if device.index is not None else torch.cuda.current_device(), _stream_ptr(device))
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        if ws is not None:
            _retired.append(ws)
        ws = torch.empty(max(nbytes, 1 << 20, 2 * ws.numel() if ws is not None else 0), dtype=torch.uint8,
                         device=device)
        _workspaces[key] = ws
    return ws


def workspace_bytes(op: int, batch: int, hq: int, hkv: int, d: int, max_seq_len: int,
                    max_tail_len: int = 0, with_scores: bool = False) -> int:
    shape = Shape(batch, hq, hkv, d, max_seq_len, max_tail_len, int(with_scores))
    out = C.c_size_t(0)
    check(lib().okv_workspace_bytes(op, C.byref(shape), C.byref(out)))
    return out.value


def _require_gpu(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise ValueError(f"{name} must be a GPU tensor (the HIP path has no CPU fallback)")


def _layout(k, v, hq: int):
    """(layout struct, k ptr, v ptr, batch, tokens) for tensors or a PagedKV."""
    if isinstance(k, PagedKV):
        pk = k
        pool_k, pool_v = pk.pool_k, pk.pool_v
        if pool_k.dim() != 4 or pool_k.stride(-1) != 1:
            raise ValueError("pool_k must be (pages, page_size, Hkv, D) with contiguous D")
        if pool_v is not None and pool_v.stride() != pool_k.stride():
            raise ValueError("pool_k and pool_v must share strides")
        pt = pk.page_table
        if pt.dtype != torch.int32 or pt.dim() != 2 or pt.stride(1) != 1:
            raise ValueError("page_table must be (bsz, max_pages) int32, rows contiguous")
        lay = KVLayout(
            _DTYPES[pool_k.dtype], hq, pool_k.shape[2], pool_k.shape[3],
            pool_k.stride(1), pool_k.stride(2), 0,
            pt.data_ptr(), pk.page_size, pt.stride(0), pool_k.stride(0),
        )
        return lay, pool_k.data_ptr(), (pool_v.data_ptr() if pool_v is not None else pool_k.data_ptr()), pt.shape[0], None
    if k.dim() != 4 or k.stride(-1) != 1:
        raise ValueError("K must be (bsz, Hkv, tokens, D) with a contiguous last dimension")
    if v is not None and (v.shape != k.shape or v.stride() != k.stride() or v.dtype != k.dtype):
        raise ValueError("K and V must share shape, strides and dtype")
    lay = KVLayout(
        _DTYPES[k.dtype], hq, k.shape[1], k.shape[3],
        k.stride(2), k.stride(1), k.stride(0), None, 0, 0, 0,
    )
    return lay, k.data_ptr(), (v.data_ptr() if v is not None else k.data_ptr()), k.shape[0], k.shape[2]


def _q3(q: torch.Tensor) -> torch.Tensor:
    if q.dim() == 4:
        if q.shape[2] != 1:
            raise ValueError("q must hold one query row per head")
        q = q[:, :, 0, :]
    return q.contiguous()


def _same_dtype(q: torch.Tensor, lay) -> None:
    if _DTYPES.get(q.dtype) != lay.dtype:
        raise ValueError("q and K/V must have the same dtype (float32, bfloat16 or float16)")


def _lens(t: Optional[torch.Tensor], batch: int, name: str) -> int:
    if t is None:
        return 0
    if t.dtype != torch.int32 or not t.is_cuda or t.numel() != batch or not t.is_contiguous():
        raise ValueError(f"{name} must be a contiguous int32 GPU tensor of {batch} entries")
    return t.data_ptr()


def score(q, k, score_len: Optional[int] = None, selector: str = "last", scale: Optional[float] = None,
          score_lens: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """(bsz, score_len) fp32 filter-layer scores; okv_score."""
    q = _q3(q)
    _require_gpu(q, "q")
    hq, d = q.shape[1], q.shape[2]
    lay, kp, _, batch, n = _layout(k, None, hq)
    _same_dtype(q, lay)
    if score_len is None:
        if n is None:
            raise ValueError("score_len is required with a paged pool")
        score_len = n
    norm, red = SELECTOR_MODES[selector]
    if out is None:
        out = torch.empty((batch, score_len), dtype=torch.float32, device=q.device)
    nbytes = workspace_bytes(_lib.OKV_OP_SCORE, batch, hq, lay.num_kv_heads, d, score_len)
    ws = _workspace(q.device, nbytes)
    check(lib().okv_score(
        q.data_ptr(), kp, C.byref(lay), _lens(score_lens, batch, "score_lens"), score_len, batch,
        _REDUCE[red], _NORM[norm], scale if scale is not None else 1.0 / math.sqrt(d),
        out.data_ptr(), out.stride(0), ws.data_ptr(), ws.numel(), _stream_ptr(q.device)))
    return out


def window_supported(q: torch.Tensor, k) -> bool:
    """Whether score_window takes these operands (else: one `score` call per position)."""
    if isinstance(k, PagedKV) or q.dim() != 4 or q.dtype not in (torch.bfloat16, torch.float16):
        return False
    hq, w = q.shape[1], q.shape[2]
    hkv = k.shape[1]
    if k.dtype != q.dtype or hkv > 8 or hq % hkv:
        return False
    return hq // hkv in (1, 2, 4, 8) and w * (hq // hkv) <= 64  # the kernel's max over a kv head's q heads pairs lanes


def score_window(q, k, score_len: Optional[int] = None, selector: str = "uniform", scale: Optional[float] = None,
                 score_lens: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """(bsz, score_len) fp32 scores of the window selectors; okv_score_window.
    q: (bsz, Hq, W, D), the last W query positions, oldest first."""
    _require_gpu(q, "q")
    if selector not in ("uniform", "exp"):
        raise ValueError(f"selector {selector!r} is not a window selector")
    if q.dim() != 4 or q.stride(3) != 1:
        raise ValueError("q must be (bsz, Hq, W, D) with contiguous D")
    hq, w, d = q.shape[1], q.shape[2], q.shape[3]
    lay, kp, _, batch, n = _layout(k, None, hq)
    _same_dtype(q, lay)
    if score_len is None:
        score_len = n
    if out is None:
        out = torch.empty((batch, score_len), dtype=torch.float32, device=q.device)
    nbytes = workspace_bytes(_lib.OKV_OP_SCORE_WINDOW, batch, hq, lay.num_kv_heads, d, score_len)
    ws = _workspace(q.device, nbytes)
    check(lib().okv_score_window(
        q.data_ptr(), q.stride(0), q.stride(1), q.stride(2), w, int(selector == "exp"), kp, C.byref(lay),
        _lens(score_lens, batch, "score_lens"), score_len, batch,
        scale if scale is not None else 1.0 / math.sqrt(d),
        out.data_ptr(), out.stride(0), ws.data_ptr(), ws.numel(), _stream_ptr(q.device)))
    return out


def dense_attn_window(q, q_window, k, v, selector: str = "uniform", seq_len: Optional[int] = None,
                      seq_lens: Optional[torch.Tensor] = None, score_len: Optional[int] = None,
                      score_lens: Optional[torch.Tensor] = None, scale: Optional[float] = None,
                      scores_out: Optional[torch.Tensor] = None):
    """A window-selector filter layer in two passes over K: (out, scores) = (dense_attn(q, k, v),
    score_window(q_window, k, score_len)) with the first scoring pass done inside the attention's;
    okv_dense_attn_window.  q: (bsz, Hq, D) or (bsz, Hq, 1, D); q_window: (bsz, Hq, W, D), oldest first."""
    q = _q3(q)
    _require_gpu(q, "q")
    _require_gpu(q_window, "q_window")
    if selector not in ("uniform", "exp"):
        raise ValueError(f"selector {selector!r} is not a window selector")
    if q_window.dim() != 4 or q_window.stride(3) != 1 or q_window.dtype != q.dtype:
        raise ValueError("q_window must be (bsz, Hq, W, D) with contiguous D and q's dtype")
    hq, d = q.shape[1], q.shape[2]
    if q_window.shape[0] != q.shape[0] or q_window.shape[1] != hq or q_window.shape[3] != d:
        raise ValueError("q_window does not match q")
    lay, kp, vp, batch, n = _layout(k, v, hq)
    _same_dtype(q, lay)
    if seq_len is None:
        seq_len = n
    if score_len is None:
        score_len = seq_len
    out = torch.empty_like(q)
    scores = scores_out
    if scores is None:
        scores = torch.empty((batch, score_len), dtype=torch.float32, device=q.device)
    elif scores.shape != (batch, score_len) or scores.dtype != torch.float32 or scores.stride(1) != 1:
        raise ValueError("scores_out must be (bsz, score_len) float32 with contiguous rows")
    nbytes = workspace_bytes(_lib.OKV_OP_DENSE_ATTN_WINDOW, batch, hq, lay.num_kv_heads, d, seq_len)
    ws = _workspace(q.device, nbytes)
    check(lib().okv_dense_attn_window(
        q.data_ptr(), q_window.data_ptr(), q_window.stride(0), q_window.stride(1), q_window.stride(2),
        q_window.shape[2], int(selector == "exp"), kp, vp, C.byref(lay), _lens(seq_lens, batch, "seq_lens"), seq_len,
        batch, scale if scale is not None else 1.0 / math.sqrt(d), out.data_ptr(),
        _lens(score_lens, batch, "score_lens"), score_len, scores.data_ptr(), scores.stride(0),
        ws.data_ptr(), ws.numel(), _stream_ptr(q.device)))
    return out, scores


def topk(scores: torch.Tensor, k: int, seq_lens: Optional[torch.Tensor] = None,
         k_per_seg: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """(bsz, min(k, N)) int32 ascending indices of the k largest scores; okv_topk."""
    _require_gpu(scores, "scores")
    if scores.dtype != torch.float32 or scores.dim() != 2 or scores.stride(1) != 1:
        raise ValueError("scores must be (bsz, N) float32 with contiguous rows")
    batch, n = scores.shape
    kk = min(k, n)
    if out is None:
        if seq_lens is None and k_per_seg is None:
            out = torch.empty((batch, kk), dtype=torch.int32, device=scores.device)
        else:  # ragged: the kernels leave entries beyond a request's own k untouched -> padding is -1
            out = torch.full((batch, kk), -1, dtype=torch.int32, device=scores.device)
    if kk == 0:
        return out
    ws = _workspace(scores.device, workspace_bytes(_lib.OKV_OP_TOPK, batch, 0, 0, 0, n))
    check(lib().okv_topk(
        scores.data_ptr(), scores.stride(0), _lens(seq_lens, batch, "seq_lens"), n,
        _lens(k_per_seg, batch, "k_per_seg"), k, batch, out.data_ptr(), out.stride(0),
        ws.data_ptr(), ws.numel(), _stream_ptr(scores.device)))
    return out


def dense_attn(q, k, v=None, seq_len: Optional[int] = None, seq_lens: Optional[torch.Tensor] = None,
               scale: Optional[float] = None, selector: Optional[str] = None,
               score_len: Optional[int] = None, score_lens: Optional[torch.Tensor] = None,
               scores_out: Optional[torch.Tensor] = None, select_k: Optional[int] = None,
               k_per_seg: Optional[torch.Tensor] = None, idx_out: Optional[torch.Tensor] = None):
    """Dense GQA decode attention; with `selector` also returns the filter-layer
    scores of the first score_len tokens from the same pass (okv_dense_attn), and with
    `select_k` on top of that the ascending indices of the select_k largest of them, as
    topk(scores, select_k, score_lens, k_per_seg) would: (out, scores, idx), the whole filter
    layer in one call (okv_dense_attn_select)."""
    q = _q3(q)
    _require_gpu(q, "q")
    hq, d = q.shape[1], q.shape[2]
    lay, kp, vp, batch, n = _layout(k, v, hq)
    _same_dtype(q, lay)
    if seq_len is None:
        if n is None:
            raise ValueError("seq_len is required with a paged pool")
        seq_len = n
    out = torch.empty_like(q)
    scores = None
    sp, ss, red, norm = None, 0, 0, 0
    if select_k is not None and selector is None:
        raise ValueError("select_k needs a selector")
    if selector is not None:
        norm_s, red_s = SELECTOR_MODES[selector]
        red, norm = _REDUCE[red_s], _NORM[norm_s]
        if score_len is None:
            score_len = seq_len
        scores = scores_out
        if scores is None:
            scores = torch.empty((batch, score_len), dtype=torch.float32, device=q.device)
        elif scores.shape != (batch, score_len) or scores.dtype != torch.float32 or scores.stride(1) != 1:
            raise ValueError("scores_out must be (bsz, score_len) float32 with contiguous rows")
        sp, ss = scores.data_ptr(), scores.stride(0)
    sc = scale if scale is not None else 1.0 / math.sqrt(d)
    if select_k is None:
        nbytes = workspace_bytes(_lib.OKV_OP_DENSE_ATTN, batch, hq, lay.num_kv_heads, d, seq_len,
                                 with_scores=selector is not None)
        ws = _workspace(q.device, nbytes)
        check(lib().okv_dense_attn(
            q.data_ptr(), kp, vp, C.byref(lay), _lens(seq_lens, batch, "seq_lens"), seq_len, batch,
            sc, out.data_ptr(), _lens(score_lens, batch, "score_lens"), score_len or 0, red, norm, sp, ss,
            ws.data_ptr(), ws.numel(), _stream_ptr(q.device)))
        return (out, scores) if selector is not None else out
    kk = min(select_k, score_len)
    idx = idx_out
    if idx is None:
        if score_lens is None and k_per_seg is None:
            idx = torch.empty((batch, kk), dtype=torch.int32, device=q.device)
        else:  # ragged: entries beyond a request's own k are left untouched -> padding is -1
            idx = torch.full((batch, kk), -1, dtype=torch.int32, device=q.device)
    elif idx.shape != (batch, kk) or idx.dtype != torch.int32 or idx.stride(1) != 1:
        raise ValueError("idx_out must be (bsz, min(select_k, score_len)) int32 with contiguous rows")
    nbytes = workspace_bytes(_lib.OKV_OP_DENSE_ATTN_SELECT, batch, hq, lay.num_kv_heads, d, seq_len,
                             with_scores=True)
    ws = _workspace(q.device, nbytes)
    check(lib().okv_dense_attn_select(
        q.data_ptr(), kp, vp, C.byref(lay), _lens(seq_lens, batch, "seq_lens"), seq_len, batch,
        sc, out.data_ptr(), _lens(score_lens, batch, "score_lens"), score_len, red, norm, sp, ss,
        _lens(k_per_seg, batch, "k_per_seg"), select_k, idx.data_ptr(), idx.stride(0),
        ws.data_ptr(), ws.numel(), _stream_ptr(q.device)))
    return out, scores, idx


def sparse_attn(q, k, v=None, idx: Optional[torch.Tensor] = None, sel_len: Optional[int] = None,
                sel_lens: Optional[torch.Tensor] = None, tail_k: Optional[torch.Tensor] = None,
                tail_v: Optional[torch.Tensor] = None, tail_len: Optional[int] = None,
                tail_lens: Optional[torch.Tensor] = None, scale: Optional[float] = None,
                slots: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention over rows idx of K/V followed by the tail rows; okv_sparse_attn.

    idx (bsz, k) int32 ascending, or None for rows [0, sel_len).  tail_k / tail_v
    are (bsz, Hkv, T, D) with any strides (last dimension contiguous)."""
    q = _q3(q)
    _require_gpu(q, "q")
    hq, d = q.shape[1], q.shape[2]
    if slots is not None:
        # rows of a paged pool addressed as token slots (PagedKV.slot_index): no page table
        if not isinstance(k, PagedKV) or idx is not None:
            raise ValueError("slots go with a PagedKV and replace idx")
        pool_k, pool_v = k.pool_k, k.pool_v
        lay = KVLayout(_DTYPES[pool_k.dtype], hq, pool_k.shape[2], pool_k.shape[3], pool_k.stride(1),
                       pool_k.stride(2), 0, None, 0, 0, 0)
        kp, vp, batch, n, idx = pool_k.data_ptr(), pool_v.data_ptr(), slots.shape[0], None, slots
    else:
        lay, kp, vp, batch, n = _layout(k, v, hq)
    _same_dtype(q, lay)
    ip, istride = None, 0
    if idx is not None:
        if idx.dtype != torch.int32 or idx.dim() != 2 or idx.stride(1) != 1 or not idx.is_cuda:
            raise ValueError("idx must be a (bsz, k) int32 GPU tensor with contiguous rows")
        ip, istride = idx.data_ptr(), idx.stride(0)
        if sel_len is None:
            sel_len = idx.shape[1]
    elif sel_len is None:
        sel_len = n
    tkp = tvp = None
    tts = ths = tbs = 0
    if tail_k is not None:
        if tail_k.dim() != 4 or tail_k.stride(-1) != 1 or tail_v.stride() != tail_k.stride():
            raise ValueError("tail_k / tail_v must be (bsz, Hkv, T, D), same strides, contiguous D")
        if tail_k.dtype != q.dtype:
            raise ValueError("tail dtype differs from q")
        if tail_len is None:
            tail_len = tail_k.shape[2]
        tkp, tvp = tail_k.data_ptr(), tail_v.data_ptr()
        tts, ths, tbs = tail_k.stride(2), tail_k.stride(1), tail_k.stride(0)
    tail_len = tail_len or 0
    out = torch.empty_like(q)
    nbytes = workspace_bytes(_lib.OKV_OP_SPARSE_ATTN, batch, hq, lay.num_kv_heads, d, sel_len, tail_len)
    ws = _workspace(q.device, nbytes)
    check(lib().okv_sparse_attn(
        q.data_ptr(), kp, vp, C.byref(lay), ip, istride, _lens(sel_lens, batch, "sel_lens"), sel_len,
        tkp, tvp, tts, ths, tbs, _lens(tail_lens, batch, "tail_lens"), tail_len, batch,
        scale if scale is not None else 1.0 / math.sqrt(d), out.data_ptr(),
        ws.data_ptr(), ws.numel(), _stream_ptr(q.device)))
    return out


def gather_rows(src, idx: torch.Tensor, out: Optional[torch.Tensor] = None,
                sel_lens: Optional[torch.Tensor] = None, hq: Optional[int] = None) -> torch.Tensor:
    """out[b, g, j, :] = src[b, g, idx[b, j], :]; okv_gather_rows.

    `out` may be any (bsz, Hkv, k, D) tensor with a contiguous last dimension;
    by default it is token-major storage viewed in that shape."""
    if idx.dtype != torch.int32 or idx.dim() != 2 or idx.stride(1) != 1 or not idx.is_cuda:
        raise ValueError("idx must be a (bsz, k) int32 GPU tensor with contiguous rows")
    probe = src.pool_k if isinstance(src, PagedKV) else src
    hkv = probe.shape[2] if isinstance(src, PagedKV) else probe.shape[1]
    lay, sp, _, batch, _ = _layout(src, None, hq or hkv)
    ksel = idx.shape[1]
    d = probe.shape[-1]
    if out is None:
        out = torch.empty((batch, ksel, hkv, d), dtype=probe.dtype, device=idx.device).permute(0, 2, 1, 3)
    if out.stride(-1) != 1 or out.shape != (batch, hkv, ksel, d):
        raise ValueError("out must be (bsz, Hkv, k, D) with a contiguous last dimension")
    check(lib().okv_gather_rows(
        sp, C.byref(lay), idx.data_ptr(), idx.stride(0), _lens(sel_lens, batch, "sel_lens"), ksel,
        batch, out.data_ptr(), out.stride(2), out.stride(1), out.stride(0), _stream_ptr(idx.device)))
    return out


# ---------------------------------------------------------------- per-token layer operations
def _same(*ts):
    t0 = ts[0]
    for t in ts:
        _require_gpu(t, "tensor")
        if t.dtype != t0.dtype or not t.is_contiguous():
            raise ValueError("operands must be contiguous GPU tensors of one dtype")
    if t0.dtype not in _DTYPES:
        raise ValueError("dtype must be float32, bfloat16 or float16")
    return _DTYPES[t0.dtype]


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, residual: Optional[torch.Tensor] = None):
    """weight * rms_normalise(x [+ residual]) over the last dimension; okv_rmsnorm.  Returns the
    normalised tensor, or (normalised, x + residual) when a residual is given."""
    dt = _same(x, weight) if residual is None else _same(x, weight, residual)
    hidden = x.shape[-1]
    rows = x.numel() // hidden
    out = torch.empty_like(x)
    total = torch.empty_like(x) if residual is not None else None
    check(lib().okv_rmsnorm(x.data_ptr(), residual.data_ptr() if residual is not None else None, weight.data_ptr(),
                            float(eps), rows, hidden, dt, total.data_ptr() if total is not None else None,
                            out.data_ptr(), _stream_ptr(x.device)))
    return out if residual is None else (out, total)


def _check_rope_tables(cos: torch.Tensor, sin: torch.Tensor, bsz: int, d: int) -> None:
    """The kernels read one row of d cos / sin values per request, back to back: a broadcast (1, 1, d) table
    next to bsz > 1 would be read past its end."""
    if d != 128:
        raise ValueError("the rotary kernels are built for head_dim 128")
    if tuple(cos.shape) != (bsz, 1, d) or tuple(sin.shape) != (bsz, 1, d):
        raise ValueError(f"cos / sin must be (bsz, 1, head_dim) = ({bsz}, 1, {d}), one row per request; "
                         f"got {tuple(cos.shape)} and {tuple(sin.shape)} (expand a shared row first)")


def rope(q: torch.Tensor, k: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, num_q_heads: int,
         num_kv_heads: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Rotary embedding of one position per request: q (bsz, 1, Hq*D) and k (bsz, 1, Hkv*D) as the
    projections leave them, cos / sin (bsz, 1, D); returns (bsz, Hq, 1, D) and (bsz, Hkv, 1, D).  okv_rope."""
    dt = _same(q, k, cos, sin)
    bsz = q.shape[0]
    d = cos.shape[-1]
    if q.shape[1] != 1 or q.shape[-1] != num_q_heads * d or k.shape[-1] != num_kv_heads * d:
        raise ValueError("q / k must be (bsz, 1, heads * head_dim)")
    _check_rope_tables(cos, sin, bsz, d)
    q_out = torch.empty((bsz, num_q_heads, 1, d), dtype=q.dtype, device=q.device)
    k_out = torch.empty((bsz, num_kv_heads, 1, d), dtype=q.dtype, device=q.device)
    check(lib().okv_rope(q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0), cos.data_ptr(), sin.data_ptr(), bsz,
                         num_q_heads, num_kv_heads, d, dt, q_out.data_ptr(), k_out.data_ptr(), _stream_ptr(q.device)))
    return q_out, k_out


def rope_append(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                num_q_heads: int, num_kv_heads: int, k_store: torch.Tensor, v_store: torch.Tensor,
                pos) -> torch.Tensor:
    """`rope` whose rotated k row and the v row are written into k_store / v_store (bsz, Hkv, capacity, D) at
    token position `pos` (an int, or a one-element int64 GPU tensor read by the kernel); returns the rotated
    q (bsz, Hq, 1, D).  Every request of the batch is written at the SAME position (the static decode
    path advances all requests together); nothing on the device checks a device position against the
    store's capacity -- the cache's host-side step count does.  okv_rope_append."""
    dt = _same(q, k, v, cos, sin)
    bsz, d = q.shape[0], cos.shape[-1]
    _check_rope_tables(cos, sin, bsz, d)
    if k_store.dtype != q.dtype or k_store.stride() != v_store.stride() or k_store.stride(-1) != 1:
        raise ValueError("k_store / v_store must share dtype with q and strides with each other")
    if k_store.shape[0] != bsz or k_store.shape[1] != num_kv_heads or k_store.shape[3] != d:
        raise ValueError("stores must be (bsz, Hkv, capacity, D)")
    q_out = torch.empty((bsz, num_q_heads, 1, d), dtype=q.dtype, device=q.device)
    on_dev = isinstance(pos, torch.Tensor)
    if on_dev and (pos.dtype != torch.int64 or not pos.is_cuda or pos.numel() != 1):
        raise ValueError("a device position must be a one-element int64 GPU tensor")
    if not on_dev and not 0 <= int(pos) < k_store.shape[2]:
        raise ValueError("position outside the store")
    check(lib().okv_rope_append(q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0),
                                cos.data_ptr(), sin.data_ptr(), bsz, num_q_heads, num_kv_heads, d, dt, q_out.data_ptr(),
                                k_store.data_ptr(), v_store.data_ptr(), k_store.stride(2), k_store.stride(1),
                                k_store.stride(0), pos.data_ptr() if on_dev else None, 0 if on_dev else int(pos),
                                _stream_ptr(q.device)))
    return q_out


def silu_mul(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """silu(gate) * up; okv_silu_mul."""
    dt = _same(gate, up)
    out = torch.empty_like(gate)
    check(lib().okv_silu_mul(gate.data_ptr(), up.data_ptr(), gate.numel(), dt, out.data_ptr(), _stream_ptr(gate.device)))
    return out
