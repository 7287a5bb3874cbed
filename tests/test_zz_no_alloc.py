"""The sparse-attention entry point that allocates nothing (okv_sparse_attn_noalloc), called
through the C ABI: its output must equal okv_sparse_attn's bit for bit (same kernels, the
partial results in the library's fixed per-GPU array instead of a caller's workspace), on
consecutive calls that reuse the array with different sizes, and no device memory may be
taken by a call."""
import ctypes as C
import math

import pytest
import torch

from omnikv_amd import _lib, ops
from omnikv_amd._lib import KVLayout, check, lib

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
HQ, HKV, D = 32, 8, 128


def _call_noalloc(q, k, v, idx, tail_k, tail_v, out):
    """Straight ctypes call: pointers, strides and the current stream; nothing else."""
    lay = KVLayout(_lib.OKV_BF16, HQ, HKV, D, k.stride(2), k.stride(1), k.stride(0), None, 0, 0, 0)
    t = tail_k.shape[2] if tail_k is not None else 0
    return lib().okv_sparse_attn_noalloc(
        q.data_ptr(), k.data_ptr(), v.data_ptr(), C.byref(lay), idx.data_ptr(), idx.stride(0), None, idx.shape[1],
        tail_k.data_ptr() if t else None, tail_v.data_ptr() if t else None,
        tail_k.stride(2) if t else 0, tail_k.stride(1) if t else 0, tail_k.stride(0) if t else 0, None, t,
        q.shape[0], 1.0 / math.sqrt(D), out.data_ptr(), torch.cuda.current_stream().cuda_stream)


def _case(n, kk, tail, bsz, seed):
    g = torch.Generator(device=DEV).manual_seed(seed)
    k = torch.randn((bsz, HKV, n, D), generator=g, device=DEV).to(torch.bfloat16)
    v = torch.randn((bsz, HKV, n, D), generator=g, device=DEV).to(torch.bfloat16)
    q = torch.randn((bsz, HQ, D), generator=g, device=DEV).to(torch.bfloat16)
    idx = torch.stack([torch.randperm(n, generator=g, device=DEV)[:kk].sort().values for _ in range(bsz)]).to(torch.int32)
    tk = torch.randn((bsz, HKV, max(tail, 1), D), generator=g, device=DEV).to(torch.bfloat16)[:, :, :tail]
    tv = torch.randn((bsz, HKV, max(tail, 1), D), generator=g, device=DEV).to(torch.bfloat16)[:, :, :tail]
    return q, k, v, idx, (tk if tail else None), (tv if tail else None)


def test_noalloc_sparse_attention_equals_the_workspace_entry_point():
    assert lib().okv_noalloc_scratch_bytes() == 4 << 20
    # large first, then smaller ones that reuse the front of the same array, then large again
    cases = [(131072, 8781, 1, 1, 1), (20000, 1340, 3, 1, 2), (4096, 274, 0, 1, 3), (9000, 603, 2, 4, 4),
             (131072, 8781, 1, 1, 1)]
    prepared = [(_case(*c), c) for c in cases]
    want = [ops.sparse_attn(q, k, v, idx=idx, tail_k=tk, tail_v=tv) for (q, k, v, idx, tk, tv), _ in prepared]
    outs = [torch.full_like(w, float("nan")) for w in want]
    torch.cuda.synchronize()
    # a first call on the device looks the array's address up; no call may take device memory
    check(_call_noalloc(*prepared[1][0], outs[1]))
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    alloc0 = torch.cuda.memory_allocated()
    for ((q, k, v, idx, tk, tv), c), out in zip(prepared, outs):
        check(_call_noalloc(q, k, v, idx, tk, tv, out))
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0 and torch.cuda.memory_allocated() == alloc0
    for w, o, (_, c) in zip(want, outs, prepared):
        assert torch.equal(o, w), c
    assert torch.equal(outs[0], outs[-1])  # the small calls in between left nothing behind that matters


def test_noalloc_refuses_shapes_beyond_its_fixed_scratch():
    bsz, kk = 64, 40000  # 64 requests x 32 heads x many splits of partials: far beyond 4 MiB
    need = ops.workspace_bytes(_lib.OKV_OP_SPARSE_ATTN, bsz, HQ, HKV, D, kk, 0)
    assert need > lib().okv_noalloc_scratch_bytes()
    q = torch.zeros((bsz, HQ, D), dtype=torch.bfloat16, device=DEV)
    k = torch.zeros((1, HKV, 64, D), dtype=torch.bfloat16, device=DEV)
    idx = torch.zeros((bsz, kk), dtype=torch.int32, device=DEV)
    out = torch.zeros_like(q)
    rc = _call_noalloc(q, k, k, idx, None, None, out)  # refused on sizes alone: nothing is launched
    assert rc == -3  # OKV_ERR_WORKSPACE
    assert b"fixed scratch" in lib().okv_last_error()
