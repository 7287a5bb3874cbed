"""GPU parity: HIP kernels (through the C ABI) against the CPU oracle on the same
seeded inputs.  Bars: indices bit-exact on identical fp32 scores; attention
outputs within 1e-4 (fp32) / 2e-2 (bf16, fp16) max-abs; scores within 1e-4
relative to the row's largest magnitude when both sides see the same input values.
"""
import math

import pytest
import torch

from omnikv_amd import ops, synth
from oracle import okv_oracle as orc
from parity_helpers import assert_near_tie_only

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
ATTN_TOL = {torch.float32: 1e-4, torch.bfloat16: 2e-2, torch.float16: 2e-2}


def _rel_err(a: torch.Tensor, b: torch.Tensor) -> float:
    return float((a - b).abs().max() / b.abs().max().clamp_min(1e-30))


# ------------------------------------------------------------------ top-k
def _check_topk(scores_cpu: torch.Tensor, k: int):
    got = ops.topk(scores_cpu.to(DEV), k).cpu().to(torch.int64)
    want = orc.select_topk_stable(scores_cpu, k)
    assert got.shape == want.shape
    assert torch.equal(got, want)
    if not orc.has_boundary_tie(scores_cpu, k) and not torch.isnan(scores_cpu).any():
        assert torch.equal(got, orc.select_topk(scores_cpu, k))


@pytest.mark.parametrize("n,k", [(1, 1), (7, 3), (64, 64), (100, 1), (1000, 67), (4096, 274),
                                 (5000, 4999), (65537, 4391), (131072, 8781), (131072, 8782),
                                 (450000, 30150)])
def test_topk_random(n, k):
    g = torch.Generator().manual_seed(n * 31 + k)
    _check_topk(torch.randn((1, n), generator=g), k)


@pytest.mark.parametrize("levels", [2, 5, 100])
def test_topk_heavy_ties(levels):
    g = torch.Generator().manual_seed(levels)
    s = torch.randint(0, levels, (2, 20000), generator=g).float() * 0.25 - 3.0
    for k in (1, 100, 1340, 19999):
        _check_topk(s, k)


def test_topk_special_values():
    n = 3000
    s = torch.zeros((1, n))
    _check_topk(s, 17)  # all equal -> [0, 17)
    assert torch.equal(ops.topk(s.to(DEV), 17).cpu(), torch.arange(17, dtype=torch.int32)[None])
    s = torch.randn((1, n), generator=torch.Generator().manual_seed(5))
    s[0, 10] = float("inf")
    s[0, 11] = float("-inf")
    s[0, 12] = 0.0
    s[0, 13] = -0.0
    s[0, 2000] = float("inf")
    for k in (1, 2, 3, 1500, n - 1, n):
        _check_topk(s, k)
    z = torch.tensor([[0.0, -0.0, 0.0, -0.0, -1.0, -0.0]])
    assert ops.topk(z.to(DEV), 3).cpu().tolist() == [[0, 1, 2]]  # -0.0 ties with +0.0
    s[0, 77] = float("nan")
    s[0, 2999] = float("nan")
    got = ops.topk(s.to(DEV), 3).cpu()[0].tolist()
    assert got == [10, 77, 2999]  # NaN ranks above +inf; lowest index wins among the infs


def test_topk_narrow_range_and_softmax_scores():
    g = torch.Generator().manual_seed(9)
    s = 2.0 + 1e-4 * torch.rand((1, 50000), generator=g)  # keys within a few thousand ulps
    _check_topk(s, 3350)
    p = torch.softmax(4.0 * torch.randn((1, 131072), generator=g), dim=-1) * 32
    _check_topk(p, 8781)
    neg = -torch.rand((1, 9000), generator=g) - 0.5 + torch.randn((1, 9000), generator=g)
    _check_topk(neg, 603)


def test_topk_ragged_batch():
    g = torch.Generator().manual_seed(11)
    lens = torch.tensor([5000, 17, 32768, 1, 9001], dtype=torch.int32)
    ks = torch.tensor([335, 20, 2195, 1, 0], dtype=torch.int32)
    nmax = int(lens.max())
    s = torch.randn((len(lens), nmax), generator=g)
    out = torch.full((len(lens), int(ks.max())), -7, dtype=torch.int32, device=DEV)
    ops.topk(s.to(DEV), int(ks.max()), seq_lens=lens.to(DEV), k_per_seg=ks.to(DEV), out=out)
    out = out.cpu()
    for b in range(len(lens)):
        kb = min(int(ks[b]), int(lens[b]))
        want = orc.select_topk_stable(s[b:b + 1, : int(lens[b])], kb)[0].to(torch.int32)
        assert torch.equal(out[b, :kb], want)
        assert (out[b, kb:] == -7).all()  # untouched beyond k_b


# ---------------------------------------------------------------- scoring
def _inputs(n, dtype, layout):
    q, k, v = synth.filter_layer_inputs(n)
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    kd, vd = k.to(DEV), v.to(DEV)
    if layout == "token_major":
        kd, vd = synth.token_major(kd), synth.token_major(vd)
    return q, k, v, kd, vd


@pytest.mark.parametrize("selector", ["last", "softmax_before_last", "softmax_sum_last"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("layout", ["hf", "token_major"])
def test_score_matches_oracle(selector, dtype, layout):
    n = 4096
    q, k, v, kd, vd = _inputs(n, dtype, layout)
    got = ops.score(q.to(DEV), kd, selector=selector).cpu()
    want = orc.score_tokens(q.float(), k.float(), n, selector)  # same values, fp32 math
    assert got.shape == want.shape
    assert _rel_err(got, want) < 1e-4
    if "softmax" in selector and "sum" in selector:
        assert abs(float(got.sum()) - 32.0) < 1e-2  # each head's softmax sums to one
    # selected sets agree except for provable near-ties at the cut
    kk = orc.num_selected_tokens(0.067, n)
    assert_near_tie_only(got[0], want[0], ops.topk(got.to(DEV), kk).cpu()[0], orc.select_topk_stable(want, kk)[0], kk)


def test_score_partial_length_and_odd_sizes():
    for n, consider in [(1000, 1000), (1000, 777), (65, 64), (4099, 4099), (300, 1)]:
        q, k, _ = synth.filter_layer_inputs(n, seed=77)
        for selector in ("last", "softmax_sum_last"):
            got = ops.score(q.to(DEV), k.to(DEV), score_len=consider, selector=selector).cpu()
            want = orc.score_tokens(q, k, consider, selector)
            assert got.shape == (1, consider)
            assert _rel_err(got, want) < 1e-4


# -------------------------------------------------------------- attention
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("layout", ["hf", "token_major"])
@pytest.mark.parametrize("n", [1, 63, 4096, 20011])
def test_dense_attention(dtype, layout, n):
    q, k, v, kd, vd = _inputs(n, dtype, layout)
    got = ops.dense_attn(q.to(DEV), kd, vd).cpu().float()
    want = orc.gqa_attention(q.float(), k.float(), v.float())[:, :, 0, :]
    assert (got - want).abs().max() < ATTN_TOL[dtype]
    if dtype != torch.float32:  # and against the oracle run in the low precision itself
        low = orc.gqa_attention(q, k, v)[:, :, 0, :].float()
        assert (got - low).abs().max() < 2 * ATTN_TOL[dtype]


@pytest.mark.parametrize("selector", ["last", "softmax_before_last", "softmax_sum_last"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_dense_attention_with_fused_scores(selector, dtype):
    n, consider = 4096 + 37, 4096
    q, k, v, kd, vd = _inputs(n, dtype, "token_major")
    out, scores = ops.dense_attn(q.to(DEV), kd, vd, selector=selector, score_len=consider)
    want_o = orc.gqa_attention(q.float(), k.float(), v.float())[:, :, 0, :]
    want_s = orc.score_tokens(q.float(), k.float(), consider, selector)
    assert (out.cpu().float() - want_o).abs().max() < ATTN_TOL[dtype]
    assert _rel_err(scores.cpu(), want_s) < 1e-4
    alone = ops.score(q.to(DEV), kd, score_len=consider, selector=selector)
    assert _rel_err(scores.cpu(), alone.cpu()) < 1e-5


@pytest.mark.parametrize("selector", ["last", "softmax_sum_last"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,consider,ksel", [(4096 + 37, 4096, 274), (14336, 14336, 960), (20011, 20000, 1340),
                                              (70001, 69990, 4689), (70001, 69990, 69990), (40000, 39999, 1)])
def test_filter_layer_in_one_call_equals_attention_then_topk(selector, dtype, n, consider, ksel):
    """okv_dense_attn_select against okv_dense_attn followed by okv_topk on the same inputs: the same
    bits in all three outputs (below and above the length at which top-k goes to many workgroups),
    and the indices against the oracle's stable top-k of those scores."""
    q, k, v, kd, vd = _inputs(n, dtype, "hf")
    qd = q.to(DEV)
    out2, scores2 = ops.dense_attn(qd, kd, vd, selector=selector, score_len=consider)
    idx2 = ops.topk(scores2, ksel)
    for _ in range(2):  # the second call finds the workspace as the first left it
        out1, scores1, idx1 = ops.dense_attn(qd, kd, vd, selector=selector, score_len=consider, select_k=ksel)
        assert torch.equal(out1, out2) and torch.equal(scores1, scores2)
        assert torch.equal(idx1, idx2)
    want = orc.select_topk_stable(scores1.cpu(), ksel)
    assert torch.equal(idx1.cpu().to(torch.int64), want)


def test_filter_layer_in_one_call_where_the_topk_chunking_changes():
    """262145 rows attended, 262144 scored: the workspace is sized by the attention's length, whose top-k
    would use 33 chunks of two tiles, while the scores' own length makes 64 chunks of one."""
    n = 64 * 4096
    g = torch.Generator().manual_seed(5)
    k = torch.randn((1, 8, n + 1, 128), generator=g).to(torch.bfloat16).to(DEV)
    v = torch.randn((1, 8, n + 1, 128), generator=g).to(torch.bfloat16).to(DEV)
    q = torch.randn((1, 32, 1, 128), generator=g).to(torch.bfloat16).to(DEV)
    ksel = int(0.067 * n)
    out2, scores2 = ops.dense_attn(q, k, v, selector="softmax_sum_last", score_len=n)
    out1, scores1, idx1 = ops.dense_attn(q, k, v, selector="softmax_sum_last", score_len=n, select_k=ksel)
    assert torch.equal(out1, out2) and torch.equal(scores1, scores2)
    assert torch.equal(idx1, ops.topk(scores2, ksel))
    assert torch.equal(idx1.cpu().to(torch.int64), orc.select_topk_stable(scores1.cpu(), ksel))


def test_filter_layer_in_one_call_ragged_batch_and_both_block_sizes():
    """Requests of different lengths (one empty, one shorter than a score-finishing block, two ending
    inside one) with per-request k, at the automatic split size and at one small enough that the
    score-finishing blocks take 1024 tokens instead of 512."""
    from omnikv_amd._lib import check, lib
    g = torch.Generator().manual_seed(77)
    lens = torch.tensor([30000, 0, 300, 16385, 24577], dtype=torch.int32)
    ks = torch.tensor([2010, 5, 20, 16385, 0], dtype=torch.int32)
    hq, hkv, d, nmax = 32, 8, 128, int(lens.max())
    k = torch.randn((len(lens), hkv, nmax + 1, d), generator=g).to(torch.bfloat16)
    v = torch.randn((len(lens), hkv, nmax + 1, d), generator=g).to(torch.bfloat16)
    q = torch.randn((len(lens), hq, 1, d), generator=g).to(torch.bfloat16)
    kd, vd, qd, ld, ksd = k.to(DEV), v.to(DEV), q.to(DEV), lens.to(DEV), ks.to(DEV)
    seq = (lens + 1).to(DEV)  # every request attends to one row more than is scored
    kmax = int(ks.max())
    try:
        for split_rows in (0, 64):
            check(lib().okv_set_option(b"split_rows", split_rows))
            for sel in ("last", "softmax_sum_last"):
                out2, sc2 = ops.dense_attn(qd, kd, vd, seq_len=nmax + 1, seq_lens=seq, selector=sel, score_len=nmax,
                                           score_lens=ld)
                idx2 = ops.topk(sc2, kmax, seq_lens=ld, k_per_seg=ksd)
                out1, sc1, idx1 = ops.dense_attn(qd, kd, vd, seq_len=nmax + 1, seq_lens=seq, selector=sel,
                                                 score_len=nmax, score_lens=ld, select_k=kmax, k_per_seg=ksd)
                assert torch.equal(out1, out2)
                for b, n in enumerate(int(x) for x in lens):
                    kb = min(int(ks[b]), n)
                    assert torch.equal(sc1[b, :n], sc2[b, :n])
                    assert torch.equal(idx1[b, :kb], idx2[b, :kb]), (split_rows, sel, b)
                    assert (idx1[b, kb:] == -1).all()
                    want = orc.select_topk_stable(sc1[b:b + 1, :n].cpu(), kb)[0]
                    assert torch.equal(idx1[b, :kb].cpu().to(torch.int64), want), (split_rows, sel, b)
    finally:
        check(lib().okv_set_option(b"split_rows", 0))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("layout", ["hf", "token_major"])
@pytest.mark.parametrize("n,ksel,tail", [(4096, 274, 0), (4096, 274, 5), (4096, 1, 1), (20000, 1340, 100),
                                         (512, 512, 3), (300, 0, 7)])
def test_sparse_attention(dtype, layout, n, ksel, tail):
    q, k, v, kd, vd = _inputs(n, dtype, layout)
    g = torch.Generator().manual_seed(n + ksel + tail)
    idx = torch.sort(torch.randperm(n, generator=g)[:ksel]).values
    qn = synth.fresh_q().to(dtype)
    tk = torch.randn((1, 8, tail, 128), generator=g).to(dtype)
    tv = torch.randn((1, 8, tail, 128), generator=g).to(dtype)
    pk = torch.cat([orc.gather_rows(k, idx), tk], dim=-2)
    pv = torch.cat([orc.gather_rows(v, idx), tv], dim=-2)
    want = orc.gqa_attention(qn.float(), pk.float(), pv.float())[:, :, 0, :]
    idx_d = idx.to(torch.int32)[None].to(DEV) if ksel > 0 else torch.zeros((1, 0), dtype=torch.int32, device=DEV)
    got = ops.sparse_attn(qn.to(DEV), kd, vd, idx=idx_d,
                          tail_k=tk.to(DEV) if tail else None, tail_v=tv.to(DEV) if tail else None)
    assert (got.cpu().float() - want).abs().max() < ATTN_TOL[dtype]
    # an already gathered buffer (idx=None) gives the same answer
    if ksel > 0:
        got2 = ops.sparse_attn(qn.to(DEV), pk[:, :, :ksel].to(DEV).contiguous(), pv[:, :, :ksel].to(DEV).contiguous(),
                               tail_k=tk.to(DEV) if tail else None, tail_v=tv.to(DEV) if tail else None)
        assert (got2.cpu().float() - want).abs().max() < ATTN_TOL[dtype]


def test_sparse_with_all_rows_equals_dense():
    n = 3000
    q, k, v, kd, vd = _inputs(n, torch.bfloat16, "token_major")
    idx = torch.arange(n, dtype=torch.int32, device=DEV)[None]
    a = ops.sparse_attn(q.to(DEV), kd, vd, idx=idx).float()
    b = ops.dense_attn(q.to(DEV), kd, vd).float()
    assert (a - b).abs().max() < 1e-2


# ----------------------------------------------------------------- gather
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("layout", ["hf", "token_major"])
def test_gather_rows_bit_exact(dtype, layout):
    n, ksel = 5000, 335
    q, k, v, kd, vd = _inputs(n, dtype, layout)
    idx = torch.sort(torch.randperm(n, generator=torch.Generator().manual_seed(3))[:ksel]).values
    got = ops.gather_rows(kd, idx.to(torch.int32)[None].to(DEV))
    assert got.shape == (1, 8, ksel, 128)
    assert torch.equal(got.cpu(), orc.gather_rows(k, idx))
    dst = torch.empty((1, 8, ksel, 128), dtype=dtype, device=DEV)  # the reference's own layout
    ops.gather_rows(vd, idx.to(torch.int32)[None].to(DEV), out=dst)
    assert torch.equal(dst.cpu(), orc.gather_rows(v, idx))


# ------------------------------------------------ the CPU-runnable config, end to end
@pytest.mark.parametrize("selector", ["last", "softmax_sum_last"])
def test_filter_layer_op_config0(selector):
    n = 4096
    kk = orc.num_selected_tokens(0.067, n)
    assert kk == 274
    q, k, v = synth.filter_layer_inputs(n)
    _, k2, v2 = synth.filter_layer_inputs(n, seed=synth.SEED_DATA + 100)
    qn = synth.fresh_q()
    idx_w, scores_w, out_w = orc.filter_layer_op(q, k, v2, k2, qn, kk, selector)
    scores = ops.score(q.to(DEV), k.to(DEV), selector=selector)
    idx = ops.topk(scores, kk)
    out = ops.sparse_attn(qn.to(DEV), k2.to(DEV), v2.to(DEV), idx=idx)
    # identical fp32 scores -> identical indices
    assert torch.equal(ops.topk(scores_w.to(DEV), kk).cpu().to(torch.int64), idx_w)
    # own scores: identical up to provable near-ties at the cut
    assert_near_tie_only(scores[0].cpu(), scores_w[0], idx.cpu()[0], idx_w[0], kk)
    # the downstream layer on the ORACLE's rows, always; and on the kernel's own selection
    # (one swapped near-tie row of 274 moves the output by far less than the tolerance)
    out_on_oracle_idx = ops.sparse_attn(qn.to(DEV), k2.to(DEV), v2.to(DEV), idx=idx_w.to(torch.int32).to(DEV))
    assert (out_on_oracle_idx.cpu() - out_w[:, :, 0, :]).abs().max() < 1e-4
    own = orc.gqa_attention(qn, orc.gather_rows(k2, idx.cpu()[0].long()), orc.gather_rows(v2, idx.cpu()[0].long()))
    assert (out.cpu() - own[:, :, 0, :]).abs().max() < 1e-4


# ------------------------------------------------ long vectors: the chunked multi-workgroup path
def _topk_single_workgroup(scores_dev, k):
    """The one-workgroup-per-request kernel, selected by passing no workspace."""
    import ctypes as C

    from omnikv_amd._lib import check, lib
    out = torch.empty((scores_dev.shape[0], min(k, scores_dev.shape[1])), dtype=torch.int32, device=DEV)
    check(lib().okv_topk(scores_dev.data_ptr(), scores_dev.stride(0), None, scores_dev.shape[1], None, k,
                         scores_dev.shape[0], out.data_ptr(), out.stride(0), None, 0,
                         torch.cuda.current_stream().cuda_stream))
    return out


@pytest.mark.parametrize("n", [14336, 14337, 16385, 40000, 131072 + 3])
def test_topk_long_special_values_and_both_kernels(n):
    g = torch.Generator().manual_seed(n)
    s = torch.randn((2, n), generator=g)
    s[0, 5] = float("inf"); s[0, n - 1] = float("inf"); s[0, 6] = float("-inf")
    s[0, 100:200] = 0.0; s[0, 150:160] = -0.0
    s[1, 7] = float("nan"); s[1, n - 2] = float("nan")
    s[1, 4096:8192] = 1.25  # a whole chunk of one value
    for k in (1, 2, 3, 150, n // 15, n - 1, n):
        _check_topk(s, k)
        sd = s.to(DEV)
        assert torch.equal(_topk_single_workgroup(sd, k), ops.topk(sd, k))
    z = torch.zeros((1, n))
    assert torch.equal(ops.topk(z.to(DEV), 1000).cpu(), torch.arange(1000, dtype=torch.int32)[None])
    # unaligned score rows (a view starting one float into a buffer)
    buf = torch.randn((n + 1,), generator=g).to(DEV)
    view = buf[1:][None]
    assert torch.equal(ops.topk(view, 500).cpu().to(torch.int64), orc.select_topk_stable(view.cpu(), 500))


def test_topk_repeated_calls_leave_workspace_clean():
    g = torch.Generator().manual_seed(77)
    for i in range(6):  # same workspace, different lengths and distributions each time
        n = [131072, 20000, 450000, 16384, 70001, 131072][i]
        s = torch.randn((1, n), generator=g) * (10.0 ** (i - 3))
        if i % 2:
            s = torch.softmax(s * 3, dim=-1)
        _check_topk(s, max(1, int(0.067 * n)))


def test_topk_multi_tile_chunks_and_many_candidates():
    """Lengths whose chunks hold several tiles (2 at 450K; the 15-tile cap and more than 64 chunks
    at 4.2M), and score sets whose threshold bin holds more candidates than the last launch
    caches in LDS (a few distinct values; a narrow band), checked against the stable sort."""
    g = torch.Generator().manual_seed(5)
    for n in (450000, 4_200_000):
        s = torch.randn((1, n), generator=g)
        _check_topk(s, int(0.067 * n))
        _check_topk(torch.round(s * 2) / 2, int(0.067 * n))            # ~10 distinct values
        _check_topk(1.0 + s * 1e-3, n // 3)                              # everything inside one level-0 bin
    s = torch.randn((3, 300000), generator=g)
    s[1] = torch.round(s[1] * 8) / 8
    lens = torch.tensor([300000, 262145, 4097], dtype=torch.int32)
    kper = torch.tensor([20000, 262144, 4097], dtype=torch.int32)
    out = torch.full((3, 262144), -1, dtype=torch.int32, device=DEV)
    ops.topk(s.to(DEV), 262144, seq_lens=lens.to(DEV), k_per_seg=kper.to(DEV), out=out)
    for b in range(3):
        want = orc.select_topk_stable(s[b:b + 1, :int(lens[b])], int(kper[b]))[0]
        assert torch.equal(out[b, :int(kper[b])].cpu().to(torch.int64), want), b


# ------------------------------------------------------------------ window selectors
def _window_inputs(n, w, hq, hkv, dtype, seed=3, bsz=1):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn((bsz, hq, w, 128), generator=g).to(dtype)
    k = torch.randn((bsz, hkv, n, 128), generator=g)
    k[:, :, 0] *= 4.0  # a sink token, so that the softmax is peaked like a real one
    return q, k.to(dtype)


@pytest.mark.parametrize("selector", ["uniform", "exp"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("w,hq,hkv,n", [(1, 32, 8, 1000), (3, 32, 8, 4096), (16, 32, 8, 4099), (16, 32, 8, 70001),
                                        (8, 32, 4, 3000), (5, 8, 8, 2048), (7, 16, 8, 777), (8, 8, 1, 1500)])
def test_window_scores_match_oracle(selector, dtype, w, hq, hkv, n):
    """All window positions in two passes over K (matrix cores) against the oracle's
    position-by-position loop on the same 16-bit values."""
    q, k = _window_inputs(n, w, hq, hkv, dtype)
    assert ops.window_supported(q.to(DEV), k.to(DEV))
    consider = n - 3
    got = ops.score_window(q.to(DEV), k.to(DEV), score_len=consider, selector=selector).cpu()
    want = orc.score_tokens(q.float(), k.float(), consider, selector)
    assert got.shape == want.shape
    assert _rel_err(got, want) < 1e-4
    kk = max(1, int(0.067 * consider))
    assert_near_tie_only(got[0], want[0], ops.topk(got.to(DEV), kk).cpu()[0], orc.select_topk_stable(want, kk)[0], kk)


@pytest.mark.parametrize("selector", ["uniform", "exp"])
def test_window_scores_equal_the_per_position_kernels(selector):
    """The fused window kernel and one okv_score call per position compute the same
    sums in the same order: agreement to fp32 rounding of the softmax terms."""
    q, k = _window_inputs(20000, 16, 32, 8, torch.bfloat16, seed=9)
    qd, kd = q.to(DEV), k.to(DEV)
    fused = ops.score_window(qd, kd, selector=selector)
    loop = None
    for t in range(16):
        s = ops.score(qd[:, :, t:t + 1], kd, selector="softmax_before_last")
        loop = s if loop is None else (loop + s if selector == "uniform" else loop * 0.5 + s)
    assert _rel_err(fused.cpu(), loop.cpu()) < 2e-5
    # every position's head-max softmax lies in (0, 1]: bounds of the sums
    top = 16.0 if selector == "uniform" else 2.0
    assert float(fused.min()) >= 0.0 and float(fused.max()) <= top


def test_window_scores_ragged_batch_and_strided_q():
    """Per-request lengths, and q taken as a view of a longer (bsz, Hq, L, D) tensor."""
    lens = [5000, 37, 2048, 1]
    q_all, k = _window_inputs(5000, 24, 32, 8, torch.bfloat16, seed=21, bsz=4)
    q = q_all[:, :, 8:24]  # the last 16 positions: a strided view
    sl = torch.tensor(lens, dtype=torch.int32, device=DEV)
    got = ops.score_window(q.to(DEV)[:, :, :], k.to(DEV), score_len=5000, selector="exp", score_lens=sl).cpu()
    qv = q_all.to(DEV)[:, :, 8:24]
    assert not qv.is_contiguous()
    got_view = ops.score_window(qv, k.to(DEV), score_len=5000, selector="exp", score_lens=sl).cpu()
    for b, n in enumerate(lens):
        want = orc.score_tokens(q[b:b + 1].float(), k[b:b + 1].float(), n, "exp")
        assert _rel_err(got[b:b + 1, :n], want) < 1e-4
        assert torch.equal(got[b, :n], got_view[b, :n])


@pytest.mark.parametrize("selector", ["uniform", "exp"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("w,hq,hkv,n,extra", [(16, 32, 8, 4099, 1), (16, 32, 8, 70001, 1), (16, 32, 8, 20000, 37),
                                              (3, 32, 8, 4096, 1), (8, 32, 4, 3000, 5), (5, 8, 8, 2048, 1),
                                              (7, 16, 8, 777, 0)])
def test_window_filter_layer_in_two_passes(selector, dtype, w, hq, hkv, n, extra):
    """okv_dense_attn_window: the layer's attention over n + extra rows and the window scores of the first
    n from one call, against the oracle and against the two separate calls (the attention's pass over K
    computes the window columns' log-sum-exps, grouped by its own splits)."""
    q, k = _window_inputs(n + extra, w, hq, hkv, dtype)
    g = torch.Generator().manual_seed(n + w)
    v = torch.randn(k.shape, generator=g).to(dtype)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    q_last = qd[:, :, -1:].contiguous()
    out, scores = ops.dense_attn_window(q_last, qd, kd, vd, selector=selector, score_len=n)
    want_o = orc.gqa_attention(q[:, :, -1:].float(), k.float(), v.float())[:, :, 0, :]
    want_s = orc.score_tokens(q.float(), k.float(), n, selector)
    assert (out.cpu().float() - want_o).abs().max() < ATTN_TOL[dtype]
    assert scores.shape == want_s.shape
    assert _rel_err(scores.cpu(), want_s) < 1e-4
    assert (out.float() - ops.dense_attn(q_last, kd, vd).float()).abs().max() < 1e-2
    assert _rel_err(scores.cpu(), ops.score_window(qd, kd, score_len=n, selector=selector).cpu()) < 2e-5
    kk = max(1, int(0.067 * n))
    assert_near_tie_only(scores[0].cpu(), want_s[0], ops.topk(scores, kk).cpu()[0], orc.select_topk_stable(want_s, kk)[0], kk)


def test_window_filter_layer_ragged_batch_static_shapes():
    """Per-request lengths on the device, K/V buffers longer than any request (the captured decode
    step's shapes), and an attention query that is not the window's last row."""
    lens = [5000, 37, 2048, 640, 0]  # the last request scores nothing and attends to its two new rows
    cap = 5200
    qw, k = _window_inputs(cap, 16, 32, 8, torch.bfloat16, seed=33, bsz=5)
    g = torch.Generator().manual_seed(34)
    v = torch.randn(k.shape, generator=g).to(torch.bfloat16)
    qa = torch.randn((5, 32, 1, 128), generator=g).to(torch.bfloat16)
    seq = torch.tensor([n + 2 for n in lens], dtype=torch.int32, device=DEV)
    sl = torch.tensor(lens, dtype=torch.int32, device=DEV)
    out, scores = ops.dense_attn_window(qa.to(DEV), qw.to(DEV), k.to(DEV), v.to(DEV), selector="uniform", seq_len=cap,
                                        seq_lens=seq, score_len=5000, score_lens=sl)
    for b, n in enumerate(lens):
        want_o = orc.gqa_attention(qa[b:b + 1].float(), k[b:b + 1, :, :n + 2].float(), v[b:b + 1, :, :n + 2].float())[0, :, 0]
        assert (out[b].cpu().float() - want_o).abs().max() < 2e-2, b
        if n == 0:
            continue
        want_s = orc.score_tokens(qw[b:b + 1].float(), k[b:b + 1].float(), n, "uniform")
        assert _rel_err(scores[b:b + 1, :n].cpu(), want_s) < 1e-4, b


def test_window_unsupported_shapes_are_refused():
    q, k = _window_inputs(256, 17, 32, 8, torch.bfloat16)  # 17 positions x group 4 > 64 columns
    assert not ops.window_supported(q.to(DEV), k.to(DEV))
    with pytest.raises(Exception, match="unsupported"):
        ops.score_window(q.to(DEV), k.to(DEV), selector="uniform")
    q32, k32 = _window_inputs(256, 4, 32, 8, torch.float32)
    assert not ops.window_supported(q32.to(DEV), k32.to(DEV))
    with pytest.raises(Exception, match="unsupported"):
        ops.score_window(q32.to(DEV), k32.to(DEV), selector="uniform")
    q3, k3 = _window_inputs(256, 4, 24, 8, torch.bfloat16)  # three q heads per kv head: the head max pairs lanes
    assert not ops.window_supported(q3.to(DEV), k3.to(DEV))
    with pytest.raises(Exception, match="unsupported"):
        ops.score_window(q3.to(DEV), k3.to(DEV), selector="uniform")
    v3 = torch.zeros_like(k3)
    with pytest.raises(Exception, match="unsupported"):
        ops.dense_attn_window(q3.to(DEV)[:, :, -1:].contiguous(), q3.to(DEV), k3.to(DEV), v3.to(DEV), selector="uniform")


# ------------------------------------------------------------------ other GQA group sizes
@pytest.mark.parametrize("hq,hkv", [(8, 8), (16, 8), (64, 8), (4, 1), (32, 4)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_group_sizes_one_two_eight(hq, hkv, dtype):
    """Groups of 1, 2 and 8 q heads per kv head (the benchmark geometry is 4): dense with fused
    scores, raw scoring, top-k and the sparse pass against the oracle."""
    n, tail, kk = 3001, 3, 200
    g = torch.Generator().manual_seed(hq * 100 + hkv)
    q = torch.randn((1, hq, 1, 128), generator=g).to(dtype)
    k = torch.randn((1, hkv, n + tail, 128), generator=g).to(dtype)
    v = torch.randn((1, hkv, n + tail, 128), generator=g).to(dtype)
    k[:, :, 0] *= 6
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    out, sc = ops.dense_attn(q.to(DEV), k.to(DEV), v.to(DEV), selector="softmax_before_last", score_len=n)
    assert (out.cpu().float() - orc.gqa_attention(q.float(), k.float(), v.float())[:, :, 0]).abs().max() < tol
    want = orc.score_tokens(q.float(), k.float(), n, "softmax_before_last")
    assert _rel_err(sc.cpu(), want) < 1e-4
    raw = ops.score(q.to(DEV), k.to(DEV)[:, :, :n], selector="last")
    assert _rel_err(raw.cpu(), orc.score_tokens(q.float(), k.float(), n, "last")) < 1e-4
    idx = ops.topk(sc, kk)
    assert torch.equal(idx.cpu().to(torch.int64), orc.select_topk_stable(sc.cpu(), kk))
    sp = ops.sparse_attn(q.to(DEV), k.to(DEV)[:, :, :n], v.to(DEV)[:, :, :n], idx=idx,
                         tail_k=k.to(DEV)[:, :, n:], tail_v=v.to(DEV)[:, :, n:])
    ks = torch.cat([orc.gather_rows(k[:, :, :n], idx.cpu().to(torch.int64)), k[:, :, n:]], dim=2)
    vs = torch.cat([orc.gather_rows(v[:, :, :n], idx.cpu().to(torch.int64)), v[:, :, n:]], dim=2)
    assert (sp.cpu().float() - orc.gqa_attention(q.float(), ks.float(), vs.float())[:, :, 0]).abs().max() < tol


def test_empty_requests_in_a_batch():
    """A request of length zero next to ordinary ones: its attention output is defined as
    zero, it gets no scores and selects nothing; the others are unaffected."""
    lens = [0, 5, 300, 0, 1]
    g = torch.Generator().manual_seed(31)
    nmax = max(lens)
    q = torch.randn((len(lens), 32, 1, 128), generator=g).to(torch.bfloat16)
    k = torch.randn((len(lens), 8, nmax, 128), generator=g).to(torch.bfloat16)
    v = torch.randn((len(lens), 8, nmax, 128), generator=g).to(torch.bfloat16)
    sl = torch.tensor(lens, dtype=torch.int32, device=DEV)
    for sel in ("last", "softmax_sum_last"):
        out, sc = ops.dense_attn(q.to(DEV), k.to(DEV), v.to(DEV), seq_len=nmax, seq_lens=sl, selector=sel,
                                 score_len=nmax, score_lens=sl)
        for b, n in enumerate(lens):
            if n == 0:
                assert float(out[b].float().abs().max()) == 0.0
                continue
            want = orc.gqa_attention(q[b:b + 1].float(), k[b:b + 1, :, :n].float(), v[b:b + 1, :, :n].float())[0, :, 0]
            assert (out[b].cpu().float() - want).abs().max() < 2e-2
            ws = orc.score_tokens(q[b:b + 1].float(), k[b:b + 1].float(), n, sel)[0]
            assert _rel_err(sc[b:b + 1, :n].cpu(), ws[None]) < 1e-4
    k_per = torch.tensor([0, 2, 20, 0, 1], dtype=torch.int32)
    idx = torch.full((len(lens), 20), -1, dtype=torch.int32, device=DEV)
    ops.topk(sc, 20, seq_lens=sl, k_per_seg=k_per.to(DEV), out=idx)
    assert (idx[0] == -1).all() and (idx[3] == -1).all() and (idx[1, 2:] == -1).all()
    sp = ops.sparse_attn(q.to(DEV), k.to(DEV), v.to(DEV), idx=idx, sel_len=20, sel_lens=k_per.to(DEV))
    assert float(sp[0].float().abs().max()) == 0.0 and float(sp[3].float().abs().max()) == 0.0
    for b in (1, 2, 4):
        ii = idx[b, :int(k_per[b])].cpu().to(torch.int64)[None]
        want = orc.gqa_attention(q[b:b + 1].float(), orc.gather_rows(k[b:b + 1], ii).float(),
                                 orc.gather_rows(v[b:b + 1], ii).float())[0, :, 0]
        assert (sp[b].cpu().float() - want).abs().max() < 2e-2


def test_mismatched_dtypes_are_refused():
    q = torch.randn((1, 32, 1, 128), device=DEV)
    k = torch.randn((1, 8, 64, 128), device=DEV).to(torch.bfloat16)
    for call in (lambda: ops.score(q, k), lambda: ops.dense_attn(q, k, k), lambda: ops.sparse_attn(q, k, k),
                 lambda: ops.score_window(q.expand(1, 32, 4, 128).contiguous(), k)):
        with pytest.raises(ValueError, match="same dtype"):
            call()


def test_matrix_core_and_portable_kernels_agree_on_random_shapes():
    """Seeded random geometries (lengths around tile / split boundaries, ragged batches, tails,
    index lists, both layouts): the matrix-core kernels against the portable VALU kernels of
    the same library, which share no load path, tile logic or split code with them."""
    from omnikv_amd._lib import check, lib
    rng = torch.Generator().manual_seed(2024)

    def ri(lo, hi):
        return int(torch.randint(lo, hi + 1, (1,), generator=rng))

    try:
        for case in range(24):
            bsz = [1, 1, 2, 5][case % 4]
            hkv = [8, 2, 4, 1][case % 4]
            hq = hkv * [4, 8, 1, 2][(case // 4) % 4]
            n = [1, 15, 16, 17, 63, 64, 65, 255, 256, 257, 1409, 2817, 5000][ri(0, 12)] + (ri(0, 3) if case % 3 else 0)
            tail = [0, 1, 7, 40][ri(0, 3)]
            lens = torch.tensor([ri(1, n) for _ in range(bsz)], dtype=torch.int32)
            lens[ri(0, bsz - 1)] = n
            dtype = [torch.bfloat16, torch.float16][case % 2]
            q = torch.randn((bsz, hq, 1, 128), generator=rng).to(dtype).to(DEV)
            k = torch.randn((bsz, hkv, n + tail, 128), generator=rng).to(dtype).to(DEV)
            v = torch.randn((bsz, hkv, n + tail, 128), generator=rng).to(dtype).to(DEV)
            if case % 5 == 0:
                k, v = synth.token_major(k), synth.token_major(v)
            ld = lens.to(DEV)
            ksel = max(1, n // 7)
            kper = torch.tensor([min(ksel, int(l)) for l in lens], dtype=torch.int32)
            idx = torch.zeros((bsz, ksel), dtype=torch.int32)  # ascending per request, zero padded
            for b in range(bsz):
                idx[b, :int(kper[b])] = torch.randperm(int(lens[b]), generator=rng)[:int(kper[b])].sort().values
            idx = idx.to(DEV)
            res = {}
            for variant in (0, 1):
                check(lib().okv_set_option(b"attn_variant", variant))
                o, sc = ops.dense_attn(q, k[:, :, :n], v[:, :, :n], seq_len=n, seq_lens=ld, selector="softmax_sum_last",
                                       score_len=n, score_lens=ld)
                raw = ops.score(q, k[:, :, :n], score_len=n, selector="last", score_lens=ld)
                sp = ops.sparse_attn(q, k[:, :, :n], v[:, :, :n], idx=idx, sel_len=ksel, sel_lens=kper.to(DEV),
                                     tail_k=k[:, :, n:] if tail else None, tail_v=v[:, :, n:] if tail else None)
                res[variant] = (o.float(), sc, raw, sp.float())
            for b in range(bsz):
                lb = int(lens[b])
                assert (res[0][0][b] - res[1][0][b]).abs().max() < 2e-2, (case, "dense", b)
                assert _rel_err(res[0][1][b:b + 1, :lb].cpu(), res[1][1][b:b + 1, :lb].cpu()) < 1e-4, (case, "scores", b)
                assert _rel_err(res[0][2][b:b + 1, :lb].cpu(), res[1][2][b:b + 1, :lb].cpu()) < 1e-4, (case, "raw", b)
                assert (res[0][3][b] - res[1][3][b]).abs().max() < 2e-2, (case, "sparse", b)
    finally:
        check(lib().okv_set_option(b"attn_variant", 0))


def test_topk_random_lengths_and_distributions_bit_exact():
    """Seeded random lengths on both sides of the single- / multi-workgroup switch, k from 1 to
    n, smooth, quantised (many ties) and softmax-like scores, ragged batches: the indices must
    equal the oracle's stable selection exactly."""
    rng = torch.Generator().manual_seed(77)

    def ri(lo, hi):
        return int(torch.randint(lo, hi + 1, (1,), generator=rng))

    for case in range(30):
        bsz = [1, 1, 3][case % 3]
        nmax = [ri(1, 300), ri(4000, 17000), ri(16384, 70000), ri(100000, 200000)][case % 4]
        s = torch.randn((bsz, nmax), generator=rng)
        kind = case % 5
        if kind == 1:
            s = torch.round(s * 4) / 4            # a few dozen distinct values: ties everywhere
        elif kind == 2:
            s = torch.softmax(s * 6, dim=-1)      # many tiny values, a few large
        elif kind == 3:
            s = s * 1e-30                         # near the subnormal range
        elif kind == 4:
            s[:, ::7] = 0.0
            s[:, 1::13] = -0.0
        lens = torch.tensor([ri(1, nmax) for _ in range(bsz)], dtype=torch.int32)
        lens[ri(0, bsz - 1)] = nmax
        kper = torch.tensor([ri(1, int(l)) if case % 2 else max(1, int(0.067 * int(l))) for l in lens], dtype=torch.int32)
        kmax = int(kper.max())
        out = torch.full((bsz, kmax), -1, dtype=torch.int32, device=DEV)
        ops.topk(s.to(DEV), kmax, seq_lens=lens.to(DEV), k_per_seg=kper.to(DEV), out=out)
        for b in range(bsz):
            kb, lb = int(kper[b]), int(lens[b])
            want = orc.select_topk_stable(s[b:b + 1, :lb], kb)[0]
            assert torch.equal(out[b, :kb].cpu().to(torch.int64), want), (case, b, lb, kb)
            assert (out[b, kb:] == -1).all()


def test_c_abi_from_a_native_host_program():
    """tests/native/abi_smoke.cpp (built beforehand next to its source) links the library, owns
    its device memory through the HIP runtime, and checks scores, selection, dense and sparse
    attention and the row gather against loops of its own: the C ABI needs no Python around it."""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "native", "abi_smoke")
    assert os.path.exists(exe), "build first: python -c 'import __graft_entry__ as g; g.build()'"
    res = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert res.returncode == 0, res.stdout
    assert "abi smoke ok" in res.stdout


def test_topk_degenerate_score_vectors():
    """Vectors made of one value, of two, of NaN, of infinities, of zeros of both signs, of
    subnormals, and monotone ones: every key falls into one or two histogram bins, so the
    selection is decided by the tie rule and the chunk offsets alone."""
    n = 50021
    cases = {
        "all_nan": torch.full((1, n), float("nan")),
        "all_inf": torch.full((1, n), float("inf")),
        "all_ninf": torch.full((1, n), float("-inf")),
        "all_negative": torch.full((1, n), -3.5),
        "zeros_of_both_signs": torch.zeros((1, n)),
        "every_other_nan": torch.randn((1, n), generator=torch.Generator().manual_seed(3)),
        "subnormal": torch.randn((1, n), generator=torch.Generator().manual_seed(4)) * 1e-42,
        "two_values": (torch.arange(n) % 2).float()[None],
        "descending": torch.arange(n, 0, -1).float()[None],
        "ascending": torch.arange(n).float()[None],
    }
    cases["zeros_of_both_signs"][0, ::2] = -0.0
    cases["every_other_nan"][0, ::2] = float("nan")
    for name, s in cases.items():
        for k in (1, 7, 3351, n // 2, n - 1, n):
            got = ops.topk(s.to(DEV), k).cpu().to(torch.int64)
            assert torch.equal(got, orc.select_topk_stable(s, k)), (name, k)
