"""GPU parity on the batched / paged layout (page tables shuffled from a seed,
per-request lengths, ragged top-k) and size-independent properties at the
benchmark's full context lengths."""
import pytest
import torch

from omnikv_amd import ops, synth
from oracle import okv_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
HQ, HKV, D = 32, 8, 128


def _paged_batch(lens, page_size, dtype, seed=0):
    """Random K/V per request scattered into a shuffled page pool."""
    g = torch.Generator().manual_seed(seed)
    table, total = synth.shuffled_page_table(lens, page_size)
    pool_k = torch.zeros((total, page_size, HKV, D), dtype=dtype)
    pool_v = torch.zeros((total, page_size, HKV, D), dtype=dtype)
    ks, vs = [], []
    for b, n in enumerate(int(x) for x in lens):
        k = torch.randn((1, HKV, n, D), generator=g).to(dtype)
        v = torch.randn((1, HKV, n, D), generator=g).to(dtype)
        k[:, :, 0] *= 8
        ks.append(k)
        vs.append(v)
        t = torch.arange(n)
        pool_k[table[b, t // page_size].long(), t % page_size] = k[0].permute(1, 0, 2)
        pool_v[table[b, t // page_size].long(), t % page_size] = v[0].permute(1, 0, 2)
    q = torch.randn((len(lens), HQ, 1, D), generator=g).to(dtype)
    return q, ks, vs, pool_k, pool_v, table


@pytest.mark.parametrize("page_size", [1, 8, 12, 16, 64])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_paged_ragged_batch(page_size, dtype):
    lens = torch.tensor([700, 33, 1500, 1, 16, 1024, 257], dtype=torch.int32)
    q, ks, vs, pool_k, pool_v, table = _paged_batch(lens, page_size, dtype)
    # the page pool is addressed exactly as the oracle's paged_rows says
    for b in (0, 2):
        assert torch.equal(orc.paged_rows(pool_k, table[b], int(lens[b]), page_size), ks[b])
    kv = ops.PagedKV(pool_k.to(DEV), pool_v.to(DEV), table.to(DEV), page_size)
    lens_d = lens.to(DEV)
    nmax = int(lens.max())
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    for sel in ("last", "softmax_sum_last"):
        out, scores = ops.dense_attn(q.to(DEV), kv, seq_len=nmax, seq_lens=lens_d, selector=sel, score_len=nmax,
                                     score_lens=lens_d)
        k_per = torch.tensor([max(1, int(0.067 * int(n))) for n in lens], dtype=torch.int32)
        idx = torch.full((len(lens), int(k_per.max())), -1, dtype=torch.int32, device=DEV)
        ops.topk(scores, int(k_per.max()), seq_lens=lens_d, k_per_seg=k_per.to(DEV), out=idx)
        qn = torch.randn((len(lens), HQ, 1, D), generator=torch.Generator().manual_seed(3)).to(dtype)
        sparse = ops.sparse_attn(qn.to(DEV), kv, idx=idx, sel_len=int(k_per.max()), sel_lens=k_per.to(DEV))
        for b, n in enumerate(int(x) for x in lens):
            want_o = orc.gqa_attention(q[b:b + 1].float(), ks[b].float(), vs[b].float())[0, :, 0]
            assert (out[b].cpu().float() - want_o).abs().max() < tol
            want_s = orc.score_tokens(q[b:b + 1].float(), ks[b].float(), n, sel)[0]
            got_s = scores[b, :n].cpu()
            assert float((got_s - want_s).abs().max() / want_s.abs().max()) < 1e-4
            kb = int(k_per[b])
            # ragged top-k: bit-exact on the kernel's own scores
            want_idx = orc.select_topk_stable(got_s[None], kb)[0]
            assert torch.equal(idx[b, :kb].cpu().to(torch.int64), want_idx)
            assert (idx[b, kb:] == -1).all()
            # page-indirected gather + attention over exactly those rows
            want_sp = orc.gqa_attention(qn[b:b + 1].float(), orc.gather_rows(ks[b], want_idx).float(),
                                        orc.gather_rows(vs[b], want_idx).float())[0, :, 0]
            assert (sparse[b].cpu().float() - want_sp).abs().max() < tol
        # the same rows through token slots composed once (one lookup per row instead of two)
        slots = kv.slot_index(idx)
        assert slots.dtype == torch.int32 and ((slots < 0) == (idx < 0)).all()
        b0, k0 = 2, int(k_per[2])
        t = idx[b0, :k0].cpu().long()
        assert torch.equal(slots[b0, :k0].cpu().long(), table[b0, t // page_size].long() * page_size + t % page_size)
        via_slots = ops.sparse_attn(qn.to(DEV), kv, slots=slots, sel_len=int(k_per.max()), sel_lens=k_per.to(DEV))
        assert torch.equal(via_slots, sparse)  # identical rows in identical order: bit-identical output
    # LightLLM's own score: unscaled q.k, max over heads (rank-equivalent to `last`)
    raw = ops.score(q.to(DEV), kv, score_len=nmax, selector="last", scale=1.0, score_lens=lens_d)
    for b in (0, 5):
        n = int(lens[b])
        want = orc.lightllm_raw_head_max_score(q[b:b + 1].float(), ks[b].float())[0]
        assert float((raw[b, :n].cpu() - want).abs().max() / want.abs().max()) < 1e-4


@pytest.mark.parametrize("page_size", [16, 64])
def test_paged_scores_over_an_unaligned_prefix(page_size):
    """The filter layer's decode step on a paged pool: scores over the prompt only, attention
    over prompt + generated tokens.  The rows behind a scoring boundary that is not a multiple
    of 16 are read in 16-row tiles that straddle pages."""
    dtype = torch.bfloat16
    lens = torch.tensor([2100, 133, 700, 4099, 64, 37], dtype=torch.int32)
    cut = torch.tensor([37, 33, 1, 100, 16, 36], dtype=torch.int32)  # generated tokens per request
    score_lens = lens - cut
    q, ks, vs, pool_k, pool_v, table = _paged_batch(lens, page_size, dtype, seed=21)
    kv = ops.PagedKV(pool_k.to(DEV), pool_v.to(DEV), table.to(DEV), page_size)
    nmax, smax = int(lens.max()), int(score_lens.max())
    for sel in ("last", "softmax_sum_last"):
        out, scores = ops.dense_attn(q.to(DEV), kv, seq_len=nmax, seq_lens=lens.to(DEV), selector=sel,
                                     score_len=smax, score_lens=score_lens.to(DEV))
        for b, n in enumerate(int(x) for x in lens):
            a = int(score_lens[b])
            want_o = orc.gqa_attention(q[b:b + 1].float(), ks[b].float(), vs[b].float())[0, :, 0]
            assert (out[b].cpu().float() - want_o).abs().max() < 2e-2, (sel, b)
            want_s = orc.score_tokens(q[b:b + 1].float(), ks[b].float(), a, sel)[0]
            assert float((scores[b, :a].cpu() - want_s).abs().max() / want_s.abs().max()) < 1e-4
            # the same request stored contiguously: same tiles, same order of additions
            o1, s1 = ops.dense_attn(q[b:b + 1].to(DEV), ks[b].to(DEV), vs[b].to(DEV), selector=sel, score_len=a)
            op, sp = ops.dense_attn(q[b:b + 1].to(DEV), ops.PagedKV(kv.pool_k, kv.pool_v, kv.page_table[b:b + 1].contiguous(),
                                                                      page_size), seq_len=n, selector=sel, score_len=a)
            assert torch.equal(op, o1) and torch.equal(sp, s1), (sel, b)


def test_ragged_topk_pads_with_minus_one_by_default():
    """ops.topk without `out` on a ragged batch: entries beyond a request's own k are -1, which
    is what PagedKV.slot_index treats as padding."""
    g = torch.Generator().manual_seed(12)
    lens = torch.tensor([900, 40, 20000], dtype=torch.int32)
    ks = torch.tensor([60, 2, 1340], dtype=torch.int32)
    s = torch.randn((3, int(lens.max())), generator=g)
    idx = ops.topk(s.to(DEV), int(ks.max()), seq_lens=lens.to(DEV), k_per_seg=ks.to(DEV))
    for b in range(3):
        kb = int(ks[b])
        assert torch.equal(idx[b, :kb].cpu().long(), orc.select_topk_stable(s[b:b + 1, : int(lens[b])], kb)[0])
        assert (idx[b, kb:] == -1).all()
    table, total = synth.shuffled_page_table(lens, 16)
    pool = torch.zeros((total, 16, HKV, D), dtype=torch.bfloat16, device=DEV)
    slots = ops.PagedKV(pool, pool, table.to(DEV), 16).slot_index(idx)
    assert ((slots < 0) == (idx < 0)).all() and int(slots.max()) < total * 16


def test_paged_gather_rows():
    lens = torch.tensor([300, 90], dtype=torch.int32)
    q, ks, vs, pool_k, pool_v, table = _paged_batch(lens, 16, torch.bfloat16, seed=4)
    kv = ops.PagedKV(pool_k.to(DEV), pool_v.to(DEV), table.to(DEV), 16)
    idx = torch.tensor([[0, 5, 17, 299, 31], [1, 2, 3, 88, 89]], dtype=torch.int32)
    got = ops.gather_rows(kv, idx.to(DEV)).cpu()
    for b in range(2):
        assert torch.equal(got[b:b + 1], orc.gather_rows(ks[b], idx[b].long()))


@pytest.mark.parametrize("n", [131072, 450000])
def test_full_context_properties(n):
    """At the benchmark's context lengths: properties that need no CPU attention."""
    g = torch.Generator(device=DEV).manual_seed(n)
    k = torch.empty((1, n, HKV, D), dtype=torch.bfloat16, device=DEV).normal_(generator=g).permute(0, 2, 1, 3)
    v = torch.empty((1, n, HKV, D), dtype=torch.bfloat16, device=DEV).normal_(generator=g).permute(0, 2, 1, 3)
    q = torch.randn((1, HQ, 1, D), generator=g, device=DEV).to(torch.bfloat16)
    kk = int(0.067 * n)
    out, s_sum = ops.dense_attn(q, k, v, selector="softmax_sum_last", score_len=n)
    # each head's softmax sums to one
    assert abs(float(s_sum.double().sum()) - HQ) < 1e-2
    # fused scores == stand-alone scores
    assert float((ops.score(q, k, selector="softmax_sum_last") - s_sum).abs().max() / s_sum.max()) < 1e-5
    # top-k: ascending, right size, bit-exact against the CPU oracle on the same fp32 scores
    idx = ops.topk(s_sum, kk)
    i64 = idx.cpu().to(torch.int64)
    assert i64.shape == (1, kk) and torch.all(i64[0, 1:] > i64[0, :-1])
    assert torch.equal(i64, orc.select_topk_stable(s_sum.cpu(), kk))
    sel = s_sum[0, idx[0].long()]
    mask = torch.ones(n, dtype=torch.bool, device=DEV)
    mask[idx[0].long()] = False
    assert float(sel.min()) >= float(s_sum[0, mask].max())
    # selecting everything reproduces dense attention; splitting rows into (selected, rest as tail) too
    all_idx = torch.arange(n, dtype=torch.int32, device=DEV)[None]
    assert (ops.sparse_attn(q, k, v, idx=all_idx).float() - out.float()).abs().max() < 1e-2
    cut = n - 37
    two = ops.sparse_attn(q, k, v, idx=all_idx[:, :cut], tail_k=k[:, :, cut:], tail_v=v[:, :, cut:])
    assert (two.float() - out.float()).abs().max() < 1e-2
    # LSE linearity: attention over the selected rows and over the complement merge to the dense result
    raw = ops.score(q, k, selector="last")
    assert torch.equal(ops.topk(raw, kk).cpu().to(torch.int64), orc.select_topk_stable(raw.cpu(), kk))
    # the gather is a pure copy
    rows = ops.gather_rows(k, idx)
    assert torch.equal(rows, k[:, :, idx[0].long()])
