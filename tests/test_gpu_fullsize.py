"""GPU parity against the CPU oracle AT the benchmark's sizes: 131072 and 450000 tokens
(batch 1, bf16, the sink + heavy-hitter key distribution) and the batch of 16 ragged
requests of 8192..32768 tokens on a paged pool with 16-token pages.

Selectors: `last`, `softmax_before_last` (the reference's default, omnikv.py:139), the benchmark's
`softmax_sum_last`, and the window selectors `uniform` / `exp` with 16 positions.

Bars: scores within 1e-4 of the oracle's relative to the row's largest magnitude; top-k
bit-exact on identical fp32 scores; on the kernel's own scores every index that differs from
the oracle's selection is a provable near-tie (parity_helpers.assert_near_tie_only); attention within
2e-2 max-abs (bf16).
"""
import pytest
import torch

from omnikv_amd import ops, synth
from oracle import okv_oracle as orc
from parity_helpers import assert_near_tie_only

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
HQ, HKV, D = 32, 8, 128
DT = torch.bfloat16
SCORE_TOL, ATTN_TOL = 1e-4, 2e-2


def _rel(got, want):
    return float((got - want).abs().max() / want.abs().max())


@pytest.mark.parametrize("n,ks", [(131072, (8781, 8782)), (450000, (30150,))])
def test_filter_layer_op_matches_oracle_at_benchmark_size(n, ks):
    q, k, v = synth.filter_layer_inputs(n)
    q, k, v = q.to(DT), k.to(DT), v.to(DT)
    g = torch.Generator().manual_seed(n)
    tk, tv = torch.randn((1, HKV, 1, D), generator=g).to(DT), torch.randn((1, HKV, 1, D), generator=g).to(DT)
    # prompt rows + the decode step's own row, as the filter layer sees them
    kd = torch.cat([k, tk], dim=2).to(DEV)
    vd = torch.cat([v, tv], dim=2).to(DEV)
    qd = q.to(DEV)
    qf, kf, vf = q.float(), k.float(), v.float()
    by_head = n > 200000  # bound the host memory of the 4x repeated K
    want_dense = (orc.gqa_attention_by_kv_head if by_head else orc.gqa_attention)(
        qf, torch.cat([kf, tk.float()], 2), torch.cat([vf, tv.float()], 2))[0, :, 0]
    got_dense = ops.dense_attn(qd, kd, vd)
    assert (got_dense[0].cpu().float() - want_dense).abs().max() < ATTN_TOL

    qn = synth.fresh_q().to(DT)
    for sel in ("last", "softmax_before_last", "softmax_sum_last"):
        want = (orc.score_tokens_by_kv_head if by_head else orc.score_tokens)(qf, kf, n, sel)
        alone = ops.score(qd, kd[:, :, :n], selector=sel)
        out, fused = ops.dense_attn(qd, kd, vd, selector=sel, score_len=n)
        assert alone.shape == fused.shape == (1, n)
        assert _rel(alone.cpu(), want) < SCORE_TOL, sel
        assert _rel(fused.cpu(), want) < SCORE_TOL, sel
        # the fused pass also is the layer's attention, over all n + 1 rows
        assert (out[0].cpu().float() - want_dense).abs().max() < ATTN_TOL
        if sel == "softmax_sum_last":
            assert abs(float(fused.double().sum()) - HQ) < 1e-2
        for kk in ks:
            want_idx = orc.select_topk_stable(want, kk)
            if not orc.has_boundary_tie(want, kk):
                assert torch.equal(want_idx, orc.select_topk(want, kk))  # the reference's own topk + sort
            # identical fp32 scores -> identical indices
            idx = ops.topk(want.to(DEV), kk)
            assert torch.equal(idx.cpu().to(torch.int64), want_idx), (sel, kk)
            # attention, scores and selection in one call: the same bits as the separate calls
            out1, sc1, idx1 = ops.dense_attn(qd, kd, vd, selector=sel, score_len=n, select_k=kk)
            assert torch.equal(out1, out) and torch.equal(sc1, fused) and torch.equal(idx1, ops.topk(fused, kk))
            # the kernels' own scores: differences are near-ties only
            for got in (alone, fused):
                own = ops.topk(got, kk).cpu()[0].to(torch.int64)
                assert torch.all(own[1:] > own[:-1])
                assert_near_tie_only(got[0].cpu(), want[0], own, want_idx[0], kk)
            # downstream layer: fused gather + sparse attention over the oracle's rows + the tail row
            pk = torch.cat([orc.gather_rows(kf, want_idx[0]), tk.float()], dim=-2)
            pv = torch.cat([orc.gather_rows(vf, want_idx[0]), tv.float()], dim=-2)
            want_sp = orc.gqa_attention(qn.float(), pk, pv)[0, :, 0]
            got_sp = ops.sparse_attn(qn.to(DEV), kd[:, :, :n], vd[:, :, :n], idx=idx,
                                     tail_k=kd[:, :, n:], tail_v=vd[:, :, n:])
            assert (got_sp[0].cpu().float() - want_sp).abs().max() < ATTN_TOL, (sel, kk)
            # the materialised gather is a pure copy of the oracle's rows
            assert torch.equal(ops.gather_rows(kd[:, :, :n], idx).cpu(), orc.gather_rows(k, want_idx[0]))


@pytest.mark.parametrize("n", [131072, 450000])
def test_window_selectors_match_oracle_at_benchmark_size(n):
    """`uniform` and `exp` (modeling/omnikv.py:59-105) with a window of 16 positions at the benchmark's
    context lengths, through okv_score_window and through the filter layer's two-pass form
    okv_dense_attn_window, against the oracle evaluated one kv head at a time.  450000 rows are where the
    window passes take their largest split count."""
    w = 16
    q1, k, v = synth.filter_layer_inputs(n)
    g = torch.Generator().manual_seed(n + 5)
    # the window: the benchmark's query as the newest position, fifteen older ones scattered around it
    qw = torch.cat([q1 + 0.5 * torch.randn((1, HQ, w - 1, D), generator=g), q1], dim=2).to(DT)
    k, v = k.to(DT), v.to(DT)
    tk, tv = torch.randn((1, HKV, 1, D), generator=g).to(DT), torch.randn((1, HKV, 1, D), generator=g).to(DT)
    kd = torch.cat([k, tk], dim=2).to(DEV)
    vd = torch.cat([v, tv], dim=2).to(DEV)
    qd = qw.to(DEV)
    assert ops.window_supported(qd, kd)
    q_last = qd[:, :, -1:].contiguous()
    want_dense = orc.gqa_attention_by_kv_head(qw[:, :, -1:].float(), torch.cat([k, tk], 2).float(),
                                              torch.cat([v, tv], 2).float())[0, :, 0]
    kk = int(0.067 * n)
    for sel in ("uniform", "exp"):
        want = orc.score_window_by_kv_head(qw.float(), k.float(), n, sel)
        alone = ops.score_window(qd, kd[:, :, :n], score_len=n, selector=sel)
        out, fused = ops.dense_attn_window(q_last, qd, kd, vd, selector=sel, score_len=n)
        assert alone.shape == fused.shape == want.shape == (1, n)
        assert _rel(alone.cpu(), want) < SCORE_TOL, sel
        assert _rel(fused.cpu(), want) < SCORE_TOL, sel
        assert (out[0].cpu().float() - want_dense).abs().max() < ATTN_TOL, sel
        want_idx = orc.select_topk_stable(want, kk)
        assert torch.equal(ops.topk(want.to(DEV), kk).cpu().to(torch.int64), want_idx), sel
        for got in (alone, fused):
            own = ops.topk(got, kk).cpu()[0].to(torch.int64)
            assert torch.all(own[1:] > own[:-1])
            assert_near_tie_only(got[0].cpu(), want[0], own, want_idx[0], kk)


def test_batch16_ragged_paged_matches_oracle_at_benchmark_size():
    """16 requests of 8192..32768 tokens (seeded), 16-token pages shuffled from a seed,
    per-request k = int(0.067 * length): scores, ragged top-k and page-indirected sparse
    attention of every request against the oracle; slot_index against the table by hand."""
    page = 16
    lens = synth.ragged_lengths()
    assert lens.shape == (16,)
    table, total = synth.shuffled_page_table(lens, page)
    g = torch.Generator().manual_seed(synth.SEED_DATA)
    pool_k = torch.zeros((total, page, HKV, D), dtype=DT)
    pool_v = torch.zeros((total, page, HKV, D), dtype=DT)
    reqs = []
    for b, n in enumerate(int(x) for x in lens):
        qb, kb, vb = synth.filter_layer_inputs(n, seed=synth.SEED_DATA + 10 * b)
        qb, kb, vb = qb.to(DT), kb.to(DT), vb.to(DT)
        t = torch.arange(n)
        pool_k[table[b, t // page].long(), t % page] = kb[0].permute(1, 0, 2)
        pool_v[table[b, t // page].long(), t % page] = vb[0].permute(1, 0, 2)
        reqs.append((qb, kb, vb))
    for b in (0, 7):
        assert torch.equal(orc.paged_rows(pool_k, table[b], int(lens[b]), page), reqs[b][1])
    kv = ops.PagedKV(pool_k.to(DEV), pool_v.to(DEV), table.to(DEV), page)
    q = torch.cat([r[0] for r in reqs], dim=0).to(DEV)
    qn = torch.randn((16, HQ, 1, D), generator=g).to(DT)
    lens_d = lens.to(DEV)
    nmax = int(lens.max())
    k_per = torch.tensor([int(0.067 * int(n)) for n in lens], dtype=torch.int32)
    kmax = int(k_per.max())
    for sel in ("last", "softmax_sum_last"):
        alone = ops.score(q, kv, score_len=nmax, selector=sel, score_lens=lens_d)
        out, fused = ops.dense_attn(q, kv, seq_len=nmax, seq_lens=lens_d, selector=sel, score_len=nmax,
                                    score_lens=lens_d)
        want_scores = torch.full((16, nmax), -float("inf"))
        for b, n in enumerate(int(x) for x in lens):
            qb, kb, vb = reqs[b]
            want = orc.score_tokens(qb.float(), kb.float(), n, sel)[0]
            want_scores[b, :n] = want
            assert _rel(alone[b, :n].cpu(), want) < SCORE_TOL, (sel, b)
            assert _rel(fused[b, :n].cpu(), want) < SCORE_TOL, (sel, b)
            want_o = orc.gqa_attention(qb.float(), kb.float(), vb.float())[0, :, 0]
            assert (out[b].cpu().float() - want_o).abs().max() < ATTN_TOL, (sel, b)
        # ragged top-k on the ORACLE's scores: bit-exact, padding -1
        idx = ops.topk(want_scores.to(DEV), kmax, seq_lens=lens_d, k_per_seg=k_per.to(DEV))
        own = ops.topk(fused, kmax, seq_lens=lens_d, k_per_seg=k_per.to(DEV)).cpu()
        out1, sc1, idx1 = ops.dense_attn(q, kv, seq_len=nmax, seq_lens=lens_d, selector=sel, score_len=nmax,
                                         score_lens=lens_d, select_k=kmax, k_per_seg=k_per.to(DEV))
        assert torch.equal(out1, out) and torch.equal(idx1.cpu(), own)  # the one-call filter layer
        slots = kv.slot_index(idx)
        sparse = ops.sparse_attn(qn.to(DEV), kv, idx=idx, sel_len=kmax, sel_lens=k_per.to(DEV))
        via_slots = ops.sparse_attn(qn.to(DEV), kv, slots=slots, sel_len=kmax, sel_lens=k_per.to(DEV))
        assert torch.equal(sparse, via_slots)
        for b, n in enumerate(int(x) for x in lens):
            qb, kb, vb = reqs[b]
            kb_sel = int(k_per[b])
            want_idx = orc.select_topk_stable(want_scores[b:b + 1, :n], kb_sel)[0]
            assert torch.equal(idx[b, :kb_sel].cpu().to(torch.int64), want_idx), (sel, b)
            assert (idx[b, kb_sel:] == -1).all()
            assert_near_tie_only(fused[b, :n].cpu(), want_scores[b, :n], own[b, :kb_sel].to(torch.int64), want_idx,
                                  kb_sel)
            t = want_idx
            assert torch.equal(slots[b, :kb_sel].cpu().long(), table[b, t // page].long() * page + t % page)
            assert (slots[b, kb_sel:] == -1).all()
            want_sp = orc.gqa_attention(qn[b:b + 1].float(), orc.gather_rows(kb, want_idx).float(),
                                        orc.gather_rows(vb, want_idx).float())[0, :, 0]
            assert (sparse[b].cpu().float() - want_sp).abs().max() < ATTN_TOL, (sel, b)
