"""GPU parity of the host-side mirror of the reference interface: the multi-stage
cache (update / set_idx_on_gpu / attend, with and without the host offload tier),
the selector with the reference's signature, and the committed golden vectors."""
import math
import os

import numpy as np
import pytest
import torch

from omnikv_amd import ops, selector, synth
from omnikv_amd.cache import OmniKVMultiStageCache
from omnikv_amd.config import OmniKVConfig
from oracle import okv_oracle as orc
from parity_helpers import assert_near_tie_only

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
TOL = {torch.float32: 1e-4, torch.bfloat16: 2e-2}


def _rel(got, want):
    return float((got - want).abs().max() / want.abs().max())


# ------------------------------------------------------------------ golden vectors
@pytest.mark.parametrize("n,tail", [(64, 0), (1000, 3), (4096, 1)])
def test_kernels_against_golden(n, tail):
    z = np.load(os.path.join(GOLDEN, f"filter_op_n{n}.npz"))
    kk = int(z["k"])
    q, k, v = synth.filter_layer_inputs(n)
    _, k2, v2 = synth.filter_layer_inputs(n, seed=synth.SEED_DATA + 100)
    qn = synth.fresh_q()
    g = torch.Generator().manual_seed(4242 + n)
    tk = torch.randn((1, 8, tail, 128), generator=g)
    tv = torch.randn((1, 8, tail, 128), generator=g)
    dense = ops.dense_attn(q.to(DEV), k.to(DEV), v.to(DEV)).cpu()
    assert np.abs(dense[0].numpy() - z["dense_out"]).max() < 1e-4
    for sel in ("last", "softmax_before_last", "softmax_sum_last"):
        want_scores = torch.from_numpy(z[f"scores_{sel}"])[None]
        want_idx = torch.from_numpy(z[f"idx_{sel}"])[None]
        got_scores = ops.score(q.to(DEV), k.to(DEV), selector=sel).cpu()
        assert float((got_scores - want_scores).abs().max() / want_scores.abs().max()) < 1e-4
        # bit-exact indices on identical fp32 scores
        assert torch.equal(ops.topk(want_scores.to(DEV), kk).cpu(), want_idx)
        out = ops.sparse_attn(qn.to(DEV), k2.to(DEV), v2.to(DEV), idx=want_idx.to(DEV),
                              tail_k=tk.to(DEV) if tail else None, tail_v=tv.to(DEV) if tail else None).cpu()
        assert np.abs(out[0].numpy() - z[f"sparse_out_{sel}"]).max() < 1e-4


def test_topk_against_golden_ties():
    z = np.load(os.path.join(GOLDEN, "topk_ties.npz"))
    s = torch.from_numpy(z["scores"]).to(DEV)
    for k in z["ks"]:
        assert np.array_equal(ops.topk(s, int(k)).cpu().numpy(), z[f"idx_k{int(k)}"])


# ------------------------------------------------------------------ cache vs oracle cache
class _Bag:
    """A plain object carrying whatever attributes a test gives it."""

    def __init__(self, **kw):
        self.__dict__.update(kw)


def _run_decode(dtype, real_offload, offload_mode, n=777, steps=3, L=8, sel_layers=(1, 4), wait=1, ratio=0.1,
                cls=OmniKVMultiStageCache, adopt=None):
    """adopt: None = prefill through update(); "lists" / "layers" / "lists_cpu" = the prompt
    arrives as a populated cache object through from_dynamic_cache (key_cache / value_cache
    lists on the GPU, `.layers[i].keys/.values`, or lists of CPU tensors)."""
    hq, hkv, d = 32, 8, 128
    g = torch.Generator().manual_seed(n + L)
    full = orc.full_attn_layers_from_select_layers(list(sel_layers), L)
    ref = orc.OracleMultiStageCache(full, L, wait, real_offload)
    kw = dict(max_new_tokens=16, offload_mode=offload_mode, cpu_num_threads=2)
    dut = cls(full, L, wait, real_offload, **kw) if adopt is None else None
    kk = orc.num_selected_tokens(ratio, n)
    # prefill
    prompt = []
    for i in range(L):
        k = torch.randn((1, hkv, n, d), generator=g).to(dtype)
        v = torch.randn((1, hkv, n, d), generator=g).to(dtype)
        rk, rv = ref.update(k, v, i)
        if adopt is None:
            dk, dv = dut.update(k.to(DEV), v.to(DEV), i)
            assert torch.equal(dk.cpu(), rk) and torch.equal(dv.cpu(), rv)
        else:
            prompt.append((k.clone(), v.clone()) if adopt == "lists_cpu" else (k.to(DEV), v.to(DEV)))
    if adopt is not None:
        if adopt == "layers":
            src = _Bag(layers=[_Bag(keys=k, values=v) for k, v in prompt])
        else:
            src = _Bag(key_cache=[k for k, _ in prompt], value_cache=[v for _, v in prompt], _seen_tokens=n)
        dut = cls.from_dynamic_cache(src, full, L, wait, real_offload, **kw)
        assert type(dut) is cls and dut.stage == "prefill"
        for i in range(L):  # the reference-visible lists hold the adopted values, tiered by the constructor's rule
            assert torch.equal(dut.key_cache[i].cpu(), ref.key_cache[i]) and torch.equal(dut.value_cache[i].cpu(), ref.value_cache[i])
            assert dut.key_cache[i].is_cuda == (not (real_offload and dut.layer_state[i][0]))
        prompt[0][0].zero_()  # adopted rows were copied: the donor may be reused
    assert dut._seen_tokens == ref._seen_tokens == n
    ref.stage = dut.stage = "decoding"
    for step in range(steps):
        for i in range(L):
            q = torch.randn((1, hq, 1, d), generator=g).to(dtype)
            k = torch.randn((1, hkv, 1, d), generator=g).to(dtype)
            v = torch.randn((1, hkv, 1, d), generator=g).to(dtype)
            if i in sel_layers:
                # the reference selects before the layer's own update (omnikv.py:189-212)
                scores = orc.score_tokens(q.float(), ref.key_cache[i].float(), n, "last")
                idx = orc.select_topk(scores, kk)
                ref.set_idx_on_gpu(idx, i)
                got = selector.select_from_query(q.to(DEV), dut.key_cache[i], kk, n, "last")
                assert got.dtype == torch.int64 and got.shape == idx.shape
                own = selector.score_from_query(q.to(DEV), dut.key_cache[i], n, "last")
                assert_near_tie_only(own[0].cpu(), scores[0], got.cpu()[0], orc.select_topk_stable(scores, kk)[0], kk)
                dut.set_idx_on_gpu(idx.to(DEV), i)  # identical selection on both sides from here on
            rk, rv = ref.update(k, v, i)
            want = orc.gqa_attention(q.float(), rk.float(), rv.float())[:, :, 0]
            # native path: append + attend
            dut.append(k.to(DEV), v.to(DEV), i)
            out = dut.attend(q.to(DEV), i).cpu().float()
            assert (out - want).abs().max() < TOL[dtype], (step, i)
        # reference-style consumption of the same state: update() must return the reference's tensors
        if step == steps - 1:
            for i in range(L):
                k = torch.randn((1, hkv, 1, d), generator=g).to(dtype)
                v = torch.randn((1, hkv, 1, d), generator=g).to(dtype)
                rk, rv = ref.update(k, v, i)
                dk, dv = dut.update(k.to(DEV), v.to(DEV), i)
                assert dk.shape == rk.shape
                assert torch.equal(dk.cpu(), rk) and torch.equal(dv.cpu(), rv), i
    return dut


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_cache_matches_reference_semantics_on_gpu(dtype):
    dut = _run_decode(dtype, real_offload=False, offload_mode="memcpy")
    assert sorted(dut._host_kv) == []
    assert dut.device is None


@pytest.mark.parametrize("mode", ["memcpy", "zero_copy", "incremental"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_cache_with_host_offload_tier(dtype, mode):
    dut = _run_decode(dtype, real_offload=True, offload_mode=mode)
    # layers that only ever read selected rows keep their prompt K/V in pinned host memory
    sparse = sorted(i for i, s in dut.layer_state.items() if s[0])
    assert sorted(dut._host_kv) == sparse and sparse
    for i in sparse:
        assert dut._host_kv[i].is_pinned() and not dut.key_cache[i].is_cuda
    dut._join_worker()


@pytest.mark.parametrize("adopt", ["lists", "layers", "lists_cpu"])
@pytest.mark.parametrize("real_offload", [False, True])
@pytest.mark.parametrize("name", ["multi", "without_pack"])
def test_from_dynamic_cache_adopts_a_populated_cache(name, real_offload, adopt):
    """modeling/spec_cache.py:371-385 (called at omnikv.py:339-341): a cache object that already
    holds the prompt is adopted, then decode steps (selection, update, attend) match the oracle
    cache that saw the same prompt through update()."""
    from omnikv_amd.cache import get_cache_cls

    cls = get_cache_cls(OmniKVConfig(cache_cls=name))
    dut = _run_decode(torch.bfloat16, real_offload, "zero_copy", n=500, steps=2, cls=cls, adopt=adopt)
    sparse = sorted(i for i, s in dut.layer_state.items() if s[0])
    assert sorted(dut._host_kv) == (sparse if real_offload else [])
    dut._join_worker()


def test_from_dynamic_cache_of_an_empty_cache():
    """What the reference's first forward does: the adopted DynamicCache is empty."""
    full = orc.full_attn_layers_from_select_layers([1, 4], 8)
    c = OmniKVMultiStageCache.from_dynamic_cache(_Bag(key_cache=[], value_cache=[], _seen_tokens=0), full, 8, 1, True)
    assert c.key_cache == [] and c._seen_tokens == 0 and c.stage == "prefill" and c.device == "cpu"
    assert c.layer_state == orc.layer_schedule(full, 8, 1)


@pytest.mark.parametrize("real_offload,mode", [(False, "zero_copy"), (True, "zero_copy"), (True, "memcpy")])
def test_without_pack_cache_fetches_rows_per_layer(real_offload, mode):
    """cache_cls `without_pack`: same results as `multi`; with the host tier nothing is
    staged at selection time, each sparse layer stages its own rows when it runs."""
    from omnikv_amd.cache import WOPackCache, get_cache_cls
    from omnikv_amd.config import OmniKVConfig
    assert get_cache_cls(OmniKVConfig(cache_cls="without_pack")) is WOPackCache
    staged = []
    orig = WOPackCache._start_offload

    def spy(self, idx32, layers):
        staged.append(list(layers))
        return orig(self, idx32, layers)

    WOPackCache._start_offload = spy
    try:
        dut = _run_decode(torch.bfloat16, real_offload=real_offload, offload_mode=mode, cls=WOPackCache)
    finally:
        WOPackCache._start_offload = orig
    if real_offload:
        assert staged and all(len(l) == 1 for l in staged)  # one layer at a time, never a group
        dut._join_worker()
    else:
        assert staged == []


@pytest.mark.parametrize("overlap", [0.0, 0.5, 0.9, 1.0])
def test_incremental_staging_fetches_only_rows_that_are_new(overlap):
    """offload_mode='incremental': consecutive selections that share a fraction `overlap` of their
    tokens.  After every selection the staged rows are exactly the selected set, only the rows
    the previous selection did not hold crossed the host link, every sparse layer's attention
    matches the oracle cache (which gathers everything anew, modeling/spec_cache.py:290-306), and
    update() still hands out the reference's tensors in the reference's order."""
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(int(overlap * 100) + 3)
    n, kk, L, hq, hkv, d = 5000, 500, 6, 32, 8, 128
    full = orc.full_attn_layers_from_select_layers([0], L)  # filter 0, wait 1, sparse 2..5
    ref = orc.OracleMultiStageCache(full, L, 1, True)
    dut = OmniKVMultiStageCache(full, L, 1, True, max_new_tokens=16, offload_mode="incremental")
    for i in range(L):
        k = torch.randn((1, hkv, n, d), generator=g).to(dtype)
        v = torch.randn((1, hkv, n, d), generator=g).to(dtype)
        ref.update(k, v, i)
        dut.update(k.to(DEV), v.to(DEV), i)
    ref.stage = dut.stage = "decoding"
    sparse = [i for i, st in dut.layer_state.items() if st[0]]
    assert sparse == [2, 3, 4, 5]
    prev = None
    for step in range(4):
        if prev is None:
            idx = torch.randperm(n, generator=g)[:kk].sort().values
        else:
            keep = prev[torch.randperm(kk, generator=g)[: int(round(overlap * kk))]]
            rest = torch.tensor(sorted(set(range(n)) - set(prev.tolist())))
            fresh = rest[torch.randperm(len(rest), generator=g)[: kk - len(keep)]]
            idx = torch.cat([keep, fresh]).sort().values
        ref.set_idx_on_gpu(idx[None], 0)
        dut.set_idx_on_gpu(idx[None].to(DEV), 0)
        expect_fetch = kk if prev is None else kk - len(set(idx.tolist()) & set(prev.tolist()))
        for i in range(L):
            q = torch.randn((1, hq, 1, d), generator=g).to(dtype)
            k = torch.randn((1, hkv, 1, d), generator=g).to(dtype)
            v = torch.randn((1, hkv, 1, d), generator=g).to(dtype)
            rk, rv = ref.update(k, v, i)
            want = orc.gqa_attention(q.float(), rk.float(), rv.float())[:, :, 0]
            dut.append(k.to(DEV), v.to(DEV), i)
            out = dut.attend(q.to(DEV), i).cpu().float()
            assert (out - want).abs().max() < TOL[dtype], (step, i)
        assert dut.last_fetch_count(0) == expect_fetch, step
        plan = dut._plan[0]
        assert torch.equal(plan["slot_tok"].cpu().sort().values.long(), idx)  # the staged set is the selection
        assert torch.equal(plan["slot_of"].cpu()[idx].sort().values, torch.arange(kk, dtype=torch.int32))
        assert int((plan["slot_of"] >= 0).sum()) == kk
        for i in sparse:  # the staged rows themselves: slot s holds token slot_tok[s]'s K and V
            st = plan["slot_tok"].cpu().long()
            assert torch.equal(dut._part[i][0, :, 0].cpu(), ref.key_cache[i][0, :, st].permute(1, 0, 2))
            assert torch.equal(dut._part[i][0, :, 1].cpu(), ref.value_cache[i][0, :, st].permute(1, 0, 2))
        prev = idx
    # reference-style consumption: update() returns gathered rows ++ tail in ascending token order
    for i in range(L):
        k = torch.randn((1, hkv, 1, d), generator=g).to(dtype)
        v = torch.randn((1, hkv, 1, d), generator=g).to(dtype)
        rk, rv = ref.update(k, v, i)
        dk, dv = dut.update(k.to(DEV), v.to(DEV), i)
        assert torch.equal(dk.cpu(), rk) and torch.equal(dv.cpu(), rv), i


def test_second_prompt_of_the_same_length_invalidates_what_incremental_staging_remembers():
    """The pinned rows of an offloaded layer are rewritten in place by a second prefill of the same
    length.  The slot maps of the incremental mode then describe rows of the OLD prompt: a selection that
    repeats tokens of the previous one must fetch them again, not reuse the stale staged rows."""
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(77)
    n, kk, L, hq, hkv, d = 1200, 120, 4, 32, 8, 128
    full = orc.full_attn_layers_from_select_layers([0], L)  # filter 0, wait 1, sparse 2..3
    dut = OmniKVMultiStageCache(full, L, 1, True, max_new_tokens=8, offload_mode="incremental")
    idx = torch.randperm(n, generator=g)[:kk].sort().values
    for prompt in range(2):
        dut.stage = "prefill"
        keys = [torch.randn((1, hkv, n, d), generator=g).to(dtype) for _ in range(L)]
        vals = [torch.randn((1, hkv, n, d), generator=g).to(dtype) for _ in range(L)]
        if prompt == 1:  # a fresh prompt in the same cache object: dense stores start over
            for st in dut._store.values():
                st.len = 0
            dut._tail.clear()
            dut.tail_k.clear()
            dut.tail_v.clear()
        for i in range(L):
            dut.update(keys[i].to(DEV), vals[i].to(DEV), i)
        dut.stage = "decoding"
        dut.set_idx_on_gpu(idx[None].to(DEV), 0)  # the SAME tokens both times
        assert dut.last_fetch_count(0) == kk, prompt  # nothing of the first prompt's staging is reused
        for i in (2, 3):
            q = torch.randn((1, hq, 1, d), generator=g).to(dtype)
            k1 = torch.randn((1, hkv, 1, d), generator=g).to(dtype)
            v1 = torch.randn((1, hkv, 1, d), generator=g).to(dtype)
            dut.append(k1.to(DEV), v1.to(DEV), i)
            pk = torch.cat([orc.gather_rows(keys[i], idx), k1], dim=-2)
            pv = torch.cat([orc.gather_rows(vals[i], idx), v1], dim=-2)
            want = orc.gqa_attention(q.float(), pk.float(), pv.float())[:, :, 0]
            out = dut.attend(q.to(DEV), i).cpu().float()
            assert (out - want).abs().max() < TOL[dtype], (prompt, i)


def test_incremental_staging_is_refused_where_layers_stage_themselves():
    from omnikv_amd.cache import WOPackCache
    with pytest.raises(ValueError, match="incremental"):
        WOPackCache([0, 4], 4, 1, True, offload_mode="incremental")


def test_lazy_reselection_skips_similar_selections():
    """skip_threshold (OmniKVLazyCache.set_out_idx): a selection that overlaps the one in
    use by more than the threshold is dropped, the rows already staged stay in use."""
    from omnikv_amd.cache import get_idx_iou_score
    g = torch.Generator().manual_seed(8)
    n, kk, L = 600, 60, 4
    full = orc.full_attn_layers_from_select_layers([0], L)
    dut = OmniKVMultiStageCache(full, L, 1, False, max_new_tokens=8, skip_threshold=0.5)
    for i in range(L):
        dut.update(torch.randn((1, 8, n, 128), generator=g).to(DEV), torch.randn((1, 8, n, 128), generator=g).to(DEV), i)
    dut.stage = "decoding"
    a = torch.arange(0, kk, device=DEV)[None]
    b = torch.cat([torch.arange(0, 40), torch.arange(100, 120)]).to(DEV)[None]   # 40/60 shared: skipped
    c = torch.cat([torch.arange(0, 20), torch.arange(200, 240)]).to(DEV)[None]   # 20/60 shared: taken
    assert get_idx_iou_score(b[0], a[0]) == pytest.approx(orc.idx_overlap_score(b[0].cpu(), a[0].cpu()))
    assert get_idx_iou_score(b[0], a[0]) == pytest.approx(40 / 60)
    dut.set_idx_on_gpu(a, 0)
    dut.set_idx_on_gpu(b, 0)
    assert dut.num_skipped_selections == 1 and torch.equal(dut._idx[0].cpu(), a.cpu().to(torch.int32))
    dut.set_idx_on_gpu(c, 0)
    assert dut.num_skipped_selections == 1 and torch.equal(dut._idx[0].cpu(), c.cpu().to(torch.int32))
    # cache_cls: lazy is that cache with the reference's threshold of 0.4: b (2/3 shared) is skipped, c (1/3) taken
    from omnikv_amd.cache import get_cache_cls
    from omnikv_amd.config import OmniKVConfig
    lazy = get_cache_cls(OmniKVConfig(cache_cls="lazy"))(full, L, 1, False, max_new_tokens=8)
    for i in range(L):
        lazy.update(torch.randn((1, 8, n, 128), generator=g).to(DEV), torch.randn((1, 8, n, 128), generator=g).to(DEV), i)
    lazy.stage = "decoding"
    for sel in (a, b, c):
        lazy.set_idx_on_gpu(sel, 0)
    assert lazy.num_skipped_selections == 1 and torch.equal(lazy._idx[0].cpu(), c.cpu().to(torch.int32))
    # default: every selection is taken, as the reference's multi-stage cache does
    ref = OmniKVMultiStageCache(full, L, 1, False)
    ref.set_idx_on_gpu(a, 0)
    ref.set_idx_on_gpu(b, 0)
    assert ref.num_skipped_selections == 0 and torch.equal(ref._idx[0].cpu(), b.cpu().to(torch.int32))


def test_offload_stage_packs_rows():
    # the C entry point alone: pinned rows -> staging -> device, runs of consecutive indices included
    n, row = 5000, 1024
    host = torch.randn((n, row), generator=torch.Generator().manual_seed(1)).pin_memory()
    idx = torch.tensor(sorted(set([0, 1, 2, 3, 77, 78, 4999] + list(range(100, 3000, 7)))), dtype=torch.int32)
    k = idx.numel()
    stg = torch.empty((k, row)).pin_memory()
    dst = torch.empty((k, row), device=DEV)
    stream = torch.cuda.Stream()
    ev = torch.cuda.Event()
    from omnikv_amd._lib import check, lib
    for threads in (1, 4):
        dst.zero_()
        torch.cuda.synchronize()
        check(lib().okv_offload_stage(host.data_ptr(), row * 4, idx.data_ptr(), k, stg.data_ptr(), threads,
                                      dst.data_ptr(), stream.cuda_stream, None))
        ev.record(stream)
        ev.synchronize()
        assert torch.equal(dst.cpu(), host[idx.long()])


# ------------------------------------------------------------------ selector with the reference's signature
class _Rotary(torch.nn.Module):
    def __init__(self, d, theta=500000.0):
        super().__init__()
        self.inv = 1.0 / (theta ** (torch.arange(0, d, 2, dtype=torch.float32) / d))

    def forward(self, x, position_ids):
        ang = position_ids[:, :, None].float() * self.inv.to(position_ids.device)[None, None, :]
        emb = torch.cat([ang, ang], dim=-1)
        return emb.cos().to(x.dtype), emb.sin().to(x.dtype)


class _Attn(torch.nn.Module):
    def __init__(self, hidden, hq, hkv, d, layer_idx):
        super().__init__()
        self.q_proj = torch.nn.Linear(hidden, hq * d, bias=False)
        self.k_proj = torch.nn.Linear(hidden, hkv * d, bias=False)
        self.num_heads, self.head_dim, self.num_key_value_heads = hq, d, hkv
        self.num_key_value_groups = hq // hkv
        self.layer_idx = layer_idx
        self.rotary_emb = _Rotary(d)
        self.config = OmniKVConfig(pretraining_tp=1)


@pytest.mark.parametrize("selector_cls", ["last", "softmax_before_last", "uniform", "exp"])
def test_select_tokens_by_attn_universal(selector_cls):
    torch.manual_seed(5)
    hidden, hq, hkv, d, n = 256, 32, 8, 128, 2000
    attn = _Attn(hidden, hq, hkv, d, layer_idx=0)
    win = 1 if "last" in selector_cls else 5
    hs = torch.randn((1, win, hidden))
    pos = torch.tensor([[n]])
    k = torch.randn((1, hkv, n, d))
    kk, consider = 134, n - 7

    class _C:
        key_cache = [k.to(DEV)]

    got = selector.select_tokens_by_attn_universal(attn.to(DEV), hs.to(DEV), pos.to(DEV), _C(), kk, consider, 0,
                                                   selector_cls)
    with torch.no_grad():  # the scores behind that selection (same device-side query)
        qd = attn.q_proj(hs.to(DEV)).view(1, win, hq, d).transpose(1, 2)
        cd, sd = attn.rotary_emb(qd, pos.to(DEV))
        qd, _ = selector.apply_rotary_pos_emb(qd, qd, cd, sd)
        own = selector.score_from_query(qd.contiguous(), k.to(DEV), consider, selector_cls)[0].cpu()
    # the same computation with the oracle on the CPU
    attn = attn.to("cpu")
    qs = attn.q_proj(hs).view(1, win, hq, d).transpose(1, 2)
    cos, sin = attn.rotary_emb(qs, pos)
    qs, _ = selector.apply_rotary_pos_emb(qs, qs, cos, sin)
    scores = orc.score_tokens(qs.detach(), k, consider, selector_cls)
    want = orc.select_topk(scores, kk)
    assert got.dtype == torch.int64 and got.shape == want.shape and got.device.type == "cuda"
    g = got.cpu()[0]
    assert torch.all(g[1:] > g[:-1]) and int(g.max()) < consider
    assert _rel(own, scores[0]) < 1e-4
    assert_near_tie_only(own, scores[0], g, orc.select_topk_stable(scores, kk)[0], kk)


def test_selector_clamps_k_and_refuses_tp():
    k = torch.randn((1, 8, 50, 128), device=DEV)
    q = torch.randn((1, 32, 1, 128), device=DEV)
    idx = selector.select_from_query(q, k, 4096, 50, "last")
    assert idx.cpu()[0].tolist() == list(range(50))  # min(k, N): everything, ascending
    attn = _Attn(64, 32, 8, 128, 0)
    attn.config = OmniKVConfig(pretraining_tp=2)

    class _C:
        key_cache = [k]

    with pytest.raises(NotImplementedError):
        selector.select_tokens_by_attn_universal(attn, torch.zeros((1, 1, 64)), torch.zeros((1, 1)), _C(), 4, 50)
