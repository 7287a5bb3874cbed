"""Pins the CPU oracle (oracle/okv_oracle.py) WITHOUT retyping its formulas:
pure-Python loops, library routines (torch SDPA, torch.sort), closed forms and
invariants that a dropped term, a wrong sign or index, or a transposed operand
would break.  The reference holds no golden vectors for this path, so these checks
are what anchors the oracle.
"""
import math

import pytest
import torch
from hypothesis import given, settings, strategies as st

from oracle import okv_oracle as orc


def _rand(shape, seed):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float64)


# ------------------------------------------------------------------ logits / scores
def _loop_logits(q, k):
    """q (Hq, D), k (Hkv, N, D) -> (Hq, N) with explicit loops; q head h reads kv head h // group."""
    hq, d = q.shape
    hkv, n, _ = k.shape
    grp = hq // hkv
    out = [[0.0] * n for _ in range(hq)]
    for h in range(hq):
        for t in range(n):
            acc = 0.0
            for i in range(d):
                acc += float(q[h, i]) * float(k[h // grp, t, i])
            out[h][t] = acc / math.sqrt(d)
    return torch.tensor(out, dtype=torch.float64)


@pytest.mark.parametrize("hq,hkv,n,d", [(4, 2, 7, 8), (8, 2, 5, 4), (6, 6, 3, 2), (4, 1, 9, 16)])
def test_attn_logits_against_loops(hq, hkv, n, d):
    q, k = _rand((1, hq, 1, d), 1), _rand((1, hkv, n, d), 2)
    want = _loop_logits(q[0, :, 0], k[0])
    got = orc.attn_logits(q, k)[0, :, 0]
    assert torch.allclose(got, want, atol=1e-12)


def test_score_selectors_against_loops():
    hq, hkv, n, d = 8, 2, 11, 4
    q, k = _rand((1, hq, 1, d), 3), _rand((1, hkv, n, d), 4)
    lg = _loop_logits(q[0, :, 0], k[0])
    # last: max over heads of raw logits
    want_last = [max(float(lg[h, t]) for h in range(hq)) for t in range(n)]
    assert torch.allclose(orc.score_tokens(q, k, n, "last")[0], torch.tensor(want_last, dtype=torch.float64))
    # softmax per head over tokens, by hand
    sm = [[0.0] * n for _ in range(hq)]
    for h in range(hq):
        mx = max(float(x) for x in lg[h])
        ex = [math.exp(float(x) - mx) for x in lg[h]]
        s = sum(ex)
        sm[h] = [e / s for e in ex]
    want_max = [max(sm[h][t] for h in range(hq)) for t in range(n)]
    want_sum = [sum(sm[h][t] for h in range(hq)) for t in range(n)]
    assert torch.allclose(orc.score_tokens(q, k, n, "softmax_before_last")[0],
                          torch.tensor(want_max, dtype=torch.float64), atol=1e-12)
    assert torch.allclose(orc.score_tokens(q, k, n, "softmax_sum_last")[0],
                          torch.tensor(want_sum, dtype=torch.float64), atol=1e-12)


def test_score_consider_len_and_last_row_only():
    hq, hkv, n, d = 4, 2, 20, 8
    q, k = _rand((1, hq, 3, d), 5), _rand((1, hkv, n, d), 6)
    # only the LAST query row counts for the `last` family, only the first consider_len tokens are scored
    a = orc.score_tokens(q, k, 13, "last")
    b = orc.score_tokens(q[:, :, -1:], k[:, :, :13], 13, "last")
    assert a.shape == (1, 13) and torch.equal(a, b)
    c = orc.score_tokens(q, k, 13, "softmax_before_last")
    d_ = orc.score_tokens(q[:, :, -1:], k[:, :, :13], 13, "softmax_before_last")
    assert torch.equal(c, d_)  # the softmax is over the considered tokens only


def test_score_invariants():
    hq, hkv, n, d = 32, 8, 300, 128
    q, k = _rand((1, hq, 1, d), 7).float(), _rand((1, hkv, n, d), 8).float()
    perm = torch.randperm(n, generator=torch.Generator().manual_seed(9))
    for sel in ("last", "softmax_before_last", "softmax_sum_last"):
        s = orc.score_tokens(q, k, n, sel)
        assert torch.allclose(orc.score_tokens(q, k[:, :, perm], n, sel), s[:, perm], rtol=1e-5, atol=1e-7)
    assert torch.allclose(orc.score_tokens(2.5 * q, k, n, "last"), 2.5 * orc.score_tokens(q, k, n, "last"), rtol=1e-5)
    # every head's softmax sums to one -> the head-summed score sums to the number of q heads
    assert abs(float(orc.score_tokens(q, k, n, "softmax_sum_last").sum()) - hq) < 1e-3
    # q head h must read kv head h // 4: zeroing kv head 1 silences exactly q heads 4..7
    k2 = k.clone()
    k2[:, 1] = 0
    lg = orc.attn_logits(q, k2)[0, :, 0]
    assert torch.all(lg[4:8] == 0) and torch.all(lg[:4] != 0) and torch.all(lg[8:] != 0)


def test_window_selectors_against_loops():
    hq, hkv, n, d, w = 4, 2, 9, 4, 3
    q, k = _rand((1, hq, w, d), 10), _rand((1, hkv, n, d), 11)
    per_pos = []
    for t in range(w):
        lg = _loop_logits(q[0, :, t], k[0])
        sm = torch.softmax(lg, dim=-1)
        per_pos.append(sm.max(dim=0).values)
    want_uniform = per_pos[0] + per_pos[1] + per_pos[2]
    # reference recurrence (modeling/omnikv.py:94-103): sum = sum/2 + score -> weights 1/4, 1/2, 1
    want_exp = per_pos[0] / 4 + per_pos[1] / 2 + per_pos[2]
    assert torch.allclose(orc.score_tokens(q, k, n, "uniform")[0], want_uniform, atol=1e-12)
    assert torch.allclose(orc.score_tokens(q, k, n, "exp")[0], want_exp, atol=1e-12)


# ------------------------------------------------------------------ top-k
def _brute_topk(vals, k):
    """Lowest-index tie rule by definition: rank by (value desc, index asc)."""
    order = sorted(range(len(vals)), key=lambda i: (-vals[i], i))
    return sorted(order[:k])


@settings(max_examples=200, deadline=None)
@given(st.lists(st.integers(-3, 3), min_size=1, max_size=24), st.integers(1, 30))
def test_topk_stable_against_brute_force(vals, k):
    s = torch.tensor([vals], dtype=torch.float32)
    kk = min(k, len(vals))
    assert orc.select_topk_stable(s, k)[0].tolist() == _brute_topk(vals, kk)


@settings(max_examples=200, deadline=None)
@given(st.lists(st.floats(-1e3, 1e3, allow_nan=False, width=32), min_size=1, max_size=40, unique=True),
       st.integers(1, 40))
def test_topk_torch_path_matches_when_no_tie(vals, k):
    s = torch.tensor([vals], dtype=torch.float32)
    kk = min(k, len(vals))
    got = orc.select_topk(s, k)[0].tolist()
    assert got == _brute_topk(vals, kk)
    assert got == orc.select_topk_stable(s, k)[0].tolist()
    assert not orc.has_boundary_tie(s, kk)


def test_topk_special_cases():
    s = torch.tensor([[0.5, 0.5, 0.5, 0.5, 0.5]])
    assert orc.select_topk_stable(s, 3)[0].tolist() == [0, 1, 2]
    assert orc.has_boundary_tie(s, 3)
    s = torch.tensor([[1.0, 3.0, 2.0]])
    assert orc.select_topk_stable(s, 3)[0].tolist() == [0, 1, 2]  # k = N: identity
    assert orc.select_topk_stable(s, 9)[0].tolist() == [0, 1, 2]  # k > N clamps (omnikv.py:47)
    assert orc.select_topk(s, 1)[0].tolist() == [1]
    s = torch.tensor([[0.0, -0.0, -1.0, -0.0, 0.0]])
    assert orc.select_topk_stable(s, 3)[0].tolist() == [0, 1, 3]  # -0.0 ties with +0.0
    s = torch.tensor([[1.0, float("inf"), float("nan"), float("-inf"), float("inf")]])
    assert orc.select_topk_stable(s, 1)[0].tolist() == [2]  # NaN ranks first, as in torch.topk
    assert orc.select_topk(s, 1)[0].tolist() == [2]
    assert orc.select_topk_stable(s, 2)[0].tolist() == [1, 2]
    assert orc.select_topk_stable(s, 4)[0].tolist() == [0, 1, 2, 4]


def test_canonical_key_is_monotone():
    vals = torch.tensor([float("-inf"), -3.5, -1e-30, -0.0, 0.0, 1e-30, 2.0, float("inf")])
    key = orc.canonical_key(vals)
    assert key[3] == key[4]
    rest = torch.cat([key[:3], key[4:]])
    assert torch.all(rest[1:] > rest[:-1])


# ------------------------------------------------------------------ integer logic
def test_num_selected_tokens_table():
    # int(ratio * N) truncates (modeling/omnikv.py:169-171)
    assert orc.num_selected_tokens(0.067, 4096) == 274
    assert orc.num_selected_tokens(0.067, 131072) == 8781
    assert orc.num_selected_tokens(0.067, 450000) == 30150
    assert orc.num_selected_tokens(2048, 131072) == 2048
    assert orc.window_adjust(274, 4096, 16, 1) == (259, 4081, 15)
    assert orc.window_adjust(274, 4096, 16, 20) == (274, 4096, 0)
    assert orc.window_adjust(5, 100, 16, 1) == (1, 85, 15)  # max(1, .)


def test_layer_schedule_tables():
    # Llama-3-8B example configuration: filters 2, 8, 18; one wait layer
    full = orc.full_attn_layers_from_select_layers([2, 8, 18], 32)
    assert full == [0, 1, 2, 8, 18, 32]
    st8 = orc.layer_schedule(full, 32, 1)
    dense = sorted(i for i, s in st8.items() if not s[0])
    assert dense == [0, 1, 2, 3, 8, 9, 18, 19]
    assert [st8[i][1] for i in (4, 7, 10, 17, 20, 31)] == [2, 2, 8, 8, 18, 18]
    assert st8[7][2] == 8 and st8[17][2] == 18 and st8[31][2] == 32
    assert sorted(st8) == list(range(32))
    # 70B serving configuration of the reference: filters 4, 19, 41 of 80 layers
    full = orc.full_attn_layers_from_select_layers([4, 19, 41], 80)
    st70 = orc.layer_schedule(full, 80, 1)
    assert sorted(i for i, s in st70.items() if not s[0]) == [0, 1, 2, 3, 4, 5, 19, 20, 41, 42]
    # two wait layers (the code's default)
    st2 = orc.layer_schedule([0, 1, 2, 8, 18, 32], 32, 2)
    assert sorted(i for i, s in st2.items() if not s[0]) == [0, 1, 2, 3, 4, 8, 9, 10, 18, 19, 20]


# ------------------------------------------------------------------ attention
@pytest.mark.parametrize("hq,hkv,n", [(32, 8, 257), (8, 8, 33), (16, 2, 64)])
def test_gqa_attention_against_sdpa(hq, hkv, n):
    d = 128
    q, k, v = _rand((1, hq, 1, d), 20).float(), _rand((1, hkv, n, d), 21).float(), _rand((1, hkv, n, d), 22).float()
    want = torch.nn.functional.scaled_dot_product_attention(q, k, v, enable_gqa=True)
    assert torch.allclose(orc.gqa_attention(q, k, v), want, atol=2e-6)


def test_gqa_attention_against_loops():
    hq, hkv, n, d = 4, 2, 6, 4
    q, k, v = _rand((1, hq, 1, d), 23), _rand((1, hkv, n, d), 24), _rand((1, hkv, n, d), 25)
    lg = _loop_logits(q[0, :, 0], k[0])
    out = torch.zeros((hq, d), dtype=torch.float64)
    for h in range(hq):
        p = torch.softmax(lg[h], dim=-1)
        for t in range(n):
            out[h] += p[t] * v[0, h // 2, t]
    assert torch.allclose(orc.gqa_attention(q, k, v)[0, :, 0], out, atol=1e-12)


def test_lse_merge_equals_joint_softmax():
    q, k, v = _rand((1, 8, 1, 16), 26).float(), _rand((1, 2, 50, 16), 27).float(), _rand((1, 2, 50, 16), 28).float()
    joint = orc.gqa_attention(q, k, v)
    for cuts in ([17], [1, 2, 49], [25, 26, 27, 40]):
        edges = [0] + cuts + [50]
        parts = [orc.attention_partial(q, k[:, :, a:b], v[:, :, a:b]) for a, b in zip(edges[:-1], edges[1:])]
        assert torch.allclose(orc.lse_merge(parts), joint, atol=1e-6)


def test_sparse_equals_dense_when_everything_is_selected():
    q, k, v = _rand((1, 8, 1, 16), 29).float(), _rand((1, 2, 40, 16), 30).float(), _rand((1, 2, 40, 16), 31).float()
    idx = torch.arange(40)
    a = orc.gqa_attention(q, orc.gather_rows(k, idx), orc.gather_rows(v, idx))
    assert torch.equal(a, orc.gqa_attention(q, k, v))


# ------------------------------------------------------------------ cache tiering
def test_oracle_cache_against_independent_bookkeeping():
    L, hkv, d, n = 6, 2, 4, 10
    full = orc.full_attn_layers_from_select_layers([1, 3], L)  # [0, 1, 3, 6]
    cache = orc.OracleMultiStageCache(full, L, num_wait_load_layers=1, real_offload=False)
    assert sorted(i for i, s in cache.layer_state.items() if s[0]) == [5]
    ks = [_rand((1, hkv, n, d), 100 + i).float() for i in range(L)]
    vs = [_rand((1, hkv, n, d), 200 + i).float() for i in range(L)]
    for i in range(L):
        k_ret, v_ret = cache.update(ks[i], vs[i], i)
        assert torch.equal(k_ret, ks[i]) and torch.equal(v_ret, vs[i])
    assert cache._seen_tokens == n
    cache.stage = "decoding"
    idx = torch.tensor([[0, 3, 4, 9]])
    new_k = [_rand((1, hkv, 1, d), 300 + i).float() for i in range(L)]
    new_v = [_rand((1, hkv, 1, d), 400 + i).float() for i in range(L)]
    for step in range(2):
        for i in range(L):
            if i == 3:
                cache.set_idx_on_gpu(idx, 3)
            k_ret, v_ret = cache.update(new_k[i] + step, new_v[i] + step, i)
            if i == 5:  # the only selected-rows layer: rows 0,3,4,9 then every decode row
                tail = [new_k[i] + s for s in range(step + 1)]
                want = torch.cat([ks[i][:, :, [0, 3, 4, 9]]] + tail, dim=-2)
                assert torch.equal(k_ret, want)
                assert v_ret.shape == want.shape
            else:
                assert k_ret.shape[-2] == n + step + 1
                assert torch.equal(k_ret[:, :, -1:], new_k[i] + step)
    assert cache._seen_tokens == n + 2


def test_idx_overlap_score_against_python_sets():
    """The lazy re-selection score is |new & old| / |new| (not over the union): checked with
    Python sets on random index lists, and on the closed cases identical / disjoint / nested."""
    g = torch.Generator().manual_seed(12)
    for n, k in [(50, 7), (1000, 67), (4096, 274)]:
        a = torch.randperm(n, generator=g)[:k].sort().values
        b = torch.randperm(n, generator=g)[:k].sort().values
        want = len(set(a.tolist()) & set(b.tolist())) / k
        assert orc.idx_overlap_score(a, b) == pytest.approx(want, abs=1e-12)
    a = torch.arange(0, 20)
    assert orc.idx_overlap_score(a, a.clone()) == 1.0
    assert orc.idx_overlap_score(a, a + 20) == 0.0
    assert orc.idx_overlap_score(torch.arange(0, 10), torch.arange(0, 40)) == 1.0   # new inside old
    assert orc.idx_overlap_score(torch.arange(0, 40), torch.arange(0, 10)) == 0.25  # old inside new


# ------------------------------------------------------------------ helpers for long contexts and pools
@pytest.mark.parametrize("sel", ["last", "softmax_before_last", "softmax_sum_last"])
def test_per_kv_head_evaluation_equals_the_whole_tensor_functions(sel):
    g = torch.Generator().manual_seed(31)
    q = torch.randn((2, 32, 1, 128), generator=g)
    k = torch.randn((2, 8, 300, 128), generator=g)
    v = torch.randn((2, 8, 300, 128), generator=g)
    whole = orc.score_tokens(q, k, 257, sel)
    by_head = orc.score_tokens_by_kv_head(q, k, 257, sel)
    # the BLAS call sees other shapes, so sums may round differently: equal to fp32 rounding
    assert torch.allclose(by_head, whole, rtol=2e-5, atol=2e-5 * float(whole.abs().max()))
    assert torch.allclose(orc.gqa_attention_by_kv_head(q, k, v), orc.gqa_attention(q, k, v), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("sel", ["uniform", "exp"])
@pytest.mark.parametrize("w,hq,hkv", [(1, 8, 8), (5, 32, 8), (16, 32, 8), (7, 16, 4)])
def test_window_scores_per_kv_head_equal_the_position_loop(sel, w, hq, hkv):
    """score_window_by_kv_head against score_tokens (the reference's position-by-position loop over
    all q heads at once), and against a brute-force evaluation in float64 with Python loops over
    positions and heads on a tiny case: a dropped position, a wrong decay or a head max taken
    over the wrong axis fails."""
    g = torch.Generator().manual_seed(40 + w)
    q = torch.randn((2, hq, w, 128), generator=g)
    k = torch.randn((2, hkv, 300, 128), generator=g)
    k[:, :, 0] *= 3.0
    whole = orc.score_tokens(q, k, 257, sel)
    by_head = orc.score_window_by_kv_head(q, k, 257, sel)
    assert by_head.shape == whole.shape == (2, 257)
    assert torch.allclose(by_head, whole, rtol=2e-5, atol=2e-5 * float(whole.abs().max()))
    # brute force, float64: score[t] = sum_w weight_w * max_h softmax_t(q_hw . k_t / sqrt(D))
    n = 23
    qd, kd = q[:1].double(), k[:1, :, :n].double()
    grp = hq // hkv
    want = torch.zeros(n, dtype=torch.float64)
    for wi in range(w):
        best = torch.zeros(n, dtype=torch.float64)
        for h in range(hq):
            logit = torch.stack([(qd[0, h, wi] * kd[0, h // grp, t]).sum() / 128 ** 0.5 for t in range(n)])
            best = torch.maximum(best, torch.softmax(logit, dim=0))
        weight = 1.0 if sel == "uniform" else 2.0 ** (wi - w + 1)
        want += weight * best
    got = orc.score_window_by_kv_head(q[:1], k[:1], n, sel)[0].double()
    assert torch.allclose(got, want, rtol=1e-5, atol=1e-7)


def test_paged_rows_round_trip_with_loops():
    """Scatter a request into a shuffled pool token by token with Python loops; paged_rows
    must read back exactly the original rows, for page sizes 1 (token slots), 4 and 16."""
    g = torch.Generator().manual_seed(32)
    for page_size, n in ((1, 9), (4, 10), (16, 33)):
        pages = (n + page_size - 1) // page_size
        table = torch.randperm(pages + 3, generator=g)[:pages]  # some pool pages stay unused
        rows = torch.randn((1, 2, n, 8), generator=g)
        pool = torch.full((pages + 3, page_size, 2, 8), float("nan"))
        for t in range(n):
            for h in range(2):
                pool[int(table[t // page_size]), t % page_size, h] = rows[0, h, t]
        assert torch.equal(orc.paged_rows(pool, table, n, page_size), rows)
        assert torch.equal(orc.paged_rows(pool, table, n - 1, page_size), rows[:, :, : n - 1])


def test_lightllm_raw_score_is_the_last_score_times_sqrt_d():
    """The serving stack's score is the dot product before sm_scale: sqrt(D) times the `last`
    selector's value (D = 64 makes the factor a power of two, so the identity is exact), and
    against explicit loops."""
    g = torch.Generator().manual_seed(33)
    q = torch.randn((1, 8, 1, 64), generator=g)
    k = torch.randn((1, 2, 50, 64), generator=g)
    got = orc.lightllm_raw_head_max_score(q, k)
    assert torch.equal(got, orc.score_tokens(q, k, 50, "last") * 8.0)
    q64, k64 = q.double(), k.double()
    want = [max(float((q64[0, h, 0] * k64[0, h // 4, t]).sum()) for h in range(8)) for t in range(50)]
    assert torch.allclose(got[0].double(), torch.tensor(want, dtype=torch.float64), atol=1e-4)
