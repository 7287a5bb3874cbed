"""CPU-side checks: golden fixtures against the oracle, the C-ABI library's exports
and argument validation (no kernel is launched), and the host logic that mirrors the
reference's Python interface."""
import ctypes as C
import os
import re

import numpy as np
import pytest
import torch

from omnikv_amd import _lib, cache as okv_cache, config as okv_config, ops, selector, synth
from oracle import okv_oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(ROOT, "tests", "golden")


# ------------------------------------------------------------------ golden vectors
@pytest.mark.parametrize("n,tail", [(64, 0), (1000, 3), (4096, 1)])
def test_oracle_reproduces_golden(n, tail):
    z = np.load(os.path.join(GOLDEN, f"filter_op_n{n}.npz"))
    kk = int(z["k"])
    assert kk == max(1, int(0.067 * n)) and int(z["tail"]) == tail
    q, k, v = synth.filter_layer_inputs(n)
    _, k2, v2 = synth.filter_layer_inputs(n, seed=synth.SEED_DATA + 100)
    qn = synth.fresh_q()
    g = torch.Generator().manual_seed(4242 + n)
    tk = torch.randn((1, 8, tail, 128), generator=g)
    tv = torch.randn((1, 8, tail, 128), generator=g)
    assert np.allclose(orc.gqa_attention(q, k, v)[0, :, 0].numpy(), z["dense_out"], atol=1e-6)
    for sel in ("last", "softmax_before_last", "softmax_sum_last"):
        idx, scores, out = orc.filter_layer_op(q, k, v2, k2, qn, kk, sel, tk if tail else None, tv if tail else None)
        assert np.array_equal(idx[0].numpy().astype(np.int32), z[f"idx_{sel}"])
        assert np.allclose(scores[0].numpy(), z[f"scores_{sel}"], rtol=1e-5, atol=1e-8)
        assert np.allclose(out[0, :, 0].numpy(), z[f"sparse_out_{sel}"], atol=1e-6)
        # the fixture's indices are the top-k of the fixture's scores under the stable rule too
        s = torch.from_numpy(z[f"scores_{sel}"])[None]
        assert np.array_equal(orc.select_topk_stable(s, kk)[0].numpy().astype(np.int32), z[f"idx_{sel}"])


def test_golden_tie_vectors():
    z = np.load(os.path.join(GOLDEN, "topk_ties.npz"))
    s = torch.from_numpy(z["scores"])
    for k in z["ks"]:
        assert np.array_equal(orc.select_topk_stable(s, int(k)).numpy().astype(np.int32), z[f"idx_k{int(k)}"])


def test_synthetic_inputs_are_deterministic_and_shaped():
    q, k, v = synth.filter_layer_inputs(512)
    q2, k2, v2 = synth.filter_layer_inputs(512)
    assert torch.equal(q, q2) and torch.equal(k, k2) and torch.equal(v, v2)
    assert q.shape == (1, 32, 1, 128) and k.shape == (1, 8, 512, 128)
    # the sink: token 0's keys are 8x larger than a unit normal's
    assert float(k[0, :, 0].std()) > 6.0 and float(k[0, :, 1:].std()) < 1.5
    # round(2%) heavy hitters stand out in the head-max score
    s = orc.score_tokens(q, k, 512, "last")[0]
    assert int((s[1:] > s[1:].median() + 2.0).sum()) >= 8
    lens = synth.ragged_lengths()
    assert lens.shape == (16,) and int(lens.min()) >= 8192 and int(lens.max()) <= 32768
    table, total = synth.shuffled_page_table(lens, 16)
    used = torch.cat([table[b, : (int(l) + 15) // 16] for b, l in enumerate(lens)])
    assert sorted(used.tolist()) == list(range(total))
    tm = synth.token_major(k)
    assert torch.equal(tm, k) and tm.stride(2) == 8 * 128 and tm.stride(1) == 128


# ------------------------------------------------------------------ the library
def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "omnikv_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(okv_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.lib()
    names = _declared_symbols()
    assert "okv_score" in names and "okv_topk" in names and "okv_sparse_attn" in names
    assert sorted(names) == sorted(_lib.EXPORTS)
    for name in names:
        assert getattr(lib, name) is not None
    assert lib.okv_version() >= 1
    assert lib.okv_strerror(0) == b"ok"
    assert lib.okv_strerror(-3) == b"workspace too small"


def test_measurement_hooks_live_in_the_measurement_build_only():
    """The product library holds the public interface and nothing of the okv_diag_* hooks (a process-wide
    switch that makes entry points skip their merge has no place in a serving process); the measurement
    build next to it holds both."""
    import ctypes as C
    hooks = ("okv_diag_split_pass_only", "okv_diag_split_geometry", "okv_diag_gather_floor", "okv_diag_empty_launch")
    product = C.CDLL(_lib.LIB_PATH)
    for name in hooks:
        assert not hasattr(product, name), name
    diag = C.CDLL(_lib.DIAG_LIB_PATH)
    for name in hooks + tuple(_lib.EXPORTS):
        assert getattr(diag, name) is not None


def test_header_is_plain_c(tmp_path):
    """The boundary is a C ABI: the header must compile as C99 and as C++ with nothing but the
    standard headers (no torch, no HIP types in the signatures)."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    src = tmp_path / "hdr.c"
    src.write_text('#include "omnikv_hip.h"\nint main(void) { okv_shape_t s; (void)s; return OKV_OK; }\n')
    inc = os.path.join(ROOT, "include")
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only", "-I", inc, str(src)])
    subprocess.check_call(["g++", "-std=c++11", "-Wall", "-Werror", "-fsyntax-only", "-x", "c++", "-I", inc, str(src)])


def test_workspace_sizes_are_consistent():
    base = ops.workspace_bytes(_lib.OKV_OP_DENSE_ATTN, 1, 32, 8, 128, 131072)
    with_scores = ops.workspace_bytes(_lib.OKV_OP_DENSE_ATTN, 1, 32, 8, 128, 131072, with_scores=True)
    assert with_scores >= base + 32 * 131072 * 4  # room for one fp32 logit per (head, token)
    assert ops.workspace_bytes(_lib.OKV_OP_SCORE, 1, 32, 8, 128, 4096) >= 32 * 4096 * 4
    small = ops.workspace_bytes(_lib.OKV_OP_SPARSE_ATTN, 1, 32, 8, 128, 274, 5)
    big = ops.workspace_bytes(_lib.OKV_OP_SPARSE_ATTN, 16, 32, 8, 128, 2195, 64)
    assert 0 < small < big
    assert ops.workspace_bytes(_lib.OKV_OP_TOPK, 1, 0, 0, 0, 450000) > 0
    # a workspace sized for a length serves every shorter one: the top-k's size never shrinks as the length
    # grows (its chunks become twice as long and half as many at 64 * 4096 + 1 scores), and the one-call filter
    # layer, sized by the attention's length, covers the attention's and the top-k's parts at any score length
    lengths = sorted(list(range(1, 700000, 4093)) + [262144, 262145, 4096 * 960, 4096 * 960 + 1, 5000000])
    for b in (1, 16):
        run = [ops.workspace_bytes(_lib.OKV_OP_TOPK, b, 0, 0, 0, n) for n in lengths]
        assert all(y >= x for x, y in zip(run, run[1:]))
    for n in (4096, 131073, 262145, 450001):
        both = ops.workspace_bytes(_lib.OKV_OP_DENSE_ATTN_SELECT, 1, 32, 8, 128, n)
        assert both >= ops.workspace_bytes(_lib.OKV_OP_DENSE_ATTN, 1, 32, 8, 128, n, with_scores=True) - 512 + \
            ops.workspace_bytes(_lib.OKV_OP_TOPK, 1, 0, 0, 0, n - 1)
    win = ops.workspace_bytes(_lib.OKV_OP_DENSE_ATTN_WINDOW, 1, 32, 8, 128, 131073)
    assert win > ops.workspace_bytes(_lib.OKV_OP_DENSE_ATTN, 1, 32, 8, 128, 131073) // 4
    out = C.c_size_t(0)
    assert _lib.lib().okv_workspace_bytes(99, C.byref(_lib.Shape(1, 32, 8, 128, 10, 0, 0)), C.byref(out)) == -1
    assert _lib.lib().okv_workspace_bytes(0, None, C.byref(out)) == -1


def test_argument_validation_happens_before_any_launch():
    """Every call below must be refused on the host (no GPU is needed or touched)."""
    lib = _lib.lib()
    lay = _lib.KVLayout(_lib.OKV_BF16, 32, 8, 128, 1024, 128, 0, None, 0, 0, 0)
    fake = C.c_void_p(0x1000)  # aligned, never dereferenced
    ws = C.c_void_p(0x2000)
    # NULL pointers
    assert lib.okv_topk(None, 8, None, 8, None, 2, 1, fake, 2, None, 0, None) == -1
    assert b"NULL" in lib.okv_last_error()
    assert lib.okv_score(None, fake, C.byref(lay), None, 8, 1, 0, 0, 1.0, fake, 8, ws, 1 << 30, None) == -1
    # unsupported geometry / dtype
    bad = _lib.KVLayout(_lib.OKV_BF16, 32, 8, 64, 512, 64, 0, None, 0, 0, 0)
    assert lib.okv_score(fake, fake, C.byref(bad), None, 8, 1, 0, 0, 1.0, fake, 8, ws, 1 << 30, None) == -2
    bad = _lib.KVLayout(7, 32, 8, 128, 1024, 128, 0, None, 0, 0, 0)
    assert lib.okv_score(fake, fake, C.byref(bad), None, 8, 1, 0, 0, 1.0, fake, 8, ws, 1 << 30, None) == -2
    bad = _lib.KVLayout(_lib.OKV_BF16, 24, 8, 128, 1024, 128, 0, None, 0, 0, 0)  # group of 3
    assert lib.okv_score(fake, fake, C.byref(bad), None, 8, 1, 0, 0, 1.0, fake, 8, ws, 1 << 30, None) == -2
    bad = _lib.KVLayout(_lib.OKV_BF16, 30, 8, 128, 1024, 128, 0, None, 0, 0, 0)  # not a multiple
    assert lib.okv_score(fake, fake, C.byref(bad), None, 8, 1, 0, 0, 1.0, fake, 8, ws, 1 << 30, None) == -1
    # misaligned base, odd stride
    assert lib.okv_score(fake, C.c_void_p(0x1004), C.byref(lay), None, 8, 1, 0, 0, 1.0, fake, 8, ws, 1 << 30, None) == -1
    bad = _lib.KVLayout(_lib.OKV_BF16, 32, 8, 128, 1020, 128, 0, None, 0, 0, 0)
    assert lib.okv_score(fake, fake, C.byref(bad), None, 8, 1, 0, 0, 1.0, fake, 8, ws, 1 << 30, None) == -1
    # bad enums, strides smaller than the row
    assert lib.okv_score(fake, fake, C.byref(lay), None, 8, 1, 5, 0, 1.0, fake, 8, ws, 1 << 30, None) == -1
    assert lib.okv_score(fake, fake, C.byref(lay), None, 8, 1, 0, 0, 1.0, fake, 4, ws, 1 << 30, None) == -1
    assert lib.okv_topk(fake, 4, None, 8, None, 2, 1, fake, 2, None, 0, None) == -1
    assert lib.okv_topk(fake, 8, None, 8, None, 4, 1, fake, 2, None, 0, None) == -1
    # workspace too small / missing
    assert lib.okv_score(fake, fake, C.byref(lay), None, 4096, 1, 0, 0, 1.0, fake, 4096, ws, 16, None) == -3
    assert b"need" in lib.okv_last_error()
    assert lib.okv_dense_attn(fake, fake, fake, C.byref(lay), None, 4096, 1, 1.0, fake, None, 0, 0, 0, None, 0,
                              None, 0, None) == -1
    # nothing to attend to, tail without pointers
    assert lib.okv_sparse_attn(fake, fake, fake, C.byref(lay), None, 0, None, 0, None, None, 0, 0, 0, None, 0, 1,
                               1.0, fake, ws, 1 << 30, None) == -1
    assert lib.okv_sparse_attn(fake, fake, fake, C.byref(lay), None, 0, None, 4, None, None, 1024, 128, 0, None, 2,
                               1, 1.0, fake, ws, 1 << 30, None) == -1
    # offload staging arguments
    assert lib.okv_offload_stage(None, 4096, fake, 1, fake, 1, fake, None, None) == -1
    assert lib.okv_offload_stage(fake, 4096, fake, 1, fake, 0, fake, None, None) == -1
    # incremental staging: NULL, too many staged rows, rows that are no multiple of 16 bytes, misaligned buffers
    assert lib.okv_offload_plan(None, 8, fake, fake, 100, fake, fake, fake, None) == -1
    assert lib.okv_offload_plan(fake, 0, fake, fake, 100, fake, fake, fake, None) == -1
    assert lib.okv_offload_plan(fake, (1 << 18) + 1, fake, fake, 1 << 20, fake, fake, fake, None) == -2
    assert lib.okv_offload_fetch(fake, 4100, fake, fake, fake, 8, fake, None) == -1
    assert lib.okv_offload_fetch(C.c_void_p(0x1008), 4096, fake, fake, fake, 8, fake, None) == -1
    assert lib.okv_offload_fetch(fake, 4096, fake, fake, None, 8, fake, None) == -1
    assert lib.okv_offload_fetch(fake, 4096, fake, fake, fake, 0, fake, None) == 0  # nothing to bound: no launch
    # the entry point without a workspace refuses what its fixed scratch cannot hold, before anything else
    assert lib.okv_noalloc_scratch_bytes() == 4 << 20
    assert lib.okv_sparse_attn_noalloc(fake, fake, fake, C.byref(lay), fake, 40000, None, 40000, None, None, 0, 0, 0,
                                       None, 0, 64, 1.0, fake, None) == -3
    assert b"fixed scratch" in lib.okv_last_error()
    assert lib.okv_sparse_attn_noalloc(fake, fake, fake, None, fake, 8, None, 8, None, None, 0, 0, 0, None, 0, 1, 1.0,
                                       fake, None) == -1
    # empty work is a successful no-op
    assert lib.okv_topk(fake, 8, None, 0, None, 2, 1, fake, 2, None, 0, None) == 0
    assert lib.okv_score(fake, fake, C.byref(lay), None, 0, 1, 0, 0, 1.0, fake, 0, ws, 1 << 30, None) == 0
    assert lib.okv_set_option(b"no_such_option", 1) == -1
    assert lib.okv_set_option(b"split_rows", 100) == -1
    assert lib.okv_set_option(b"skip_merge", 1) == -1  # measurement hooks are not options of the public interface
    assert lib.okv_set_option(b"split_rows", 0) == 0


def test_no_cpu_fallback():
    with pytest.raises(ValueError, match="GPU"):
        ops.topk(torch.zeros((1, 8)), 2)
    with pytest.raises(ValueError, match="GPU"):
        ops.score(torch.zeros((1, 32, 1, 128)), torch.zeros((1, 8, 16, 128)))
    with pytest.raises(ValueError, match="GPU"):
        ops.dense_attn(torch.zeros((1, 32, 1, 128)), torch.zeros((1, 8, 16, 128)), torch.zeros((1, 8, 16, 128)))


def test_check_raises_with_detail():
    with pytest.raises(_lib.OmniKVLibraryError, match="invalid argument"):
        _lib.check(_lib.lib().okv_topk(None, 8, None, 8, None, 2, 1, None, 2, None, 0, None))


# ------------------------------------------------------------------ host mirror of the reference interface
def test_config_get_sets_and_returns_default():
    cfg = okv_config.OmniKVConfig(do_select_layers="2,8,18", cache_cls="multi")
    assert cfg.get("do_select_layers") == "2,8,18"
    assert not hasattr(cfg, "window_size")
    assert cfg.get("window_size", 16) == 16
    assert cfg.window_size == 16  # omnikv_config.py:15-19: the default is written back
    assert okv_cache.get_cache_cls(cfg) is okv_cache.OmniKVMultiStageCache
    # `lazy` (modeling/spec_cache.py:523-557) is the multi-stage cache with re-selection skipping at 0.4
    lazy = okv_cache.get_cache_cls(okv_config.OmniKVConfig(cache_cls="lazy"))
    assert issubclass(lazy, okv_cache.OmniKVMultiStageCache)
    assert lazy([0, 4], 4, 1, False).skip_threshold == 0.4
    assert lazy([0, 4], 4, 1, False, skip_threshold=0.7).skip_threshold == 0.7
    assert okv_cache.OmniKVMultiStageCache([0, 4], 4, 1, False).skip_threshold is None
    for other in ("default", "eff"):  # other model paths of the reference
        with pytest.raises(NotImplementedError):
            okv_cache.get_cache_cls(okv_config.OmniKVConfig(cache_cls=other))


def test_cache_schedule_matches_oracle():
    for sel, L, wait in (([2, 8, 18], 32, 1), ([4, 19, 41], 80, 1), ([2, 8, 18], 32, 2), ([0], 4, 0)):
        full = orc.full_attn_layers_from_select_layers(sel, L)
        c = okv_cache.OmniKVMultiStageCache(full, L, wait, real_offload=False)
        assert c.layer_state == orc.layer_schedule(full, L, wait)
        assert c.stage == "prefill" and c.num_wait_layers == wait and c.device is None
    c = okv_cache.OmniKVMultiStageCache([0, 1, 2, 8, 18, 32], 32, 1, real_offload=True)
    assert c.device == "cpu"
    with pytest.raises(ValueError):
        okv_cache.OmniKVMultiStageCache([0, 4], 4, 1, offload_mode="nvme")


def test_unknown_selector_is_refused():
    with pytest.raises(NotImplementedError):
        selector.select_from_query(torch.zeros((1, 32, 1, 128)), torch.zeros((1, 8, 16, 128)), 4, 16, "median")


def test_rotary_matches_complex_rotation():
    # rotate-half RoPE == multiplying (x[i], x[i+D/2]) as a complex number by e^{i*theta_i*pos}
    d, pos = 8, 5
    x = torch.randn((1, 2, 1, d), generator=torch.Generator().manual_seed(3), dtype=torch.float64)
    inv = 1.0 / (500000.0 ** (torch.arange(0, d, 2, dtype=torch.float64) / d))
    ang = torch.cat([pos * inv, pos * inv])
    cos, sin = ang.cos()[None, None], ang.sin()[None, None]
    got, _ = selector.apply_rotary_pos_emb(x, x, cos, sin)
    z = torch.complex(x[..., : d // 2], x[..., d // 2:]) * torch.polar(torch.ones(d // 2, dtype=torch.float64), pos * inv)
    want = torch.cat([z.real, z.imag], dim=-1)
    assert torch.allclose(got, want, atol=1e-12)


def test_filter_layer_suggestion_follows_the_cache_schedule():
    """The tracer's schedule is the cache's own (which layers read which filter), and the
    exhaustive search returns the planted optimum of a synthetic layer-agreement matrix."""
    import itertools

    from omnikv_amd import trace
    from omnikv_amd.cache import layer_schedule

    L = 12
    for filters, wait in itertools.product([(2, 5, 9), (0, 6), (3,), (1, 2, 10)], [0, 1, 2]):
        full = list(range(0, filters[0])) + list(filters) + [L]
        want = {i: s[1] for i, s in layer_schedule(full, L, wait).items() if s[0]}
        assert trace._schedule(filters, L, wait) == want
    # layers fall into three groups that agree inside and not across; the best filters are the
    # group heads, at the price of the layers before the first one staying dense
    g = torch.tensor([0, 0, 1, 1, 1, 1, 2, 2, 2, 3, 3, 3])
    mass = torch.where(g[:, None] == g[None, :], 0.9, 0.2).double()
    layers, q = trace.suggest_filter_layers(mass, num_filters=3, num_wait_load_layers=1, max_dense_layers=8)
    assert layers == [2, 6, 9] and q == pytest.approx(0.9)
    assert trace.schedule_quality(mass, [2, 6, 9], 1) == (pytest.approx(0.9), 8)
    assert trace.schedule_quality(mass, [1, 4, 8], 1)[0] < 0.9
    with pytest.raises(ValueError):
        trace.suggest_filter_layers(mass, num_filters=3, num_wait_load_layers=1, max_dense_layers=3)
    # the recorder alone works without a GPU and round-trips through a file nothing is executed from
    import tempfile
    with tempfile.TemporaryDirectory() as d:
        tr = trace.SelectedIndexTracer(desc="cpu", save_dir=d)
        tr.append_spec_layer(torch.tensor([[3, 1]]), torch.tensor([[0.6, 0.4]]), 10, 7)
        tr.append_out("text")
        blob = trace.read_idx_tracer(tr.save_idx())
        assert blob["out"] == ["text"] and blob["layers_idx"][0][7][0]["prefill_len"] == 10
        assert torch.equal(blob["layers_idx"][0][7][0]["idx"], torch.tensor([[3, 1]]))


def test_static_decode_budget_is_counted_on_the_host():
    """Static (graph) decode appends at device positions nothing on the device checks: the
    host counts the steps and refuses the one that would run past the buffers."""
    from omnikv_amd.model import StaticDecodeGraph

    c = okv_cache.OmniKVMultiStageCache([0, 1, 3], 3, 1, real_offload=False, max_new_tokens=4)
    c._static_budget, c._static_steps = 3, 0
    assert c.static_steps_left == 3

    class FakeGraph:
        replays = 0

        def replay(self):
            self.replays += 1

    g = StaticDecodeGraph(FakeGraph(), c)
    c.note_static_step()  # an eager static step
    g.replay()
    g.replay()
    assert c.static_steps_left == 0 and g.graph.replays == 2
    with pytest.raises(RuntimeError, match="max_new_tokens"):
        g.replay()
    assert g.graph.replays == 2  # the refused replay launched nothing
    with pytest.raises(RuntimeError):
        c.note_static_step()


def test_llama_checkpoint_names_load_into_the_merged_projections():
    """q/k/v and gate/up share one weight each here; a state dict with the per-projection names of a Llama
    checkpoint fills the right rows, and the per-projection handles keep computing what separate layers would."""
    from omnikv_amd.model import LlamaShape, OmniKVMulLM

    shape = LlamaShape(hidden_size=256, intermediate_size=384, vocab_size=100, num_hidden_layers=2,
                       num_attention_heads=4, num_key_value_heads=2, head_dim=128)
    cfg = okv_config.OmniKVConfig(model_cls="multi", cache_cls="multi", do_select_layers="0", num_wait_load_layers=1,
                                  real_offload=False, dense_more=True, num_of_selected_tokens=0.5, selector_cls="last")
    lm = OmniKVMulLM(shape, cfg).float()
    g = torch.Generator().manual_seed(0)
    sd = {"model.embed_tokens.weight": torch.randn(100, 256, generator=g), "model.norm.weight": torch.randn(256, generator=g),
          "lm_head.weight": torch.randn(100, 256, generator=g)}
    for li in range(2):
        p = f"model.layers.{li}."
        sd.update({p + "self_attn.q_proj.weight": torch.randn(512, 256, generator=g),
                   p + "self_attn.k_proj.weight": torch.randn(256, 256, generator=g),
                   p + "self_attn.v_proj.weight": torch.randn(256, 256, generator=g),
                   p + "self_attn.o_proj.weight": torch.randn(256, 512, generator=g),
                   p + "mlp.gate_proj.weight": torch.randn(384, 256, generator=g),
                   p + "mlp.up_proj.weight": torch.randn(384, 256, generator=g),
                   p + "mlp.down_proj.weight": torch.randn(256, 384, generator=g),
                   p + "input_layernorm.weight": torch.randn(256, generator=g),
                   p + "post_attention_layernorm.weight": torch.randn(256, generator=g),
                   p + "self_attn.rotary_emb.inv_freq": torch.zeros(64)})
    lm.load_llama_state_dict(sd)
    x = torch.randn(1, 3, 256, generator=g)
    for li in range(2):
        a, m = lm.model.layers[li].self_attn, lm.model.layers[li].mlp
        p = f"model.layers.{li}."
        for name in ("q_proj", "k_proj", "v_proj"):
            assert torch.equal(getattr(a, name).weight, sd[p + f"self_attn.{name}.weight"])
            assert torch.allclose(getattr(a, name)(x), x @ sd[p + f"self_attn.{name}.weight"].T, atol=1e-5)
        q, k, v = a._project(x)
        assert torch.allclose(k, x @ sd[p + "self_attn.k_proj.weight"].T, atol=1e-4)
        want = (torch.nn.functional.silu(x @ sd[p + "mlp.gate_proj.weight"].T) * (x @ sd[p + "mlp.up_proj.weight"].T)) \
            @ sd[p + "mlp.down_proj.weight"].T
        assert torch.allclose(m(x), want, atol=1e-3)
    del sd["model.layers.1.mlp.up_proj.weight"]
    with pytest.raises(KeyError, match="missing"):
        lm.load_llama_state_dict(sd)
    sd["model.layers.1.mlp.up_proj.weight"] = torch.zeros(3, 3)
    with pytest.raises(ValueError, match="shape"):
        lm.load_llama_state_dict(sd)


def test_bench_scales_the_byte_counters_by_the_copy_kernel(tmp_path, monkeypatch):
    """bench.py's live roofline.traffic: the dense pass's average counter reading, scaled by what the same counter
    reads for the copy kernel's known transfer; the set-up's scoring pass and earlier copies are left out; without a
    profiler the measurement is skipped with a reason."""
    import bench

    head = '"Dispatch_Id","Kernel_Name","Grid_Size","Counter_Name","Counter_Value"\n'
    dense = "void okv::attn_stage1_mfma<okv::BF16, 4, true, 0, false>(okv::BF16 const*, okv::RowList, int, float, okv::AttnWorkspace)"
    score = "void okv::attn_stage1_mfma<okv::BF16, 4, false, 0, true>(okv::BF16 const*, okv::RowList, int, float, okv::AttnWorkspace)"
    rows = [(1, "__amd_rocclr_copyBuffer", 77.0), (2, score, 999999.0)]
    rows += [(3 + i, dense, 262256.0) for i in range(5)]
    rows += [(8 + i, "__amd_rocclr_copyBuffer", 131089.0) for i in range(3)]
    path = tmp_path / "p_counter_collection.csv"
    path.write_text(head + "".join(f'{d},"{k}",1024,"FETCH_SIZE",{v}\n' for d, k, v in rows)
                    + '20,"' + dense + '",1024,"WRITE_SIZE",5.0\n')
    got, why = bench.traffic_from_counters(str(path), "FETCH_SIZE", 268437504)
    assert why == "" and got["dispatches"] == 5
    assert abs(got["scale"] - 268437504 / (131089.0 * 1024)) < 1e-12
    assert abs(got["bytes"] - 262256.0 * 1024 * got["scale"]) < 1.0
    none, why = bench.traffic_from_counters(str(path), "WRITE_SIZE", 268437504)
    assert none is None and "1 dense" in why
    monkeypatch.setattr("shutil.which", lambda name: None)
    assert bench.live_traffic(131072, 1, "bf16") == (None, "rocprofv3 is not on PATH")
