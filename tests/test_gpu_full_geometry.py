"""The end-to-end configuration at its real model geometry: 32 layers, hidden 4096, FFN 14336,
vocabulary 128256, RoPE theta 500000, bf16, random-init N(0, 0.02), OmniKV at layers 2, 8 and 18 with one
wait layer and real_offload (the sparse layers' prompt K/V in pinned host memory, selected rows fetched per
step).  The prompt is shortened (8192 tokens) so that the test fits a test run; the layer schedule, the
tiering, the number of layers per group, the GEMM shapes and the captured step are the real ones.

What is compared:
  * graph replays against eager steps of the SAME static decode path (same kernels, same shapes: bit for
    bit), 42 replays -- more new tokens than any small test appends, twelve sparse layers in one group;
  * the static path against the ordinary eager decode path (other split sizes: within bf16 rounding);
  * a four-layer slice of the same width against the oracle runner on the CPU (fp32 arithmetic on the
    same bf16-rounded weights), the reference's layer forward (modeling/omnikv.py:143-246, 287-394).
"""
import copy

import pytest
import torch

from omnikv_amd.config import OmniKVConfig
from omnikv_amd.model import LlamaShape, OmniKVMulLM

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _config(select_layers, real_offload=True):
    return OmniKVConfig(model_cls="multi", cache_cls="multi", do_select_layers=select_layers, num_wait_load_layers=1,
                        real_offload=real_offload, dense_more=True, num_of_selected_tokens=0.067, selector_cls="last",
                        window_size=16)


def _build(shape, cfg, seed=0):
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device(DEV):
            lm = OmniKVMulLM(shape, cfg)
    finally:
        torch.set_default_dtype(torch.float32)
    return lm.init_weights(seed=seed, std=0.02)


@pytest.mark.parametrize("mode", ["zero_copy", "incremental"])
def test_full_geometry_decode_with_the_host_tier_graph_against_eager(mode):
    shape = LlamaShape()
    assert (shape.num_hidden_layers, shape.hidden_size, shape.intermediate_size, shape.vocab_size) == (32, 4096, 14336, 128256)
    lm = _build(shape, _config("2,8,18"))
    n, replays = 8192, 42
    k_sel = int(0.067 * n)
    ids = torch.randint(0, shape.vocab_size, (1, n), generator=torch.Generator().manual_seed(1)).to(DEV)

    # ---- eager steps of the static decode path
    logits0, cache = lm.forward(ids, None, max_new_tokens=64, offload_mode=mode)
    dense = sorted(i for i, s in cache.layer_state.items() if not s[0])
    assert dense == [0, 1, 2, 3, 8, 9, 18, 19]
    assert sorted(cache._host_kv) == [i for i in range(32) if i not in dense]  # 24 layers' prompt K/V in pinned memory
    assert all(h.is_pinned() and h.shape == (n, 2, 8, 128) for h in cache._host_kv.values())
    tok = logits0[:, -1].argmax(-1, keepdim=True)
    cache.enable_static_decode()
    eager = []
    for _ in range(replays + 2):
        logits, cache = lm.forward(tok, cache)
        tok = logits[:, -1].argmax(-1, keepdim=True)
        eager.append((logits.clone(), int(tok)))
    assert all(cache._part[i].shape == (1, k_sel, 2, 8, 128) for i in cache._host_kv)
    assert int(cache._len32) == n + 1 + replays + 2
    scale = float(logits0.abs().max())
    del cache

    # ---- the ordinary eager path (lengths on the host, splits sized by the rows present): same tokens
    # wherever the top two logits are apart by more than bf16 rounding of the attention outputs can move them
    logits1, cache = lm.forward(ids, None, max_new_tokens=64, offload_mode=mode)
    assert torch.equal(logits1, logits0)
    tok = logits1[:, -1].argmax(-1, keepdim=True)
    for t in range(8):
        logits, cache = lm.forward(tok, cache)
        assert (logits - eager[t][0]).abs().max() < 0.03 * scale, t
        top2 = eager[t][0][0, 0].topk(2).values
        if float(top2[0] - top2[1]) > 0.06 * scale:
            assert int(logits[0, 0].argmax()) == eager[t][1], t
        tok = torch.tensor([[eager[t][1]]], device=DEV)  # teacher forcing with the static path's token
    cache._join_worker()
    del cache

    # ---- the captured step: two eager static warm-up steps, then replays
    logits2, cache = lm.forward(ids, None, max_new_tokens=64, offload_mode=mode)
    tok = logits2[:, -1].argmax(-1, keepdim=True)
    graph, token, glogits = lm.capture_decode(cache, tok, warmup=2)
    assert int(token) == eager[1][1]
    for t in range(replays):
        graph.replay()
        torch.cuda.synchronize()
        _ = (glogits.clone() * 2).sum().item()  # other work between replays, as a real loop would have
        assert torch.equal(glogits, eager[2 + t][0]), t
        assert int(token) == eager[2 + t][1], t
    if mode == "incremental":
        # a random-init model selects at chance overlap: most rows are new every step, none more than k
        assert all(0 < cache.last_fetch_count(f) <= k_sel for f in (2, 8, 18))


def test_full_width_four_layer_slice_matches_the_oracle_runner():
    """Hidden 4096 / FFN 14336 / vocabulary 128256 with four layers (filter layer 1, wait layer 2, sparse layer
    3 on the host tier): prefill and the first decode steps against the reference's layer forward on the CPU."""
    from test_gpu_model import _OracleRunner  # the reference's forward: select -> set_idx_on_gpu -> update -> attention

    shape = LlamaShape(num_hidden_layers=4)
    cfg = _config("1")
    lm = _build(shape, cfg, seed=2)
    ref = _OracleRunner(copy.deepcopy(lm).cpu().float(), _config("1"))
    chosen = {}  # filter layer -> the oracle's latest selection
    take = ref.cache.set_idx_on_gpu

    def record(idx, sel_layer_idx):
        chosen[sel_layer_idx] = idx.view(-1).clone()
        return take(idx, sel_layer_idx)

    ref.cache.set_idx_on_gpu = record
    n, steps = 1024, 4
    ids = torch.randint(0, shape.vocab_size, (1, n), generator=torch.Generator().manual_seed(3))
    want = ref.forward(ids)
    got, cache = lm.forward(ids.to(DEV), None, max_new_tokens=16)
    scale = float(want.abs().max())
    assert got.shape == (1, 1, shape.vocab_size) and got.dtype == torch.float32
    assert (got.cpu() - want).abs().max() < 0.1 * scale
    assert sorted(i for i, s in cache.layer_state.items() if s[0]) == [3]
    for t in range(steps):
        tok = want[:, -1].argmax(-1, keepdim=True)  # teacher forcing with the oracle's token
        want = ref.forward(tok)
        got, cache = lm.forward(tok.to(DEV), cache)
        assert (got.cpu() - want).abs().max() < 0.1 * scale, t
        top2 = want[0, 0].topk(2).values
        if float(top2[0] - top2[1]) > 0.2 * scale:
            assert int(got[0, 0].argmax()) == int(want[0, 0].argmax()), t
    # the selection itself: the filter layer's indices against the oracle's, near-ties aside (bf16 hidden states
    # against fp32 ones move scores by a fraction of a percent)
    mine, theirs = set(cache._idx[1][0].tolist()), set(chosen[1].tolist())
    assert len(mine) == len(theirs) == int(0.067 * n)
    assert len(mine - theirs) <= 4
    cache._join_worker()
