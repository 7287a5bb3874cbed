"""The per-token layer operations (one HIP launch each) against the op-by-op torch chains they
replace -- transformers' LlamaRMSNorm / apply_rotary_pos_emb / act_fn(gate) * up as the model's
modules state them -- on the same GPU.  Rotary embedding and SiLU*up round exactly where the
chains round, so they must be bit-equal; RMSNorm sums the squares in another order, so its
normaliser may differ in the last fp32 bit and an output by one unit of the tensor type."""
import pytest
import torch
import torch.nn.functional as F

from omnikv_amd import model as okv_model
from omnikv_amd import ops
from omnikv_amd.config import OmniKVConfig
from omnikv_amd.model import LlamaShape, OmniKVMulLM, RMSNorm, RotaryEmbedding
from omnikv_amd.selector import apply_rotary_pos_emb

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.bfloat16, torch.float16, torch.float32]


def _ulp_close(got, want, dtype):
    """Equal up to one unit in the last place of `dtype` (relative 2^-7 / 2^-10 / 2^-22 of the value)."""
    rel = {torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10, torch.float32: 2.0 ** -21}[dtype]
    diff = (got.float() - want.float()).abs()
    assert bool((diff <= rel * want.float().abs() + 1e-30).all()), float((diff / want.float().abs().clamp_min(1e-30)).max())
    return float((diff > 0).float().mean())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,hidden", [(1, 4096), (3, 256), (2, 1000)])
def test_rmsnorm_matches_the_module_chain(dtype, rows, hidden):
    g = torch.Generator(device=DEV).manual_seed(hidden + rows)
    x = (torch.randn((rows, 1, hidden), generator=g, device=DEV) * 3).to(dtype)
    r = torch.randn((rows, 1, hidden), generator=g, device=DEV).to(dtype)
    norm = RMSNorm(hidden, 1e-5).to(DEV)
    with torch.no_grad():
        norm.weight.copy_(1 + 0.1 * torch.randn(hidden, generator=g, device=DEV))
    norm = norm.to(dtype)
    okv_model.FUSED_LAYER_OPS = False
    try:
        want = norm(x)
        want_n, want_sum = norm(x, residual=r)
    finally:
        okv_model.FUSED_LAYER_OPS = True
    got = norm(x)
    got_n, got_sum = norm(x, residual=r)
    assert torch.equal(got_sum, want_sum) and torch.equal(want_sum, r + x)  # the residual stream: bit-equal
    changed = _ulp_close(got, want, dtype)
    _ulp_close(got_n, want_n, dtype)
    if dtype != torch.float32:  # a last-bit difference of the fp32 normaliser rarely survives rounding to 16 bits
        assert changed < 0.02


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bsz", [1, 3])
def test_rope_is_bit_equal_to_apply_rotary_pos_emb(dtype, bsz):
    hq, hkv, d = 32, 8, 128
    g = torch.Generator(device=DEV).manual_seed(bsz)
    q = torch.randn((bsz, 1, hq * d), generator=g, device=DEV).to(dtype)
    k = torch.randn((bsz, 1, hkv * d), generator=g, device=DEV).to(dtype)
    pos = torch.tensor([[131072 + 7 * b] for b in range(bsz)], device=DEV)
    cos, sin = RotaryEmbedding(d, 500000.0).to(DEV)(q, pos)
    want_q, want_k = apply_rotary_pos_emb(q.view(bsz, 1, hq, d).transpose(1, 2), k.view(bsz, 1, hkv, d).transpose(1, 2),
                                          cos, sin)
    got_q, got_k = ops.rope(q, k, cos, sin, hq, hkv)
    assert got_q.shape == (bsz, hq, 1, d) and got_k.shape == (bsz, hkv, 1, d)
    assert torch.equal(got_q, want_q) and torch.equal(got_k, want_k)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("on_device", [False, True])
def test_rope_append_writes_the_rows_append_would(dtype, on_device):
    """Rotation + append in one launch: the K / V stores end up exactly as after rope() followed by
    writing the rows at that position, rows elsewhere untouched; position from the host or from device memory."""
    hq, hkv, d, bsz, cap, pos = 32, 8, 128, 2, 37, 29
    g = torch.Generator(device=DEV).manual_seed(9)
    q = torch.randn((bsz, 1, hq * d), generator=g, device=DEV).to(dtype)
    k = torch.randn((bsz, 1, hkv * d), generator=g, device=DEV).to(dtype)
    v = torch.randn((bsz, 1, hkv * d), generator=g, device=DEV).to(dtype)
    cos, sin = RotaryEmbedding(d, 500000.0).to(DEV)(q, torch.tensor([[5000], [77]], device=DEV))
    ks = torch.randn((bsz, hkv, cap, d), generator=g, device=DEV).to(dtype)
    vs = torch.randn((bsz, hkv, cap, d), generator=g, device=DEV).to(dtype)
    want_q, want_k = ops.rope(q, k, cos, sin, hq, hkv)
    want_ks, want_vs = ks.clone(), vs.clone()
    want_ks[:, :, pos] = want_k[:, :, 0]
    want_vs[:, :, pos] = v.view(bsz, hkv, d)
    where = torch.tensor([pos], dtype=torch.int64, device=DEV) if on_device else pos
    got_q = ops.rope_append(q, k, v, cos, sin, hq, hkv, ks, vs, where)
    assert torch.equal(got_q, want_q) and torch.equal(ks, want_ks) and torch.equal(vs, want_vs)
    with pytest.raises(ValueError):
        ops.rope_append(q, k, v, cos, sin, hq, hkv, ks, vs, cap)


@pytest.mark.parametrize("dtype", DTYPES)
def test_silu_mul_is_bit_equal_to_the_torch_ops(dtype):
    g = torch.Generator(device=DEV).manual_seed(5)
    gate = (torch.randn((2, 1, 14336), generator=g, device=DEV) * 4).to(dtype)
    up = torch.randn((2, 1, 14336), generator=g, device=DEV).to(dtype)
    assert torch.equal(ops.silu_mul(gate, up), F.silu(gate) * up)


def test_decode_step_with_and_without_the_fused_ops():
    """A whole decode step of the bf16 model: fused per-token ops against the op-by-op path, same
    weights and cache contents.  Only RMSNorm can differ (by one bf16 unit here and there), so the
    logits stay within bf16 noise and the selections agree."""
    shape = LlamaShape(hidden_size=512, intermediate_size=1024, vocab_size=2000, num_hidden_layers=6,
                       num_attention_heads=32, num_key_value_heads=8, head_dim=128)
    cfg = OmniKVConfig(model_cls="multi", cache_cls="multi", do_select_layers="1,3", num_wait_load_layers=1,
                       real_offload=False, dense_more=True, num_of_selected_tokens=0.1, selector_cls="last", window_size=4)
    ids = torch.randint(0, 2000, (1, 600), generator=torch.Generator().manual_seed(3)).to(DEV)
    outs = {}
    for fused in (False, True):
        okv_model.FUSED_LAYER_OPS = fused
        try:
            lm = OmniKVMulLM(shape, cfg).to(torch.bfloat16).to(DEV)
            lm.init_weights(seed=2, std=0.05)
            logits, cache = lm.forward(ids, None, max_new_tokens=8)
            steps = []
            tok = logits[:, -1].argmax(-1, keepdim=True)
            for _ in range(3):
                logits, cache = lm.forward(tok, cache)
                steps.append(logits.clone())
                tok = torch.tensor([[17]], device=DEV)  # the same token on both sides whatever the argmax
            outs[fused] = (steps, [cache._idx[l].clone() for l in (1, 3)])
        finally:
            okv_model.FUSED_LAYER_OPS = True
    for a, b in zip(outs[False][0], outs[True][0]):
        assert (a - b).abs().max() < 0.05 * a.abs().max()
    for a, b in zip(outs[False][1], outs[True][1]):
        assert len(set(a[0].tolist()) & set(b[0].tolist())) >= a.shape[1] - 3
