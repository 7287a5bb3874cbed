"""Writes the committed golden vectors of the selection path.

The reference's own tests hold no vectors for this path, so these come from the
CPU oracle (oracle/okv_oracle.py, pinned by tests/test_oracle_pinning.py) on the
seeded synthetic inputs of omnikv_amd/synth.py.  K and V are not stored: they are
regenerated from the seed.  Run from the repository root:

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from omnikv_amd import synth  # noqa: E402
from oracle import okv_oracle as orc  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
SELECTORS = ("last", "softmax_before_last", "softmax_sum_last")


def filter_case(n: int, tail: int):
    kk = max(1, orc.num_selected_tokens(0.067, n))
    q, k, v = synth.filter_layer_inputs(n)
    _, k2, v2 = synth.filter_layer_inputs(n, seed=synth.SEED_DATA + 100)
    qn = synth.fresh_q()
    g = torch.Generator().manual_seed(4242 + n)
    tk = torch.randn((1, 8, tail, 128), generator=g)
    tv = torch.randn((1, 8, tail, 128), generator=g)
    out = {"n": n, "k": kk, "tail": tail, "dense_out": orc.gqa_attention(q, k, v)[0, :, 0].numpy()}
    for sel in SELECTORS:
        idx, scores, o = orc.filter_layer_op(q, k, v2, k2, qn, kk, sel, tk if tail else None, tv if tail else None)
        assert not orc.has_boundary_tie(scores, kk)
        out[f"scores_{sel}"] = scores[0].numpy()
        out[f"idx_{sel}"] = idx[0].numpy().astype(np.int32)
        out[f"sparse_out_{sel}"] = o[0, :, 0].numpy()
    return out


def tie_cases():
    g = torch.Generator().manual_seed(99)
    s = (torch.randint(0, 7, (4, 500), generator=g).float() - 3.0) * 0.5
    s[1, 100] = float("inf")
    s[2, 7] = -0.0
    s[2, 8] = 0.0
    ks = [1, 37, 250, 499]
    out = {"scores": s.numpy(), "ks": np.array(ks, dtype=np.int32)}
    for k in ks:
        out[f"idx_k{k}"] = orc.select_topk_stable(s, k).numpy().astype(np.int32)
    return out


def main():
    for n, tail in ((64, 0), (1000, 3), (4096, 1)):
        np.savez_compressed(os.path.join(HERE, f"filter_op_n{n}.npz"), **filter_case(n, tail))
    np.savez_compressed(os.path.join(HERE, "topk_ties.npz"), **tie_cases())
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))


if __name__ == "__main__":
    main()
