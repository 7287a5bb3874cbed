"""Seeded synthetic K/V/q for the benchmark configurations.

All values are drawn on the CPU in fp32 from torch.Generator().manual_seed(seed)
and then cast / moved, so the CPU checker and the GPU path see identical numbers.
Geometry defaults to Llama-3-8B decode: 32 q heads, 8 kv heads, head_dim 128.

Distribution (the benchmark's): q, K, V ~ N(0,1); token 0's key is scaled x8 (an
attention sink); a random 2% of the other tokens are heavy hitters whose keys are
0.5*q_dir + N(0,1), where q_dir[g] is the mean of kv head g's four q rows rescaled
to norm sqrt(head_dim).
"""
from __future__ import annotations

import math
from typing import Tuple

import torch

SEED_DATA, SEED_HEAVY, SEED_QNEXT, SEED_PAGES, SEED_LENS = 1234, 1235, 1236, 1237, 1238


def filter_layer_inputs(n: int, hq: int = 32, hkv: int = 8, d: int = 128, seed: int = SEED_DATA,
                        heavy_frac: float = 0.02) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """q (1,hq,1,d), K (1,hkv,n,d), V (1,hkv,n,d), fp32 on the CPU."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn((1, hq, 1, d), generator=g)
    k = torch.randn((1, hkv, n, d), generator=g)
    v = torch.randn((1, hkv, n, d), generator=g)
    k[:, :, 0, :] *= 8.0
    n_heavy = int(round(heavy_frac * n))
    if n_heavy > 0 and n > 1:
        gh = torch.Generator().manual_seed(seed - SEED_DATA + SEED_HEAVY)
        pos = torch.randperm(n - 1, generator=gh)[:n_heavy] + 1
        grp = hq // hkv
        q_dir = q[0, :, 0, :].view(hkv, grp, d).mean(dim=1)
        q_dir = q_dir / q_dir.norm(dim=-1, keepdim=True) * math.sqrt(d)
        noise = torch.randn((hkv, n_heavy, d), generator=gh)
        k[0, :, pos, :] = 0.5 * q_dir[:, None, :] + noise
    return q, k, v


def fresh_q(hq: int = 32, d: int = 128, seed: int = SEED_QNEXT, batch: int = 1) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    return torch.randn((batch, hq, 1, d), generator=g)


def token_major(x: torch.Tensor) -> torch.Tensor:
    """(b,Hkv,N,D) values re-stored token-major (b,N,Hkv,D) and returned as a
    (b,Hkv,N,D) view: token stride Hkv*D, head stride D."""
    return x.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)


def ragged_lengths(batch: int = 16, lo: int = 8192, hi: int = 32768, seed: int = SEED_LENS) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(lo, hi + 1, (batch,), generator=g, dtype=torch.int64).to(torch.int32)


def shuffled_page_table(lengths: torch.Tensor, page_size: int = 16, seed: int = SEED_PAGES):
    """(page_table (batch, max_pages) int32 padded with 0, num_pages)."""
    g = torch.Generator().manual_seed(seed)
    pages = [(int(l) + page_size - 1) // page_size for l in lengths]
    total = sum(pages)
    perm = torch.randperm(total, generator=g).to(torch.int32)
    table = torch.zeros((len(pages), max(pages)), dtype=torch.int32)
    o = 0
    for b, p in enumerate(pages):
        table[b, :p] = perm[o:o + p]
        o += p
    return table, total
