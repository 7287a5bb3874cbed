"""Assertions shared by the GPU parity tests."""
import torch


def assert_near_tie_only(got_scores, want_scores, got_idx, want_idx, kk):
    """The kernel selected on ITS scores, the oracle on its own; both sets hold kk tokens.
    Let kth be the oracle's k-th largest value.

    Absolute band (any scores): with delta = max |got - want| over the row, the two vectors'
    k-th largest values differ by at most delta, so a token only the kernel took has an oracle
    score >= kth - 2 delta and a token only the oracle took <= kth + 2 delta.

    Relative band (positive scores: the softmax selectors, whose values span many decades, so
    the row-wide delta says little at the cut): with eps = max |got/want - 1| over the tokens
    whose oracle score is >= kth/2, and no smaller token scored above 0.75 kth by the kernel,
    the k-th values differ by a factor within (1 +- eps); a token only the kernel took has an
    oracle score >= kth (1-eps)/(1+eps), one only the oracle took <= kth (1+eps)/(1-eps).

    A token outside these bands is a real disagreement (an off-by-one in the scored range, a
    wrong row), not rounding.  Returns (#differing, delta, eps)."""
    delta = float((got_scores - want_scores).abs().max())
    kth = float(torch.topk(want_scores, kk).values[-1])
    a, b = set(got_idx.tolist()), set(want_idx.tolist())
    assert len(a) == kk and len(b) == kk
    only_kernel = torch.tensor(sorted(a - b), dtype=torch.int64)
    only_oracle = torch.tensor(sorted(b - a), dtype=torch.int64)
    assert len(only_kernel) == len(only_oracle)
    eps = None
    if bool((want_scores > 0).all()):
        near = want_scores >= kth / 2
        eps = float((got_scores[near] / want_scores[near] - 1).abs().max())
        assert eps < 1e-3, eps
        assert bool((got_scores[~near] < 0.75 * kth).all())
    if len(only_kernel):
        assert float(want_scores[only_kernel].min()) >= kth - 2 * delta
        assert float(want_scores[only_oracle].max()) <= kth + 2 * delta
        if eps is not None:
            assert float(want_scores[only_kernel].min()) >= kth * (1 - eps) / (1 + eps)
            assert float(want_scores[only_oracle].max()) <= kth * (1 + eps) / (1 - eps)
    # and the bands are narrow: rounding may swap a handful of tokens, not a percent of them
    assert len(only_kernel) <= max(2, kk // 1000), (len(only_kernel), delta, eps, kth)
    return len(only_kernel), delta, eps
