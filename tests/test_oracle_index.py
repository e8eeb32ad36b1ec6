"""Window rules of the oracle, pinned by brute force (no formula is retyped:
each check derives the answer from the definition by enumeration)."""
import pytest
import torch

from oracle import na2d_oracle as O

KS = [1, 3, 5, 7, 9, 11, 13]


def _nearest_window(i, L, k):
    """Definition: among the windows [s, s+k) inside [0, L), the one whose
    centre s + k//2 is nearest to i (unique for odd k)."""
    best = min(range(0, L - k + 1), key=lambda s: (abs(s + k // 2 - i), s))
    return best


@pytest.mark.parametrize("k", KS)
def test_win_start_is_nearest_inside_window(k):
    for L in range(k, 40):
        for i in range(L):
            assert O.win_start(i, L, k) == _nearest_window(i, L, k), (i, L, k)


@pytest.mark.parametrize("k", KS)
def test_win_start_matches_piecewise_rule_of_reference(k):
    # e_natten/pytorch.py:7-11 is written as "max(i - k//2, 0), then pull back
    # by the overshoot past the end"; evaluate that description literally.
    for L in range(k, 40):
        for i in range(L):
            s = max(i - k // 2, 0)
            overshoot = i + k // 2 - (L - 1)
            if overshoot >= 0:
                s -= overshoot
            assert O.win_start(i, L, k) == s


@pytest.mark.parametrize("k", KS)
def test_inv_range_is_exact_inverse(k):
    for L in list(range(k, 2 * k + 3)) + [14, 16, 28, 32, 64]:
        if L < k:
            continue
        for i in range(L):
            attending = [x for x in range(L)
                         if O.win_start(x, L, k) <= i < O.win_start(x, L, k) + k]
            lo, hi = O.inv_range(i, L, k)
            assert attending == list(range(lo, hi)), (i, L, k)
            # k in the interior, k + k//2 beside one edge; both edges can
            # add up when the image is narrower than 2k
            assert len(attending) <= (k + k // 2 if L >= 2 * k else k + 2 * (k // 2))


@pytest.mark.parametrize("k", KS)
def test_c_oracle_index_rules_agree(k, c_oracle):
    for L in [k, k + 1, 2 * k - 1, 2 * k, 17, 33]:
        for i in range(L):
            assert c_oracle.win_start(i, L, k) == O.win_start(i, L, k)
            assert c_oracle.inv_range(i, L, k) == O.inv_range(i, L, k)


def test_neighbour_index_and_mask_agree():
    for (H, W, k) in [(5, 6, 3), (7, 7, 7), (9, 12, 5)]:
        idx = O.neighbour_index(H, W, k)
        m = O.neighbour_mask(H, W, k)
        assert idx.shape == (H * W, k * k)
        dense = torch.zeros(H * W, H * W, dtype=torch.bool)
        dense.scatter_(1, idx, True)
        assert torch.equal(dense, m)
        assert (m.sum(1) == k * k).all()
        # every window is a contiguous k x k block inside the image
        rows = idx // W
        cols = idx % W
        assert ((rows.max(1).values - rows.min(1).values) == k - 1).all()
        assert ((cols.max(1).values - cols.min(1).values) == k - 1).all()


def test_window_is_reflection_symmetric():
    # flipping the axis maps window(i) onto window(L-1-i) for odd k
    for k in KS:
        for L in range(k, 30):
            for i in range(L):
                s = O.win_start(i, L, k)
                sf = O.win_start(L - 1 - i, L, k)
                assert sf == L - (s + k)
