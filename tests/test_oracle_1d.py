"""1D oracle pinned against independent statements."""
import pytest
import torch

from oracle import na1d_oracle as O1
from oracle import na2d_oracle as O


def _rand(shape, seed=0, n=4, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(shape, generator=g, dtype=torch.float32).to(dtype) for _ in range(n)]


@pytest.mark.parametrize("k", [3, 5, 7, 9, 11])
def test_gather_matches_dense_mask_and_brute(k):
    q, kk, v, _ = _rand((2, 3, 16, 2), 0)  # test.py:51 shape
    o = O1.natten1d_gather(q, kk, v, k)
    assert O.max_abs_err(o, O1.natten1d_dense_mask(q, kk, v, k)) < 1e-12
    assert O.max_abs_err(o, O1.natten1d_brute(q, kk, v, k)) < 1e-12


def test_special_cases():
    q, kk, v, _ = _rand((1, 2, 9, 4), 1)
    assert O.max_abs_err(O1.natten1d_gather(q, kk, v, 1), v) < 1e-14
    p = torch.softmax(q @ kk.transpose(-1, -2), dim=-1)
    assert O.max_abs_err(O1.natten1d_gather(q, kk, v, 9), p @ v) < 1e-12
    fl = lambda t: t.flip(2)
    assert O.max_abs_err(O1.natten1d_gather(fl(q), fl(kk), fl(v), 5), fl(O1.natten1d_gather(q, kk, v, 5))) < 1e-12


def test_gradcheck_recipe_of_reference():
    # gradcheck.py:6-15: double (B=2, heads=3, T=8, d=2), k=7, eps=1e-6, atol=1e-4
    q, kk, v = (t.requires_grad_(True) for t in _rand((2, 3, 8, 2), 2, 3))
    assert torch.autograd.gradcheck(lambda a, b, c: O1.natten1d_gather(a, b, c, 7), (q, kk, v),
                                    eps=1e-6, atol=1e-4)


@pytest.mark.parametrize("k", [3, 7])
def test_explicit_backward_matches_autograd_of_dense_mask(k):
    q, kk, v, g = _rand((2, 2, 13, 5), 3)
    a, b, c = (t.clone().requires_grad_(True) for t in (q, kk, v))
    O1.natten1d_dense_mask(a, b, c, k).backward(g)
    _, _, dq, dk, dv = O1.natten1d_explicit(q, kk, v, g, k)
    for x, r in ((dq, a.grad), (dk, b.grad), (dv, c.grad)):
        assert O.max_abs_err(x, r) < 1e-11


def test_loop_restatement_equals_explicit():
    q, kk, v, g = _rand((1, 2, 11, 3), 4)
    for k in (3, 5, 9):
        a, b, c = (t.clone().requires_grad_(True) for t in (q, kk, v))
        o = O1.natten1d_loops(a, b, c, k)
        o.backward(g)
        ref = O1.natten1d_explicit(q, kk, v, g, k)
        for x, r in ((o, ref[0]), (a.grad, ref[2]), (b.grad, ref[3]), (c.grad, ref[4])):
            assert O.max_abs_err(x.detach(), r) < 1e-11


def test_c_oracle_1d(c_oracle):
    q, kk, v, g = _rand((2, 3, 37, 16), 5, 4, torch.float32)
    ref = O1.natten1d_explicit(q, kk, v, g, 7, 0.5)
    o, lse = c_oracle.forward_1d(q, kk, v, 7, 0.5)
    dq, dk, dv = c_oracle.backward_1d(q, kk, v, g, 7, 0.5)
    for x, r in ((o, ref[0]), (lse, ref[1]), (dq, ref[2]), (dk, ref[3]), (dv, ref[4])):
        assert O.max_abs_err(x, r) < 1e-5
