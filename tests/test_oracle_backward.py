"""Gradients of the oracle pinned by autograd of independent forwards,
numerical differentiation and sum invariants."""
import pytest
import torch

from oracle import na2d_oracle as O


def _rand(shape, seed=0, n=4, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(shape, generator=g, dtype=torch.float32).to(dtype) for _ in range(n)]


def _autograd(fn, q, k, v, g):
    q, k, v = (t.detach().clone().requires_grad_(True) for t in (q, k, v))
    fn(q, k, v).backward(g)
    return q.grad, k.grad, v.grad


@pytest.mark.parametrize("k", [3, 5, 7, 9, 11])
def test_explicit_backward_matches_autograd_of_dense_mask(k):
    # test.py:51-53 shapes (B=2, heads=6, 16x16, d=2), all its kernel sizes
    q, kk, v, g = _rand((2, 6, 16, 16, 2), 0)
    o, lse, dq, dk, dv = O.natten2d_explicit(q, kk, v, g, k)
    rq, rk, rv = _autograd(lambda a, b, c: O.natten2d_dense_mask(a, b, c, k), q, kk, v, g)
    for x, r in ((dq, rq), (dk, rk), (dv, rv)):
        assert O.max_abs_err(x, r) < 1e-10


@pytest.mark.parametrize("shape,k,scale", [((1, 2, 9, 11, 5), 5, 1.0), ((2, 1, 14, 14, 8), 7, 0.3),
                                           ((1, 1, 13, 13, 4), 13, 1.0), ((1, 1, 19, 15, 3), 13, 1.0)])
def test_gather_grads_match_explicit(shape, k, scale):
    q, kk, v, g = _rand(shape, 1)
    a = O.natten2d_gather_grads(q, kk, v, g, k, scale)
    b = O.natten2d_explicit(q, kk, v, g, k, scale)
    for x, y in zip(a, b):
        assert O.max_abs_err(x, y) < 1e-10


def test_gradcheck_2d():
    # the reference grad-checks only 1D (gradcheck.py:6-15); same recipe in 2D
    q, kk, v = (t.requires_grad_(True) for t in _rand((1, 2, 6, 7, 2), 2, 3))
    assert torch.autograd.gradcheck(lambda a, b, c: O.natten2d_gather(a, b, c, 5),
                                    (q, kk, v), eps=1e-6, atol=1e-4)


def test_gradient_invariants():
    q, kk, v, g = _rand((2, 2, 10, 12, 6), 3)
    o, lse, dq, dk, dv = O.natten2d_explicit(q, kk, v, g, 5)
    # rows of P sum to one: total dV equals total dO per (b, n, channel)
    assert O.max_abs_err(dv.sum((2, 3)), g.sum((2, 3))) < 1e-10
    # sum_j dS_j = 0 for every query, so sum over keys of dK vanishes only
    # when weighted by nothing: sum_keys dK = sum_q (sum_j dS_j) q = 0
    assert dk.sum((2, 3)).abs().max() < 1e-10
    # k = 1: P == 1, so dQ = dK = 0 and dV = dO
    o1, _, dq1, dk1, dv1 = O.natten2d_explicit(q, kk, v, g, 1)
    assert dq1.abs().max() < 1e-13 and dk1.abs().max() < 1e-13
    assert O.max_abs_err(dv1, g) < 1e-14


def test_loop_restatement_backward_equals_explicit():
    q, kk, v, g = _rand((1, 2, 8, 9, 3), 4)
    for k in (3, 5):
        rq, rk, rv = _autograd(lambda a, b, c: O.natten2d_loops(a, b, c, k), q, kk, v, g)
        _, _, dq, dk, dv = O.natten2d_explicit(q, kk, v, g, k)
        assert O.max_abs_err(rq, dq) < 1e-11
        assert O.max_abs_err(rk, dk) < 1e-11
        assert O.max_abs_err(rv, dv) < 1e-11


@pytest.mark.parametrize("shape,k,scale", [((2, 3, 16, 16, 2), 3, 1.0), ((1, 2, 14, 14, 32), 7, 32 ** -0.5),
                                           ((1, 1, 20, 17, 8), 13, 1.0), ((1, 2, 16, 16, 2), 11, 1.0)])
def test_c_oracle_backward(shape, k, scale, c_oracle):
    q, kk, v, g = _rand(shape, 6, 4, torch.float32)
    _, _, dq, dk, dv = O.natten2d_explicit(q, kk, v, g, k, scale)
    cq, ck, cv = c_oracle.backward(q, kk, v, g, k, scale)
    for x, r in ((cq, dq), (ck, dk), (cv, dv)):
        assert O.max_abs_err(x, r) < 1e-5 * max(1.0, r.abs().max().item())
