"""Forward of the oracle pinned against independent statements."""
import pytest
import torch

from oracle import na2d_oracle as O


def _rand(shape, seed=0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(shape, generator=g, dtype=torch.float32).to(dtype) for _ in range(3)]


@pytest.mark.parametrize("shape,k", [((1, 1, 5, 6, 4), 3), ((1, 2, 6, 5, 3), 5), ((1, 1, 7, 7, 2), 7)])
def test_gather_matches_brute_force(shape, k):
    q, kk, v = _rand(shape, 1)
    o, lse = O.natten2d_gather(q, kk, v, k, return_lse=True)
    ob, lb = O.natten2d_brute(q, kk, v, k)
    assert O.max_abs_err(o, ob) < 1e-12
    assert O.max_abs_err(lse, lb) < 1e-12


@pytest.mark.parametrize("k", [3, 5, 7, 9, 11, 13])
@pytest.mark.parametrize("hw", [(16, 16), (13, 19)])
def test_gather_matches_dense_mask_sdpa(k, hw):
    H, W = hw
    if min(H, W) < k:
        pytest.skip("image smaller than window")
    q, kk, v = _rand((2, 2, H, W, 8), 2)
    o = O.natten2d_gather(q, kk, v, k)
    od = O.natten2d_dense_mask(q, kk, v, k)
    assert O.max_abs_err(o, od) < 1e-11


def test_scale_argument():
    q, kk, v = _rand((1, 2, 8, 8, 16), 3)
    a = O.natten2d_gather(q, kk, v, 3, scale=0.25)
    b = O.natten2d_gather(q * 0.25, kk, v, 3)
    c = O.natten2d_dense_mask(q, kk, v, 3, scale=0.25)
    assert O.max_abs_err(a, b) < 1e-12
    assert O.max_abs_err(a, c) < 1e-12


def test_k1_returns_v():
    q, kk, v = _rand((2, 1, 4, 5, 3), 4)
    o, lse = O.natten2d_gather(q, kk, v, 1, return_lse=True)
    assert O.max_abs_err(o, v) < 1e-14
    assert O.max_abs_err(lse, (q * kk).sum(-1)) < 1e-12


def test_full_window_is_global_attention():
    q, kk, v = _rand((1, 2, 5, 5, 4), 5)
    o = O.natten2d_gather(q, kk, v, 5)
    f = lambda t: t.reshape(1, 2, 25, 4)
    p = torch.softmax(f(q) @ f(kk).transpose(-1, -2), dim=-1)
    assert O.max_abs_err(o, (p @ f(v)).reshape(1, 2, 5, 5, 4)) < 1e-12


def test_invariances():
    q, kk, v = _rand((1, 2, 9, 10, 6), 6)
    o = O.natten2d_gather(q, kk, v, 5)
    # constant V -> constant O
    vc = torch.ones_like(v) * 3.5
    assert O.max_abs_err(O.natten2d_gather(q, kk, vc, 5), vc) < 1e-12
    # adding one vector to every key shifts all logits of a query equally
    shift = torch.randn(6, dtype=torch.float64)
    assert O.max_abs_err(O.natten2d_gather(q, kk + shift, v, 5), o) < 1e-10
    # flips and transposition of the image axes commute with the operator
    fl = lambda t: t.flip(2)
    assert O.max_abs_err(O.natten2d_gather(fl(q), fl(kk), fl(v), 5), fl(o)) < 1e-12
    tr = lambda t: t.transpose(2, 3)
    assert O.max_abs_err(O.natten2d_gather(tr(q), tr(kk), tr(v), 5), tr(o)) < 1e-12


@pytest.mark.parametrize("k", [3, 5, 7, 9])
def test_loop_restatement_clean_equals_gather(k):
    q, kk, v = _rand((2, 2, 11, 13, 4), 7)
    o = O.natten2d_gather(q, kk, v, k)
    ol = O.natten2d_loops(q, kk, v, k)
    assert O.max_abs_err(o, ol) < 1e-12


def test_loop_restatement_row_band():
    q, kk, v = _rand((1, 1, 12, 9, 4), 8)
    o = O.natten2d_gather(q, kk, v, 5)
    ol = O.natten2d_loops(q, kk, v, 5, (4, 8))
    assert O.max_abs_err(o[:, :, 4:8], ol[:, :, 4:8]) < 1e-12
    assert ol[:, :, :4].abs().max() == 0 and ol[:, :, 8:].abs().max() == 0


@pytest.mark.parametrize("shape,k", [((2, 3, 16, 16, 2), 3), ((1, 2, 14, 14, 32), 7), ((1, 1, 20, 17, 8), 13)])
def test_c_oracle_forward(shape, k, c_oracle):
    q, kk, v = _rand(shape, 10, torch.float32)
    o, lse = O.natten2d_gather(q.double(), kk.double(), v.double(), k, return_lse=True)
    oc, lc = c_oracle.forward(q, kk, v, k)
    assert O.max_abs_err(oc, o) < 2e-6
    assert O.max_abs_err(lc, lse) < 4e-6


def test_unfused_comparator_equals_fused():
    # the procedure of the reference's test.py:16-21: qk -> softmax -> av
    q, kk, v = _rand((2, 6, 16, 16, 2), 0)
    for k in [3, 5, 7, 9, 11]:
        p = torch.softmax(O.natten2d_qk(q, kk, k), dim=-1)
        assert O.max_abs_err(O.natten2d_av(p, v, k), O.natten2d_gather(q, kk, v, k)) < 1e-12


@pytest.mark.parametrize("H,W,ks,dil", [(12, 13, 3, 2), (15, 11, 3, 3), (21, 20, 5, 4), (9, 10, 3, 1)])
def test_dilated_window_rule_is_the_plain_rule_on_residue_classes(H, W, ks, dil):
    # NATTEN's dilated window start, restated in the oracle, against the statement the
    # product relies on: pixels of one residue class modulo the dilation form a sub-grid
    # on which the neighbourhood is the undilated one.
    for L in (H, W):
        for i in range(L):
            r, t = i % dil, i // dil
            Ls = (L - r + dil - 1) // dil
            assert O.dilated_win_start(i, L, ks, dil) == r + dil * O.win_start(t, Ls, ks)
    g = torch.Generator().manual_seed(5)
    q, k, v = (torch.randn(1, 2, H, W, 4, generator=g, dtype=torch.float64) for _ in range(3))
    ref = O.natten2d_dilated_dense_mask(q, k, v, ks, dil)
    got = torch.empty_like(ref)
    for i in range(dil):
        for j in range(dil):
            sub = (slice(None), slice(None), slice(i, None, dil), slice(j, None, dil))
            got[sub] = O.natten2d_gather(q[sub], k[sub], v[sub], ks)
    assert torch.allclose(got, ref, atol=1e-12)


def test_axis_window_mask_rules():
    # centred axis: the reference's rule; causal axis: the last k positions up to the
    # query's own, which for k = L is the lower triangle of ordinary causal attention
    for L in (1, 2, 5, 9, 16):
        for k in range(1, L + 1):
            mc = O.axis_window_mask(L, k, causal=True)
            for i in range(L):
                row = mc[i].nonzero().flatten().tolist()
                assert row == list(range(max(i - k + 1, 0), i + 1)), (L, k, i, row)
            if k % 2 == 1:
                m = O.axis_window_mask(L, k)
                for i in range(L):
                    s0 = O.win_start(i, L, k)
                    assert m[i].nonzero().flatten().tolist() == list(range(s0, s0 + k))
            else:
                with pytest.raises(ValueError):
                    O.axis_window_mask(L, k)
        assert torch.equal(O.axis_window_mask(L, L, causal=True),
                           torch.ones(L, L).tril().bool())


def test_window_dense_mask_special_cases():
    g = torch.Generator().manual_seed(5)
    q, k, v = (torch.randn(2, 2, 7, 9, 4, generator=g, dtype=torch.float64) for _ in range(3))
    # square centred window: the pinned dense-mask oracle of the reference's operator
    a = O.natten2d_window_dense_mask(q, k, v, (5, 5), (False, False), 0.7)
    b = O.natten2d_dense_mask(q, k, v, 5, 0.7)
    assert torch.allclose(a, b, atol=1e-12)
    # a rectangular window with one full axis: rows attend all rows, columns their 3 neighbours
    c = O.natten2d_window_dense_mask(q, k, v, (7, 3))
    s = torch.einsum("bnxyd,bnuwd->bnxyuw", q, k)
    keep = O.axis_window_mask(9, 3)[None, None, None, :, None, :].expand_as(s)
    p = torch.softmax(s.masked_fill(~keep, float("-inf")).flatten(-2), -1).view_as(s)
    assert torch.allclose(c, torch.einsum("bnxyuw,bnuwd->bnxyd", p, v), atol=1e-12)
    # 1D causal with the window as long as the sequence: textbook causal attention
    q1, k1, v1 = (t[:, :, :1] for t in (q, k, v))
    d = O.natten2d_window_dense_mask(q1, k1, v1, (1, 9), (False, True))
    ref = torch.nn.functional.scaled_dot_product_attention(q1[:, :, 0], k1[:, :, 0], v1[:, :, 0],
                                                           is_causal=True, scale=1.0)
    assert torch.allclose(d[:, :, 0], ref, atol=1e-12)
    # the first query of a causal axis only sees itself: its output is its own value
    e = O.natten2d_window_dense_mask(q, k, v, (3, 4), (True, True))
    assert torch.allclose(e[:, :, 0, 0], v[:, :, 0, 0], atol=1e-12)


def test_relative_position_bias_oracle():
    # NATTEN's published bias index (get_pb_start: ns + max(ns - i, 0) + min(L - i - 1 - ns, 0),
    # plus the position inside the window) is key - query + k - 1 for every query of every axis
    for L in (5, 8, 13):
        for k in (1, 3, 5):
            ns = k // 2
            for i in range(L):
                pb = ns + (ns - i if i < ns else 0) + (L - i - 1 - ns if i + ns >= L else 0)
                s0 = O.win_start(i, L, k)
                for j in range(k):
                    assert pb + j == (s0 + j) - i + k - 1, (L, k, i, j)
    g = torch.Generator().manual_seed(9)
    q, k, v = (torch.randn(1, 2, 6, 7, 4, generator=g, dtype=torch.float64) for _ in range(3))
    rpb = torch.randn(2, 5, 9, generator=g, dtype=torch.float64, requires_grad=True)
    base = O.natten2d_window_dense_mask(q, k, v, (3, 5), scale=0.6)
    # a zero bias and a constant bias change nothing (softmax is shift-invariant)
    assert torch.allclose(O.natten2d_window_dense_mask(q, k, v, (3, 5), scale=0.6,
                                                       rpb=torch.zeros(2, 5, 9, dtype=torch.float64)), base)
    assert torch.allclose(O.natten2d_window_dense_mask(q, k, v, (3, 5), scale=0.6,
                                                       rpb=torch.full((2, 5, 9), 1.7, dtype=torch.float64)), base)
    # brute force for one interior and one border query
    o = O.natten2d_window_dense_mask(q, k, v, (3, 5), scale=0.6, rpb=rpb)
    for (x, y) in ((3, 3), (0, 6), (5, 0)):
        x0, y0 = O.win_start(x, 6, 3), O.win_start(y, 7, 5)
        for n in range(2):
            logits, vals = [], []
            for i in range(3):
                for j in range(5):
                    kx, ky = x0 + i, y0 + j
                    logits.append(0.6 * (q[0, n, x, y] @ k[0, n, kx, ky]) + rpb[n, kx - x + 2, ky - y + 4])
                    vals.append(v[0, n, kx, ky])
            p = torch.softmax(torch.stack(logits), 0)
            assert torch.allclose(o[0, n, x, y], (p[:, None] * torch.stack(vals)).sum(0), atol=1e-12)
    # every query's dS sums to zero, so the bias gradient sums to zero per head
    (d_rpb,) = torch.autograd.grad((o * torch.randn(o.shape, generator=g, dtype=torch.float64)).sum(), rpb)
    assert d_rpb.sum((1, 2)).abs().max() < 1e-10 and d_rpb.abs().max() > 1e-3
