"""CPU oracle for 2D neighborhood attention (torch, runs without a GPU).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py, never by the product package.

The operator (reference: e_natten/pytorch.py:158-290, e_natten/triton.py:224-423):
for every query pixel (x, y) of a [B, heads, H, W, d] tensor the keys are the
k x k pixels of the window whose start on each axis is
``clamp(i - k//2, 0, L - k)``; S = q . k_j (no softmax scale in the reference;
``scale`` here defaults to 1.0), P = softmax(S), O = sum_j P_j v_j.

Four independent statements are kept here so they can be checked against each
other and against what the mathematics fixes:

  * ``natten2d_gather``      vectorised gather + autograd   (main oracle)
  * ``natten2d_explicit``    closed-form O/LSE/dQ/dK/dV, no autograd
  * ``natten2d_dense_mask``  reduction to plain masked attention (library SDPA)
  * ``natten2d_brute``       pure-Python loops, tiny inputs only
  * ``Natten2dLoops``        tile-by-tile loop restatement of the reference's
                             algorithm (its per-query softmax Jacobian and its
                             inverse-neighbourhood gather for dK/dV)

Pinning status (see tests/test_oracle_*.py):
  win_start / inv_range      brute force over all (i, L, k)
  forward O, LSE             dense-mask SDPA, brute force, k=1, k=H=W, shifts
  dQ, dK, dV                 fp64 autograd of two independent forwards,
                             torch.autograd.gradcheck, sum invariants
  Natten2dLoops              equals the gather oracle
  axis_window_mask /         (rectangular and causal windows, not in the reference) centred
  natten2d_window_dense_mask axis = win_start; causal axis with k = L = lower triangle; 1D
                             causal with k = T = torch's is_causal attention; brute-force rows
Every function here is pinned by one of those checks.  Two accidental behaviours
of e_natten/pytorch.py are deliberately NOT restated (they contradict its own
backward, the Triton kernels and the NATTEN definition): its tile offset rule
(:25-31) shifts the window of a few rows when k//2 is not a multiple of 3, and
its dQ loop (:230-231) only visits the first tile.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch


# --------------------------------------------------------------------------
# index rules
# --------------------------------------------------------------------------
def win_start(i: int, L: int, k: int) -> int:
    """First key index of the window of query ``i`` on an axis of length ``L``.

    Closed form of e_natten/pytorch.py:7-11 (and e_natten/triton.py:7-12):
    centred on ``i`` and shifted just enough to stay inside ``[0, L)``.
    """
    return min(max(i - k // 2, 0), L - k)


def inv_range(i: int, L: int, k: int) -> Tuple[int, int]:
    """Half-open range of queries whose window contains key ``i``.

    Follows e_natten/pytorch.py:13-23 (get_backward_window_start/_end).  The
    range has k entries in the interior and up to k + k//2 next to an edge,
    because the clamped windows of the first/last k//2 queries all contain the
    first/last k keys.
    """
    lo = 0 if i < k else i - k // 2
    hi = L if i >= L - k else i + k // 2 + 1
    return lo, hi


def window_starts(L: int, k: int) -> torch.Tensor:
    """win_start for every query index of an axis, as an int64 tensor."""
    i = torch.arange(L)
    return (i - k // 2).clamp(0, L - k)


def neighbour_index(H: int, W: int, k: int) -> torch.Tensor:
    """[H*W, k*k] flat key indices (row-major over the image) per query."""
    sx = window_starts(H, k)  # [H]
    sy = window_starts(W, k)  # [W]
    a = torch.arange(k)
    rows = sx[:, None] + a[None, :]  # [H, k]
    cols = sy[:, None] + a[None, :]  # [W, k]
    idx = rows[:, None, :, None] * W + cols[None, :, None, :]  # [H, W, k, k]
    return idx.reshape(H * W, k * k)


def _check(q, k, v, ks):
    if q.dim() != 5 or q.shape != k.shape or q.shape != v.shape:
        raise ValueError("q, k, v must share a [B, heads, H, W, d] shape")
    if ks < 1 or ks % 2 == 0:
        raise ValueError("kernel_size must be odd and >= 1")
    if q.shape[2] < ks or q.shape[3] < ks:
        raise ValueError("image sides must be >= kernel_size")


# --------------------------------------------------------------------------
# main oracle: vectorised gather, autograd-able
# --------------------------------------------------------------------------
def natten2d_gather(q, k, v, kernel_size: int, scale: float = 1.0,
                    return_lse: bool = False):
    """O (and optionally LSE) through an explicit gather of every window.

    Per-query math as e_natten/pytorch.py:196-202: S = q K_w^T, softmax, P V_w.
    Differentiable; use fp64 inputs for a tight oracle.
    """
    _check(q, k, v, kernel_size)
    B, N, H, W, D = q.shape
    idx = neighbour_index(H, W, kernel_size).to(q.device)  # [HW, kk]
    qf = q.reshape(B, N, H * W, D)
    kf = k.reshape(B, N, H * W, D)
    vf = v.reshape(B, N, H * W, D)
    kg = kf[:, :, idx]  # [B, N, HW, kk, D]
    vg = vf[:, :, idx]
    s = torch.einsum("bnqd,bnqjd->bnqj", qf, kg) * scale
    lse = torch.logsumexp(s, dim=-1)
    p = torch.exp(s - lse[..., None])
    o = torch.einsum("bnqj,bnqjd->bnqd", p, vg).reshape(B, N, H, W, D)
    if return_lse:
        return o, lse.reshape(B, N, H, W)
    return o


def natten2d_gather_grads(q, k, v, d_o, kernel_size: int, scale: float = 1.0,
                          compute_dtype=torch.float64, slab_chunk: int = 1):
    """(O, LSE, dQ, dK, dV) by autograd through ``natten2d_gather``.

    Inputs are cast to ``compute_dtype`` first, so bf16/fp32 test inputs are
    evaluated exactly on their rounded values.  Work is chunked over the
    flattened (batch, head) axis to bound memory.
    """
    _check(q, k, v, kernel_size)
    B, N, H, W, D = q.shape
    outs = [torch.empty(B * N, H, W, D, dtype=compute_dtype) for _ in range(4)]
    lse = torch.empty(B * N, H, W, dtype=compute_dtype)
    qs, ks_, vs, gs = (t.reshape(B * N, 1, H, W, D) for t in (q, k, v, d_o))
    for s0 in range(0, B * N, slab_chunk):
        sl = slice(s0, s0 + slab_chunk)
        qq, kk, vv = (t[sl].to(compute_dtype).detach().requires_grad_(True)
                      for t in (qs, ks_, vs))
        o, l = natten2d_gather(qq, kk, vv, kernel_size, scale, return_lse=True)
        o.backward(gs[sl].to(compute_dtype))
        outs[0][sl] = o.detach()[:, 0]
        outs[1][sl] = qq.grad[:, 0]
        outs[2][sl] = kk.grad[:, 0]
        outs[3][sl] = vv.grad[:, 0]
        lse[sl] = l.detach()[:, 0]
    shp = (B, N, H, W, D)
    return (outs[0].reshape(shp), lse.reshape(B, N, H, W),
            outs[1].reshape(shp), outs[2].reshape(shp), outs[3].reshape(shp))


# --------------------------------------------------------------------------
# closed form without autograd
# --------------------------------------------------------------------------
def natten2d_explicit(q, k, v, d_o, kernel_size: int, scale: float = 1.0,
                      compute_dtype=torch.float64):
    """(O, LSE, dQ, dK, dV) from the written-out backward.

    dP_j = dO . v_j ; delta = sum_j P_j dP_j ; dS_j = P_j (dP_j - delta)
    (the product of the softmax Jacobian diag(P) - P P^T with dP that
    e_natten/pytorch.py:252-257 and e_natten/triton.py:395-396 form);
    dQ = scale * sum_j dS_j k_j ; dK[j] += scale * dS_j q ; dV[j] += P_j dO
    (e_natten/pytorch.py:285,288, e_natten/triton.py:412-423), accumulated
    here with index_add_ over the same neighbour table.
    """
    _check(q, k, v, kernel_size)
    B, N, H, W, D = q.shape
    kk = kernel_size * kernel_size
    idx = neighbour_index(H, W, kernel_size)
    flat = lambda t: t.reshape(B * N, H * W, D).to(compute_dtype)
    qf, kf, vf, gf = flat(q), flat(k), flat(v), flat(d_o)
    o = torch.empty_like(qf)
    dq = torch.empty_like(qf)
    dk = torch.zeros_like(qf)
    dv = torch.zeros_like(qf)
    lse = torch.empty(B * N, H * W, dtype=compute_dtype)
    for s in range(B * N):
        kg = kf[s][idx]  # [HW, kk, D]
        vg = vf[s][idx]
        sc = torch.einsum("qd,qjd->qj", qf[s], kg) * scale
        l = torch.logsumexp(sc, dim=-1)
        p = torch.exp(sc - l[:, None])
        o[s] = torch.einsum("qj,qjd->qd", p, vg)
        dp = torch.einsum("qd,qjd->qj", gf[s], vg)
        delta = (p * dp).sum(-1, keepdim=True)
        ds = p * (dp - delta)
        dq[s] = torch.einsum("qj,qjd->qd", ds, kg) * scale
        dk[s].index_add_(0, idx.reshape(-1),
                         (ds[:, :, None] * qf[s][:, None, :] * scale).reshape(-1, D))
        dv[s].index_add_(0, idx.reshape(-1),
                         (p[:, :, None] * gf[s][:, None, :]).reshape(-1, D))
        lse[s] = l
    shp = (B, N, H, W, D)
    return (o.reshape(shp), lse.reshape(B, N, H, W), dq.reshape(shp),
            dk.reshape(shp), dv.reshape(shp))


# --------------------------------------------------------------------------
# reduction to library attention with a dense mask (small images only)
# --------------------------------------------------------------------------
def neighbour_mask(H: int, W: int, k: int) -> torch.Tensor:
    """[H*W, H*W] boolean: True where the key is inside the query's window."""
    sx = window_starts(H, k)
    sy = window_starts(W, k)
    r = torch.arange(H)
    c = torch.arange(W)
    row_ok = (r[None, :] >= sx[:, None]) & (r[None, :] < sx[:, None] + k)  # [Hq, Hk]
    col_ok = (c[None, :] >= sy[:, None]) & (c[None, :] < sy[:, None] + k)  # [Wq, Wk]
    m = row_ok[:, None, :, None] & col_ok[None, :, None, :]  # [Hq, Wq, Hk, Wk]
    return m.reshape(H * W, H * W)


def natten2d_dense_mask(q, k, v, kernel_size: int, scale: float = 1.0):
    """O through torch's scaled_dot_product_attention on flattened tokens."""
    _check(q, k, v, kernel_size)
    B, N, H, W, D = q.shape
    m = neighbour_mask(H, W, kernel_size).to(q.device)
    f = lambda t: t.reshape(B, N, H * W, D)
    o = torch.nn.functional.scaled_dot_product_attention(
        f(q), f(k), f(v), attn_mask=m, scale=scale)
    return o.reshape(B, N, H, W, D)


# --------------------------------------------------------------------------
# brute force (tiny inputs)
# --------------------------------------------------------------------------
def natten2d_brute(q, k, v, kernel_size: int, scale: float = 1.0):
    """O and LSE with Python loops and math.exp only; for B*N*H*W*k*k*d small."""
    _check(q, k, v, kernel_size)
    B, N, H, W, D = q.shape
    ql, kl, vl = q.tolist(), k.tolist(), v.tolist()
    o = torch.zeros(B, N, H, W, D, dtype=torch.float64)
    lse = torch.zeros(B, N, H, W, dtype=torch.float64)
    for b in range(B):
        for n in range(N):
            for x in range(H):
                x0 = win_start(x, H, kernel_size)
                for y in range(W):
                    y0 = win_start(y, W, kernel_size)
                    scores, vals = [], []
                    for a in range(x0, x0 + kernel_size):
                        for c in range(y0, y0 + kernel_size):
                            scores.append(scale * sum(
                                ql[b][n][x][y][e] * kl[b][n][a][c][e] for e in range(D)))
                            vals.append(vl[b][n][a][c])
                    m = max(scores)
                    w = [math.exp(s - m) for s in scores]
                    z = sum(w)
                    for e in range(D):
                        o[b, n, x, y, e] = sum(wi * vi[e] for wi, vi in zip(w, vals)) / z
                    lse[b, n, x, y] = m + math.log(z)
    return o, lse


# --------------------------------------------------------------------------
# loop restatement of the reference's algorithm
# --------------------------------------------------------------------------
REF_TILE = 3  # e_natten/pytorch.py:5


def _softmax_jvp(p: torch.Tensor, dp: torch.Tensor) -> torch.Tensor:
    """(diag(p) - p p^T) dp over the last axis: what the reference builds as a
    dense Jacobian (e_natten/pytorch.py:33-43) and multiplies by dP (:256)."""
    jac = torch.diag_embed(p) - p[..., :, None] * p[..., None, :]
    return torch.einsum("...ij,...j->...i", jac, dp)


class Natten2dLoops(torch.autograd.Function):
    """Tile-by-tile restatement of e_natten/pytorch.py:158-290.

    forward  : image cut into 3x3 query tiles; each tile reads one
               (3+k-1)^2 key/value slab; every query softmaxes over its own
               k x k slice of the slab (:178-202).
    backward : dQ per query from the softmax Jacobian (:244-258); dK/dV per
               key by walking the inverse neighbourhood and recomputing each
               contributing query's softmax (:261-288).

    The in-slab offset is ``win_start(query) - slab_start`` (the file's own rule,
    :25-31, is wrong for k = 3 and 9) and dQ is produced for every tile (the loop
    the reference has commented out at :228-229).
    ``rows=(r0, r1)`` restricts the outer row loops to that band so a bounded
    sample of the work can be timed; outputs outside the band stay zero.
    """

    @staticmethod
    def forward(ctx, q, k, v, kernel_size=7, rows=None):
        _check(q, k, v, kernel_size)
        B, N, H, W, D = q.shape
        ks = kernel_size
        slab = REF_TILE + ks - 1
        r0, r1 = rows if rows is not None else (0, H)
        out = torch.zeros_like(q)
        for tx in range(r0 - r0 % REF_TILE, r1, REF_TILE):
            sx0 = win_start(tx, H, ks)
            for ty in range(0, W, REF_TILE):
                sy0 = win_start(ty, W, ks)
                k_slab = k[:, :, sx0:sx0 + slab, sy0:sy0 + slab]
                v_slab = v[:, :, sx0:sx0 + slab, sy0:sy0 + slab]
                for ix in range(min(REF_TILE, H - tx)):
                    if not (r0 <= tx + ix < r1):
                        continue
                    for iy in range(min(REF_TILE, W - ty)):
                        ox = win_start(tx + ix, H, ks) - sx0
                        oy = win_start(ty + iy, W, ks) - sy0
                        kw = k_slab[:, :, ox:ox + ks, oy:oy + ks].reshape(B, N, ks * ks, D)
                        vw = v_slab[:, :, ox:ox + ks, oy:oy + ks].reshape(B, N, ks * ks, D)
                        qv = q[:, :, tx + ix, ty + iy]  # [B, N, D]
                        p = torch.softmax(torch.einsum("bnd,bnjd->bnj", qv, kw), dim=-1)
                        out[:, :, tx + ix, ty + iy] = torch.einsum("bnj,bnjd->bnd", p, vw)
        ctx.save_for_backward(q, k, v)
        ctx.ks, ctx.rows = ks, (r0, r1)
        return out

    @staticmethod
    def backward(ctx, d_o):
        q, k, v = ctx.saved_tensors
        ks, (r0, r1) = ctx.ks, ctx.rows
        B, N, H, W, D = q.shape
        slab = REF_TILE + ks - 1
        dq, dk, dv = torch.zeros_like(q), torch.zeros_like(k), torch.zeros_like(v)

        def query_terms(x, y, x0, y0):
            kw = k[:, :, x0:x0 + ks, y0:y0 + ks].reshape(B, N, ks * ks, D)
            vw = v[:, :, x0:x0 + ks, y0:y0 + ks].reshape(B, N, ks * ks, D)
            p = torch.softmax(torch.einsum("bnd,bnjd->bnj", q[:, :, x, y], kw), dim=-1)
            dp = torch.einsum("bnd,bnjd->bnj", d_o[:, :, x, y], vw)
            return p, _softmax_jvp(p, dp), kw

        # dQ, tile by tile
        for tx in range(r0 - r0 % REF_TILE, r1, REF_TILE):
            for ty in range(0, W, REF_TILE):
                for ix in range(min(REF_TILE, H - tx)):
                    if not (r0 <= tx + ix < r1):
                        continue
                    for iy in range(min(REF_TILE, W - ty)):
                        x0 = win_start(tx + ix, H, ks)
                        y0 = win_start(ty + iy, W, ks)
                        _, ds, kw = query_terms(tx + ix, ty + iy, x0, y0)
                        dq[:, :, tx + ix, ty + iy] = torch.einsum("bnj,bnjd->bnd", ds, kw)

        # dK, dV: every key gathers from the queries that attend to it
        for x in range(r0, r1):
            qx0, qx1 = inv_range(x, H, ks)
            for y in range(W):
                qy0, qy1 = inv_range(y, W, ks)
                for xi in range(qx0, qx1):
                    wx = win_start(xi, H, ks)
                    for yi in range(qy0, qy1):
                        wy = win_start(yi, W, ks)
                        p, ds, _ = query_terms(xi, yi, wx, wy)
                        slot = (x - wx) * ks + (y - wy)
                        dk[:, :, x, y] += q[:, :, xi, yi] * ds[:, :, slot, None]
                        dv[:, :, x, y] += d_o[:, :, xi, yi] * p[:, :, slot, None]
        return dq, dk, dv, None, None


def natten2d_loops(q, k, v, kernel_size=7, rows=None):
    return Natten2dLoops.apply(q, k, v, kernel_size, rows)


# --------------------------------------------------------------------------
# unfused comparator of the reference's own test (test.py:16-21)
# --------------------------------------------------------------------------
def natten2d_qk(q, k, kernel_size: int) -> torch.Tensor:
    """[B, N, H, W, k*k] raw logits q . k_j: what NATTEN's natten2dqk returns
    with dilation 1 and no bias, restated from its published definition."""
    B, N, H, W, D = q.shape
    idx = neighbour_index(H, W, kernel_size)
    kg = k.reshape(B, N, H * W, D)[:, :, idx]
    return torch.einsum("bnqd,bnqjd->bnqj", q.reshape(B, N, H * W, D), kg).reshape(
        B, N, H, W, kernel_size * kernel_size)


def natten2d_av(p, v, kernel_size: int) -> torch.Tensor:
    """[B, N, H, W, d] = sum_j p_j v_j over each query's window (natten2dav)."""
    B, N, H, W, D = v.shape
    idx = neighbour_index(H, W, kernel_size)
    vg = v.reshape(B, N, H * W, D)[:, :, idx]
    return torch.einsum("bnqj,bnqjd->bnqd", p.reshape(B, N, H * W, -1), vg).reshape(
        B, N, H, W, D)


# --------------------------------------------------------------------------
# error measures used by the parity tests
# --------------------------------------------------------------------------
# --------------------------------------------------------------------------
# dilated neighborhoods (beyond the reference, which always passes dilation 1 to its
# comparator: test.py:17,21)
# --------------------------------------------------------------------------
def dilated_win_start(i: int, L: int, k: int, dilation: int) -> int:
    """First key of query i's window on an axis of length L: its k keys are
    start, start + dilation, ..., start + (k - 1) * dilation.

    Restates the window rule of the third-party NATTEN package (SHI-Labs; the
    comparator the reference's test.py imports, absent here and un-pinned there) as
    published in its CPU/CUDA sources, `get_window_start(index, length, kernel_size,
    neighborhood_size, dilation)`: centred where it fits, otherwise the first /
    last k positions of the query's residue class modulo the dilation.
    """
    ns = k // 2
    if dilation <= 1:
        return max(i - ns, 0) + (L - i - ns - 1 if i + ns >= L else 0)
    ni = i - ns * dilation
    if ni < 0:
        return i % dilation
    if i + ns * dilation >= L:
        imodd = i % dilation
        a = (L // dilation) * dilation
        b = L - a
        if imodd < b:
            return L - b + imodd - 2 * ns * dilation
        return a + imodd - k * dilation
    return ni


def dilated_neighbour_mask(H: int, W: int, k: int, dilation: int) -> torch.Tensor:
    """[H*W, H*W] bool: query (row) attends key (column), from dilated_win_start."""
    def axis(L):
        m = torch.zeros(L, L, dtype=torch.bool)
        for i in range(L):
            s0 = dilated_win_start(i, L, k, dilation)
            for j in range(k):
                m[i, s0 + j * dilation] = True
        return m
    mr, mc = axis(H), axis(W)
    return (mr[:, None, :, None] & mc[None, :, None, :]).reshape(H * W, H * W)


def natten2d_dilated_dense_mask(q, k, v, kernel_size: int, dilation: int, scale: float = 1.0):
    """O of dilated 2D neighborhood attention through torch's
    scaled_dot_product_attention with the dense mask above; differentiable."""
    B, N, H, W, D = q.shape
    if H < kernel_size * dilation or W < kernel_size * dilation:
        raise ValueError("image sides must be >= kernel_size * dilation")
    m = dilated_neighbour_mask(H, W, kernel_size, dilation).to(q.device)
    o = torch.nn.functional.scaled_dot_product_attention(
        q.reshape(B, N, H * W, D), k.reshape(B, N, H * W, D), v.reshape(B, N, H * W, D),
        attn_mask=m, scale=scale)
    return o.reshape(B, N, H, W, D)


def axis_window_mask(L: int, k: int, causal: bool = False) -> torch.Tensor:
    """[L, L] bool, query (row) attends key (column), for one axis.  Not in the reference
    (one odd kernel_size, no causal mode); NATTEN's published rules, get_window_start /
    get_window_end for dilation 1: a centred axis has start = clamp(i - k//2, 0, L - k) and
    k keys (the reference's rule, e_natten/pytorch.py:7-11); a causal axis has
    start = max(i - k + 1, 0) and end = i + 1, the last k positions up to the query's own."""
    if k < 1 or k > L or (not causal and k % 2 == 0):
        raise ValueError("bad window %d on an axis of %d positions" % (k, L))
    m = torch.zeros(L, L, dtype=torch.bool)
    for i in range(L):
        s0 = max(i - k + 1, 0) if causal else win_start(i, L, k)
        s1 = i + 1 if causal else s0 + k
        m[i, s0:s1] = True
    return m


def natten2d_window_dense_mask(q, k, v, kernel, causal=(False, False), scale: float = 1.0,
                               rpb=None):
    """O of 2D neighborhood attention with a kernel[0] x kernel[1] window and per-axis
    causal flags, through torch's scaled_dot_product_attention with the dense mask built
    from axis_window_mask; differentiable.  A [B, N, 1, T, D] input with kernel (1, k) is
    the 1D operator.  rpb [N, 2*kh-1, 2*kw-1], if given, is NATTEN's relative position
    bias: the logit of (query, key) gets rpb[n, key_row - query_row + kh - 1,
    key_col - query_col + kw - 1] added after the scaling."""
    B, N, H, W, D = q.shape
    mr = axis_window_mask(H, kernel[0], causal[0])
    mc = axis_window_mask(W, kernel[1], causal[1])
    m = (mr[:, None, :, None] & mc[None, :, None, :]).reshape(H * W, H * W).to(q.device)
    if rpb is not None:
        ar = (torch.arange(H)[None, :] - torch.arange(H)[:, None] + kernel[0] - 1)  # [query, key]
        ac = (torch.arange(W)[None, :] - torch.arange(W)[:, None] + kernel[1] - 1)
        ar = ar.clamp(0, 2 * kernel[0] - 2)[:, None, :, None].expand(H, W, H, W)
        ac = ac.clamp(0, 2 * kernel[1] - 2)[None, :, None, :].expand(H, W, H, W)
        bias = rpb[:, ar.reshape(H * W, H * W), ac.reshape(H * W, H * W)]  # [N, HW, HW]
        m = torch.where(m[None], bias, torch.full_like(bias, float("-inf")))[None]
    o = torch.nn.functional.scaled_dot_product_attention(
        q.reshape(B, N, H * W, D), k.reshape(B, N, H * W, D), v.reshape(B, N, H * W, D),
        attn_mask=m, scale=scale)
    return o.reshape(B, N, H, W, D)


def max_abs_err(x: torch.Tensor, ref: torch.Tensor) -> float:
    return (x.double() - ref.double()).abs().max().item()


def rel_err(x: torch.Tensor, ref: torch.Tensor) -> float:
    """max |x - ref| / max |ref| : the bf16 criterion (<= 2e-2)."""
    r = ref.double()
    return ((x.double() - r).abs().max() / r.abs().max().clamp_min(1e-30)).item()
