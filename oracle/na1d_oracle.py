"""CPU oracle for 1D neighborhood attention (torch).  TEST INFRASTRUCTURE ONLY.

The 1D operator of the reference (e_natten/pytorch.py:46-156,
e_natten/triton.py:65-222, 425-485): tensors [B, heads, T, d]; query t attends
the k keys starting at ``clamp(t - k//2, 0, T - k)``; S = q . k_j (no scale),
P = softmax(S), O = sum_j P_j v_j.

Pinning (tests/test_oracle_1d.py): dense-mask reduction to library attention,
brute force, torch.autograd.gradcheck with the recipe of the reference's
gradcheck.py:6-15, the C oracle run as a 1 x k window on an image of height 1,
and the loop restatement against the gather statement.
"""
from __future__ import annotations

import math

import torch

from .na2d_oracle import REF_TILE, _softmax_jvp, inv_range, win_start, window_starts


def neighbour_index_1d(T: int, k: int) -> torch.Tensor:
    """[T, k] key indices per query."""
    return window_starts(T, k)[:, None] + torch.arange(k)[None, :]


def _check(q, k, v, ks):
    if q.dim() != 4 or q.shape != k.shape or q.shape != v.shape:
        raise ValueError("q, k, v must share a [B, heads, T, d] shape")
    if ks < 1 or ks % 2 == 0:
        raise ValueError("kernel_size must be odd and >= 1")
    if q.shape[2] < ks:
        raise ValueError("sequence must be at least kernel_size long")


def natten1d_gather(q, k, v, kernel_size: int, scale: float = 1.0, return_lse: bool = False):
    """O (and LSE) through an explicit gather; differentiable.
    Per-query math as e_natten/pytorch.py:76-81."""
    _check(q, k, v, kernel_size)
    idx = neighbour_index_1d(q.shape[2], kernel_size)
    kg, vg = k[:, :, idx], v[:, :, idx]  # [B, N, T, k, D]
    s = torch.einsum("bntd,bntjd->bntj", q, kg) * scale
    lse = torch.logsumexp(s, dim=-1)
    o = torch.einsum("bntj,bntjd->bntd", torch.exp(s - lse[..., None]), vg)
    return (o, lse) if return_lse else o


def natten1d_explicit(q, k, v, d_o, kernel_size: int, scale: float = 1.0,
                      compute_dtype=torch.float64):
    """(O, LSE, dQ, dK, dV) from the written-out backward
    (e_natten/pytorch.py:124-152 with dS = P (dP - sum P dP))."""
    _check(q, k, v, kernel_size)
    B, N, T, D = q.shape
    idx = neighbour_index_1d(T, kernel_size)
    q, k, v, d_o = (t.to(compute_dtype) for t in (q, k, v, d_o))
    kg, vg = k[:, :, idx], v[:, :, idx]
    s = torch.einsum("bntd,bntjd->bntj", q, kg) * scale
    lse = torch.logsumexp(s, dim=-1)
    p = torch.exp(s - lse[..., None])
    o = torch.einsum("bntj,bntjd->bntd", p, vg)
    dp = torch.einsum("bntd,bntjd->bntj", d_o, vg)
    ds = p * (dp - (p * dp).sum(-1, keepdim=True))
    dq = torch.einsum("bntj,bntjd->bntd", ds, kg) * scale
    dk = torch.zeros_like(k)
    dv = torch.zeros_like(v)
    flat = idx.reshape(-1)
    dk.index_add_(2, flat, (ds[..., None] * q[:, :, :, None, :] * scale).reshape(B, N, -1, D))
    dv.index_add_(2, flat, (p[..., None] * d_o[:, :, :, None, :]).reshape(B, N, -1, D))
    return o, lse, dq, dk, dv


def natten1d_dense_mask(q, k, v, kernel_size: int, scale: float = 1.0):
    """O through torch's scaled_dot_product_attention with a banded mask."""
    _check(q, k, v, kernel_size)
    T = q.shape[2]
    s0 = window_starts(T, kernel_size)
    j = torch.arange(T)
    m = (j[None, :] >= s0[:, None]) & (j[None, :] < s0[:, None] + kernel_size)
    return torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=m, scale=scale)


def natten1d_brute(q, k, v, kernel_size: int):
    """O with Python loops and math.exp only (tiny inputs)."""
    _check(q, k, v, kernel_size)
    B, N, T, D = q.shape
    ql, kl, vl = q.tolist(), k.tolist(), v.tolist()
    o = torch.zeros(B, N, T, D, dtype=torch.float64)
    for b in range(B):
        for n in range(N):
            for t in range(T):
                t0 = win_start(t, T, kernel_size)
                sc = [sum(ql[b][n][t][e] * kl[b][n][j][e] for e in range(D))
                      for j in range(t0, t0 + kernel_size)]
                m = max(sc)
                w = [math.exp(x - m) for x in sc]
                z = sum(w)
                for e in range(D):
                    o[b, n, t, e] = sum(wi * vl[b][n][t0 + i][e] for i, wi in enumerate(w)) / z
    return o


class Natten1dLoops(torch.autograd.Function):
    """Tile-by-tile restatement of e_natten/pytorch.py:46-156: queries in tiles of
    3 read one (3+k-1)-key slab (:66-81); dQ per query from the softmax Jacobian
    (:105-130); dK/dV per key over its inverse neighbourhood (:136-152).  The
    in-slab offset is win_start(query) - slab_start (the intended rule)."""

    @staticmethod
    def forward(ctx, q, k, v, kernel_size=7):
        _check(q, k, v, kernel_size)
        B, N, T, D = q.shape
        ks = kernel_size
        out = torch.zeros_like(q)
        for t0 in range(0, T, REF_TILE):
            s0 = win_start(t0, T, ks)
            k_slab = k[:, :, s0:s0 + REF_TILE + ks - 1]
            v_slab = v[:, :, s0:s0 + REF_TILE + ks - 1]
            for j in range(min(REF_TILE, T - t0)):
                off = win_start(t0 + j, T, ks) - s0
                p = torch.softmax(torch.einsum("bnd,bnjd->bnj", q[:, :, t0 + j],
                                               k_slab[:, :, off:off + ks]), dim=-1)
                out[:, :, t0 + j] = torch.einsum("bnj,bnjd->bnd", p, v_slab[:, :, off:off + ks])
        ctx.save_for_backward(q, k, v)
        ctx.ks = ks
        return out

    @staticmethod
    def backward(ctx, d_o):
        q, k, v = ctx.saved_tensors
        ks = ctx.ks
        B, N, T, D = q.shape
        dq, dk, dv = torch.zeros_like(q), torch.zeros_like(k), torch.zeros_like(v)

        def terms(t):
            w0 = win_start(t, T, ks)
            p = torch.softmax(torch.einsum("bnd,bnjd->bnj", q[:, :, t], k[:, :, w0:w0 + ks]), dim=-1)
            dp = torch.einsum("bnd,bnjd->bnj", d_o[:, :, t], v[:, :, w0:w0 + ks])
            return w0, p, _softmax_jvp(p, dp)

        for t in range(T):
            w0, _, ds = terms(t)
            dq[:, :, t] = torch.einsum("bnj,bnjd->bnd", ds, k[:, :, w0:w0 + ks])
        for i in range(T):
            lo, hi = inv_range(i, T, ks)
            for t in range(lo, hi):
                w0, p, ds = terms(t)
                dk[:, :, i] += q[:, :, t] * ds[:, :, i - w0, None]
                dv[:, :, i] += d_o[:, :, t] * p[:, :, i - w0, None]
        return dq, dk, dv, None


def natten1d_loops(q, k, v, kernel_size=7):
    return Natten1dLoops.apply(q, k, v, kernel_size)
