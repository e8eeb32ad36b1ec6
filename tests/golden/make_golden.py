"""Writes the golden vectors in this directory.

The reference repository ships no golden vectors or known-answer files for this
operator (its test.py compares against the third-party `natten` package at run
time), so these fixtures come from this repository's own fp64 CPU oracle, which
tests/test_oracle_*.py pin against library attention, brute force and closed
forms.  They freeze the oracle: a later change to oracle/ that alters any output
fails tests/test_golden.py.

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import na1d_oracle as O1  # noqa: E402
from oracle import na2d_oracle as O  # noqa: E402

CASES_2D = {  # name: (shape, kernel_size, seed, scale)
    "c1_like_b1_n1_16x16_d32_k3": ((1, 1, 16, 16, 32), 3, 0, 32 ** -0.5),
    "ragged_b1_n1_9x11_d8_k5": ((1, 1, 9, 11, 8), 5, 1, 1.0),
    "window_is_image_7x7_d4_k7": ((1, 2, 7, 7, 4), 7, 2, 1.0),
}
CASES_1D = {"gradcheck_shape_b2_n3_t8_d2_k7": ((2, 3, 8, 2), 7, 3)}


def inputs(shape, seed):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(shape, generator=g, dtype=torch.float32) for _ in range(4)]


def f32(o, lse, dq, dk, dv):
    """Outputs are stored rounded to float32 to keep the files small."""
    return {n: t.to(torch.float32).numpy() for n, t in
            (("o", o), ("lse", lse), ("dq", dq), ("dk", dk), ("dv", dv))}


def main():
    for name, (shape, ks, seed, scale) in CASES_2D.items():
        q, k, v, d_o = inputs(shape, seed)
        o, lse, dq, dk, dv = O.natten2d_explicit(q, k, v, d_o, ks, scale)
        np.savez(os.path.join(HERE, name + ".npz"), q=q.numpy(), k=k.numpy(), v=v.numpy(),
                 d_o=d_o.numpy(), kernel_size=ks, scale=scale, **f32(o, lse, dq, dk, dv))
    for name, (shape, ks, seed) in CASES_1D.items():
        q, k, v, d_o = inputs(shape, seed)
        o, lse, dq, dk, dv = O1.natten1d_explicit(q, k, v, d_o, ks)
        np.savez(os.path.join(HERE, name + ".npz"), q=q.numpy(), k=k.numpy(), v=v.numpy(),
                 d_o=d_o.numpy(), kernel_size=ks, scale=1.0, **f32(o, lse, dq, dk, dv))


if __name__ == "__main__":
    main()
