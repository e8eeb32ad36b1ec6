"""CPU oracle for fused 2D neighborhood attention.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package may import this
directory: it exists so that tests, the smoke check and the benchmark's CPU
baseline can compare the HIP kernels with an independent CPU statement of the
algorithm in the reference's ``e_natten/pytorch.py``.
"""
