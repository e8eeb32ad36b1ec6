"""Fused 2D neighborhood attention for AMD MI355X (gfx950).

Drop-in for the entry points of the reference package (e_natten/__init__.py:1):
``from e_natten_amd import natten2d``.
"""
from .ops import Natten2d, natten2d, kernel_path

__all__ = ["Natten2d", "natten2d", "kernel_path"]
