"""Fused 2D neighborhood attention for AMD MI355X (gfx950).

Drop-in for the entry points of the reference package (e_natten/__init__.py:1):
``from e_natten_amd import natten1d, natten2d``.
"""
from .ops import Natten1d, Natten2d, kernel_path, natten1d, natten2d

__all__ = ["Natten1d", "Natten2d", "natten1d", "natten2d", "kernel_path"]
