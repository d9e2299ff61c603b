"""Shim for `cuda_w4a16.kernels` (reference: src/cuda_w4a16/kernels.py)."""
from glowq_amd.kernels import load_w4a16_extension  # noqa: F401

__all__ = ["load_w4a16_extension"]
