"""MI355X-native GlowQ Step-3 hot path: W4A16 linear + group-shared low-rank correction.

Public surface (same names as the reference, src/cuda_w4a16/__init__.py:1-8 and
src/step3_eval_dataset.py:409-605):
"""
from .kernels import load_w4a16_extension
from .linear import CudaW4A16Linear, convert_to_cuda_w4a16, refresh_env_knobs
from .correction import (
    AddSVDCorrection,
    MiniGroupCache,
    patch_svd_correction_wrappers,
    patch_svd_correction_wrappers_cumulative,
)

__all__ = [
    "load_w4a16_extension",
    "CudaW4A16Linear",
    "convert_to_cuda_w4a16",
    "refresh_env_knobs",
    "AddSVDCorrection",
    "MiniGroupCache",
    "patch_svd_correction_wrappers",
    "patch_svd_correction_wrappers_cumulative",
]
