"""Shim for `cuda_w4a16.linear` (reference: src/cuda_w4a16/linear.py)."""
from glowq_amd.linear import (  # noqa: F401
    CudaW4A16Linear,
    _get_kernel_out_dtype,
    _pack_int4_to_int32,
    _quantize_per_group_w4,
    _unpack_int4_i32,
    convert_to_cuda_w4a16,
)
