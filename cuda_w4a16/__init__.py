"""Import-path shim: the reference's callers do `from cuda_w4a16.linear import convert_to_cuda_w4a16`
(src/step3_eval_dataset.py:1047) and `from cuda_w4a16 import ...` (src/cuda_w4a16/__init__.py:1-8).
Everything lives in `glowq_amd`."""
from glowq_amd.kernels import load_w4a16_extension
from glowq_amd.linear import CudaW4A16Linear, convert_to_cuda_w4a16

__all__ = ["load_w4a16_extension", "CudaW4A16Linear", "convert_to_cuda_w4a16"]
