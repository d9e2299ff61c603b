"""W4A16 quantised linear for MI355X: module, quantiser and model conversion.

Drop-in for the reference's `cuda_w4a16.linear` (src/cuda_w4a16/linear.py):

  `CudaW4A16Linear`        same constructor, buffers (`qweight_i32`, `qzeros_i32`, `scales_f16`, non-persistent
                           `gid`), attributes, `from_float`, `forward` contract and environment knobs
                           (linear.py:91-276)
  `convert_to_cuda_w4a16`  replaces every nn.Linear outside `lm_head` (linear.py:279-293)
  `_quantize_per_group_w4`, `_pack_int4_to_int32`, `_unpack_int4_i32`   (linear.py:42-88)

Differences on purpose: forward runs only on the GPU through the HIP library (no torch matmul route, no
dequantised-weight cache: the GEMM route dequantises inside the kernel, so `W4A16_DEQUANT_CACHE`,
`W4A16_DEQUANT_CHUNK` and `W4A16_GEMM_CUDA` are accepted and have nothing left to control), and the
row count at which the GEMV route hands over to the MFMA GEMM defaults to this hardware's measured
cross-over instead of 128 (still overridable through `W4A16_GEMV_M_MAX`).
"""
from __future__ import annotations

import math
import os
from typing import Optional

import torch
import torch.nn as nn

from .kernels import load_w4a16_extension

_TRUE = {"1", "true", "yes", "y", "on"}

# Rows up to which the decode kernels (wave-dot GEMV, skinny MFMA) are used; above it the tiled
# MFMA GEMM takes over.  The reference's constant is 128 (linear.py:120).
DEFAULT_GEMV_M_MAX = 64


def _env_flag(*names: str, default: bool = False) -> bool:
    for n in names:
        v = os.environ.get(n)
        if v is not None:
            return v.lower() in _TRUE
    return default


def _env_number(*names: str, default: int) -> int:
    for n in names:
        v = os.environ.get(n)
        if v:
            return int(v)
    return int(default)


def _get_kernel_out_dtype() -> torch.dtype:
    """`W4A16_KERNEL_OUT_DTYPE` (legacy `MIXED_KERNEL_OUT_DTYPE`) as the environment has it now: fp16 or fp32, default
    fp32 (linear.py:29-39)."""
    v = os.environ.get("W4A16_KERNEL_OUT_DTYPE", os.environ.get("MIXED_KERNEL_OUT_DTYPE", "fp32")).lower()
    return torch.float16 if v in ("fp16", "float16", "half") else torch.float32


_KNOB_ENV = ("W4A16_KERNEL_OUT_DTYPE", "MIXED_KERNEL_OUT_DTYPE", "W4A16_FORCE_GEMM", "CUDA_MIXED_FORCE_GEMM",
             "W4A16_FORCE_GEMV", "CUDA_MIXED_FORCE_GEMV", "W4A16_USE_GEMV", "W4A16_SPLIT_K_ITERS")


# os.environ keeps its strings in a plain dict of encoded keys: reading that dict is a fifth of the cost of
# os.environ.get (no encoding, no KeyError on a miss), and a forward reads all the switches.  Falls back to the mapping
# itself where the interpreter has no such dict.
_ENV_DATA = getattr(os.environ, "_data", None)
_KNOB_KEYS = tuple(os.environ.encodekey(k) for k in _KNOB_ENV) if (_ENV_DATA is not None and hasattr(os.environ, "encodekey")) else None


def _raw_env():
    if _KNOB_KEYS is not None:
        get = _ENV_DATA.get
        return tuple([get(k) for k in _KNOB_KEYS])
    return tuple(map(os.environ.get, _KNOB_ENV))


class _Knobs:
    """The `W4A16_*` switches a forward depends on.  The reference reads them from the environment on every forward
    (linear.py:172-177); here they are parsed once and a forward only compares the raw strings with the ones it parsed
    last (`sync`), so a switch set with `os.environ[...] = ...` after import is honoured by the next forward, as in the
    reference, without parsing anything on the calls in between."""

    __slots__ = ("out_dtype", "force_gemm", "force_gemv", "use_gemv", "split_k_iters", "_raw")

    def __init__(self):
        self.read()

    def read(self) -> None:
        self._raw = _raw_env()
        self.out_dtype = _get_kernel_out_dtype()
        self.force_gemm = _env_flag("W4A16_FORCE_GEMM", "CUDA_MIXED_FORCE_GEMM")
        self.force_gemv = _env_flag("W4A16_FORCE_GEMV", "CUDA_MIXED_FORCE_GEMV")
        self.use_gemv = _env_flag("W4A16_USE_GEMV")
        self.split_k_iters = _env_number("W4A16_SPLIT_K_ITERS", default=1)

    def sync(self) -> None:
        if _raw_env() != self._raw:
            self.read()


KNOBS = _Knobs()


def refresh_env_knobs() -> None:
    """Re-reads the `W4A16_*` environment switches (output dtype, forced routes, split-K iterations) for every module;
    every forward does the same when one of their strings has changed.  The row threshold `W4A16_GEMV_M_MAX` is read when
    a module is constructed, as in the reference (linear.py:120)."""
    KNOBS.read()


# ----------------------------------------------------------------------------------------------
# int4 packing: element i of the trailing axis goes to bits [4i, 4i+4) of one int32
# ----------------------------------------------------------------------------------------------
def _pack_int4_to_int32(u4: torch.Tensor) -> torch.Tensor:
    assert u4.dtype == torch.uint8
    if u4.shape[-1] != 8:
        raise ValueError("the trailing axis must hold the 8 codes of one int32")
    wide = u4.to(torch.int64)
    word = torch.zeros(u4.shape[:-1], dtype=torch.int64, device=u4.device)
    for i in range(8):
        word |= wide[..., i] << (4 * i)
    # fold bit 31 into the sign, as a wrapping int32 sum does
    word = torch.where(word >= 2**31, word - 2**32, word)
    return word.to(torch.int32)


def _unpack_int4_i32(packed_i32: torch.Tensor, total_vals: int) -> torch.Tensor:
    packed = packed_i32.contiguous().to(torch.int32)
    rows = packed.size(0)
    nib = torch.stack([(packed >> (4 * i)) & 0xF for i in range(8)], dim=-1)
    return nib.to(torch.uint8).reshape(rows, -1)[:, :total_vals].contiguous()


def _quantize_per_group_w4(weight: torch.Tensor, group_size: int):
    """Asymmetric min/max uint4 quantisation per (row, group) in the dtype of `weight` (fp16 at
    conversion time), following linear.py:57-88 op for op so the integer codes are identical:
    scale = ((max - min) / 15).clamp(min=1e-8); zero = round(-min / scale).clamp(0, 15);
    code = round(w / scale + zero).clamp(0, 15).  Zero-point words are padded with code 8.
    """
    if group_size % 8 != 0:
        raise ValueError("group_size must be multiple of 8 for int32 int4 packing")
    n_out, n_in = weight.shape
    tail = n_in % group_size
    if tail:
        weight = torch.nn.functional.pad(weight, (0, group_size - tail))
        n_in = weight.shape[1]
    n_groups = n_in // group_size
    grouped = weight.reshape(n_out, n_groups, group_size)
    lo, hi = grouped.amin(dim=-1), grouped.amax(dim=-1)
    scales = ((hi - lo) / 15.0).clamp(min=1e-8)
    zeros = (-lo / scales).round().clamp(0, 15)
    codes = (grouped / scales[..., None] + zeros[..., None]).round().clamp(0, 15).to(torch.uint8)
    qweight = _pack_int4_to_int32(codes.reshape(n_out, n_groups, group_size // 8, 8)).reshape(n_out, n_in // 8)

    words = (n_groups + 7) // 8
    zcodes = torch.full((n_out, words * 8), 8, dtype=torch.uint8, device=weight.device)
    zcodes[:, :n_groups] = zeros.to(torch.uint8)
    qzeros = _pack_int4_to_int32(zcodes.reshape(n_out, words, 8))
    return qweight.contiguous(), qzeros.contiguous(), scales.to(torch.float16).contiguous(), n_in


# ----------------------------------------------------------------------------------------------
# module
# ----------------------------------------------------------------------------------------------
class CudaW4A16Linear(nn.Module):
    def __init__(self, in_features: int, out_features: int, group_size: int = 128, bias: bool = False):
        super().__init__()
        self.in_features = int(in_features)
        self.out_features = int(out_features)
        self.group_size = int(group_size)
        if self.group_size <= 0 or self.group_size % 8:
            raise ValueError("group_size must be > 0 and a multiple of 8 for GlowQ int32 int4 packing")

        self.groups = math.ceil(self.in_features / self.group_size)
        self.groups_packed = (self.groups + 7) // 8
        self.register_buffer("qweight_i32", torch.empty(self.out_features, (self.in_features + 7) // 8, dtype=torch.int32))
        self.register_buffer("qzeros_i32", torch.empty(self.out_features, max(1, self.groups_packed), dtype=torch.int32))
        self.register_buffer("scales_f16", torch.empty(self.out_features, self.groups, dtype=torch.float16))
        self.register_buffer("gid", torch.arange(self.in_features, dtype=torch.long) // self.group_size, persistent=False)
        self.bias = nn.Parameter(torch.empty(self.out_features, dtype=torch.float16)) if bias else None

        self._ext = None
        self._gemv_threshold = _env_number("W4A16_GEMV_M_MAX", "CUDA_MIXED_GEMV_M_MAX", default=DEFAULT_GEMV_M_MAX)
        self._prepared = None  # descriptors of the bare module for single-call forwards (kernels.PreparedGroup)

    def extra_repr(self) -> str:
        return (f"in_features={self.in_features}, out_features={self.out_features}, "
                f"group_size={self.group_size}, bias={self.bias is not None}")

    def _get_ext(self):
        if self._ext is None:
            self._ext = load_w4a16_extension()
        return self._ext

    # -- helpers shared with the correction wrapper ------------------------------------------------
    def _as_rows(self, x: torch.Tensor) -> torch.Tensor:
        """[*, K] -> contiguous fp16 [M, K]; raises on a trailing-dim mismatch (linear.py:165-166)."""
        if x.shape[-1] != self.in_features:
            raise ValueError(f"Input dim mismatch: got {x.shape[-1]}, expected {self.in_features}")
        x2d = x.reshape(-1, self.in_features)
        if x2d.dtype != torch.float16:
            x2d = x2d.to(torch.float16)
        return x2d.contiguous()

    def _member(self, L: Optional[torch.Tensor] = None) -> dict:
        return {"qweight": self.qweight_i32, "scales": self.scales_f16, "qzeros": self.qzeros_i32, "L": L,
                "bias": None}

    def _apply(self, fn, *args, **kwargs):
        # .to() / .cuda() / .half() move the buffers: descriptors built from their addresses go with them
        from .kernels import bump_generation

        self._prepared = None
        bump_generation()
        return super()._apply(fn, *args, **kwargs)

    def _bare_group(self):
        """The module alone as a prepared group (validated once, side stream packed once); rebuilt when a buffer has
        been replaced since."""
        # the bias rides in the kernel's epilogue, y = fp16(acc + bias), where the output stays fp16; with fp32 output the
        # reference adds it in fp32 after the cast (linear.py:183-186) and so does `_finish`
        fold_bias = self.bias is not None and KNOBS.out_dtype == torch.float16
        key = (self.qweight_i32.data_ptr(), self.scales_f16.data_ptr(), self.qzeros_i32.data_ptr(),
               self.bias.data_ptr() if fold_bias else 0)
        if self._prepared is None or self._prepared[0] != key:
            from .kernels import PreparedGroup

            member = self._member()
            member["bias"] = self.bias.data if fold_bias else None
            self._prepared = (key, PreparedGroup(self._get_ext(), [member], self.in_features, self.group_size, 0.0))
        return self._prepared[1]

    def _prefer_gemv(self, m: int) -> bool:
        KNOBS.sync()
        if KNOBS.force_gemm:
            return False
        return KNOBS.force_gemv or KNOBS.use_gemv or m <= self._gemv_threshold

    def _require_gpu(self, x: torch.Tensor) -> None:
        if not x.is_cuda or not self.qweight_i32.is_cuda:
            raise RuntimeError(
                "CudaW4A16Linear.forward runs only on the GPU through the glowq HIP library; "
                "move the module and its input to the device (there is no CPU route)")

    def _finish(self, out: torch.Tensor, lead_shape, bias_applied: bool = False) -> torch.Tensor:
        if out.dtype != KNOBS.out_dtype:
            out = out.to(KNOBS.out_dtype)
        if self.bias is not None and not bias_applied:
            out = out + self.bias.to(out.dtype)
        return out.reshape(*lead_shape, self.out_features)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        lead = x.shape[:-1]
        x2d = self._as_rows(x)
        self._require_gpu(x2d)
        KNOBS.sync()
        if KNOBS.force_gemm or (not self._prefer_gemv(x2d.size(0))):
            out = self._get_ext().w4a16_gemm_forward_cuda(x2d, self.qweight_i32, self.scales_f16, self.qzeros_i32,
                                                          self.group_size, KNOBS.split_k_iters)
            return self._finish(out, lead)
        # the decode kernels through descriptors validated once (the bias rides in the kernel's epilogue)
        return self._finish(self._bare_group().run(x2d)[0], lead, bias_applied=KNOBS.out_dtype == torch.float16)

    def dequantize(self) -> torch.Tensor:
        """fp16 [out_features, in_features] weight, fp16((code - zero) * scale); the device twin of the
        reference's `_dequant_chunk` over all rows (linear.py:248-253)."""
        self._require_gpu(self.qweight_i32)
        return self._get_ext().dequant(self.qweight_i32, self.scales_f16, self.qzeros_i32, self.in_features, self.group_size)

    def _dequant_chunk(self, start: int, end: int) -> torch.Tensor:
        """fp16 rows [start, end) of the dequantised weight, [end - start, in_features] (linear.py:248-253)."""
        self._require_gpu(self.qweight_i32)
        start, end = max(0, int(start)), min(self.out_features, int(end))
        if end <= start:
            return torch.empty((0, self.in_features), dtype=torch.float16, device=self.qweight_i32.device)
        return self._get_ext().dequant(self.qweight_i32[start:end], self.scales_f16[start:end], self.qzeros_i32[start:end],
                                       self.in_features, self.group_size)

    @classmethod
    def from_float(cls, linear_layer: nn.Linear, group_size: int):
        src = linear_layer.weight
        mod = cls(linear_layer.in_features, linear_layer.out_features, group_size,
                  bias=linear_layer.bias is not None).to(src.device)
        qweight, qzeros, scales, _ = _quantize_per_group_w4(src.data.to(torch.float16), group_size)
        for name, val in (("qweight_i32", qweight), ("qzeros_i32", qzeros), ("scales_f16", scales)):
            buf = getattr(mod, name)
            buf.resize_(val.shape)
            buf.copy_(val)
        if linear_layer.bias is not None:
            mod.bias.data.copy_(linear_layer.bias.data.to(torch.float16))
        return mod


def convert_to_cuda_w4a16(model: nn.Module, group_size: int = 128) -> nn.Module:
    """Swaps every nn.Linear whose qualified name has no "lm_head" for a `CudaW4A16Linear`
    (linear.py:279-293).  A module whose conversion raises is left as it was, as in the reference."""
    targets = [(name, mod) for name, mod in model.named_modules()
               if isinstance(mod, nn.Linear) and "lm_head" not in name]
    for name, mod in targets:
        *path, leaf = name.split(".")
        owner = model
        for p in path:
            owner = getattr(owner, p)
        try:
            setattr(owner, leaf, CudaW4A16Linear.from_float(mod, group_size))
        except Exception:
            continue
    if torch.cuda.is_available():
        torch.cuda.empty_cache()
    return model


__all__ = ["CudaW4A16Linear", "convert_to_cuda_w4a16", "refresh_env_knobs", "DEFAULT_GEMV_M_MAX"]
