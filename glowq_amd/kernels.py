"""Loader and tensor-level front end of libglowq_w4a16.so (hand-written HIP for gfx950).

Mirrors the reference's extension loader (src/cuda_w4a16/kernels.py:16-59) and the three functions
its pybind module exports (src/cuda_w4a16/csrc/pybind.cpp:19-34):

    ext = load_w4a16_extension()
    y = ext.w4a16_gemv_forward_cuda(x, qweight, scales, qzeros, group_size)
    y = ext.w4a16_gemm_forward_cuda(x, qweight, scales, qzeros, group_size, split_k_iters)
    y = ext.gemv_w4a16_asym(...)                      # alias of the GEMV entry

plus the group-level entry points this implementation adds (`shared_proj`, `group_forward`,
`dequant`, `unpack_int4`).  The library itself is a plain C ABI (include/glowq_w4a16.h); torch is used
only for device memory and the current HIP stream.  There is no CPU or eager fallback: a missing
library raises, as the reference's loader does (kernels.py:24-32).
"""
from __future__ import annotations

import ctypes
import os
from typing import List, Optional, Sequence

import torch

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "libglowq_w4a16.so")
MAX_MEMBERS = 4

_ext = None

_P = ctypes.c_void_p
_I = ctypes.c_int


class _Member(ctypes.Structure):
    _fields_ = [
        ("qweight", _P), ("scales", _P), ("qzeros", _P), ("L", _P), ("bias", _P), ("y", _P),
        ("N", ctypes.c_int32), ("ldw_i32", ctypes.c_int32), ("lds", ctypes.c_int32),
        ("ldz_i32", ctypes.c_int32), ("ldy", ctypes.c_int32), ("side_rank", ctypes.c_int32),
        ("side", _P), ("tiled", _P), ("tiled_L", _P), ("tiled_rank", ctypes.c_int32), ("reserved", ctypes.c_int32),
    ]


class _Chain(ctypes.Structure):
    _fields_ = [
        ("prologue", ctypes.c_int), ("epilogue", ctypes.c_int), ("norm_weight", _P), ("eps", ctypes.c_float),
        ("acc_in", _P), ("resid", _P), ("next_norm_weight", _P), ("next_Rt", _P), ("acc_out", _P), ("act", _P),
    ]


# prologues and epilogues of the chained single-token group launch, and the size of one accumulator
CHAIN_PRO_PLAIN, CHAIN_PRO_ACC, CHAIN_PRO_NORM_ACC = 0, 1, 2
CHAIN_EPI_NONE, CHAIN_EPI_RESIDUAL, CHAIN_EPI_SWIGLU = 0, 1, 2
CHAIN_ACC_BYTES = (16 * 256 + 8) * 8

_SIGNATURES = {
    "glowq_version": (ctypes.c_int, []),
    "glowq_last_error": (ctypes.c_char_p, []),
    "glowq_w4a16_gemv_forward": (_I, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P]),
    "glowq_w4a16_gemm_forward": (_I, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _P]),
    "glowq_w4a16_dequant": (_I, [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P]),
    "glowq_unpack_int4": (_I, [_P, _P, _I, _I, _I, _P]),
    "glowq_shared_proj": (_I, [_P, _P, _P, _I, _I, _I, _P]),
    "glowq_shared_proj_ws": (_I, [_P, _P, _P, _I, _I, _I, _P, ctypes.c_size_t, _P]),
    "glowq_proj_workspace_bytes": (ctypes.c_size_t, [_I, _I, _I]),
    "glowq_w4a16_group_forward_ws": (_I, [_P, _P, ctypes.POINTER(_Member), _I, _I, _I, _I, _I, ctypes.c_float, _P,
                                          ctypes.c_size_t, _P]),
    "glowq_w4a16_group_forward_fused_ws": (_I, [_P, _P, _P, ctypes.POINTER(_Member), _I, _I, _I, _I, _I, ctypes.c_float,
                                                _P, ctypes.c_size_t, _P]),
    "glowq_w4a16_group_forward_fused_static": (_I, [_P, _P, _P, ctypes.POINTER(_Member), _I, _I, _I, _I, _I, ctypes.c_float, _P]),
    "glowq_static_scratch_bytes": (ctypes.c_size_t, []),
    "glowq_static_scratch_prepare": (_I, []),
    "glowq_side_bytes": (ctypes.c_size_t, [_I, _I, _I, _I]),
    "glowq_pack_side": (_I, [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P]),
    "glowq_w4a16_group_forward": (_I, [_P, _P, ctypes.POINTER(_Member), _I, _I, _I, _I, _I, ctypes.c_float, _P]),
    "glowq_w4a16_group_forward_fused": (_I, [_P, _P, _P, ctypes.POINTER(_Member), _I, _I, _I, _I, _I, ctypes.c_float, _P]),
    "glowq_w4a16_group_forward_chained": (_I, [_P, _P, ctypes.POINTER(_Member), _I, _I, _I, _I, ctypes.c_float,
                                               ctypes.POINTER(_Chain), _P]),
    "glowq_w4a16_route": (_I, [_I, _I, _I, _I, _I]),
    "glowq_w4a16_route_tiled": (_I, [_I, _I, _I, _I, _I]),
    "glowq_last_launch": (_I, [ctypes.c_char_p, ctypes.c_size_t, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int),
                                ctypes.POINTER(ctypes.c_int)]),
    "glowq_probe_stream_read": (_I, [_P, ctypes.c_size_t, _P, _I, _I, _P]),
    "glowq_probe_empty_launch": (_I, [_I, _I, _P]),
    "glowq_tiled_bytes": (ctypes.c_size_t, [_I, _I, _I]),
    "glowq_pack_tiled": (_I, [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P]),
    "glowq_tiled_left_bytes": (ctypes.c_size_t, [_I, _I]),
    "glowq_pack_tiled_left": (_I, [_P, _P, _I, _I, _P]),
    "glowq_set_tuning": (_I, [ctypes.c_char_p, _I]),
    "glowq_add_rmsnorm": (_I, [_P, _P, _P, _P, _I, _I, ctypes.c_float, _P]),
    "glowq_silu_mul": (_I, [_P, _P, _P, ctypes.c_long, _P]),
    "glowq_add_rmsnorm_proj": (_I, [_P, _P, _P, _P, _P, _P, _P, _I, _I, ctypes.c_float, _P]),
    "glowq_silu_mul_proj": (_I, [_P, _P, _P, _P, _P, _I, _I, _P]),
    "glowq_rope_attend": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, ctypes.c_float, _P]),
    "glowq_rope_attend_split": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, ctypes.c_float, _P]),
    "glowq_attend_combine_proj": (_I, [_P, _P, _P, _P, _I, _I, _I, _I, _P]),
    "glowq_argmax_advance": (_I, [_P, _I, _P, _P, _P, _P]),
}


# Calls with this many token rows and more bring the tiled copy of the weights along when they build descriptors per call.
TILED_MIN_ROWS = 2


def tiled_enabled() -> bool:
    """GLOWQ_TILED=0 keeps every route on the canonical buffers (no second copy of the weights in device memory)."""
    return os.environ.get("GLOWQ_TILED", "1").lower() not in {"0", "false", "no", "off"}


# The raw handle of torch's current stream of a device: the accessor behind `torch.cuda.current_stream(dev).cuda_stream`,
# without building the Stream object (a forward makes this call once).
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None) or (lambda idx: torch.cuda.current_stream(idx).cuda_stream)


def _check(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


class W4A16Extension:
    """Tensor-level wrappers over the C ABI.  Every call launches on torch's current stream."""

    def __init__(self, lib: ctypes.CDLL):
        self.lib = lib
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        self.version = lib.glowq_version()
        self._workspaces = {}

    # ------------------------------------------------------------------ helpers
    def _raise(self, rc: int, what: str):
        msg = self.lib.glowq_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{what}: {msg} (code {rc})")

    @staticmethod
    def _stream(dev: torch.device) -> int:
        idx = dev.index
        return _raw_stream(idx if idx is not None else torch.cuda.current_device())

    WORKSPACE_BYTES = 64 << 20

    HANDOVER_BYTES = 8192

    def _workspace(self, dev: torch.device, rows: int):
        """(pointer, bytes) of the workspace of the current stream of `dev`: one per stream, because calls that share
        one must not overlap.  Calls with two and more token rows get the large one (many-row projection, split-K of the
        GEMM and of the skinny kernels, hand-over words of the launches that compute r themselves); single-token calls
        a small one, through which a group launch that computes r itself hands it from the waves that produce it to the
        others.  A stream that meets
        its first such call while it is being captured into a graph goes without (the buffer would come from the
        graph's own memory pool)."""
        small = rows <= 1
        key = (dev.index if dev.index is not None else torch.cuda.current_device(), self._stream(dev), small)
        ws = self._workspaces.get(key)
        if ws is None:
            if torch.cuda.is_current_stream_capturing():
                return None, 0
            ws = torch.zeros(self.HANDOVER_BYTES if small else self.WORKSPACE_BYTES, dtype=torch.uint8, device=dev)
            self._workspaces[key] = ws
        return ws.data_ptr(), ws.numel()

    @staticmethod
    def _check_quant(x, qweight, scales, qzeros, group_size):
        _check(x.is_cuda, "inputs must be CUDA")
        _check(qweight.is_cuda, "qweight must be CUDA")
        _check(scales.is_cuda, "scales must be CUDA")
        _check(qzeros.is_cuda, "qzeros must be CUDA")
        _check(x.dtype == torch.float16, "inputs must be fp16")
        _check(qweight.dtype == torch.int32, "qweight must be int32 (8x int4 packed)")
        _check(scales.dtype == torch.float16, "scales must be fp16")
        _check(qzeros.dtype == torch.int32, "qzeros must be int32 (8x int4 packed)")
        _check(x.dim() == 2, "inputs must be [M, IC]")
        _check(qweight.dim() == 2, "qweight must be [OC, packed_i32]")
        _check(scales.dim() == 2, "scales must be [OC, groups]")
        _check(qzeros.dim() == 2, "qzeros must be [OC, groups_packed]")
        _check(group_size > 0, "group_size must be > 0")
        _check(group_size % 8 == 0, "group_size must be a multiple of 8")
        _check(scales.size(0) == qweight.size(0), "scales OC mismatch")
        _check(qzeros.size(0) == qweight.size(0), "qzeros OC mismatch")

    # ------------------------------------------------------------------ reference-named entry points
    def w4a16_gemv_forward_cuda(self, x, qweight, scales, qzeros, group_size: int) -> torch.Tensor:
        self._check_quant(x, qweight, scales, qzeros, group_size)
        x, qweight, scales, qzeros = x.contiguous(), qweight.contiguous(), scales.contiguous(), qzeros.contiguous()
        M, K = x.shape
        N = qweight.size(0)
        out = torch.empty((M, N), dtype=torch.float16, device=x.device)
        if M == 0 or N == 0:
            return out
        with torch.cuda.device(x.device):
            rc = self.lib.glowq_w4a16_gemv_forward(
                x.data_ptr(), qweight.data_ptr(), scales.data_ptr(), qzeros.data_ptr(), out.data_ptr(),
                M, K, N, int(group_size), qweight.size(1), scales.size(1), qzeros.size(1), self._stream(x.device))
        if rc:
            self._raise(rc, "w4a16_gemv_forward")
        return out

    gemv_w4a16_asym = w4a16_gemv_forward_cuda

    def w4a16_gemm_forward_cuda(self, x, qweight, scales, qzeros, group_size: int, split_k_iters: int = 1) -> torch.Tensor:
        self._check_quant(x, qweight, scales, qzeros, group_size)
        x, qweight, scales, qzeros = x.contiguous(), qweight.contiguous(), scales.contiguous(), qzeros.contiguous()
        M, K = x.shape
        N = qweight.size(0)
        out = torch.empty((M, N), dtype=torch.float16, device=x.device)
        if M == 0 or N == 0:
            return out
        with torch.cuda.device(x.device):
            rc = self.lib.glowq_w4a16_gemm_forward(
                x.data_ptr(), qweight.data_ptr(), scales.data_ptr(), qzeros.data_ptr(), out.data_ptr(),
                M, K, N, int(group_size), int(split_k_iters), qweight.size(1), scales.size(1), qzeros.size(1),
                self._stream(x.device))
        if rc:
            self._raise(rc, "w4a16_gemm_forward")
        return out

    # ------------------------------------------------------------------ additional entry points
    def dequant(self, qweight, scales, qzeros, in_features: int, group_size: int) -> torch.Tensor:
        _check(qweight.is_cuda and scales.is_cuda and qzeros.is_cuda, "dequant: tensors must be CUDA")
        _check(qweight.dtype == torch.int32 and qzeros.dtype == torch.int32 and scales.dtype == torch.float16,
               "dequant: qweight/qzeros must be int32 and scales fp16")
        qweight, scales, qzeros = qweight.contiguous(), scales.contiguous(), qzeros.contiguous()
        N = qweight.size(0)
        out = torch.empty((N, in_features), dtype=torch.float16, device=qweight.device)
        with torch.cuda.device(qweight.device):
            rc = self.lib.glowq_w4a16_dequant(
                qweight.data_ptr(), scales.data_ptr(), qzeros.data_ptr(), out.data_ptr(), N, int(in_features),
                int(group_size), qweight.size(1), scales.size(1), qzeros.size(1), self._stream(qweight.device))
        if rc:
            self._raise(rc, "w4a16_dequant")
        return out

    def unpack_int4(self, packed, total_vals: int) -> torch.Tensor:
        _check(packed.is_cuda and packed.dtype == torch.int32 and packed.dim() == 2, "unpack: packed must be CUDA int32 [rows, W]")
        packed = packed.contiguous()
        rows = packed.size(0)
        out = torch.empty((rows, total_vals), dtype=torch.uint8, device=packed.device)
        with torch.cuda.device(packed.device):
            rc = self.lib.glowq_unpack_int4(packed.data_ptr(), out.data_ptr(), rows, int(total_vals), packed.size(1),
                                            self._stream(packed.device))
        if rc:
            self._raise(rc, "unpack_int4")
        return out

    def pack_side(self, scales, qzeros, L, in_features: int, group_size: int, rank: int) -> Optional[torch.Tensor]:
        """The member's side stream for single-token calls (scales, zero-points and the rows of L, which may be None, in
        the order the decode GEMV reads them; include/glowq_w4a16.h) as a uint8 tensor, or None where the layout does
        not cover the shape.  `rank` is the rank of the calls it will serve (0: calls without correction)."""
        _check(scales.is_cuda and qzeros.is_cuda and scales.dtype == torch.float16 and qzeros.dtype == torch.int32
               and scales.dim() == 2 and qzeros.dim() == 2 and scales.is_contiguous() and qzeros.is_contiguous()
               and scales.size(0) == qzeros.size(0), "pack_side: scales fp16 [OC, groups] and qzeros int32 [OC, groups_packed] on the GPU")
        N = scales.size(0)
        if L is not None:
            _check(L.is_cuda and L.dtype == torch.float16 and L.is_contiguous() and tuple(L.shape) == (N, rank),
                   "pack_side: L must be a contiguous CUDA fp16 [OC, rank] tensor")
        size = self.lib.glowq_side_bytes(N, int(in_features), int(group_size), int(rank))
        if size == 0:
            return None
        out = torch.empty(size, dtype=torch.uint8, device=scales.device)
        with torch.cuda.device(scales.device):
            rc = self.lib.glowq_pack_side(scales.data_ptr(), qzeros.data_ptr(), L.data_ptr() if L is not None else None,
                                          out.data_ptr(), N, int(in_features), int(group_size), int(rank), scales.size(1),
                                          qzeros.size(1), self._stream(scales.device))
        if rc:
            self._raise(rc, "pack_side")
        return out

    def pack_tiled(self, qweight, scales, qzeros, in_features: int, group_size: int) -> Optional[torch.Tensor]:
        """The tiled copy of a member's weights for the matrix-core routes (a uint8 tensor; layout in csrc/tiled.hpp), or
        None where the layout does not apply.  Built once per weight tensor and kept on it (`qweight._glowq_tiled`) until
        the tensor is written to in place; a module moved with `.to()` gets new tensors and with them a new copy."""
        if not tiled_enabled():
            return None
        N = qweight.size(0)
        nbytes = self.lib.glowq_tiled_bytes(N, int(in_features), int(group_size))
        if nbytes == 0 or not qweight.is_cuda:
            return None
        key = (qweight._version, scales.data_ptr(), scales._version, qzeros.data_ptr(), qzeros._version, int(in_features), int(group_size))
        hit = getattr(qweight, "_glowq_tiled", None)
        if hit is not None and hit[0] == key:
            return hit[1]
        if torch.cuda.is_current_stream_capturing():
            return None  # not under a graph capture: the copy would come from the graph's own memory pool
        _check(qweight.dtype == torch.int32 and scales.dtype == torch.float16 and qzeros.dtype == torch.int32 and
               qweight.is_contiguous() and scales.is_contiguous() and qzeros.is_contiguous(), "pack_tiled: contiguous canonical buffers")
        out = torch.empty(nbytes, dtype=torch.uint8, device=qweight.device)
        with torch.cuda.device(qweight.device):
            rc = self.lib.glowq_pack_tiled(qweight.data_ptr(), scales.data_ptr(), qzeros.data_ptr(), out.data_ptr(), N, int(in_features),
                                           int(group_size), qweight.size(1), scales.size(1), qzeros.size(1), self._stream(qweight.device))
        if rc:
            self._raise(rc, "pack_tiled")
        qweight._glowq_tiled = (key, out)
        return out

    def pack_tiled_left(self, L) -> Optional[torch.Tensor]:
        """The tiled copy of a left factor [N, rank] (fp16 B operand of the correction blocks), kept on the tensor."""
        if not tiled_enabled() or L is None or not L.is_cuda:
            return None
        N, rank = L.shape
        nbytes = self.lib.glowq_tiled_left_bytes(int(N), int(rank))
        if nbytes == 0:
            return None
        hit = getattr(L, "_glowq_tiled", None)
        if hit is not None and hit[0] == L._version:
            return hit[1]
        if torch.cuda.is_current_stream_capturing():
            return None
        _check(L.dtype == torch.float16 and L.is_contiguous(), "pack_tiled_left: contiguous fp16 [OC, rank]")
        out = torch.empty(nbytes, dtype=torch.uint8, device=L.device)
        with torch.cuda.device(L.device):
            rc = self.lib.glowq_pack_tiled_left(L.data_ptr(), out.data_ptr(), int(N), int(rank), self._stream(L.device))
        if rc:
            self._raise(rc, "pack_tiled_left")
        L._glowq_tiled = (L._version, out)
        return out

    def wants_tiled(self, M: int, K: int, N_total: int, group_size: int, ldw_i32: int) -> bool:
        """Whether a group of this shape would take the route that reads the tiled copies: they are built (and kept in device
        memory beside the canonical buffers) only for such groups."""
        if M < TILED_MIN_ROWS or not tiled_enabled():
            return False
        route = self.lib.glowq_w4a16_route_tiled(int(M), int(K), int(N_total), int(group_size), int(ldw_i32))
        # 8: the kernel that streams the copy at 5..64 rows (2..4 on the longest streams); 2: the MFMA GEMM, which takes its B operand from the copy where
        # the layout applies (its lane order is the matrix instruction's)
        return route == 8 or (route == 2 and self.lib.glowq_tiled_bytes(int(N_total), int(K), int(group_size)) > 0)

    def _set_tiled(self, e, qw, sc, qz, L, in_features: int, group_size: int):
        """Fills the tiled fields of descriptor `e`; returns what has to stay alive with it."""
        tw = self.pack_tiled(qw, sc, qz, in_features, group_size)
        if tw is None:
            return None
        tl = self.pack_tiled_left(L) if L is not None else None
        if L is not None and tl is None:
            return None
        e.tiled = tw.data_ptr()
        e.tiled_L = tl.data_ptr() if tl is not None else None
        e.tiled_rank = int(L.size(1)) if L is not None else 0
        return (tw, tl)

    def shared_proj(self, x, R, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """r = fp16(x @ R^T); x [M, K] fp16, R [rank, K] fp16."""
        _check(x.is_cuda and R.is_cuda, "shared_proj: tensors must be CUDA")
        _check(x.dtype == torch.float16 and R.dtype == torch.float16, "shared_proj: tensors must be fp16")
        _check(x.dim() == 2 and R.dim() == 2 and x.size(1) == R.size(1), "shared_proj: x [M, K] and R [rank, K] must agree on K")
        x, R = x.contiguous(), R.contiguous()
        M, K = x.shape
        rank = R.size(0)
        if out is None:
            out = torch.empty((M, rank), dtype=torch.float16, device=x.device)
        with torch.cuda.device(x.device):
            ws, ws_bytes = self._workspace(x.device, M)
            rc = self.lib.glowq_shared_proj_ws(x.data_ptr(), R.data_ptr(), out.data_ptr(), M, K, rank, ws, ws_bytes,
                                               self._stream(x.device))
        if rc:
            self._raise(rc, "shared_proj")
        return out

    def group_forward(self, x, r, members: Sequence[dict], group_size: int, alpha: float,
                      outs: Optional[List[torch.Tensor]] = None, R: Optional[torch.Tensor] = None) -> List[torch.Tensor]:
        """One launch for a group.  Each member is a dict with `qweight`, `scales`, `qzeros` and optional
        `L` ([N, rank] fp16 or None), `bias` ([N] fp16 or None) and `side` (a (side stream, rank) pair from
        `pack_side`).  Returns the [M, N_i] fp16 outputs.
        With `R` ([rank, K] fp16) the launch computes r = x R^T itself and writes it into `r` (an
        [M, rank] fp16 buffer) for the caller's cache; without it `r` is an input."""
        _check(1 <= len(members) <= MAX_MEMBERS, f"group_forward: 1..{MAX_MEMBERS} members")
        _check(x.is_cuda and x.dtype == torch.float16 and x.dim() == 2, "inputs must be CUDA fp16 [M, IC]")
        x = x.contiguous()
        M, K = x.shape
        arr = (_Member * len(members))()
        keep = []
        rank = 0
        if R is not None:
            _check(R.is_cuda and R.dtype == torch.float16 and R.dim() == 2 and R.size(1) == K and R.is_contiguous(),
                   "group_forward: R must be a contiguous CUDA fp16 [rank, K] tensor")
            _check(r is not None and tuple(r.shape) == (M, R.size(0)), "group_forward: r must be an [M, rank] output buffer when R is given")
        if r is not None:
            _check(r.is_cuda and r.dtype == torch.float16 and r.dim() == 2 and r.size(0) == M and r.is_contiguous(),
                   "group_forward: r must be a contiguous CUDA fp16 [M, rank] tensor")
            rank = r.size(1)
        want_tiled = self.wants_tiled(M, K, sum(int(m["qweight"].size(0)) for m in members), group_size,
                                      int(members[0]["qweight"].size(1)))
        result = []
        for i, m in enumerate(members):
            qw, sc, qz = m["qweight"], m["scales"], m["qzeros"]
            self._check_quant(x, qw, sc, qz, group_size)
            _check(qw.is_contiguous() and sc.is_contiguous() and qz.is_contiguous(), "group_forward: buffers must be contiguous")
            N = qw.size(0)
            L = m.get("L")
            bias = m.get("bias")
            if L is not None:
                _check(r is not None, "group_forward: a member has L but no r was given")
                _check(L.is_cuda and L.dtype == torch.float16 and L.is_contiguous() and tuple(L.shape) == (N, rank),
                       "group_forward: L must be a contiguous CUDA fp16 [OC, rank] tensor")
            if bias is not None:
                _check(bias.is_cuda and bias.dtype == torch.float16 and bias.is_contiguous() and bias.numel() == N,
                       "group_forward: bias must be a contiguous CUDA fp16 [OC] tensor")
            y = outs[i] if outs is not None else torch.empty((M, N), dtype=torch.float16, device=x.device)
            _check(y.is_cuda and y.dtype == torch.float16 and tuple(y.shape) == (M, N) and y.stride(1) == 1,
                   "group_forward: output must be CUDA fp16 [M, OC]")
            side = m.get("side")
            keep.append((qw, sc, qz, L, bias, y, side))
            e = arr[i]
            if side is not None:
                e.side, e.side_rank = side[0].data_ptr(), int(side[1])
            e.qweight, e.scales, e.qzeros = qw.data_ptr(), sc.data_ptr(), qz.data_ptr()
            e.L = L.data_ptr() if L is not None else None
            e.bias = bias.data_ptr() if bias is not None else None
            e.y = y.data_ptr()
            e.N, e.ldw_i32, e.lds, e.ldz_i32, e.ldy = N, qw.size(1), sc.size(1), qz.size(1), y.stride(0)
            if want_tiled:
                keep.append(self._set_tiled(e, qw, sc, qz, L, K, group_size))
            result.append(y)
        if M == 0:
            return result
        with torch.cuda.device(x.device):
            if R is not None:
                ws, ws_bytes = self._workspace(x.device, M)
                rc = self.lib.glowq_w4a16_group_forward_fused_ws(
                    x.data_ptr(), R.data_ptr(), r.data_ptr(), arr, len(members), M, K, int(group_size),
                    int(rank), float(alpha), ws, ws_bytes, self._stream(x.device))
            else:
                ws, ws_bytes = self._workspace(x.device, M)
                rc = self.lib.glowq_w4a16_group_forward_ws(
                    x.data_ptr(), r.data_ptr() if r is not None else None, arr, len(members), M, K, int(group_size),
                    int(rank), float(alpha), ws, ws_bytes, self._stream(x.device))
        if rc:
            self._raise(rc, "w4a16_group_forward")
        return result

    # ------------------------------------------------------------------ single-token decode step around the linears
    @staticmethod
    def _f16(t, what):
        _check(t.is_cuda and t.dtype == torch.float16 and t.is_contiguous(), f"{what} must be a contiguous CUDA fp16 tensor")

    def add_rmsnorm(self, x, delta, weight, h, eps: float) -> None:
        """x += delta (delta may be None), h = rmsnorm(x) * weight; x and h are [M, H] fp16, x is updated in place."""
        self._f16(x, "x"), self._f16(weight, "weight"), self._f16(h, "h")
        _check(x.dim() == 2 and h.shape == x.shape and weight.numel() == x.size(1), "add_rmsnorm: x, h [M, H] and weight [H]")
        if delta is not None:
            self._f16(delta, "delta")
            _check(delta.shape == x.shape, "add_rmsnorm: delta must have the shape of x")
        with torch.cuda.device(x.device):
            rc = self.lib.glowq_add_rmsnorm(x.data_ptr(), delta.data_ptr() if delta is not None else None, weight.data_ptr(),
                                            h.data_ptr(), x.size(0), x.size(1), float(eps), self._stream(x.device))
        if rc:
            self._raise(rc, "add_rmsnorm")

    def silu_mul(self, gate, up, out) -> None:
        for t, n in ((gate, "gate"), (up, "up"), (out, "out")):
            _check(t.is_cuda and t.dtype == torch.float16 and t.stride(-1) == 1, f"silu_mul: {n} must be CUDA fp16")
        _check(gate.numel() == up.numel() == out.numel(), "silu_mul: sizes differ")
        _check(gate.is_contiguous() and up.is_contiguous() and out.is_contiguous(), "silu_mul: tensors must be contiguous")
        with torch.cuda.device(out.device):
            rc = self.lib.glowq_silu_mul(gate.data_ptr(), up.data_ptr(), out.data_ptr(), gate.numel(), self._stream(out.device))
        if rc:
            self._raise(rc, "silu_mul")

    def add_rmsnorm_proj(self, x_in, delta, weight, x_out, h, R, r, eps: float) -> None:
        """One token: x_out = x_in + delta, h = rmsnorm(x_out) * weight, r = h R^T (R [rank, H], r [1, rank])."""
        for t, n in ((x_in, "x_in"), (weight, "weight"), (x_out, "x_out"), (h, "h"), (R, "R"), (r, "r")):
            self._f16(t, n)
        H = x_in.numel()
        _check(x_out.numel() == H and h.numel() == H and weight.numel() == H and R.dim() == 2 and R.size(1) == H
               and r.numel() == R.size(0), "add_rmsnorm_proj: shape mismatch")
        if delta is not None:
            self._f16(delta, "delta")
            _check(delta.numel() == H, "add_rmsnorm_proj: delta must have the size of x")
        with torch.cuda.device(x_in.device):
            rc = self.lib.glowq_add_rmsnorm_proj(x_in.data_ptr(), delta.data_ptr() if delta is not None else None, weight.data_ptr(),
                                                 x_out.data_ptr(), h.data_ptr(), R.data_ptr(), r.data_ptr(), H, R.size(0),
                                                 float(eps), self._stream(x_in.device))
        if rc:
            self._raise(rc, "add_rmsnorm_proj")

    def silu_mul_proj(self, gate, up, out, R, r) -> None:
        """One token: out = silu(gate) * up, r = out R^T."""
        for t, n in ((gate, "gate"), (up, "up"), (out, "out"), (R, "R"), (r, "r")):
            self._f16(t, n)
        n = gate.numel()
        _check(up.numel() == n and out.numel() == n and R.dim() == 2 and R.size(1) == n and r.numel() == R.size(0),
               "silu_mul_proj: shape mismatch")
        with torch.cuda.device(out.device):
            rc = self.lib.glowq_silu_mul_proj(gate.data_ptr(), up.data_ptr(), out.data_ptr(), R.data_ptr(), r.data_ptr(), n,
                                              R.size(0), self._stream(out.device))
        if rc:
            self._raise(rc, "silu_mul_proj")

    def rope_attend(self, q, k_new, v_new, cos_table, sin_table, pos, cache_k, cache_v, out, scale: float) -> None:
        """q [heads, d], k_new / v_new [kv_heads, d] of one token, tables [max_len, d] fp32, pos int64[1] on the device,
        caches [kv_heads, max_len, d]: rotary embedding, cache append at pos, attention over 0..pos into out [heads, d]."""
        for t, n in ((q, "q"), (k_new, "k_new"), (v_new, "v_new"), (cache_k, "cache_k"), (cache_v, "cache_v"), (out, "out")):
            self._f16(t, n)
        _check(cos_table.is_cuda and cos_table.dtype == torch.float32 and cos_table.is_contiguous()
               and sin_table.dtype == torch.float32 and sin_table.is_contiguous() and sin_table.shape == cos_table.shape,
               "rope_attend: tables must be contiguous CUDA fp32 [max_len, d]")
        _check(pos.is_cuda and pos.dtype == torch.int64 and pos.numel() == 1, "rope_attend: pos must be one int64 on the device")
        kv_heads, max_len, d = cache_k.shape
        heads = q.numel() // d
        _check(cache_v.shape == cache_k.shape and k_new.numel() == kv_heads * d and v_new.numel() == kv_heads * d
               and out.numel() == heads * d and tuple(cos_table.shape) == (max_len, d), "rope_attend: shape mismatch")
        with torch.cuda.device(q.device):
            rc = self.lib.glowq_rope_attend(q.data_ptr(), k_new.data_ptr(), v_new.data_ptr(), cos_table.data_ptr(),
                                            sin_table.data_ptr(), pos.data_ptr(), cache_k.data_ptr(), cache_v.data_ptr(),
                                            out.data_ptr(), heads, kv_heads, d, max_len, float(scale), self._stream(q.device))
        if rc:
            self._raise(rc, "rope_attend")

    def rope_attend_split(self, q, k_new, v_new, cos_table, sin_table, pos, cache_k, cache_v, partials, scale: float) -> None:
        """As rope_attend, with the context split over partials.size(1) workgroups per head; partials is a
        [heads, splits, d + 4] fp32 buffer that receives {max, sum, 2 unused, unnormalised acc} of every split."""
        for t, n in ((q, "q"), (k_new, "k_new"), (v_new, "v_new"), (cache_k, "cache_k"), (cache_v, "cache_v")):
            self._f16(t, n)
        kv_heads, max_len, d = cache_k.shape
        heads = q.numel() // d
        _check(partials.is_cuda and partials.dtype == torch.float32 and partials.is_contiguous() and partials.dim() == 3
               and partials.size(0) == heads and partials.size(2) == d + 4, "rope_attend_split: partials must be fp32 [heads, splits, d + 4]")
        _check(cos_table.dtype == torch.float32 and cos_table.is_contiguous() and sin_table.dtype == torch.float32
               and sin_table.is_contiguous() and tuple(cos_table.shape) == (max_len, d) and sin_table.shape == cos_table.shape,
               "rope_attend_split: tables must be contiguous CUDA fp32 [max_len, d]")
        _check(pos.is_cuda and pos.dtype == torch.int64 and pos.numel() == 1, "rope_attend_split: pos must be one int64 on the device")
        _check(cache_v.shape == cache_k.shape and k_new.numel() == kv_heads * d and v_new.numel() == kv_heads * d,
               "rope_attend_split: shape mismatch")
        with torch.cuda.device(q.device):
            rc = self.lib.glowq_rope_attend_split(q.data_ptr(), k_new.data_ptr(), v_new.data_ptr(), cos_table.data_ptr(),
                                                  sin_table.data_ptr(), pos.data_ptr(), cache_k.data_ptr(), cache_v.data_ptr(),
                                                  partials.data_ptr(), partials.size(1), heads, kv_heads, d, max_len, float(scale),
                                                  self._stream(q.device))
        if rc:
            self._raise(rc, "rope_attend_split")

    def attend_combine_proj(self, partials, out, R=None, r=None) -> None:
        """out [heads * d] fp16 from the split partials; with R [rank, heads * d] also r = out R^T ([rank] fp16)."""
        self._f16(out, "out")
        heads, splits, d2 = partials.shape
        d = d2 - 4
        _check(partials.is_cuda and partials.dtype == torch.float32 and partials.is_contiguous() and out.numel() == heads * d,
               "attend_combine_proj: partials fp32 [heads, splits, d + 4], out [heads * d]")
        _check((R is None) == (r is None), "attend_combine_proj: R and r go together")
        if R is not None:
            self._f16(R, "R"), self._f16(r, "r")
            _check(R.dim() == 2 and R.size(1) == heads * d and r.numel() == R.size(0), "attend_combine_proj: R [rank, heads * d], r [rank]")
        with torch.cuda.device(out.device):
            rc = self.lib.glowq_attend_combine_proj(partials.data_ptr(), out.data_ptr(), R.data_ptr() if R is not None else None,
                                                    r.data_ptr() if r is not None else None, heads, d, splits,
                                                    R.size(0) if R is not None else 0, self._stream(out.device))
        if rc:
            self._raise(rc, "attend_combine_proj")

    def argmax_advance(self, logits, next_token, token=None, pos=None) -> None:
        """next_token[0] = first argmax of logits; then token[0] = next_token[0] and pos[0] += 1 when given."""
        self._f16(logits, "logits")
        for t in (next_token, token, pos):
            _check(t is None or (t.is_cuda and t.dtype == torch.int64 and t.numel() == 1), "argmax_advance: int64[1] on the device")
        with torch.cuda.device(logits.device):
            rc = self.lib.glowq_argmax_advance(logits.data_ptr(), logits.numel(), next_token.data_ptr(),
                                               token.data_ptr() if token is not None else None,
                                               pos.data_ptr() if pos is not None else None, self._stream(logits.device))
        if rc:
            self._raise(rc, "argmax_advance")

    def last_launch(self) -> dict:
        """The kernel the calling thread's last group launch used (name with template arguments where the launcher records
        them, else the route's name), its grid and its workgroup size."""
        buf = ctypes.create_string_buffer(160)
        gx, gy, blk = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int(0)
        self.lib.glowq_last_launch(buf, 160, ctypes.byref(gx), ctypes.byref(gy), ctypes.byref(blk))
        return {"kernel": buf.value.decode(), "grid": [gx.value, gy.value], "block": blk.value}

    def route(self, M: int, K: int, N: int, group_size: int = 128, tiled: Optional[bool] = None) -> str:
        names = {0: "wave_dot_gemv", 1: "skinny_mfma", 2: "tiled_mfma_gemm", 3: "generic", 4: "quad_mfma_gemv", 5: "stream_gemv",
                 6: "quad_stream_gemv", 7: "skinny_codes_mfma", 8: "skinny_tiled_mfma"}
        fn = self.lib.glowq_w4a16_route_tiled if (tiled_enabled() if tiled is None else tiled) else self.lib.glowq_w4a16_route
        return names[fn(int(M), int(K), int(N), int(group_size), (int(K) + 7) // 8)]

    def set_tuning(self, key: str, value: int) -> int:
        """Sets a route limit of the process ("quad_max_m", "quad_min_m", "wave_dot_max_m", "skinny_max_m",
        "small_group_mb", "stream_max_m", "stream_shape_rule", "qstream_max_m", "qstream_shape_rule",
        "skinny_codes_max_m"); returns the old value."""
        old = self.lib.glowq_set_tuning(key.encode(), int(value))
        if old < 0:
            raise ValueError(self.lib.glowq_last_error().decode())
        return old


# Bumped whenever a module that may own member tensors is moved or cast (`nn.Module._apply`): descriptors built from
# tensor addresses before that are stale.  Holders of a PreparedGroup compare its `generation` with `generation()`.
_generation = 0


def generation() -> int:
    return _generation


def bump_generation() -> None:
    global _generation
    _generation += 1


class PreparedGroup:
    """A group of members validated once, with its descriptors and side streams built once: what a module (or a fused
    decode step) keeps so that a forward is one output allocation and one library call.  The member tensors are held
    alive; a caller whose buffers move (`.to()`, a reassigned factor) builds a new one."""

    def __init__(self, ext: W4A16Extension, members: Sequence[dict], in_features: int, group_size: int, alpha: float,
                 R: Optional[torch.Tensor] = None, side_streams: Optional[bool] = None):
        _check(1 <= len(members) <= MAX_MEMBERS, f"group: 1..{MAX_MEMBERS} members")
        self.ext, self.lib = ext, ext.lib
        if side_streams is None:
            # Off unless asked for: with every request of a wave already in flight up front, fetching scales, zero-points
            # and L rows as one packed stream measured no faster than the three canonical arrays (8B-shape layer at one
            # token: gate|up 12.9 us either way, q|k|v 5.04 -> 4.97, o_proj 4.27 -> 4.19, down_proj 8.55 -> 8.69) and
            # costs 7 % more memory.  GLOWQ_SIDE_STREAMS=1 switches it on for measurements.
            side_streams = os.environ.get("GLOWQ_SIDE_STREAMS", "0").lower() in {"1", "true", "yes", "y", "on"}
        self.generation = _generation
        self.K, self.group_size, self.alpha = int(in_features), int(group_size), float(alpha)
        self.R = R
        dev = members[0]["qweight"].device
        self.device = dev
        ranks = {m["L"].size(1) for m in members if m.get("L") is not None}
        _check(len(ranks) <= 1, "group: the members' left factors must share one rank")
        self.rank = ranks.pop() if ranks else (R.size(0) if R is not None else 0)
        if R is not None:
            _check(R.is_cuda and R.dtype == torch.float16 and R.dim() == 2 and R.is_contiguous()
                   and tuple(R.shape) == (self.rank, self.K), "group: R must be a contiguous CUDA fp16 [rank, K] tensor")
        corrected = self.alpha != 0.0 and any(m.get("L") is not None for m in members)
        self.arr = (_Member * len(members))()
        self.Ns, self.keep = [], []
        x_probe = torch.empty(0, self.K, dtype=torch.float16, device=dev)
        for e, m in zip(self.arr, members):
            qw, sc, qz, L, bias = m["qweight"], m["scales"], m["qzeros"], m.get("L"), m.get("bias")
            ext._check_quant(x_probe, qw, sc, qz, self.group_size)
            _check(qw.is_contiguous() and sc.is_contiguous() and qz.is_contiguous(), "group: buffers must be contiguous")
            N = qw.size(0)
            if L is not None:
                _check(L.is_cuda and L.dtype == torch.float16 and L.is_contiguous() and tuple(L.shape) == (N, self.rank),
                       "group: L must be a contiguous CUDA fp16 [OC, rank] tensor")
            if bias is not None:
                _check(bias.is_cuda and bias.dtype == torch.float16 and bias.is_contiguous() and bias.numel() == N,
                       "group: bias must be a contiguous CUDA fp16 [OC] tensor")
            side = None
            if side_streams:
                side_rank = self.rank if corrected else 0
                side = ext.pack_side(sc, qz, L if corrected else None, self.K, self.group_size, side_rank)
                if side is not None:
                    e.side, e.side_rank = side.data_ptr(), side_rank
            e.qweight, e.scales, e.qzeros = qw.data_ptr(), sc.data_ptr(), qz.data_ptr()
            e.L = L.data_ptr() if L is not None else None
            e.bias = bias.data_ptr() if bias is not None else None
            e.N, e.ldw_i32, e.lds, e.ldz_i32 = N, qw.size(1), sc.size(1), qz.size(1)
            self.Ns.append(N)
            self.keep.append((qw, sc, qz, L, bias, side))
        self.corrected = corrected
        self._tiled_keep = None  # the tiled copies of the members' weights: built by the first call with five token rows or more
        self._n_total = sum(self.Ns)

    def run(self, x: torch.Tensor, r: Optional[torch.Tensor] = None, outs: Optional[List[torch.Tensor]] = None,
            project: bool = True) -> List[torch.Tensor]:
        """x [M, K] contiguous fp16 on the group's device.  With a right factor and `project`, r = x R^T is computed by
        the call (into `r`, allocated when not given, and kept as `self.last_r`); otherwise `r` is an input (needed when
        the group is corrected).  Returns the members' [M, N_i] outputs (`outs` when given)."""
        if not (x.is_cuda and x.dtype is torch.float16 and x.dim() == 2 and x.size(1) == self.K and x.is_contiguous()):
            raise RuntimeError("inputs must be contiguous CUDA fp16 [M, IC]")
        M = x.size(0)
        dev = x.device
        if self._tiled_keep is None and M >= TILED_MIN_ROWS and self.ext.wants_tiled(M, self.K, self._n_total, self.group_size,
                                                                                    self.arr[0].ldw_i32):
            self._tiled_keep = [self.ext._set_tiled(e, k[0], k[1], k[2], k[3] if self.corrected else None, self.K, self.group_size)
                                for e, k in zip(self.arr, self.keep)]
        Ns = self.Ns
        if outs is None:
            outs = [torch.empty((M, N), dtype=torch.float16, device=dev) for N in Ns]
            for e, y in zip(self.arr, outs):
                e.y, e.ldy = y.data_ptr(), y.stride(0)
        else:
            for e, y, N in zip(self.arr, outs, Ns):
                _check(y.dtype == torch.float16 and tuple(y.shape) == (M, N) and y.stride(1) == 1, "output must be CUDA fp16 [M, OC]")
                e.y, e.ldy = y.data_ptr(), y.stride(0)
        if M == 0:
            return outs
        fused = project and self.R is not None
        if r is None:
            if fused or self.corrected:
                _check(fused, "group: a corrected group needs r (or a right factor to compute it from)")
                r = torch.empty((M, self.rank), dtype=torch.float16, device=dev)
        elif not (r.dtype is torch.float16 and r.dim() == 2 and r.size(0) == M and r.size(1) == self.rank and r.is_contiguous()):
            raise RuntimeError("r must be fp16 [M, rank]")
        self.last_r = r
        ext = self.ext
        idx = dev.index
        # the library launches on the current device: switch only when the tensors live on another one
        ctx = None
        if idx is not None and idx != torch.cuda.current_device():
            ctx = torch.cuda.device(dev)
            ctx.__enter__()
        try:
            ws, ws_bytes = ext._workspace(dev, M)
            stream = ext._stream(dev)
            if fused:
                rc = self.lib.glowq_w4a16_group_forward_fused_ws(
                    x.data_ptr(), self.R.data_ptr(), r.data_ptr(), self.arr, len(Ns), M, self.K, self.group_size,
                    self.rank, self.alpha, ws, ws_bytes, stream)
            else:
                rc = self.lib.glowq_w4a16_group_forward_ws(
                    x.data_ptr(), r.data_ptr() if (r is not None and self.corrected) else None, self.arr, len(Ns), M,
                    self.K, self.group_size, self.rank if self.corrected else 0, self.alpha, ws, ws_bytes, stream)
        finally:
            if ctx is not None:
                ctx.__exit__(None, None, None)
        if rc:
            ext._raise(rc, "w4a16_group_forward")
        return outs

    def run_chained(self, x: torch.Tensor, prologue: int, epilogue: int, *, r: Optional[torch.Tensor] = None,
                    outs: Optional[List[Optional[torch.Tensor]]] = None, norm_weight=None, eps: float = 0.0, acc_in=None,
                    resid=None, next_norm_weight=None, next_Rt=None, acc_out=None, act=None) -> None:
        """One token through the chained form of the group launch (`glowq_w4a16_group_forward_chained`): `prologue` says
        where the activations and r come from (as given / r from the accumulator `acc_in` / RMSNorm of the residual stream
        `x` with `norm_weight`, `eps` and r from `acc_in`), `epilogue` where the outputs go (the members' `outs` / added
        into the residual stream `resid` / gated into `act`) and, with `next_Rt` ([N, rank], the next group's right
        factor transposed), that the projection of the result on it is added into the accumulator `acc_out`.
        Accumulators are uint8 tensors of CHAIN_ACC_BYTES, zero before the producer runs.  `outs` may hold None for
        members whose own output nobody reads (epilogues other than CHAIN_EPI_NONE)."""
        _check(x.is_cuda and x.dtype == torch.float16 and x.numel() == self.K and x.is_contiguous(),
               "inputs must be one contiguous CUDA fp16 token row [IC]")
        _check(self.corrected, "chained: the group needs a correction")
        keep = [x, r, norm_weight, acc_in, resid, next_norm_weight, next_Rt, acc_out, act]
        for e, N, y in zip(self.arr, self.Ns, outs if outs is not None else [None] * len(self.Ns)):
            if y is None:
                _check(epilogue != CHAIN_EPI_NONE, "chained: without an epilogue every member needs an output")
                e.y, e.ldy = None, N
            else:
                _check(y.dtype == torch.float16 and y.numel() == N and y.is_contiguous(), "output must be CUDA fp16 [OC]")
                e.y, e.ldy = y.data_ptr(), N
        for t, what in ((norm_weight, "norm_weight"), (resid, "resid"), (next_norm_weight, "next_norm_weight"), (act, "act")):
            if t is not None:
                ext_f16 = t.is_cuda and t.dtype == torch.float16 and t.is_contiguous()
                _check(ext_f16, f"chained: {what} must be a contiguous CUDA fp16 tensor")
        for t, what in ((acc_in, "acc_in"), (acc_out, "acc_out")):
            if t is not None:
                _check(t.is_cuda and t.is_contiguous() and t.numel() * t.element_size() >= CHAIN_ACC_BYTES,
                       f"chained: {what} must hold CHAIN_ACC_BYTES")
        n_total = sum(self.Ns) if epilogue != CHAIN_EPI_SWIGLU else self.Ns[0]
        if next_Rt is not None:
            _check(next_Rt.is_cuda and next_Rt.dtype == torch.float16 and next_Rt.is_contiguous()
                   and tuple(next_Rt.shape) == (n_total, self.rank), "chained: next_Rt must be fp16 [N, rank] of this group's rank")
        if resid is not None:
            _check(resid.numel() == n_total, "chained: resid must have one entry per output row")
        if act is not None:
            _check(act.numel() == n_total, "chained: act must have one entry per gate row")
        if norm_weight is not None:
            _check(norm_weight.numel() == self.K, "chained: norm_weight must have IC entries")
        if r is not None:
            _check(r.dtype == torch.float16 and r.numel() == self.rank and r.is_contiguous(), "r must be fp16 [rank]")
        ptr = lambda t: t.data_ptr() if t is not None else None
        ch = _Chain(int(prologue), int(epilogue), ptr(norm_weight), float(eps), ptr(acc_in), ptr(resid),
                    ptr(next_norm_weight), ptr(next_Rt), ptr(acc_out), ptr(act))
        with torch.cuda.device(x.device):
            rc = self.lib.glowq_w4a16_group_forward_chained(
                x.data_ptr(), ptr(r), self.arr, len(self.Ns), self.K, self.group_size, self.rank, self.alpha,
                ctypes.byref(ch), self.ext._stream(x.device))
        del keep
        if rc:
            self.ext._raise(rc, "w4a16_group_forward_chained")


def library_path() -> str:
    return LIB_PATH


def load_w4a16_extension(verbose: Optional[bool] = None) -> W4A16Extension:
    """Loads the prebuilt in-tree library (python -m glowq_amd.build).  Raises RuntimeError when it is
    missing or does not load; nothing falls back to torch.  With W4A16_ALLOW_JIT=1 -- the reference's switch for
    compiling its extension at run time when the prebuilt one is missing (src/cuda_w4a16/kernels.py:24-59) -- a
    library that does not load is built once with hipcc (`glowq_amd.build.build`, about a minute) and loaded again."""
    global _ext
    if _ext is not None:
        return _ext
    truthy = {"1", "true", "yes", "y", "on"}
    want_verbose = bool(verbose) or os.environ.get("W4A16_VERBOSE", os.environ.get("CUDA_MIXED_VERBOSE", "")).lower() in truthy

    def load():
        return W4A16Extension(ctypes.CDLL(LIB_PATH))

    try:
        ext = load()
    except (OSError, AttributeError) as exc:
        if os.environ.get("W4A16_ALLOW_JIT", "").lower() not in truthy:
            raise RuntimeError(
                "Failed to load the prebuilt glowq W4A16 HIP library "
                f"({LIB_PATH}). Build it first with:\n  python -m glowq_amd.build\n"
                "If you intentionally want it built at run time, set W4A16_ALLOW_JIT=1.\n"
                "There is no CPU or torch fallback for this path."
            ) from exc
        from . import build as _build

        _build.build(verbose=want_verbose)
        try:
            ext = load()
        except (OSError, AttributeError) as exc2:
            raise RuntimeError(f"Built the glowq W4A16 HIP library at run time, but it still does not load ({LIB_PATH})") from exc2
    if want_verbose:
        print(f"[glowq_amd] loaded {LIB_PATH} (version {ext.version})")
    _ext = ext
    return _ext


__all__ = ["load_w4a16_extension", "W4A16Extension", "PreparedGroup", "library_path", "LIB_PATH", "MAX_MEMBERS"]
