"""CPU oracle for the GlowQ Step-3 hot path (W4A16 linear + group-shared low-rank correction).

TEST INFRASTRUCTURE ONLY.  This module is the checker the HIP path is compared against.  Only
tests, the smoke check and the benchmark's ``cpu_baseline`` leg may import it; the product
package never does, and has no CPU fallback.

Everything is restated in numpy from the reference's algorithm (paths relative to the
reference checkout):

  pack_int4_to_int32   src/cuda_w4a16/linear.py:42-46
  unpack_int4_i32      src/cuda_w4a16/linear.py:49-54   (device twin csrc/gemv_w4a16.cu:16-18)
  quantize_per_group_w4 src/cuda_w4a16/linear.py:57-88
  dequant              src/cuda_w4a16/linear.py:248-253 (device twin csrc/gemm_w4a16.cu:19-50)
  gemv_ref             src/cuda_w4a16/csrc/gemv_w4a16.cu:34-142   (fp32-accumulate semantics)
  gemm_ref             src/cuda_w4a16/csrc/gemm_w4a16.cu:76-135   (dequant to fp16, then matmul)
  shared_proj / correction / group_forward   src/step3_eval_dataset.py:470-511
  MiniGroupCacheModel  src/step3_eval_dataset.py:417-444
  rmsnorm / swiglu / residual_add   the decoder-layer modules around the wrappers' forward.  The reference runs them
                       through Hugging Face transformers' LlamaRMSNorm and LlamaMLP (transformers is a pip dependency
                       of the reference, requirements.txt, not vendored); restated from their published definitions:
                       fp32 variance, x * rsqrt(var + eps) rounded to the input dtype, then times the weight;
                       act_fn(gate) * up with SiLU; hidden = residual + hidden in fp16.

How each function is pinned (tests/test_oracle_*.py):
  * pack / unpack / quantize / dequant / the CPU forward: bit-exact against golden vectors that
    tests/golden/make_golden.py wrote by running the reference's own functions once in the build
    container (tests/golden/*.npz), plus exhaustive brute force over all nibble values/positions.
  * gemv_ref / gemm_ref / linear_exact / linear_rounded_exact: reduce to ``x @ dequant(W).T`` (a library
    matmul on the golden-pinned dequant) and to one-hot inputs that select single dequantised columns exactly;
    linear_rounded_exact rounded to fp16 is gemm_ref.
  * correction / group_forward: closed form ``z + alpha * (x R^T) L^T`` against a float64 library
    matmul; alpha = 0 identity; linearity in alpha; group == independent solo results.
  * rmsnorm / swiglu / residual_add: against torch's own fp32 formulas (torch.nn.functional.silu, the variance written
    out) on seeded inputs, the norm's scale invariance rmsnorm(c x) = rmsnorm(x) for eps = 0, and hand-computed
    vectors (tests/test_oracle.py).
  * quantize on constant groups (scale underflows to 0 in fp16 -> NaN zero-point) is UNDEFINED in
    the reference; it is excluded from parity and documented as such.
"""
from __future__ import annotations

import numpy as np

F16 = np.float16


# --------------------------------------------------------------------------------------
# int4 <-> int32 packing
# --------------------------------------------------------------------------------------
def pack_int4_to_int32(u4: np.ndarray) -> np.ndarray:
    """[..., 8] uint8 codes -> [...] int32; element i sits in bits 4i..4i+3 (LSB first).

    The reference sums ``code << 4i`` in int32, so a code >= 8 in nibble 7 sets the sign bit.
    """
    if u4.dtype != np.uint8:
        raise TypeError("codes must be uint8")
    if u4.shape[-1] != 8:
        raise ValueError("last dim must be 8")
    acc = np.zeros(u4.shape[:-1], dtype=np.uint32)
    for i in range(8):
        acc = acc | (u4[..., i].astype(np.uint32) << np.uint32(4 * i))
    return np.asarray(acc, dtype=np.uint32).view(np.int32)


def unpack_int4_i32(packed: np.ndarray, total_vals: int) -> np.ndarray:
    """[rows, W] int32 -> [rows, total_vals] uint8, nibble ``k & 7`` of word ``k >> 3``."""
    packed = np.ascontiguousarray(packed).astype(np.int32, copy=False)
    rows = packed.shape[0]
    u = packed.view(np.uint32)
    shifts = (np.arange(8, dtype=np.uint32) * 4).reshape(1, 1, 8)
    vals = ((u[..., None] >> shifts) & np.uint32(0xF)).astype(np.uint8)
    return np.ascontiguousarray(vals.reshape(rows, -1)[:, :total_vals])


# --------------------------------------------------------------------------------------
# quantiser (fp16 arithmetic, one rounding per elementwise op, round-half-to-even)
# --------------------------------------------------------------------------------------
def _h(x) -> np.ndarray:
    return np.asarray(x, dtype=F16)


def quantize_per_group_w4(weight: np.ndarray, group_size: int):
    """Asymmetric min/max uint4 quantiser on an fp16 weight [N, K].

    Returns (qweight int32 [N, Kp/8], qzeros int32 [N, ceil(G/8)], scales fp16 [N, G], Kp).
    Every elementwise op rounds its result to fp16, as a chain of fp16 tensor ops does.
    """
    w = _h(weight)
    oc, ic = w.shape
    if ic % group_size != 0:
        pad = group_size - ic % group_size
        w = np.concatenate([w, np.zeros((oc, pad), dtype=F16)], axis=1)
        ic = w.shape[1]
    groups = ic // group_size
    wg = w.reshape(oc, groups, group_size)
    w_min = wg.min(axis=-1)
    w_max = wg.max(axis=-1)
    with np.errstate(all="ignore"):
        diff = _h(w_max.astype(np.float32) - w_min.astype(np.float32))
        scales = _h(diff.astype(np.float32) / np.float32(15.0))
        # clamp(min=1e-8): 1e-8 is below the smallest fp16 subnormal, the floor is 0 in fp16.
        scales = _h(np.maximum(scales.astype(np.float32), np.float32(1e-8)))
        neg_min = _h(-w_min.astype(np.float32))
        zf = _h(neg_min.astype(np.float32) / scales.astype(np.float32))
        zf = _h(np.rint(zf.astype(np.float32)))
        zeros_fp = _h(np.clip(zf.astype(np.float32), 0.0, 15.0))
        t = _h(wg.astype(np.float32) / scales[..., None].astype(np.float32))
        t = _h(t.astype(np.float32) + zeros_fp[..., None].astype(np.float32))
        t = _h(np.rint(t.astype(np.float32)))
        q = np.clip(t.astype(np.float32), 0.0, 15.0)
    if group_size % 8 != 0:
        raise ValueError("group_size must be multiple of 8 for int32 int4 packing")
    q = np.nan_to_num(q, nan=0.0).astype(np.uint8)
    q_packed = pack_int4_to_int32(q.reshape(oc, groups, group_size // 8, 8))

    zeros_u8 = np.nan_to_num(zeros_fp.astype(np.float32), nan=0.0).astype(np.uint8)
    groups_packed = (groups + 7) // 8
    pad_groups = groups_packed * 8 - groups
    zeros_base = np.concatenate(
        [zeros_u8, np.full((oc, pad_groups), 8, dtype=np.uint8)], axis=1
    )
    zeros_packed = pack_int4_to_int32(zeros_base.reshape(oc, groups_packed, 8))
    return (
        np.ascontiguousarray(q_packed.reshape(oc, ic // 8)),
        np.ascontiguousarray(zeros_packed),
        np.ascontiguousarray(scales),
        ic,
    )


# --------------------------------------------------------------------------------------
# dequantisation
# --------------------------------------------------------------------------------------
def codes_and_params(qweight, qzeros, scales, in_features: int, group_size: int):
    """Unpacked (codes uint8 [N,K], zeros uint8 [N,G], scales fp16 [N,G], gid int64 [K])."""
    groups = -(-in_features // group_size)
    groups_packed = (groups + 7) // 8
    codes = unpack_int4_i32(qweight, in_features)
    zeros = unpack_int4_i32(np.ascontiguousarray(qzeros[:, :groups_packed]), groups)
    gid = np.arange(in_features) // group_size
    return codes, zeros, _h(scales)[:, :groups], gid


def dequant(qweight, qzeros, scales, in_features: int, group_size: int) -> np.ndarray:
    """fp16 W[n,k] = fp16((code - zero[n,k//g]) * scale[n,k//g]); the difference is exact, the
    product is rounded once."""
    codes, zeros, sc, gid = codes_and_params(qweight, qzeros, scales, in_features, group_size)
    d = codes.astype(np.float32) - zeros[:, gid].astype(np.float32)
    return _h(d * sc[:, gid].astype(np.float32))


# --------------------------------------------------------------------------------------
# linear forward, both reference semantics
# --------------------------------------------------------------------------------------
def gemv_ref(x, qweight, qzeros, scales, group_size: int, acc=np.float64) -> np.ndarray:
    """GEMV-kernel semantics: y[m,n] = fp16(sum_k (code - z) * s * x[m,k]); the dequantised
    weight is NOT rounded to fp16.  Accumulates in ``acc`` (float64: the order-free value the
    kernel's fp32 tree sum approximates)."""
    x = _h(x)
    k = x.shape[1]
    codes, zeros, sc, gid = codes_and_params(qweight, qzeros, scales, k, group_size)
    w = (codes.astype(acc) - zeros[:, gid].astype(acc)) * sc[:, gid].astype(acc)
    return _h(x.astype(acc) @ w.T)


def gemm_ref(x, qweight, qzeros, scales, group_size: int, acc=np.float64) -> np.ndarray:
    """GEMM-path semantics: dequantise to fp16 (one rounding), matmul with wide accumulate, fp16 out."""
    x = _h(x)
    w = dequant(qweight, qzeros, scales, x.shape[1], group_size)
    return _h(x.astype(acc) @ w.astype(acc).T)


def linear_exact(x, qweight, qzeros, scales, group_size: int) -> np.ndarray:
    """float64 value of sum_k (code - z) * s * x with no output rounding: the yardstick both
    reference semantics and the HIP kernels are measured against."""
    x = _h(x)
    k = x.shape[1]
    codes, zeros, sc, gid = codes_and_params(qweight, qzeros, scales, k, group_size)
    w = (codes.astype(np.float64) - zeros[:, gid].astype(np.float64)) * sc[:, gid].astype(np.float64)
    return x.astype(np.float64) @ w.T


def linear_rounded_exact(x, qweight, qzeros, scales, group_size: int) -> np.ndarray:
    """float64 value of x @ dequant(W)^T with the dequantised weight rounded to fp16 first and no output rounding:
    the "dequantise, then matmul" route (src/cuda_w4a16/csrc/gemm_w4a16.cu:46-49,132) without the library GEMM's own
    rounding.  ``gemm_ref`` is this value rounded to fp16."""
    x = _h(x)
    w = dequant(qweight, qzeros, scales, x.shape[1], group_size)
    return x.astype(np.float64) @ w.astype(np.float64).T


# --------------------------------------------------------------------------------------
# group-shared low-rank correction
# --------------------------------------------------------------------------------------
def shared_proj(x, R, acc=np.float64) -> np.ndarray:
    """r = fp16(x @ R^T): the shared right-factor projection (R is [rank, K])."""
    return _h(_h(x).astype(acc) @ _h(R).astype(acc).T)


def correction(z, r, L, alpha: float, acc=np.float64) -> np.ndarray:
    """z + alpha * (r @ L^T) with the reference's roundings: the product to fp16, then one fp16
    add (computed wide, rounded once).  L is [N_i, rank]."""
    svd = _h(_h(r).astype(acc) @ _h(L).astype(acc).T)
    return _h(_h(z).astype(np.float32) + np.float32(alpha) * svd.astype(np.float32))


def corrected_linear_exact(x, qweight, qzeros, scales, group_size, R, L, alpha) -> np.ndarray:
    """float64, unrounded z + alpha * (x R^T) L^T."""
    z = linear_exact(x, qweight, qzeros, scales, group_size)
    r = _h(x).astype(np.float64) @ _h(R).astype(np.float64).T
    return z + float(alpha) * (r @ _h(L).astype(np.float64).T)


def corrected_linear_rounded_exact(x, qweight, qzeros, scales, group_size, R, L, alpha) -> np.ndarray:
    """float64, unrounded x @ fp16(dequant(W))^T + alpha * (x R^T) L^T: the dequantise-then-matmul-plus-correction
    value (gemm_w4a16.cu:76-135 followed by step3_eval_dataset.py:484-511) before any output rounding."""
    z = linear_rounded_exact(x, qweight, qzeros, scales, group_size)
    r = _h(x).astype(np.float64) @ _h(R).astype(np.float64).T
    return z + float(alpha) * (r @ _h(L).astype(np.float64).T)


def rmsnorm(x, weight, eps: float) -> np.ndarray:
    """fp16(fp16(x * rsqrt(mean(x^2) + eps)) * weight) over the last axis, statistics in fp32 (LlamaRMSNorm)."""
    x32 = _h(x).astype(np.float32)
    var = np.mean(x32.astype(np.float64) ** 2, axis=-1, keepdims=True).astype(np.float32)
    n = _h(x32 * (np.float32(1.0) / np.sqrt(var + np.float32(eps))))
    return _h(n.astype(np.float32) * _h(weight).astype(np.float32))


def rmsnorm_factor(x, eps: float) -> np.ndarray:
    """rsqrt(mean(x^2) + eps) in float64: the one scalar per row that keeps RMSNorm from being linear."""
    x64 = _h(x).astype(np.float64)
    return 1.0 / np.sqrt(np.mean(x64 ** 2, axis=-1, keepdims=True) + float(eps))


def swiglu(gate, up) -> np.ndarray:
    """fp16(fp16(silu(gate)) * up): act_fn(gate_proj(x)) * up_proj(x) of LlamaMLP on fp16 tensors."""
    g = _h(gate).astype(np.float64)
    a = _h(g / (1.0 + np.exp(-g)))
    return _h(a.astype(np.float32) * _h(up).astype(np.float32))


def residual_add(residual, hidden) -> np.ndarray:
    """fp16(residual + hidden): the decoder layer's residual connection on fp16 tensors."""
    return _h(_h(residual).astype(np.float32) + _h(hidden).astype(np.float32))


def group_forward(x, members, R, alpha: float, semantics: str = "gemv"):
    """One QKV / MLP group: every member shares r = x R^T.

    ``members`` is a list of dicts with keys qweight, qzeros, scales, group_size and L (or None for
    an uncorrected member).  Returns the list of fp16 outputs, reference roundings applied.
    """
    lin = gemv_ref if semantics == "gemv" else gemm_ref
    r = shared_proj(x, R) if R is not None else None
    outs = []
    for m in members:
        z = lin(x, m["qweight"], m["qzeros"], m["scales"], m["group_size"])
        if m.get("L") is not None and r is not None and alpha != 0.0:
            z = correction(z, r, m["L"], alpha)
        outs.append(z)
    return outs


class MiniGroupCacheModel:
    """State machine of the use-counted one-slot cache (set / consume / clear)."""

    def __init__(self):
        self.r = None
        self.valid = False
        self.uses_left = 0

    def set(self, r, uses: int):
        self.r, self.valid, self.uses_left = r, True, uses

    def consume(self):
        if self.valid and self.uses_left > 0:
            self.uses_left -= 1
            out = self.r
            if self.uses_left == 0:
                self.valid = False
                self.r = None
            return out, True
        return None, False

    def clear(self):
        self.r, self.valid, self.uses_left = None, False, 0


# --------------------------------------------------------------------------------------
# algorithmic work per launch (the numerator of the roofline)
# --------------------------------------------------------------------------------------
def algorithmic_bytes(M: int, K: int, N: int, rank: int = 0, group_size: int = 128) -> int:
    G = -(-K // group_size)
    b = N * K // 2 + 2 * N * G + 4 * N * (-(-G // 8)) + 2 * M * K + 2 * M * N
    if rank:
        b += 2 * rank * K + 2 * N * rank
    return b


def algorithmic_flops(M: int, K: int, N: int, rank: int = 0) -> int:
    f = 2 * M * N * K
    if rank:
        f += 2 * M * rank * K + 2 * M * N * rank
    return f
