"""The quantiser of GlowQ's step 1 next to the one of the W4A16 path: layout converter and validator.

Step 1 measures the quantisation error E = W - deq(Q(W)) that the low-rank factors are fitted to, with the quantiser of
its Triton layer (src/step1_quantize.py:215-260): same min/max asymmetric uint4 arithmetic as the W4A16 path
(src/cuda_w4a16/linear.py:57-88), but
  * the zero-point is NOT clamped to [0, 15] before it is stored (step1_quantize.py:234 vs linear.py:69), and
  * codes and zero-points are packed two per uint8, low nibble = even index (step1_quantize.py:244-253), where the
    W4A16 path packs eight per int32.
Whenever every zero-point lies in [0, 15] (every group's range straddles or touches zero) the two quantisers produce the
same codes, zero-points and scales, and a step-1 layer converts losslessly into the W4A16 buffers.  A group whose
zero-point falls outside (all-positive or all-negative group) is stored truncated to a nibble by step 1 and clamped by the
W4A16 path: the factors were then fitted to a different error than the one the kernel leaves, which is what `validate`
reports.

    python -m glowq_amd.step1_compat --weights original_weights.pt [--group-size 128]

Parity of `quantize_step1` / `dequant_step1`: bit for bit against vectors the reference's own layer wrote on CPU
tensors (tests/golden/step1_golden.npz) for weights whose zero-points are in range.  On out-of-range zero-points the
reference stores whatever its float -> uint8 conversion yields (implementation-defined; on CPU the value modulo 256,
whose upper bits then overwrite the neighbouring group's nibble): flagged here, not reproduced.  The reference's layer
raises for in_features that are not a multiple of the group size and for an odd number of groups (its buffers are sized
in_features / 2 and groups // 2); this module pads both, which only a caller outside the reference's domain can see.
"""
from __future__ import annotations

import argparse
import json
from typing import Dict, Tuple

import torch

from .linear import _pack_int4_to_int32, _quantize_per_group_w4, _unpack_int4_i32


def quantize_step1(weight: torch.Tensor, group_size: int):
    """(qweight_u8 [O, I_pad/2], qzeros_u8 [O, ceil(G/2)], scales [O, G], zeros_float [O, G]) in the dtype arithmetic of
    `weight`, op for op as step1_quantize.py:222-253.  `zeros_float` is the unclamped zero-point; the packed zero-points
    hold its low nibble (what `qzeros & 0x0F` recovers when it is in range)."""
    n_out, n_in = weight.shape
    if n_in % group_size:
        weight = torch.nn.functional.pad(weight, (0, group_size - n_in % group_size))
    n_pad = weight.shape[1]
    grouped = weight.reshape(n_out, n_pad // group_size, group_size)
    lo, hi = grouped.min(dim=-1).values, grouped.max(dim=-1).values
    scales = ((hi - lo) / 15.0).clamp(min=1e-8)
    zeros_float = (-lo / scales).round()
    codes = torch.round(grouped / scales.unsqueeze(-1) + zeros_float.unsqueeze(-1)).clamp(0, 15).to(torch.uint8)
    qweight = ((codes[:, :, 1::2] << 4) | codes[:, :, 0::2]).reshape(n_out, n_pad // 2)
    znib = (zeros_float.to(torch.int64) & 0xF).to(torch.uint8)
    if znib.shape[1] % 2:
        znib = torch.nn.functional.pad(znib, (0, 1))
    qzeros = (znib[:, 1::2] << 4) | znib[:, 0::2]
    return qweight.contiguous(), qzeros.contiguous(), scales.to(torch.float16), zeros_float


def unpack_step1(qweight_u8: torch.Tensor, qzeros_u8: torch.Tensor, n_groups: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """uint8 codes [O, I_pad] and zero-points [O, G] of a step-1 layer (step1_quantize.py:268-277)."""
    codes = torch.stack((qweight_u8 & 0x0F, qweight_u8 >> 4), dim=-1).reshape(qweight_u8.size(0), -1)
    zeros = torch.stack((qzeros_u8 & 0x0F, qzeros_u8 >> 4), dim=-1).reshape(qzeros_u8.size(0), -1)[:, :n_groups]
    return codes, zeros.contiguous()


def step1_to_w4a16(qweight_u8: torch.Tensor, qzeros_u8: torch.Tensor, scales: torch.Tensor, group_size: int):
    """Re-packs a step-1 layer into the W4A16 buffers (qweight_i32 [O, I_pad/8], qzeros_i32 [O, ceil(G/8)] padded with
    code 8, scales_f16 [O, G]); the codes themselves are untouched."""
    n_groups = scales.size(1)
    codes, zeros = unpack_step1(qweight_u8, qzeros_u8, n_groups)
    n_out, n_pad = codes.shape
    if n_pad != n_groups * group_size:
        raise ValueError(f"step-1 layer holds {n_pad} codes per row, expected {n_groups} groups of {group_size}")
    qweight = _pack_int4_to_int32(codes.reshape(n_out, n_pad // 8, 8))
    words = (n_groups + 7) // 8
    zfull = torch.full((n_out, words * 8), 8, dtype=torch.uint8, device=codes.device)
    zfull[:, :n_groups] = zeros
    qzeros = _pack_int4_to_int32(zfull.reshape(n_out, words, 8))
    return qweight.contiguous(), qzeros.contiguous(), scales.to(torch.float16).contiguous()


def dequant_step1(qweight_u8, qzeros_u8, scales, in_features: int, group_size: int) -> torch.Tensor:
    """(code - zero) * scale in the dtype of `scales`, as step1_quantize.py:263-290."""
    n_groups = scales.size(1)
    codes, zeros = unpack_step1(qweight_u8, qzeros_u8, n_groups)
    grouped = codes.reshape(codes.size(0), n_groups, group_size)
    deq = (grouped.to(scales.dtype) - zeros.unsqueeze(-1).to(scales.dtype)) * scales.unsqueeze(-1)
    return deq.reshape(codes.size(0), -1)[:, :in_features].contiguous()


def validate(weight: torch.Tensor, group_size: int = 128) -> Dict[str, float]:
    """Quantises `weight` both ways and reports where they differ: groups with a zero-point outside [0, 15], whether the
    buffers agree bit for bit on all other groups after layout conversion, and the largest difference of the two
    dequantised weights."""
    weight = weight.to(torch.float16)
    n_out, n_in = weight.shape
    q1, z1, s1, zf = quantize_step1(weight, group_size)
    qw, qz, sc, n_pad = _quantize_per_group_w4(weight, group_size)
    n_groups = sc.size(1)
    out_of_range = (zf < 0) | (zf > 15)
    cw, cz, cs = step1_to_w4a16(q1, z1, s1, group_size)
    codes_a = _unpack_int4_i32(cw, n_pad).reshape(n_out, n_groups, group_size)
    codes_b = _unpack_int4_i32(qw, n_pad).reshape(n_out, n_groups, group_size)
    zer_a = _unpack_int4_i32(cz, n_groups)
    zer_b = _unpack_int4_i32(qz, n_groups)
    ok = ~out_of_range
    same_codes = bool((codes_a[ok] == codes_b[ok]).all()) if ok.any() else True
    same_zeros = bool((zer_a[ok] == zer_b[ok]).all()) if ok.any() else True
    same_scales = bool(torch.equal(cs.view(torch.int16), sc.view(torch.int16)))
    d1 = dequant_step1(q1, z1, s1, n_in, group_size).float()
    # the W4A16 path's dequantisation: exact difference, one rounding of the product to fp16 (linear.py:248-253)
    d2 = ((codes_b.float() - zer_b.float().unsqueeze(-1)) * sc.float().unsqueeze(-1)).half().float().reshape(n_out, -1)[:, :n_in]
    return {
        "groups": int(out_of_range.numel()),
        "groups_zero_point_out_of_range": int(out_of_range.sum()),
        "in_range_codes_identical": same_codes,
        "in_range_zero_points_identical": same_zeros,
        "scales_identical": same_scales,
        "max_abs_dequant_difference": float((d1 - d2).abs().max()),
    }


def main():
    ap = argparse.ArgumentParser(description="Compare the step-1 quantiser with the W4A16 quantiser on a weight file.")
    ap.add_argument("--weights", help="dict name -> 2-D tensor saved by step 1 (--out_original_weights); loaded with "
                                      "weights_only=True.  Without it: a random matrix with some all-positive groups.")
    ap.add_argument("--group-size", type=int, default=128)
    ap.add_argument("--device", default="cuda" if torch.cuda.is_available() else "cpu")
    args = ap.parse_args()
    if args.weights:
        tensors = torch.load(args.weights, map_location="cpu", weights_only=True)
    else:
        g = torch.Generator().manual_seed(0)
        w = torch.randn(256, 1024, generator=g) * 0.02
        w[:8, :128] = w[:8, :128].abs() + 0.01
        tensors = {"synthetic": w}
    total = {"groups": 0, "groups_zero_point_out_of_range": 0}
    for name, w in tensors.items():
        if not torch.is_tensor(w) or w.dim() != 2:
            continue
        rep = validate(w.to(args.device), args.group_size)
        total["groups"] += rep["groups"]
        total["groups_zero_point_out_of_range"] += rep["groups_zero_point_out_of_range"]
        print(json.dumps({"tensor": name, **rep}))
    print(json.dumps({"total": total}))


if __name__ == "__main__":
    main()
