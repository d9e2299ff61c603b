"""CPU restatement of the reference's torch execution path, for the benchmark's cpu_baseline leg and
for cross-checks in tests.  TEST / MEASUREMENT INFRASTRUCTURE ONLY: never imported by the product.

Follows, op for op, what the reference runs when no device kernel is involved:

  dequant_chunk / linear_chunked   src/cuda_w4a16/linear.py:229-238,248-253
        unpack codes and zero-points, gather per-column zero and scale through `gid`, fp16
        `(q - z) * s`, then `torch.matmul(x, W_chunk^T)` per 512-row chunk
  corrected_group                  src/step3_eval_dataset.py:470-511
        r = F.linear(x, R) once per group (leader), F.linear(r, L_i) per member, in-place add with alpha

Pinned by tests/test_oracle.py against the numpy oracle and the golden vectors under tests/golden.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F


def unpack_i32(packed: torch.Tensor, total: int) -> torch.Tensor:
    shifts = (torch.arange(8, dtype=torch.int32) * 4).view(1, 1, 8)
    vals = ((packed.to(torch.int32).unsqueeze(-1) >> shifts) & 0xF).to(torch.uint8)
    return vals.reshape(packed.size(0), -1)[:, :total].contiguous()


def dequant_chunk(qweight, qzeros, scales, gid, in_features, groups, start, end) -> torch.Tensor:
    q = unpack_i32(qweight[start:end], in_features).to(torch.float16)
    z = unpack_i32(qzeros[start:end, : (groups + 7) // 8], groups).to(torch.float16)
    return (q - z.index_select(1, gid)) * scales[start:end].index_select(1, gid)


def linear_chunked(x, member, chunk: int = 512, compute_dtype=torch.float16) -> torch.Tensor:
    """x [M, K] fp16 -> [M, N] fp16, dequantising `chunk` output rows at a time."""
    qweight, qzeros, scales = member["qweight"], member["qzeros"], member["scales"]
    n_out, in_features = qweight.size(0), x.size(1)
    gs = member["group_size"]
    groups = -(-in_features // gs)
    gid = torch.arange(in_features, dtype=torch.long) // gs
    out = torch.empty((x.size(0), n_out), dtype=torch.float16)
    xc = x.to(compute_dtype)
    for start in range(0, n_out, chunk):
        end = min(start + chunk, n_out)
        w = dequant_chunk(qweight, qzeros, scales, gid, in_features, groups, start, end)
        out[:, start:end] = torch.matmul(xc, w.to(compute_dtype).t()).to(torch.float16)
    return out


def corrected_group(x, members, R, alpha: float = 1.0, chunk: int = 512, compute_dtype=torch.float16):
    """One QKV / MLP group the way the reference executes it: the leader computes r, followers reuse it."""
    r = None
    outs = []
    for m in members:
        z = linear_chunked(x, m, chunk, compute_dtype)
        if alpha != 0.0 and R is not None and m.get("L") is not None:
            if r is None:
                r = F.linear(x.to(compute_dtype), R.to(compute_dtype)).to(torch.float16)
            svd = F.linear(r.to(compute_dtype), m["L"].to(compute_dtype)).to(torch.float16)
            z.add_(svd, alpha=alpha)
        outs.append(z)
    return outs


def cached_dequant_group(x, dense_members, R, alpha: float = 1.0):
    """Variant with the weights dequantised once beforehand (the reference's optional
    W4A16_DEQUANT_CACHE idea, linear.py:212-227) and fp32 matmuls: the CPU figure without the Python
    dequantisation cost."""
    xf = x.float()
    r = None
    outs = []
    for m in dense_members:
        z = xf @ m["w_f32"].t()
        if alpha != 0.0 and R is not None and m.get("L") is not None:
            if r is None:
                r = xf @ R.float().t()
            z = z + alpha * (r @ m["L"].float().t())
        outs.append(z.half())
    return outs
