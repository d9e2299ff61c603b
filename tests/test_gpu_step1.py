"""A layer quantised by GlowQ's step 1 (src/step1_quantize.py:215-290: two codes per byte, zero-point not clamped) carried
through the layout converter into the W4A16 buffers and through the HIP path: the device dequantisation of the converted
buffers equals what the reference's own layer dequantises to, bit for bit, and a GEMV on them matches the oracle.  The
vectors in tests/golden/step1_golden.npz were written by the reference's TritonTrue4BitLinear.from_float and
dequantize_from_triton_layer on CPU tensors."""
import os

import numpy as np
import pytest
import torch

import glowq_oracle as oracle
from glowq_amd import step1_compat as s1
from helpers import assert_close, dev

pytestmark = pytest.mark.gpu


def _golden():
    return np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "step1_golden.npz"))


@pytest.mark.parametrize("name", ["in_range", "many_groups", "small_groups"])
def test_converted_step1_layer_dequantises_like_the_reference_layer(ext, name):
    g = _golden()
    gs = int(g[f"{name}_gs"][0])
    K = g[f"{name}_w"].shape[1]
    qw, qz, sc = s1.step1_to_w4a16(torch.from_numpy(g[f"{name}_qweight"]), torch.from_numpy(g[f"{name}_qzeros"]),
                                   torch.from_numpy(g[f"{name}_scales"]), gs)
    got = ext.dequant(qw.cuda(), sc.cuda(), qz.cuda(), K, gs).cpu().numpy()
    np.testing.assert_array_equal(got.view(np.uint16), g[f"{name}_deq"].view(np.uint16))
    codes = ext.unpack_int4(qw.cuda(), K).cpu().numpy()
    want_codes, _ = s1.unpack_step1(torch.from_numpy(g[f"{name}_qweight"]), torch.from_numpy(g[f"{name}_qzeros"]), sc.size(1))
    np.testing.assert_array_equal(codes, want_codes.numpy()[:, :K])


@pytest.mark.parametrize("name", ["in_range", "many_groups", "small_groups"])
@pytest.mark.parametrize("M", [1, 3, 8, 40])
def test_gemv_on_a_converted_step1_layer(ext, name, M):
    """Every small-M kernel and the MFMA routes on buffers that came out of the converter, against the exact value of the
    reference layer's own dequantised weight."""
    g = _golden()
    gs = int(g[f"{name}_gs"][0])
    w = g[f"{name}_w"]
    K = w.shape[1]
    qw, qz, sc = s1.step1_to_w4a16(torch.from_numpy(g[f"{name}_qweight"]), torch.from_numpy(g[f"{name}_qzeros"]),
                                   torch.from_numpy(g[f"{name}_scales"]), gs)
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(17 + M)).half().numpy()
    y = ext.w4a16_gemv_forward_cuda(dev(x), qw.cuda(), sc.cuda(), qz.cuda(), gs)
    torch.cuda.synchronize()
    want = oracle.linear_exact(x, qw.numpy(), qz.numpy(), sc.numpy(), gs)
    assert_close(y.cpu().numpy(), want, f"step-1 layer {name} M={M}")
    # and against the matmul on the reference layer's own dequantised weight: the same thing up to the fp16 rounding of
    # (code - zero) * scale, which the GEMV arithmetic does not apply
    deq = g[f"{name}_deq"].astype(np.float64)
    ref = x.astype(np.float64) @ deq.T
    assert np.all(np.abs(y.cpu().numpy().astype(np.float64) - ref) <= 2e-2 + 2e-3 * np.abs(ref))


def test_one_sided_groups_are_flagged_and_clean_rows_still_match(ext):
    """Groups without a sign change: step 1 stores a zero-point outside [0, 15] truncated, the W4A16 path clamps.
    `validate` reports them; rows without such a group convert and dequantise on the device like the reference layer."""
    g = _golden()
    w, gs = torch.from_numpy(g["one_sided_w"]), int(g["one_sided_gs"][0])
    rep = s1.validate(w, gs)
    assert rep["groups_zero_point_out_of_range"] == 2 and rep["max_abs_dequant_difference"] > 0.0
    q, z, s, zf = s1.quantize_step1(w, gs)
    out = ((zf < 0) | (zf > 15)).numpy()
    qw, qz, sc = s1.step1_to_w4a16(q, z, s, gs)
    got = ext.dequant(qw.cuda(), sc.cuda(), qz.cuda(), w.shape[1], gs).cpu().numpy()
    clean = ~out.any(axis=1)
    assert clean.any()
    np.testing.assert_array_equal(got[clean].view(np.uint16), g["one_sided_deq"][clean].view(np.uint16))
