"""The step-1 (two codes per byte, unclamped zero-point) quantiser against the W4A16 quantiser: identical codes where
every zero-point is in range, lossless layout conversion, and detection of the groups where the two disagree."""
import numpy as np
import torch

import glowq_oracle as oracle
from glowq_amd import step1_compat as s1
from glowq_amd.linear import _quantize_per_group_w4


def _w(seed, rows=48, cols=512, std=0.02):
    return (torch.randn(rows, cols, generator=torch.Generator().manual_seed(seed)) * std).half()


def test_byte_layout_low_nibble_is_the_even_index():
    # one row, one group of 8: a ramp min..max hits every second code exactly
    w = torch.linspace(-7, 8, 16).half().reshape(1, 16)
    q, z, s, zf = s1.quantize_step1(w, 16)
    codes, zeros = s1.unpack_step1(q, z, 1)
    assert codes.tolist() == [list(range(16))] and zeros.tolist() == [[7]] and float(zf) == 7.0
    assert q[0, 0].item() == (1 << 4) | 0 and q[0, 7].item() == (15 << 4) | 14        # high nibble = odd index
    assert float(s) == 1.0


def test_in_range_groups_quantise_identically_and_convert_losslessly():
    w = _w(1)
    rep = s1.validate(w, 128)
    assert rep == {"groups": 48 * 4, "groups_zero_point_out_of_range": 0, "in_range_codes_identical": True,
                   "in_range_zero_points_identical": True, "scales_identical": True, "max_abs_dequant_difference": 0.0}
    q, z, s, _ = s1.quantize_step1(w, 128)
    qw, qz, sc = s1.step1_to_w4a16(q, z, s, 128)
    rw, rz, rs, _ = _quantize_per_group_w4(w, 128)
    assert torch.equal(qw, rw) and torch.equal(qz, rz) and torch.equal(sc, rs)
    # the converted buffers dequantise (oracle) to what step 1 dequantises itself
    want = s1.dequant_step1(q, z, s, 512, 128).numpy()
    got = oracle.dequant(qw.numpy(), qz.numpy(), sc.numpy(), 512, 128)
    np.testing.assert_array_equal(got.view(np.uint16), want.view(np.uint16))


def test_ragged_in_features_and_odd_group_count():
    w = _w(2, rows=5, cols=3 * 64 - 10)
    q, z, s, _ = s1.quantize_step1(w, 64)
    assert q.shape == (5, 96) and z.shape == (5, 2) and s.shape == (5, 3)
    qw, qz, sc = s1.step1_to_w4a16(q, z, s, 64)
    rw, rz, rs, _ = _quantize_per_group_w4(w, 64)
    assert torch.equal(qw, rw) and torch.equal(qz, rz) and torch.equal(sc, rs)


def test_one_sided_groups_are_reported():
    w = _w(3)
    w[:4, :128] = w[:4, :128].abs() + 0.05          # all positive: zero-point negative
    w[4:6, 128:256] = -w[4:6, 128:256].abs() - 0.05  # all negative: zero-point above 15
    rep = s1.validate(w, 128)
    assert rep["groups_zero_point_out_of_range"] == 6
    assert rep["in_range_codes_identical"] and rep["in_range_zero_points_identical"] and rep["scales_identical"]
    assert rep["max_abs_dequant_difference"] > 0.0
