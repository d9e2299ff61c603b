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


# ---------------------------------------------------------------- golden vectors written by the reference's own layer
def _golden():
    import os

    return np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "step1_golden.npz"))


def test_in_range_weights_match_the_reference_layer_bit_for_bit():
    """TritonTrue4BitLinear.from_float and dequantize_from_triton_layer (src/step1_quantize.py:215-290) on CPU tensors,
    recorded by tests/golden/make_golden.py: codes, zero-point bytes, scales and dequantised weight."""
    g = _golden()
    for name in ("in_range", "many_groups", "small_groups"):
        w, gs = torch.from_numpy(g[f"{name}_w"]), int(g[f"{name}_gs"][0])
        q, z, s, zf = s1.quantize_step1(w, gs)
        assert not ((zf < 0) | (zf > 15)).any()
        np.testing.assert_array_equal(q.numpy(), g[f"{name}_qweight"])
        np.testing.assert_array_equal(z.numpy(), g[f"{name}_qzeros"])
        np.testing.assert_array_equal(s.numpy().view(np.uint16), g[f"{name}_scales"].view(np.uint16))
        d = s1.dequant_step1(q, z, s, w.shape[1], gs)
        np.testing.assert_array_equal(d.numpy().view(np.uint16), g[f"{name}_deq"].view(np.uint16))
        codes, zeros = s1.unpack_step1(torch.from_numpy(g[f"{name}_qweight"]), torch.from_numpy(g[f"{name}_qzeros"]), s.size(1))
        want_codes, want_zeros = oracle.codes_and_params(*(t.numpy() for t in s1.step1_to_w4a16(q, z, s, gs)[:2]), s.numpy(), w.shape[1], gs)[:2]
        np.testing.assert_array_equal(codes.numpy().reshape(want_codes.shape), want_codes)
        np.testing.assert_array_equal(zeros.numpy(), want_zeros)


def test_one_sided_groups_of_the_reference_layer():
    """Groups without a sign change give a zero-point outside [0, 15].  Codes and scales still agree bit for bit; the
    reference's zero-point byte holds whatever its float -> uint8 conversion produced (on CPU the value modulo 256, so
    a zero-point of -16 in an even group sets the bits of its odd neighbour's nibble: byte 240 where the nibbles 0 and
    7 would give 112).  That byte is not reproduced: `validate` reports the groups, and every other byte is equal."""
    g = _golden()
    w, gs = torch.from_numpy(g["one_sided_w"]), int(g["one_sided_gs"][0])
    q, z, s, zf = s1.quantize_step1(w, gs)
    np.testing.assert_array_equal(q.numpy(), g["one_sided_qweight"])
    np.testing.assert_array_equal(s.numpy().view(np.uint16), g["one_sided_scales"].view(np.uint16))
    out = ((zf < 0) | (zf > 15)).numpy()
    assert out.sum() == 2 and out[0, 0] and out[1, 1]
    assert s1.validate(w, gs)["groups_zero_point_out_of_range"] == 2
    ref_bytes = g["one_sided_qzeros"]
    touched = out[:, 0::2] | out[:, 1::2]                         # bytes that hold an out-of-range zero-point
    np.testing.assert_array_equal(z.numpy()[~touched], ref_bytes[~touched])
    assert ref_bytes[0, 0] == 240 and z.numpy()[0, 0] == 112     # the spill described above
    assert ref_bytes[1, 0] == z.numpy()[1, 0] == 184             # an odd group's excess bits are shifted out
    # rows without such a group dequantise identically
    d = s1.dequant_step1(q, z, s, w.shape[1], gs).numpy()
    clean = ~out.any(axis=1)
    np.testing.assert_array_equal(d[clean].view(np.uint16), g["one_sided_deq"][clean].view(np.uint16))
