"""Activations with outlier channels (a seeded 1 % of the columns 200 times larger than the rest, everything scaled by
4: values in the thousands among values of order one) through every kernel route of the group entry point.

On such inputs the reference's two routes differ from each other by more than the tolerance (shown on the CPU in
tests/test_oracle.py::test_two_reference_semantics_part_on_outlier_activations), so each kernel is judged against the
semantics it implements:
  * the stream, wave-dot and 4x4x4 GEMV, the skinny kernel's raw-code form and the kernel that streams the tiled copy of
    the weights keep the dequantised weight unrounded, like the reference's GEMV kernel
    (src/cuda_w4a16/csrc/gemv_w4a16.cu:96-112): yardstick `corrected_linear_exact`;
  * the skinny MFMA kernel and the tiled MFMA GEMM round the dequantised weight to fp16 once, like the reference's
    dequantise-then-matmul route (src/cuda_w4a16/csrc/gemm_w4a16.cu:46-49,132): yardstick
    `corrected_linear_rounded_exact`.
Tolerance |a - b| <= 1e-2 + 1e-3 |b| in both cases, plus the effect of rounding r = x R^T to fp16 (the path under test
and the reference both hand r on as fp16, step3_eval_dataset.py:484): |r| 2^-11 carried through |L|."""
import numpy as np
import pytest
import torch

import glowq_oracle as oracle
from helpers import ABS_TOL, REL_TOL, dev, make_group, outlier_activations

pytestmark = pytest.mark.gpu

UNROUNDED = {"wave_dot_gemv", "quad_mfma_gemv", "generic", "stream_gemv", "quad_stream_gemv", "skinny_codes_mfma", "skinny_tiled_mfma"}

# (token rows, K, member widths, rank, route mode); the default limits send 1 row to the wave-dot GEMV, 2..4 rows to the
# wave-dot GEMV, the 4x4x4 GEMV or the skinny kernel by group size, 5..32 to the skinny kernel, 33..64 to the kernel that
# streams the tiled copy of the weights, more to the tiled GEMM
CASES = [
    (1, 4096, [512, 128], 128, "default"), (1, 14336, [128], 128, "default"), (1, 4096, [512, 128], 128, "classic"),
    (2, 4096, [4096], 128, "stream"), (3, 2048, [300], 64, "stream"), (4, 14336, [2048, 2048], 128, "stream"),
    (2, 4096, [4096], 128, "default"), (2, 14336, [8192], 128, "default"),
    (3, 2048, [300], 64, "default"), (4, 4096, [2048, 2048], 64, "default"),
    (4, 4096, [2048, 2048], 64, "quad"), (4, 4096, [2048, 2048], 64, "classic"),
    (8, 4096, [512], 128, "default"), (8, 4096, [512], 128, "quad"), (4, 4096, [512], 128, "qstream"),
    (4, 14336, [8192], 128, "qstream"), (3, 4096, [2048, 2048], 256, "qstream"),
    (16, 14336, [256], 128, "default"), (16, 4096, [1024, 256], 128, "quad"),
    (64, 4096, [512, 96], 256, "default"), (130, 2048, [512], 128, "default"), (300, 4096, [256, 128], 128, "default"),
]


@pytest.fixture()
def tuned(ext):
    saved = {}

    def apply(mode):
        if mode == "default":
            return
        if mode == "stream":
            saved["stream_max_m"] = ext.set_tuning("stream_max_m", 4)
            saved["stream_shape_rule"] = ext.set_tuning("stream_shape_rule", 0)
            saved["qstream_max_m"] = ext.set_tuning("qstream_max_m", 0)
            return
        if mode == "qstream":
            saved["qstream_max_m"] = ext.set_tuning("qstream_max_m", 4)
            saved["qstream_shape_rule"] = ext.set_tuning("qstream_shape_rule", 0)
            return
        for key, value in (("quad_max_m", 16 if mode == "quad" else 0), ("quad_min_m", 1), ("small_group_mb", 0),
                           ("stream_max_m", 0), ("qstream_max_m", 0)):
            saved[key] = ext.set_tuning(key, value)

    yield apply
    for key, value in saved.items():
        ext.set_tuning(key, value)


@pytest.mark.parametrize("case", CASES, ids=lambda c: f"M{c[0]}-K{c[1]}-N{'_'.join(map(str, c[2]))}-r{c[3]}-{c[4]}")
def test_outlier_channels_against_the_semantics_of_the_route(ext, tuned, case):
    M, K, Ns, rank, mode = case
    print(f"case {case}", flush=True)
    tuned(mode)
    x, members, R = make_group(40 + M + K // 64, M, K, Ns, rank)
    x = outlier_activations(x, seed=M + K)
    mem = [{"qweight": dev(m["qweight"]), "scales": dev(m["scales"]), "qzeros": dev(m["qzeros"]), "L": dev(m["L"])} for m in members]
    r = torch.empty(M, rank, dtype=torch.float16, device="cuda")
    outs = ext.group_forward(dev(x), r, mem, 128, 1.0, R=dev(R))
    torch.cuda.synchronize()
    route = ext.route(M, K, sum(Ns))
    r64 = x.astype(np.float64) @ R.astype(np.float64).T
    assert np.all(np.abs(r.cpu().numpy().astype(np.float64) - r64) <= ABS_TOL + REL_TOL * np.abs(r64))
    yardstick = oracle.corrected_linear_exact if route in UNROUNDED else oracle.corrected_linear_rounded_exact
    for j, (m, y) in enumerate(zip(members, outs)):
        got = y.cpu().numpy()
        assert np.isfinite(got).all()
        want = yardstick(x, m["qweight"], m["qzeros"], m["scales"], 128, R, m["L"], 1.0)
        slack = (np.abs(r64) * 2.0 ** -11) @ np.abs(m["L"].astype(np.float64)).T
        err = np.abs(got.astype(np.float64) - want)
        bound = ABS_TOL + REL_TOL * np.abs(want) + slack
        worst = np.unravel_index(np.argmax(err - bound), err.shape)
        assert np.all(err <= bound), (f"member {j} on {route}: err {err[worst]:.4f} > bound {bound[worst]:.4f} at {worst} "
                                      f"(max |y| {np.abs(want).max():.1f})")
        # and the check tells the two semantics apart where it matters: the other yardstick is further away
        other = (oracle.corrected_linear_rounded_exact if route in UNROUNDED else oracle.corrected_linear_exact)(
            x, m["qweight"], m["qzeros"], m["scales"], 128, R, m["L"], 1.0)
        assert np.abs(got.astype(np.float64) - want).mean() <= np.abs(got.astype(np.float64) - other).mean() + 1e-3
