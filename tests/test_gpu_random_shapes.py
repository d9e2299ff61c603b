"""Seeded random sweep over token rows, K, member widths, ranks, group sizes, bias and selective members: one group
launch per case through the C ABI against the float64 oracle, whatever kernel route the shape takes."""
import os

import numpy as np
import pytest
import torch

import glowq_oracle as oracle
from helpers import assert_close, dev, make_group

pytestmark = pytest.mark.gpu

ROWS = [1, 2, 3, 4, 5, 7, 8, 13, 16, 17, 31, 32, 33, 48, 64, 65, 100, 130, 257]
ROUTES = {0: "wave_dot_gemv", 1: "skinny_mfma", 2: "tiled_mfma_gemm", 3: "generic", 4: "quad_mfma_gemv", 5: "stream_gemv",
          6: "quad_stream_gemv", 7: "skinny_codes_mfma"}


def random_cases(n, seed=20240):
    rng = np.random.default_rng(seed)
    cases = []
    for i in range(n):
        gs = int(rng.choice([32, 64, 128, 128, 128, 256]))
        kind = rng.random()
        if kind < 0.6:
            K = 256 * int(rng.integers(1, 25))
        elif kind < 0.85:
            K = 64 * int(rng.integers(1, 97))
        else:
            K = 8 * int(rng.integers(4, 400))
        if K % gs and rng.random() < 0.7:
            K = max(gs, K // gs * gs)  # most cases keep whole groups; the rest exercise the zero-padded tail group
        M = int(rng.choice(ROWS))
        Ns = [int(rng.integers(1, 700)) for _ in range(int(rng.integers(1, 5)))]
        rank = int(rng.choice([0, 0, 5, 8, 12, 24, 64, 96, 128, 256]))
        alpha = float(rng.choice([1.0, 0.5, 2.0]))
        bias = bool(rng.random() < 0.4)
        bare = [bool(rank and rng.random() < 0.2) for _ in Ns]  # members of a corrected group without their own L
        # extra columns behind the ones in use (the reference takes row strides from size(1): any width at or above the
        # needed one is valid) and the members' outputs as column slices of one wide buffer (row stride above N)
        pads = (int(rng.choice([0, 0, 1, 4, 8])), int(rng.choice([0, 0, 1, 2, 8])), int(rng.choice([0, 0, 1, 3])))
        wide_out = bool(rng.random() < 0.4)
        cases.append((i, M, K, Ns, rank, gs, alpha, bias, bare, pads, wide_out))
    return cases


@pytest.fixture(params=["default", "stream", "qstream", "quad", "classic"])
def route_mode(request, ext):
    """The library's own route limits, the stream GEMV for every case of 1..4 rows it can take, the stream-scheduled
    4x4x4 matrix-core GEMV for every case of 2..4 rows it can take, the 4x4x4 matrix-core GEMV for every case of 1..16
    rows it can take, or all switched off (wave-dot GEMV up to 4 rows, skinny MFMA kernel above)."""
    if request.param == "default":
        yield request.param
        return
    if request.param == "qstream":
        old = ext.set_tuning("qstream_max_m", 4), ext.set_tuning("qstream_shape_rule", 0)
        yield request.param
        ext.set_tuning("qstream_max_m", old[0]), ext.set_tuning("qstream_shape_rule", old[1])
        return
    if request.param == "stream":
        old = ext.set_tuning("stream_max_m", 4), ext.set_tuning("stream_shape_rule", 0), ext.set_tuning("qstream_max_m", 0)
        yield request.param
        ext.set_tuning("stream_max_m", old[0]), ext.set_tuning("stream_shape_rule", old[1]), ext.set_tuning("qstream_max_m", old[2])
        return
    old = [ext.set_tuning("quad_max_m", 16 if request.param == "quad" else 0), ext.set_tuning("quad_min_m", 1),
           ext.set_tuning("small_group_mb", 0), ext.set_tuning("stream_max_m", 0), ext.set_tuning("qstream_max_m", 0)]
    yield request.param
    for key, value in zip(("quad_max_m", "quad_min_m", "small_group_mb", "stream_max_m", "qstream_max_m"), old):
        ext.set_tuning(key, value)


# GLOWQ_RANDOM_CASES / GLOWQ_RANDOM_SEED widen or move the sweep for a hunting run; the defaults are what the suite runs
@pytest.mark.parametrize("case", random_cases(int(os.environ.get("GLOWQ_RANDOM_CASES", "32")), int(os.environ.get("GLOWQ_RANDOM_SEED", "20240"))), ids=lambda c: f"{c[0]}-M{c[1]}-K{c[2]}-N{'_'.join(map(str, c[3]))}-r{c[4]}-g{c[5]}")
def test_random_group_matches_oracle(ext, route_mode, case):
    i, M, K, Ns, rank, gs, alpha, bias, bare, pads, wide_out = case
    print(f"case {case}", flush=True)
    x, members, R = make_group(9000 + i, M, K, Ns, rank, group_size=gs, with_bias=bias)
    mem, want = [], []
    for m, no_l in zip(members, bare):
        L = None if (not rank or no_l) else m["L"]
        rng = np.random.default_rng(77 + i)
        qw = np.concatenate([m["qweight"], rng.integers(-2**31, 2**31 - 1, (m["qweight"].shape[0], pads[0]), dtype=np.int64).astype(np.int32)], axis=1)
        sc = np.concatenate([m["scales"], np.full((m["scales"].shape[0], pads[1]), 3.0e4, dtype=np.float16)], axis=1)
        qz = np.concatenate([m["qzeros"], rng.integers(-2**31, 2**31 - 1, (m["qzeros"].shape[0], pads[2]), dtype=np.int64).astype(np.int32)], axis=1)
        mem.append({"qweight": dev(qw), "scales": dev(sc), "qzeros": dev(qz),
                    "L": dev(L) if L is not None else None, "bias": dev(m["bias"]) if bias else None})
        w = (oracle.corrected_linear_exact(x, m["qweight"], m["qzeros"], m["scales"], gs, R, L, alpha) if L is not None
             else oracle.linear_exact(x, m["qweight"], m["qzeros"], m["scales"], gs))
        want.append(w + (m["bias"].astype(np.float64)[None, :] if bias else 0.0))
    r = torch.empty(M, rank, dtype=torch.float16, device="cuda") if rank else None
    bufs = None
    if wide_out:
        wide = torch.full((M, sum(Ns) + 3), float("nan"), dtype=torch.float16, device="cuda")
        starts = np.concatenate([[1], 1 + np.cumsum(Ns)])  # odd first column: outputs aligned to 2 bytes only
        bufs = [wide[:, int(a):int(a) + n] for a, n in zip(starts, Ns)]
    outs = ext.group_forward(dev(x), r, mem, gs, alpha, outs=bufs, R=dev(R) if rank else None)
    torch.cuda.synchronize()
    route = ROUTES.get(ext.lib.glowq_w4a16_route(M, K, sum(Ns), gs, members[0]["qweight"].shape[1] + pads[0]), "?")
    if wide_out:  # nothing written outside the members' columns
        assert torch.isnan(wide[:, 0]).all() and torch.isnan(wide[:, 1 + sum(Ns):]).all()
    for j, (w, y) in enumerate(zip(want, outs)):
        assert y.shape == (M, Ns[j])
        assert_close(y.cpu().numpy(), w, f"case {i} member {j} route {route} ({route_mode})")
    if rank:
        want_r = x.astype(np.float64) @ R.astype(np.float64).T
        assert_close(r.cpu().numpy(), want_r, f"case {i} shared projection")
