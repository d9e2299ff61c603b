"""The stream-scheduled 4x4x4 matrix-core GEMV (2..4 token rows) through the C ABI against the float64 oracle: row
lengths of one step and less, of two, of an odd number of steps (the last slice half empty), long rows cut into
slices, ranks on either side of the 16-byte chunking of L, group sizes up to one group per step, members whose row
count is no multiple of four, members without L, bias, token counts between the staged ones."""
import numpy as np
import pytest
import torch

import glowq_oracle as oracle
from helpers import assert_close, dev, make_group

pytestmark = pytest.mark.gpu

ROUTE = 6  # quad_stream_gemv


@pytest.fixture()
def qstream(ext):
    old = ext.set_tuning("qstream_max_m", 4), ext.set_tuning("qstream_shape_rule", 0)
    yield ext
    ext.set_tuning("qstream_max_m", old[0]), ext.set_tuning("qstream_shape_rule", old[1])


CASES = [
    # M, K, Ns, rank, group_size, bias, bare (members of a corrected group without L)
    (2, 256, [7], 0, 128, False, ()),
    (2, 4096, [300, 64], 128, 128, True, ()),
    (3, 2048, [130], 64, 128, False, ()),
    (4, 4096, [1024, 256, 256], 128, 128, False, (1,)),
    (4, 5120, [257], 256, 128, True, ()),
    (4, 14336, [96, 33], 128, 128, False, ()),
    (2, 14336, [64], 0, 128, False, ()),
    (3, 4096, [200], 8, 256, False, ()),
    (4, 3584, [64, 64, 19], 128, 128, True, (0,)),
    (4, 4096, [512], 128, 128, False, ()),
    (3, 4096, [66], 0, 2048, False, ()),
    (2, 2048, [40], 256, 512, False, ()),
    (4, 16384, [48], 128, 128, False, ()),
    (3, 12288, [36, 4], 256, 128, True, ()),
    (4, 8192, [100], 64, 128, False, ()),
    (3, 5120, [24, 9], 128, 128, False, ()),
    (4, 1024, [1, 2, 3, 5], 24, 128, False, ()),
    (3, 4096, [5000], 64, 128, True, ()),   # between one and two workgroups per compute unit: three tiles per workgroup
    (4, 4096, [20000], 128, 128, False, ()),  # more workgroups than the compute units hold: each walks a list of tiles
    (2, 2048, [9000, 9000, 2000], 0, 128, True, ()),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: f"M{c[0]}-K{c[1]}-N{'_'.join(map(str, c[2]))}-r{c[3]}-g{c[4]}")
def test_qstream_group_matches_oracle(qstream, case):
    ext = qstream
    M, K, Ns, rank, gs, bias, bare = case
    print(f"case {case}", flush=True)
    assert ext.lib.glowq_w4a16_route(M, K, sum(Ns), gs, K // 8) == ROUTE
    x, members, R = make_group(5100 + M + K // 64 + len(Ns), M, K, Ns, rank, group_size=gs, with_bias=bias)
    mem, want = [], []
    for j, m in enumerate(members):
        L = None if (not rank or j in bare) else m["L"]
        mem.append({"qweight": dev(m["qweight"]), "scales": dev(m["scales"]), "qzeros": dev(m["qzeros"]),
                    "L": dev(L) if L is not None else None, "bias": dev(m["bias"]) if bias else None})
        w = (oracle.corrected_linear_exact(x, m["qweight"], m["qzeros"], m["scales"], gs, R, L, 0.5) if L is not None
             else oracle.linear_exact(x, m["qweight"], m["qzeros"], m["scales"], gs))
        want.append(w + (m["bias"].astype(np.float64)[None, :] if bias else 0.0))
    # the members' outputs as column slices of one wide buffer: nothing may land outside them
    wide = torch.full((M, sum(Ns) + 2), float("nan"), dtype=torch.float16, device="cuda")
    starts = np.concatenate([[1], 1 + np.cumsum(Ns)])
    bufs = [wide[:, int(a):int(a) + n] for a, n in zip(starts, Ns)]
    r = torch.empty(M, rank, dtype=torch.float16, device="cuda") if rank else None
    outs = ext.group_forward(dev(x), r, mem, gs, 0.5, outs=bufs, R=dev(R) if rank else None)
    torch.cuda.synchronize()
    assert torch.isnan(wide[:, 0]).all() and torch.isnan(wide[:, -1]).all()
    for j, (w, y) in enumerate(zip(want, outs)):
        assert_close(y.cpu().numpy(), w, f"member {j}")


def test_qstream_is_exact_on_integer_inputs(qstream):
    """Integer-valued activations and unit scales: every product and partial sum is exact in fp32, so the result must
    equal the float64 oracle bit for bit after the one rounding to fp16, whatever the order of summation."""
    ext = qstream
    M, K, N, gs = 4, 4096, 64, 128
    rng = np.random.default_rng(3)
    x = rng.integers(-3, 4, (M, K)).astype(np.float16)
    codes = rng.integers(0, 16, (N, K)).astype(np.uint8)
    qw = oracle.pack_int4_to_int32(codes.reshape(N, K // 8, 8))
    zeros = rng.integers(0, 16, (N, K // gs)).astype(np.uint8)
    qz = oracle.pack_int4_to_int32(zeros.reshape(N, K // gs // 8, 8))
    sc = np.ones((N, K // gs), dtype=np.float16)
    assert ext.lib.glowq_w4a16_route(M, K, N, gs, K // 8) == ROUTE
    y = ext.w4a16_gemv_forward_cuda(dev(x), dev(qw), dev(sc), dev(qz), gs)
    torch.cuda.synchronize()
    want = oracle.linear_exact(x, qw, qz, sc, gs)
    assert np.array_equal(y.cpu().numpy(), want.astype(np.float16))
