"""The raw-code form of the skinny MFMA kernel (5..64 token rows, groups of 128 columns) through the C ABI against the
float64 oracle of the unrounded arithmetic: the wide tile (two column tiles per wave), the narrow one, two row tiles,
the two passes of 32 rows on wide groups, scales fetched per super-block and in runs of eight, K cut into slices through the
wrapper's workspace, members without L, bias, row counts that are no multiple of the tiles."""
import numpy as np
import pytest
import torch

import glowq_oracle as oracle
from helpers import assert_close, dev, make_group

pytestmark = pytest.mark.gpu

ROUTE = 7  # skinny_codes_mfma


@pytest.fixture()
def codes(ext):
    old = ext.set_tuning("skinny_codes_max_m", 64)
    yield ext
    ext.set_tuning("skinny_codes_max_m", old)


CASES = [
    # M, K, Ns, rank, bias, bare (members of a corrected group without L)
    (5, 256, [7], 0, False, ()),
    (8, 4096, [300, 64], 128, True, ()),
    (6, 2048, [130], 64, False, ()),
    (8, 4096, [1024, 256, 256], 128, False, (1,)),
    (7, 5120, [257], 256, True, ()),
    (16, 4096, [9000, 9000], 128, False, ()),     # wide tile, runs of eight super-blocks
    (8, 2048, [9000, 8000], 64, True, (0,)),      # wide tile, scales per super-block
    (5, 14336, [96, 33], 128, False, ()),
    (8, 14336, [1024], 128, False, ()),     # few column tiles, long K: cut into slices through the workspace
    (33, 4096, [200], 128, True, ()),             # two row tiles
    (64, 3584, [64, 64, 19], 128, False, (0,)),
    (40, 2048, [9000, 8000], 0, False, ()),       # wide group above 32 rows: two passes of the wide tile
    (64, 4096, [8192, 8192], 128, True, ()),
    (12, 1024, [1, 2, 3, 5], 16, False, ()),
    (3, 4096, [512], 128, False, ()),             # three rows of a small group
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: f"M{c[0]}-K{c[1]}-N{'_'.join(map(str, c[2]))}-r{c[3]}")
def test_skinny_codes_group_matches_oracle(codes, case):
    ext = codes
    M, K, Ns, rank, bias, bare = case
    gs = 128
    print(f"case {case}", flush=True)
    saved = None
    if M == 3:  # leave the small group to the skinny kernel
        saved = ext.set_tuning("qstream_max_m", 0), ext.set_tuning("stream_max_m", 0)
    try:
        assert ext.lib.glowq_w4a16_route(M, K, sum(Ns), gs, K // 8) == ROUTE
        x, members, R = make_group(7100 + M + K // 64 + len(Ns), M, K, Ns, rank, group_size=gs, with_bias=bias)
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
    finally:
        if saved is not None:
            ext.set_tuning("qstream_max_m", saved[0]), ext.set_tuning("stream_max_m", saved[1])
    assert torch.isnan(wide[:, 0]).all() and torch.isnan(wide[:, -1]).all()
    for j, (w, y) in enumerate(zip(want, outs)):
        assert_close(y.cpu().numpy(), w, f"member {j}")


def test_skinny_codes_is_exact_on_integer_inputs(codes):
    """Integer-valued activations (multiples of 16, so that their sixteenth is exact) and a power-of-two scale: every
    product and partial sum is exact in fp32, so the result must equal the float64 oracle bit for bit after the one
    rounding to fp16, whatever the order of summation."""
    ext = codes
    M, K, N, gs = 8, 4096, 96, 128
    rng = np.random.default_rng(4)
    x = (16 * rng.integers(-3, 4, (M, K))).astype(np.float16)
    cd = rng.integers(0, 16, (N, K)).astype(np.uint8)
    qw = oracle.pack_int4_to_int32(cd.reshape(N, K // 8, 8))
    zeros = rng.integers(0, 16, (N, K // gs)).astype(np.uint8)
    qz = oracle.pack_int4_to_int32(zeros.reshape(N, K // gs // 8, 8))
    sc = np.full((N, K // gs), 1.0 / 64, dtype=np.float16)
    assert ext.lib.glowq_w4a16_route(M, K, N, gs, K // 8) == ROUTE
    y = ext.w4a16_gemv_forward_cuda(dev(x), dev(qw), dev(sc), dev(qz), gs)
    torch.cuda.synchronize()
    want = oracle.linear_exact(x, qw, qz, sc, gs)
    assert np.array_equal(y.cpu().numpy(), want.astype(np.float16))
