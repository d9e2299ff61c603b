"""GPU parity of the entry point that produces the shared projection r = x R^T and runs the group in one call."""
import os

import numpy as np
import pytest
import torch

import glowq_oracle as oracle
from helpers import assert_close, dev, make_group

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CASES = [(1, 2048, [256, 128, 128], 64, 1.0), (2, 4096, [512, 96], 128, 0.5), (1, 4096, [300], 256, 1.0),
         (4, 1024, [64, 64, 64, 64], 32, 2.0), (1, 14336, [128], 128, 1.0), (1, 1024, [16], 128, 1.0),
         (3, 512, [40, 24], 16, 1.0), (8, 1024, [128, 64], 64, 1.0), (40, 1024, [128], 64, 1.0), (1, 200, [9], 24, 1.0)]


def run_cases(ext, repeats=2):
    for (M, K, Ns, rank, alpha) in CASES:
        print(f"case M={M} K={K} Ns={Ns} rank={rank}", flush=True)
        gs = 128 if K % 128 == 0 else 40
        x, members, R = make_group(3 + K + rank + M, M, K, Ns, rank, group_size=gs, with_bias=True)
        mem = [{"qweight": dev(m["qweight"]), "scales": dev(m["scales"]), "qzeros": dev(m["qzeros"]),
                "L": dev(m["L"]) if i != 1 else None, "bias": dev(m["bias"])} for i, m in enumerate(members)]
        xd, Rd = dev(x), dev(R)
        for _ in range(repeats):
            r = torch.full((M, rank), float("nan"), dtype=torch.float16, device="cuda")
            outs = ext.group_forward(xd, r, mem, gs, alpha, R=Rd)
            torch.cuda.synchronize()
            r_want = x.astype(np.float64) @ R.astype(np.float64).T
            assert_close(r.cpu().numpy(), r_want, "r written by the fused launch")
            for i, (m, y) in enumerate(zip(members, outs)):
                if i == 1:
                    want = oracle.linear_exact(x, m["qweight"], m["qzeros"], m["scales"], gs)
                else:
                    want = oracle.corrected_linear_exact(x, m["qweight"], m["qzeros"], m["scales"], gs, R, m["L"], alpha)
                assert_close(y.cpu().numpy(), want + m["bias"].astype(np.float64)[None, :], f"fused member {i}")


def test_fused_projection_matches_oracle(ext, small_m_route):
    run_cases(ext)


def test_fused_equals_two_launch_form(ext, small_m_route):
    M, K, Ns, rank = 1, 4096, [1024, 256, 256], 128
    x, members, R = make_group(91, M, K, Ns, rank)
    mem = [{"qweight": dev(m["qweight"]), "scales": dev(m["scales"]), "qzeros": dev(m["qzeros"]), "L": dev(m["L"])} for m in members]
    r1 = ext.shared_proj(dev(x), dev(R))
    two = ext.group_forward(dev(x), r1, mem, 128, 1.0)
    r2 = torch.empty_like(r1)
    one = ext.group_forward(dev(x), r2, mem, 128, 1.0, R=dev(R))
    torch.cuda.synchronize()
    # r is rounded to fp16 either way; the two forms may differ in the summation order of r only
    assert np.abs(r1.float().cpu().numpy() - r2.float().cpu().numpy()).max() <= 2e-3
    for a, b in zip(one, two):
        assert np.abs(a.float().cpu().numpy() - b.float().cpu().numpy()).max() <= 4e-3


@pytest.mark.parametrize("M", [1, 3])
@pytest.mark.parametrize("rank", [384, 512])
def test_fused_call_with_a_rank_above_the_stream_gemv(ext, M, rank):
    """The stream GEMV holds at most 256 columns of L per row; a fused call (r still to be produced from R when the
    route is picked) with a larger rank has to land on a route that applies all of L r."""
    K, Ns = 4096, [192, 64]
    x, members, R = make_group(500 + rank + M, M, K, Ns, rank)
    mem = [{"qweight": dev(m["qweight"]), "scales": dev(m["scales"]), "qzeros": dev(m["qzeros"]), "L": dev(m["L"])} for m in members]
    r = torch.full((M, rank), float("nan"), dtype=torch.float16, device="cuda")
    outs = ext.group_forward(dev(x), r, mem, 128, 1.0, R=dev(R))
    torch.cuda.synchronize()
    for i, (m, y) in enumerate(zip(members, outs)):
        want = oracle.corrected_linear_exact(x, m["qweight"], m["qzeros"], m["scales"], 128, R, m["L"], 1.0)
        assert_close(y.cpu().numpy(), want, f"rank {rank} member {i}")
        # the correction is not small against the tolerance here: losing the columns past 256 would be seen
        bare = oracle.linear_exact(x, m["qweight"], m["qzeros"], m["scales"], 128)
        assert np.abs(want - bare).max() > 5e-2
