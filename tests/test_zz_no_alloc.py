"""`glowq_w4a16_group_forward_fused_static` (the entry point that allocates nothing: its workspace is a static device
array inside the library) against `glowq_w4a16_group_forward_fused_ws` with a caller workspace of the same size, through
the C ABI, on shapes where both users of the workspace take part (the many-row MFMA projection with its split of K and
the skinny kernel's split of K): the two plan the same launches and add their partial tiles in the same order, so the
outputs are equal bit for bit.  Two calls in a row, the second on a smaller input, with the static array left as the
first call wrote it; then the refusals."""

import numpy as np
import pytest
import torch

import glowq_oracle as oracle
from glowq_amd.kernels import _Member
from helpers import assert_close

pytestmark = pytest.mark.gpu

GS = 128


def _random_member(g, N, K, rank):
    return {"qweight": torch.randint(-2**31, 2**31 - 1, (N, K // 8), device="cuda", generator=g, dtype=torch.int64).to(torch.int32),
            "scales": (torch.rand(N, K // GS, device="cuda", generator=g) * 0.008 + 0.002).half(),
            "qzeros": torch.randint(-2**31, 2**31 - 1, (N, (K // GS + 7) // 8), device="cuda", generator=g, dtype=torch.int64).to(torch.int32),
            "L": (torch.randn(N, rank, device="cuda", generator=g) * 0.01).half()}


def _descriptors(members, outs):
    arr = (_Member * len(members))()
    for e, m, y in zip(arr, members, outs):
        e.qweight, e.scales, e.qzeros, e.L = m["qweight"].data_ptr(), m["scales"].data_ptr(), m["qzeros"].data_ptr(), m["L"].data_ptr()
        e.bias, e.y = None, y.data_ptr()
        e.N, e.ldw_i32, e.lds, e.ldz_i32, e.ldy = m["qweight"].size(0), m["qweight"].size(1), m["scales"].size(1), m["qzeros"].size(1), y.stride(0)
    return arr


def _both(ext, M, K, Ns, rank, seed, ws):
    g = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.randn(M, K, device="cuda", generator=g).half()
    R = (torch.randn(rank, K, device="cuda", generator=g) * K ** -0.5).half()
    members = [_random_member(g, N, K, rank) for N in Ns]
    stream = torch.cuda.current_stream().cuda_stream
    res = []
    for static in (False, True):
        outs = [torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda") for N in Ns]
        r = torch.full((M, rank), float("nan"), dtype=torch.float16, device="cuda")
        arr = _descriptors(members, outs)
        if static:
            rc = ext.lib.glowq_w4a16_group_forward_fused_static(x.data_ptr(), R.data_ptr(), r.data_ptr(), arr, len(Ns), M, K, GS,
                                                                rank, 1.0, stream)
        else:
            rc = ext.lib.glowq_w4a16_group_forward_fused_ws(x.data_ptr(), R.data_ptr(), r.data_ptr(), arr, len(Ns), M, K, GS,
                                                            rank, 1.0, ws.data_ptr(), ws.numel(), stream)
        assert rc == 0, ext.lib.glowq_last_error()
        torch.cuda.synchronize()
        res.append((outs, r))
    (outs_ws, r_ws), (outs_st, r_st) = res
    assert torch.equal(r_ws, r_st)
    for a, b in zip(outs_ws, outs_st):
        assert torch.equal(a, b) and torch.isfinite(b.float()).all()
    # and both are right: sampled output rows against the oracle (the skinny kernel rounds the weight to fp16 once)
    rows = np.unique(np.concatenate(([0, 1, Ns[0] - 1], np.random.default_rng(seed).integers(0, Ns[0], 12))))
    idx = torch.from_numpy(rows).cuda()
    m0 = members[0]
    want = oracle.corrected_linear_rounded_exact(x.cpu().numpy(), m0["qweight"][idx].cpu().numpy(), m0["qzeros"][idx].cpu().numpy(),
                                                 m0["scales"][idx].cpu().numpy(), GS, R.cpu().numpy(), m0["L"][idx].cpu().numpy(), 1.0)
    assert_close(outs_st[0][:, idx].cpu().numpy(), want, f"static entry point M={M} K={K}")


def test_static_scratch_entry_point_matches_the_workspace_entry_point(ext):
    size = ext.lib.glowq_static_scratch_bytes()
    assert size == 8 << 20
    ws = torch.empty(size, dtype=torch.uint8, device="cuda")
    # long K, few columns, 48 rows: MFMA projection split over K and the skinny kernel's split of K both use the workspace
    assert ext.lib.glowq_proj_workspace_bytes(48, 14336, 128) > 0
    print("static scratch case 1: M=48 K=14336 N=4096 rank=128", flush=True)
    _both(ext, 48, 14336, [4096], 128, seed=1, ws=ws)
    # straight after it a smaller input (fewer rows, fewer columns in two members; both splits still take part): the array
    # still holds the first call's tiles
    assert ext.lib.glowq_proj_workspace_bytes(20, 14336, 256) > 0
    print("static scratch case 2: M=20 K=14336 N=1024+512 rank=256", flush=True)
    _both(ext, 20, 14336, [1024, 512], 256, seed=2, ws=ws)
    # a single row uses no workspace at all and goes through just the same
    print("static scratch case 3: M=1 K=4096 N=4096 rank=128", flush=True)
    _both(ext, 1, 4096, [4096], 128, seed=3, ws=ws)


def test_static_scratch_entry_point_refuses_what_it_cannot_hold(ext):
    g = torch.Generator(device="cuda").manual_seed(5)
    K, N, rank, M = 4096, 256, 64, 65
    x = torch.randn(M, K, device="cuda", generator=g).half()
    R = (torch.randn(rank, K, device="cuda", generator=g) * K ** -0.5).half()
    mem = _random_member(g, N, K, rank)
    y = torch.zeros(M, N, dtype=torch.float16, device="cuda")
    r = torch.zeros(M, rank, dtype=torch.float16, device="cuda")
    arr = _descriptors([mem], [y])
    rc = ext.lib.glowq_w4a16_group_forward_fused_static(x.data_ptr(), R.data_ptr(), r.data_ptr(), arr, 1, M, K, GS, rank, 1.0,
                                                        torch.cuda.current_stream().cuda_stream)
    assert rc == -4 and b"at most 64" in ext.lib.glowq_last_error()
    torch.cuda.synchronize()
    assert not y.any() and not r.any()                        # nothing was launched
    rc = ext.lib.glowq_w4a16_group_forward_fused_static(x.data_ptr(), None, r.data_ptr(), arr, 1, 8, K, GS, rank, 1.0,
                                                        torch.cuda.current_stream().cuda_stream)
    assert rc == -1                                            # the argument checks of the workspace entry point apply


def test_static_scratch_entry_point_under_graph_capture(ext):
    """Recorded into a HIP graph after glowq_static_scratch_prepare() and replayed with eager work in between: every
    replay equals the workspace entry point bit for bit."""
    assert ext.lib.glowq_static_scratch_prepare() == 0
    g = torch.Generator(device="cuda").manual_seed(9)
    M, K, Ns, rank = 24, 14336, [1024, 256], 128
    x = torch.randn(M, K, device="cuda", generator=g).half()
    R = (torch.randn(rank, K, device="cuda", generator=g) * K ** -0.5).half()
    members = [_random_member(g, N, K, rank) for N in Ns]
    ws = torch.empty(ext.lib.glowq_static_scratch_bytes(), dtype=torch.uint8, device="cuda")
    outs_ws = [torch.empty((M, N), dtype=torch.float16, device="cuda") for N in Ns]
    r_ws = torch.empty((M, rank), dtype=torch.float16, device="cuda")
    outs_st = [torch.empty((M, N), dtype=torch.float16, device="cuda") for N in Ns]
    r_st = torch.empty((M, rank), dtype=torch.float16, device="cuda")
    arr_ws, arr_st = _descriptors(members, outs_ws), _descriptors(members, outs_st)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            rc = ext.lib.glowq_w4a16_group_forward_fused_static(x.data_ptr(), R.data_ptr(), r_st.data_ptr(), arr_st, len(Ns), M, K,
                                                                GS, rank, 1.0, side.cuda_stream)
    assert rc == 0, ext.lib.glowq_last_error()
    torch.cuda.synchronize()
    for rep in range(3):
        x.copy_(torch.randn(M, K, device="cuda", generator=g).half())   # eager work between the replays
        for t in outs_st + [r_st]:
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        rc = ext.lib.glowq_w4a16_group_forward_fused_ws(x.data_ptr(), R.data_ptr(), r_ws.data_ptr(), arr_ws, len(Ns), M, K, GS,
                                                        rank, 1.0, ws.data_ptr(), ws.numel(), torch.cuda.current_stream().cuda_stream)
        assert rc == 0, ext.lib.glowq_last_error()
        torch.cuda.synchronize()
        assert torch.equal(r_ws, r_st), f"replay {rep}"
        for a, b in zip(outs_ws, outs_st):
            assert torch.equal(a, b) and torch.isfinite(b.float()).all(), f"replay {rep}"
