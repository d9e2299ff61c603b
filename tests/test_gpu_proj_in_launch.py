"""GPU tests of the single-token group launch that computes the shared projection r = R x itself: the first waves of
the grid produce the entries, the others pick them up through tagged words in the caller's workspace.  The results have
to be the bits of the two-launch form (projection launch in front, group launch on the r it left), on every launch and
every replay of a captured graph, whatever the words still hold from earlier launches."""
import re

import numpy as np
import pytest
import torch

import glowq_oracle as oracle
from helpers import assert_close, dev, make_group, tuning

pytestmark = pytest.mark.gpu

# (K, member rows, rank): the three summation forms of the projection (up to 4096 columns, up to 8192, above), ranks up
# to the 256 the stream GEMV holds, ragged row counts, a K that is no multiple of 2048
CASES = [(4096, [1024, 256, 256], 128), (2048, [256, 128, 128], 64), (4096, [600], 256), (8192, [300, 40], 128),
         (14336, [512], 128), (4128, [256, 96], 32), (8224, [384], 64), (1024, [250], 16)]


@pytest.fixture(autouse=True)
def stream_gemv_for_every_shape(ext):
    """The stream GEMV serves the single-token launches of this file whatever their size."""
    with tuning(ext, stream_max_m=4, stream_shape_rule=0):
        yield


def in_launch(ext) -> bool:
    """Whether the calling thread's last group launch was the stream GEMV with the projection inside (prologue 3)."""
    name = ext.last_launch()["kernel"]
    if not name.startswith("gemv_stream_kernel<"):
        return False
    return name[name.index("<") + 1:-1].split(",")[4] == "3"


def members_on_device(members, drop_left=None, with_bias=False):
    return [{"qweight": dev(m["qweight"]), "scales": dev(m["scales"]), "qzeros": dev(m["qzeros"]),
             "L": None if i == drop_left else dev(m["L"]), "bias": dev(m["bias"]) if with_bias else None}
            for i, m in enumerate(members)]


def two_launch(ext, xd, Rd, mem, alpha):
    r = ext.shared_proj(xd, Rd)
    return r, ext.group_forward(xd, r, mem, 128, alpha)


@pytest.mark.parametrize("K,Ns,rank", CASES)
def test_same_bits_as_the_projection_launch_in_front(ext, K, Ns, rank):
    print(f"case K={K} Ns={Ns} rank={rank}", flush=True)
    x, members, R = make_group(7 + K + rank, 1, K, Ns, rank, with_bias=True)
    mem = members_on_device(members, drop_left=1 if len(Ns) > 1 else None, with_bias=True)
    xd, Rd = dev(x), dev(R)
    r_two, y_two = two_launch(ext, xd, Rd, mem, 0.75)
    for rep in range(3):
        r = torch.full((1, rank), float("nan"), dtype=torch.float16, device="cuda")
        y = ext.group_forward(xd, r, mem, 128, 0.75, R=Rd)
        assert in_launch(ext), ext.last_launch()
        torch.cuda.synchronize()
        assert torch.equal(r, r_two), f"r, launch {rep}"
        for a, b in zip(y, y_two):
            assert torch.equal(a, b), f"launch {rep}"
    # and both are right
    assert_close(r_two.cpu().numpy(), x.astype(np.float64) @ R.astype(np.float64).T, "r")
    for i, (m, got) in enumerate(zip(members, y_two)):
        want = (oracle.linear_exact(x, m["qweight"], m["qzeros"], m["scales"], 128) if mem[i]["L"] is None else
                oracle.corrected_linear_exact(x, m["qweight"], m["qzeros"], m["scales"], 128, R, m["L"], 0.75))
        assert_close(got.cpu().numpy(), want + m["bias"].astype(np.float64)[None, :], f"member {i}")


def test_side_streams_and_prepared_group(ext):
    """The prepared group (side streams, one call per token) takes the same route and gives the same bits."""
    from glowq_amd.kernels import PreparedGroup
    K, Ns, rank = 4096, [512, 128, 128], 128
    x, members, R = make_group(11, 1, K, Ns, rank)
    mem = members_on_device(members)
    xd, Rd = dev(x), dev(R)
    r_two, y_two = two_launch(ext, xd, Rd, mem, 1.0)
    pg = PreparedGroup(ext, mem, K, 128, 1.0, R=Rd, side_streams=True)
    outs = pg.run(xd)
    assert in_launch(ext), ext.last_launch()
    assert ext.last_launch()["kernel"].split(",")[3] == "1"      # from the side streams
    torch.cuda.synchronize()
    assert torch.equal(pg.last_r, r_two)
    for a, b in zip(outs, y_two):
        assert torch.equal(a, b)


def test_every_launch_sees_its_own_r(ext):
    """Launch after launch through the same words, each with another x (and, in between, another group with another
    rank through the same words): no launch may pick up what an earlier one left."""
    K, Ns, rank = 4096, [384, 128], 128
    _, members, R = make_group(23, 1, K, Ns, rank)
    _, members_b, R_b = make_group(24, 1, 2048, [256], 64)
    mem, mem_b = members_on_device(members), members_on_device(members_b)
    Rd, Rd_b = dev(R), dev(R_b)
    g = torch.Generator().manual_seed(5)
    for it in range(12):
        xd = torch.randn(1, K, generator=g).half().cuda()
        r = torch.empty((1, rank), dtype=torch.float16, device="cuda")
        y = ext.group_forward(xd, r, mem, 128, 1.0, R=Rd)
        assert in_launch(ext)
        r_two, y_two = two_launch(ext, xd, Rd, mem, 1.0)
        torch.cuda.synchronize()
        assert torch.equal(r, r_two), f"launch {it}"
        for a, b in zip(y, y_two):
            assert torch.equal(a, b), f"launch {it}"
        xb = torch.randn(1, 2048, generator=g).half().cuda()
        rb = torch.empty((1, 64), dtype=torch.float16, device="cuda")
        yb = ext.group_forward(xb, rb, mem_b, 128, 1.0, R=Rd_b)
        rb_two, yb_two = two_launch(ext, xb, Rd_b, mem_b, 1.0)
        torch.cuda.synchronize()
        assert torch.equal(rb, rb_two) and torch.equal(yb[0], yb_two[0]), f"launch {it}, second group"


def test_replays_of_a_captured_graph(ext):
    """A replay runs with the arguments of the capture; the tag of the hand-over words must still be new every time.
    Eager work and synchronisations lie between the replays, and every replay is checked."""
    K, Ns, rank = 4096, [1024, 256, 256], 128
    _, members, R = make_group(31, 1, K, Ns, rank)
    mem = members_on_device(members)
    Rd = dev(R)
    g = torch.Generator().manual_seed(6)
    xs = torch.randn(1, K, generator=g).half().cuda()
    r = torch.empty((1, rank), dtype=torch.float16, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ext.group_forward(xs, r, mem, 128, 1.0, R=Rd)      # outside the capture first: buffers and kernel attributes
        assert in_launch(ext)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            outs = ext.group_forward(xs, r, mem, 128, 1.0, R=Rd)
            again = ext.group_forward(xs, r, mem, 128, 1.0, R=Rd)   # two launches per replay through the same words
        assert in_launch(ext)
    torch.cuda.synchronize()
    for rep in range(6):
        xs.copy_(torch.randn(1, K, generator=g).half())
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        r_two, y_two = two_launch(ext, xs, Rd, mem, 1.0)
        torch.cuda.synchronize()
        assert torch.equal(r, r_two), f"replay {rep}"
        for a, b, c in zip(outs, again, y_two):
            assert torch.equal(a, c) and torch.equal(b, c), f"replay {rep}"


def test_readers_that_never_hear_from_the_producers(ext):
    """With the producers muted every reader runs into the poll limit and computes its entry itself (fp32, column
    order): the caller still gets r from the producers, and the outputs are right within the tolerance."""
    K, Ns, rank = 2048, [192, 64], 64
    x, members, R = make_group(41, 1, K, Ns, rank)
    mem = members_on_device(members)
    xd, Rd = dev(x), dev(R)
    r_two, _ = two_launch(ext, xd, Rd, mem, 1.0)
    for limit in (0, 3):
        with tuning(ext, proj_in_launch=2, proj_spin_limit=limit):
            r = torch.full((1, rank), float("nan"), dtype=torch.float16, device="cuda")
            y = ext.group_forward(xd, r, mem, 128, 1.0, R=Rd)
            assert in_launch(ext)
            torch.cuda.synchronize()
        assert torch.equal(r, r_two)
        for m, got in zip(members, y):
            assert_close(got.cpu().numpy(), oracle.corrected_linear_exact(x, m["qweight"], m["qzeros"], m["scales"], 128, R, m["L"], 1.0),
                         f"limit {limit}")
    # a reader that does not wait at all (limit 0) but is served in time gives the usual bits
    with tuning(ext, proj_spin_limit=0):
        r = torch.empty((1, rank), dtype=torch.float16, device="cuda")
        y = ext.group_forward(xd, r, mem, 128, 1.0, R=Rd)
        torch.cuda.synchronize()
    for m, got in zip(members, y):
        assert_close(got.cpu().numpy(), oracle.corrected_linear_exact(x, m["qweight"], m["qzeros"], m["scales"], 128, R, m["L"], 1.0),
                     "no waiting")


def test_calls_that_cannot_hand_r_over_keep_the_projection_launch(ext):
    """No workspace, one that is too small, the switch turned off: the projection launch goes in front as before, and
    the results are the same bits."""
    K, Ns, rank = 4096, [512, 128], 128
    x, members, R = make_group(51, 1, K, Ns, rank)
    mem = members_on_device(members)
    xd, Rd = dev(x), dev(R)
    r_two, y_two = two_launch(ext, xd, Rd, mem, 1.0)
    with tuning(ext, proj_in_launch=0):
        r = torch.empty((1, rank), dtype=torch.float16, device="cuda")
        y = ext.group_forward(xd, r, mem, 128, 1.0, R=Rd)
        assert not in_launch(ext)
        torch.cuda.synchronize()
        assert torch.equal(r, r_two) and all(torch.equal(a, b) for a, b in zip(y, y_two))
    # (a group with fewer waves than entries of r is no exception: the entries come from workgroups of their own)
    xs, small, Rs = make_group(52, 1, 2048, [64, 32], 128)
    ms = members_on_device(small)
    r = torch.empty((1, 128), dtype=torch.float16, device="cuda")
    y = ext.group_forward(dev(xs), r, ms, 128, 1.0, R=dev(Rs))
    assert in_launch(ext)
    rs_two, ys_two = two_launch(ext, dev(xs), dev(Rs), ms, 1.0)
    torch.cuda.synchronize()
    assert torch.equal(r, rs_two) and all(torch.equal(a, b) for a, b in zip(y, ys_two))
    for m, got in zip(small, y):
        assert_close(got.cpu().numpy(), oracle.corrected_linear_exact(xs, m["qweight"], m["qzeros"], m["scales"], 128, Rs, m["L"], 1.0), "small group")
    # through the C ABI: a workspace one byte short of the hand-over words, and none at all
    from glowq_amd.kernels import _Member
    n = len(mem)
    marr = (_Member * n)()
    ys = []
    for e, m, N in zip(marr, mem, Ns):
        yb = torch.empty((1, N), dtype=torch.float16, device="cuda")
        e.qweight, e.scales, e.qzeros, e.L, e.y = (m["qweight"].data_ptr(), m["scales"].data_ptr(), m["qzeros"].data_ptr(),
                                                   m["L"].data_ptr(), yb.data_ptr())
        e.N, e.ldw_i32, e.lds, e.ldz_i32, e.ldy = N, m["qweight"].size(1), m["scales"].size(1), m["qzeros"].size(1), N
        ys.append(yb)
    ws = torch.zeros(6144, dtype=torch.uint8, device="cuda")     # what the hand-over takes: the block, and 4096 bytes behind it 256 staging words
    stream = ext._stream(xd.device)
    for ws_bytes, want_in in ((6143, False), (6144, True), (0, False)):
        r = torch.empty((1, rank), dtype=torch.float16, device="cuda")
        rc = ext.lib.glowq_w4a16_group_forward_fused_ws(xd.data_ptr(), Rd.data_ptr(), r.data_ptr(), marr, n, 1, K, 128, rank, 1.0,
                                                        ws.data_ptr() if ws_bytes else None, ws_bytes, stream)
        assert rc == 0, ext.lib.glowq_last_error().decode()
        assert in_launch(ext) == want_in, (ws_bytes, ext.last_launch())
        torch.cuda.synchronize()
        assert torch.equal(r, r_two), ws_bytes
        for a, b in zip(ys, y_two):
            assert torch.equal(a, b), ws_bytes


def test_two_streams_with_their_own_words(ext):
    """Two streams run launches of the same groups at the same time; each stream has its own hand-over words (the Python
    layer keeps them per stream), so neither picks up the other's r.  Every result is the two-launch form's."""
    K, Ns, rank = 4096, [768, 256], 128
    _, members, R = make_group(61, 1, K, Ns, rank)
    _, members_b, R_b = make_group(62, 1, K, Ns, rank)
    mem, mem_b = members_on_device(members), members_on_device(members_b)
    Rd, Rd_b = dev(R), dev(R_b)
    g = torch.Generator().manual_seed(8)
    xs = [torch.randn(1, K, generator=g).half().cuda() for _ in range(8)]
    want = [(two_launch(ext, x, Rd, mem, 1.0), two_launch(ext, x, Rd_b, mem_b, 1.0)) for x in xs]
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    got = []
    for x in xs:
        with torch.cuda.stream(s1):
            r1 = torch.empty((1, rank), dtype=torch.float16, device="cuda")
            y1 = ext.group_forward(x, r1, mem, 128, 1.0, R=Rd)
            assert in_launch(ext)
        with torch.cuda.stream(s2):
            r2 = torch.empty((1, rank), dtype=torch.float16, device="cuda")
            y2 = ext.group_forward(x, r2, mem_b, 128, 1.0, R=Rd_b)
            assert in_launch(ext)
        got.append(((r1, y1), (r2, y2)))
    torch.cuda.synchronize()
    for i, (w, h) in enumerate(zip(want, got)):
        for (rw, yw), (rg, yg) in zip(w, h):
            assert torch.equal(rw, rg), f"token {i}"
            for a, b in zip(yw, yg):
                assert torch.equal(a, b), f"token {i}"


# ---- the skinny kernel at a handful of token rows ----------------------------------------------------------------------
# (M, K, member rows, rank, alpha): the raw-code form (up to 8 rows) and the dequantising form, one and two column-tile
# members, a member without L, K slices through the workspace (few column tiles, long K), rank 256, a scale on the
# correction
SKINNY_CASES = [(8, 4096, [1024, 256, 256], 128, 1.0), (16, 5120, [640, 320], 128, 1.0), (8, 5120, [640, 320], 256, 1.0), (5, 1024, [96, 64], 64, 0.5),
                (8, 14336, [512], 128, 1.0), (12, 2048, [200], 32, 2.0), (32, 4096, [512, 128], 128, 1.0)]


def skinny_in_launch(ext) -> bool:
    return ext.last_launch()["kernel"].startswith("skinny_group_kernel<") and ext.last_launch()["kernel"].endswith(",1>")


@pytest.fixture
def skinny_routes(ext):
    """The skinny kernel on the canonical buffers serves these launches (not the kernel that streams the tiled copy)."""
    with tuning(ext, tiled_max_m=0):
        yield


@pytest.mark.parametrize("M,K,Ns,rank,alpha", SKINNY_CASES)
def test_skinny_kernel_computes_r_itself(ext, skinny_routes, M, K, Ns, rank, alpha):
    print(f"case M={M} K={K} Ns={Ns} rank={rank}", flush=True)
    x, members, R = make_group(70 + M + K + rank, M, K, Ns, rank, with_bias=True)
    mem = members_on_device(members, drop_left=1 if len(Ns) > 1 else None, with_bias=True)
    xd, Rd = dev(x), dev(R)
    with tuning(ext, proj_in_launch=0):
        r_two = torch.empty((M, rank), dtype=torch.float16, device="cuda")
        y_two = ext.group_forward(xd, r_two, mem, 128, alpha, R=Rd)
        assert not skinny_in_launch(ext)
    for rep in range(3):
        r = torch.full((M, rank), float("nan"), dtype=torch.float16, device="cuda")
        y = ext.group_forward(xd, r, mem, 128, alpha, R=Rd)
        assert skinny_in_launch(ext), ext.last_launch()
        torch.cuda.synchronize()
        assert_close(r.cpu().numpy(), x.astype(np.float64) @ R.astype(np.float64).T, f"r, launch {rep}")
        for i, (m, got) in enumerate(zip(members, y)):
            want = (oracle.linear_exact(x, m["qweight"], m["qzeros"], m["scales"], 128) if mem[i]["L"] is None else
                    oracle.corrected_linear_exact(x, m["qweight"], m["qzeros"], m["scales"], 128, R, m["L"], alpha))
            assert_close(got.cpu().numpy(), want + m["bias"].astype(np.float64)[None, :], f"member {i}, launch {rep}")
            # and next to the two-launch form: the same weights' sums, the correction added behind instead of in front
            assert np.abs(got.float().cpu().numpy() - y_two[i].float().cpu().numpy()).max() <= 4e-3 * max(1.0, float(np.abs(want).max()))


def test_skinny_launches_and_replays_see_their_own_r(ext, skinny_routes):
    """Launch after launch and replay after replay through the same workspace, each with other activations."""
    M, K, Ns, rank = 8, 4096, [768, 256], 128
    _, members, R = make_group(81, M, K, Ns, rank)
    mem = members_on_device(members)
    Rd = dev(R)
    g = torch.Generator().manual_seed(9)
    xs = torch.randn(M, K, generator=g).half().cuda()
    r = torch.empty((M, rank), dtype=torch.float16, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ext.group_forward(xs, r, mem, 128, 1.0, R=Rd)
        assert skinny_in_launch(ext)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            outs = ext.group_forward(xs, r, mem, 128, 1.0, R=Rd)
            again = ext.group_forward(xs, r, mem, 128, 1.0, R=Rd)
        assert skinny_in_launch(ext)
    torch.cuda.synchronize()
    for rep in range(5):
        xs.copy_(torch.randn(M, K, generator=g).half())
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        xn = xs.cpu().numpy()
        assert_close(r.cpu().numpy(), xn.astype(np.float64) @ R.astype(np.float64).T, f"r, replay {rep}")
        for m, a, b in zip(members, outs, again):
            want = oracle.corrected_linear_exact(xn, m["qweight"], m["qzeros"], m["scales"], 128, R, m["L"], 1.0)
            assert_close(a.cpu().numpy(), want, f"replay {rep}")
            assert torch.equal(a, b), f"replay {rep}: two launches of one replay"


def test_skinny_waves_that_never_see_the_ready_word(ext, skinny_routes):
    """With the producers' flags held down no wave ever sees the ready word: each computes the part of r it needs
    itself; the caller still gets r from the producers."""
    M, K, Ns, rank = 6, 1024, [96, 32], 64
    x, members, R = make_group(91, M, K, Ns, rank)
    mem = members_on_device(members)
    xd, Rd = dev(x), dev(R)
    with tuning(ext, proj_in_launch=2):
        r = torch.full((M, rank), float("nan"), dtype=torch.float16, device="cuda")
        y = ext.group_forward(xd, r, mem, 128, 1.0, R=Rd)
        assert skinny_in_launch(ext), ext.last_launch()
        torch.cuda.synchronize()
    assert_close(r.cpu().numpy(), x.astype(np.float64) @ R.astype(np.float64).T, "r")
    for m, got in zip(members, y):
        assert_close(got.cpu().numpy(), oracle.corrected_linear_exact(x, m["qweight"], m["qzeros"], m["scales"], 128, R, m["L"], 1.0), "own r")


# ---- the kernel that streams the tiled copy (5..16 token rows, groups whose column tiles fill the chip without K slices) ----
# (M, K, member rows, rank, alpha): one and two K groups per workgroup (K of four super-blocks / eight and more), one to
# three members with a ragged last tile, a member without L, rank 256, a scale on the correction
TILED_CASES = [(8, 1024, [12288, 4608], 64, 1.0), (5, 2048, [16640], 128, 1.0), (12, 1024, [9000, 9000], 32, 2.0),
               (16, 2048, [20000], 256, 1.0), (9, 4096, [8192, 8192, 1000], 128, 0.5)]


def tiled_in_launch(ext) -> bool:
    return re.match(r"skinny_tiled_kernel<\d+,\d+,\d+,1> ", ext.last_launch()["kernel"]) is not None


@pytest.fixture
def tiled_routes(ext):
    """The kernel that streams the tiled copy serves these launches whatever the length of the stream."""
    with tuning(ext, tiled_shape_rule=0):
        yield


@pytest.mark.parametrize("M,K,Ns,rank,alpha", TILED_CASES)
def test_tiled_kernel_computes_r_itself(ext, tiled_routes, M, K, Ns, rank, alpha):
    print(f"case M={M} K={K} Ns={Ns} rank={rank}", flush=True)
    x, members, R = make_group(170 + M + K + rank, M, K, Ns, rank, with_bias=True)
    mem = members_on_device(members, drop_left=1 if len(Ns) > 1 else None, with_bias=True)
    xd, Rd = dev(x), dev(R)
    with tuning(ext, proj_in_launch=0):
        r_two = torch.empty((M, rank), dtype=torch.float16, device="cuda")
        y_two = ext.group_forward(xd, r_two, mem, 128, alpha, R=Rd)
        assert ext.last_launch()["kernel"].startswith("skinny_tiled_kernel<") and not tiled_in_launch(ext), ext.last_launch()
    for rep in range(3):
        r = torch.full((M, rank), float("nan"), dtype=torch.float16, device="cuda")
        y = ext.group_forward(xd, r, mem, 128, alpha, R=Rd)
        assert tiled_in_launch(ext), ext.last_launch()
        torch.cuda.synchronize()
        # the producers in front add an entry of r up like the projection launch, and the correction is applied in the
        # same place: the same bits
        assert torch.equal(r, r_two), f"r, launch {rep}"
        for a, b in zip(y, y_two):
            assert torch.equal(a, b), f"launch {rep}"
    assert_close(r_two.cpu().numpy(), x.astype(np.float64) @ R.astype(np.float64).T, "r")
    for i, (m, got) in enumerate(zip(members, y_two)):
        want = (oracle.linear_exact(x, m["qweight"], m["qzeros"], m["scales"], 128) if mem[i]["L"] is None else
                oracle.corrected_linear_exact(x, m["qweight"], m["qzeros"], m["scales"], 128, R, m["L"], alpha))
        assert_close(got.cpu().numpy(), want + m["bias"].astype(np.float64)[None, :], f"member {i}")


def test_tiled_launches_and_replays_see_their_own_r(ext, tiled_routes):
    """Launch after launch and replay after replay through the same workspace, each with other activations."""
    M, K, Ns, rank = 8, 1024, [16384, 2048], 128
    _, members, R = make_group(181, M, K, Ns, rank)
    mem = members_on_device(members)
    Rd = dev(R)
    g = torch.Generator().manual_seed(19)
    xs = torch.randn(M, K, generator=g).half().cuda()
    r = torch.empty((M, rank), dtype=torch.float16, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ext.group_forward(xs, r, mem, 128, 1.0, R=Rd)
        assert tiled_in_launch(ext), ext.last_launch()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            outs = ext.group_forward(xs, r, mem, 128, 1.0, R=Rd)
            again = ext.group_forward(xs, r, mem, 128, 1.0, R=Rd)
        assert tiled_in_launch(ext)
    torch.cuda.synchronize()
    for rep in range(5):
        xs.copy_(torch.randn(M, K, generator=g).half())
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        xn = xs.cpu().numpy()
        assert_close(r.cpu().numpy(), xn.astype(np.float64) @ R.astype(np.float64).T, f"r, replay {rep}")
        for m, a, b in zip(members, outs, again):
            want = oracle.corrected_linear_exact(xn, m["qweight"], m["qzeros"], m["scales"], 128, R, m["L"], 1.0)
            assert_close(a.cpu().numpy(), want, f"replay {rep}")
            assert torch.equal(a, b), f"replay {rep}: two launches of one replay"


@pytest.mark.parametrize("spin", [None, 0])
def test_tiled_waves_that_never_see_the_ready_word(ext, tiled_routes, spin):
    """With the producers' flags held down (or no patience at all) the waves that stage r for their workgroup compute
    the pieces they would have loaded themselves; the caller still gets r from the producers in front."""
    M, K, Ns, rank = 7, 512, [16640], 64
    x, members, R = make_group(191, M, K, Ns, rank)
    mem = members_on_device(members)
    xd, Rd = dev(x), dev(R)
    knobs = {"proj_in_launch": 2} if spin is None else {"proj_spin_limit": spin}
    with tuning(ext, **knobs):
        r = torch.full((M, rank), float("nan"), dtype=torch.float16, device="cuda")
        y = ext.group_forward(xd, r, mem, 128, 1.0, R=Rd)
        assert tiled_in_launch(ext), ext.last_launch()
        torch.cuda.synchronize()
    assert_close(r.cpu().numpy(), x.astype(np.float64) @ R.astype(np.float64).T, "r")
    for m, got in zip(members, y):
        assert_close(got.cpu().numpy(), oracle.corrected_linear_exact(x, m["qweight"], m["qzeros"], m["scales"], 128, R, m["L"], 1.0), "own r")


def test_tiled_launch_that_leaves_no_room_keeps_the_projection_launch(ext, tiled_routes):
    """Column tiles for every compute unit, K slices through the workspace, more than 16 rows: the projection launch goes
    ahead as before, with the same results."""
    for M, K, Ns, rank in [(8, 512, [40000], 64), (8, 4096, [2048], 64), (24, 1024, [16640], 64)]:
        x, members, R = make_group(201 + M, M, K, Ns, rank)
        mem = members_on_device(members)
        r = torch.full((M, rank), float("nan"), dtype=torch.float16, device="cuda")
        y = ext.group_forward(dev(x), r, mem, 128, 1.0, R=dev(R))
        assert ext.last_launch()["kernel"].startswith("skinny_tiled_kernel<") and not tiled_in_launch(ext), ext.last_launch()
        torch.cuda.synchronize()
        assert_close(r.cpu().numpy(), x.astype(np.float64) @ R.astype(np.float64).T, "r")
        for m, got in zip(members, y):
            assert_close(got.cpu().numpy(), oracle.corrected_linear_exact(x, m["qweight"], m["qzeros"], m["scales"], 128, R, m["L"], 1.0), f"M={M} K={K}")


# ---- three and four token rows: the fused call takes the skinny kernel where its launch computes r itself ------------------
@pytest.mark.parametrize("M,K,Ns,rank", [(4, 4096, [4096, 1024, 1024], 128), (3, 5120, [5120], 256), (3, 4096, [4096], 64)])
def test_three_and_four_rows_take_the_launch_that_computes_r(ext, M, K, Ns, rank):
    print(f"case M={M} K={K} Ns={Ns} rank={rank}", flush=True)
    x, members, R = make_group(270 + M + K + rank, M, K, Ns, rank, with_bias=True)
    mem = members_on_device(members, drop_left=1 if len(Ns) > 1 else None, with_bias=True)
    xd, Rd = dev(x), dev(R)
    with tuning(ext, small_rows_in_launch=0):
        r_two = torch.empty((M, rank), dtype=torch.float16, device="cuda")
        y_two = ext.group_forward(xd, r_two, mem, 128, 1.0, R=Rd)
        assert not skinny_in_launch(ext), ext.last_launch()
    r = torch.full((M, rank), float("nan"), dtype=torch.float16, device="cuda")
    y = ext.group_forward(xd, r, mem, 128, 1.0, R=Rd)
    assert skinny_in_launch(ext), ext.last_launch()
    torch.cuda.synchronize()
    assert_close(r.cpu().numpy(), x.astype(np.float64) @ R.astype(np.float64).T, "r")
    for i, (m, got) in enumerate(zip(members, y)):
        want = (oracle.linear_exact(x, m["qweight"], m["qzeros"], m["scales"], 128) if mem[i]["L"] is None else
                oracle.corrected_linear_exact(x, m["qweight"], m["qzeros"], m["scales"], 128, R, m["L"], 1.0))
        assert_close(got.cpu().numpy(), want + m["bias"].astype(np.float64)[None, :], f"member {i}")
        assert np.abs(got.float().cpu().numpy() - y_two[i].float().cpu().numpy()).max() <= 4e-3 * max(1.0, float(np.abs(want).max()))
