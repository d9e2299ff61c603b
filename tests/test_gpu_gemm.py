"""GPU parity of the MFMA GEMM route (large M) and of the shared projection, through the C ABI."""
import numpy as np
import pytest
import torch

import glowq_oracle as oracle
from helpers import assert_close, dev, make_group, tuning

pytestmark = pytest.mark.gpu


def test_identity_input_reproduces_dequantised_weight_exactly(ext):
    """x = I_K: y[m, n] = fp16((code - zero) * scale) of weight element [n, m], so the in-kernel
    dequantisation (every nibble position, zero-point and scale path) is checked bit for bit."""
    K, N, gs = 256, 320, 128
    _, (m,), _ = make_group(21, 1, K, [N], 0, group_size=gs)
    x = np.eye(K, dtype=np.float16)
    y = ext.w4a16_gemm_forward_cuda(dev(x), dev(m["qweight"]), dev(m["scales"]), dev(m["qzeros"]), gs, 1).cpu().numpy()
    want = oracle.dequant(m["qweight"], m["qzeros"], m["scales"], K, gs).T
    np.testing.assert_array_equal(y.view(np.uint16), np.ascontiguousarray(want).view(np.uint16))


@pytest.mark.parametrize("M,K,N,gs", [
    (256, 512, 256, 128), (200, 1024, 300, 128), (33, 256, 64, 64), (2048, 1024, 512, 128), (129, 2048, 1000, 128),
    (64, 3584, 512, 128), (17, 512, 1024, 32),
])
def test_gemm_matches_oracle(ext, M, K, N, gs):
    print(f"case M={M} K={K} N={N} gs={gs}", flush=True)
    x, (m,), _ = make_group(31 + M + N, M, K, [N], 0, group_size=gs)
    y = ext.w4a16_gemm_forward_cuda(dev(x), dev(m["qweight"]), dev(m["scales"]), dev(m["qzeros"]), gs, 1)
    torch.cuda.synchronize()
    # yardstick: the reference's GEMM semantics (weights rounded to fp16 once) in float64
    w = oracle.dequant(m["qweight"], m["qzeros"], m["scales"], K, gs).astype(np.float64)
    want = x.astype(np.float64) @ w.T
    assert_close(y.cpu().numpy(), want, f"gemm M={M} K={K} N={N}")


def test_gemm_route_falls_back_on_odd_shapes(ext):
    M, K, N, gs = 70, 200, 37, 40
    x, (m,), _ = make_group(77, M, K, [N], 0, group_size=gs)
    y = ext.w4a16_gemm_forward_cuda(dev(x), dev(m["qweight"]), dev(m["scales"]), dev(m["qzeros"]), gs, 1)
    want = oracle.linear_exact(x, m["qweight"], m["qzeros"], m["scales"], gs)
    assert_close(y.cpu().numpy(), want, "generic from gemm entry")


@pytest.mark.parametrize("M,K,rank", [(1, 2048, 64), (3, 4096, 128), (8, 1024, 256), (300, 1024, 128), (2048, 512, 64),
                                      (70, 3584, 256), (5, 200, 24), (64, 17408, 256), (17, 4096, 128), (100, 14336, 40),
                                      (33, 5184, 96), (512, 4160, 128)])
def test_shared_proj(ext, M, K, rank):
    g = torch.Generator().manual_seed(M + K + rank)
    x = torch.randn(M, K, generator=g).half().numpy()
    R = (torch.randn(rank, K, generator=g) * K ** -0.5).half().numpy()
    r = ext.shared_proj(dev(x), dev(R)).cpu().numpy()
    want = x.astype(np.float64) @ R.astype(np.float64).T
    assert_close(r, want, f"shared_proj M={M}")


@pytest.mark.parametrize("M,K,Ns,rank,alpha", [(256, 1024, [256, 128], 128, 1.0), (100, 512, [300], 64, 0.5),
                                               (40, 1024, [128, 128, 64], 128, 1.0), (16, 2048, [256], 64, 1.0)])
def test_group_forward_large_m(ext, M, K, Ns, rank, alpha):
    """Rows above the GEMV capacity: MFMA route with the correction as a K-extension."""
    print(f"case M={M} K={K} Ns={Ns} rank={rank}", flush=True)
    x, members, R = make_group(57 + M, M, K, Ns, rank, with_bias=True)
    r = ext.shared_proj(dev(x), dev(R))
    mem = [{"qweight": dev(m["qweight"]), "scales": dev(m["scales"]), "qzeros": dev(m["qzeros"]),
            "L": dev(m["L"]) if i != 1 else None, "bias": dev(m["bias"])} for i, m in enumerate(members)]
    outs = ext.group_forward(dev(x), r, mem, 128, alpha)
    torch.cuda.synchronize()
    for i, (m, y) in enumerate(zip(members, outs)):
        if i == 1:
            want = oracle.linear_exact(x, m["qweight"], m["qzeros"], m["scales"], 128)
        else:
            want = oracle.corrected_linear_exact(x, m["qweight"], m["qzeros"], m["scales"], 128, R, m["L"], alpha)
        want = want + m["bias"].astype(np.float64)[None, :]
        assert_close(y.cpu().numpy(), want, f"group large M member {i}")


# ---------------------------------------------------------------- skinny MFMA route (5 <= M <= 64)
@pytest.mark.parametrize("M,K,N,gs", [(5, 512, 64, 128), (8, 4096, 1024, 128), (16, 1024, 300, 128), (32, 2048, 96, 64),
                                      (33, 1024, 200, 128), (64, 14336, 128, 128), (64, 64, 32, 32), (7, 192, 40, 64),
                                      (8, 2816, 200, 128), (24, 5632, 96, 128), (16, 18944, 64, 128), (40, 2304, 72, 128)])
def test_skinny_route_matches_oracle(ext, small_m_route, M, K, N, gs):
    print(f"case M={M} K={K} N={N} gs={gs}", flush=True)
    if small_m_route not in ("stream", "qstream"):  # those modes leave the limits of the other kernels at their defaults
        assert ext.lib.glowq_w4a16_route(M, K, N, gs, K // 8) in ((4,) if small_m_route == "quad" and M <= 16 else (1, 7))
    x, (m,), _ = make_group(41 + M + N, M, K, [N], 0, group_size=gs)
    with tuning(ext, tiled_max_m=0):  # (above 32 rows the kernel that streams the tiled copy would take over)
        y = ext.w4a16_gemv_forward_cuda(dev(x), dev(m["qweight"]), dev(m["scales"]), dev(m["qzeros"]), gs)
        torch.cuda.synchronize()
    w = oracle.dequant(m["qweight"], m["qzeros"], m["scales"], K, gs).astype(np.float64)
    assert_close(y.cpu().numpy(), x.astype(np.float64) @ w.T, f"skinny M={M} K={K} N={N}")


@pytest.mark.parametrize("M,K,Ns,rank", [(8, 14336, [256, 64], 128), (16, 14336, [4096], 128), (33, 14336, [128], 64),
                                         (64, 12288, [96], 128), (5, 18432, [40, 300], 0)])
def test_skinny_split_k_through_workspace(ext, M, K, Ns, rank):
    """Few column tiles and a long K: the skinny kernel cuts K into slices through the workspace (the correction rides
    on the first slice only) and a second launch adds them up; without a workspace the same call runs unsplit."""
    print(f"case M={M} K={K} Ns={Ns} rank={rank}", flush=True)
    assert ext.lib.glowq_w4a16_route(M, K, sum(Ns), 128, K // 8) in (1, 7)  # 7: the raw-code form, up to eight rows
    x, members, R = make_group(733 + M, M, K, Ns, rank, with_bias=True)
    mem = [{"qweight": dev(m["qweight"]), "scales": dev(m["scales"]), "qzeros": dev(m["qzeros"]),
            "L": dev(m["L"]) if rank else None, "bias": dev(m["bias"])} for m in members]
    want = [(oracle.corrected_linear_exact(x, m["qweight"], m["qzeros"], m["scales"], 128, R, m["L"], 0.5) if rank else
             oracle.linear_exact(x, m["qweight"], m["qzeros"], m["scales"], 128)) + m["bias"].astype(np.float64)[None, :] for m in members]
    r = torch.empty(M, rank, dtype=torch.float16, device="cuda") if rank else None
    old_tiled = ext.set_tuning("tiled_max_m", 0)  # (above 32 rows the kernel that streams the tiled copy would take over)
    outs = ext.group_forward(dev(x), r, mem, 128, 0.5, R=dev(R) if rank else None)
    torch.cuda.synchronize()
    for i, (w, y) in enumerate(zip(want, outs)):
        assert_close(y.cpu().numpy(), w, f"split skinny member {i}")
    saved = ext.WORKSPACE_BYTES, dict(ext._workspaces)
    try:
        ext.WORKSPACE_BYTES = 64  # too small for a single slice: the call must fall back to the unsplit launch
        ext._workspaces.clear()
        outs2 = ext.group_forward(dev(x), r, mem, 128, 0.5, R=dev(R) if rank else None)
        torch.cuda.synchronize()
        for i, (w, y) in enumerate(zip(want, outs2)):
            assert_close(y.cpu().numpy(), w, f"unsplit skinny member {i}")
    finally:
        ext.set_tuning("tiled_max_m", old_tiled)
        ext.WORKSPACE_BYTES = saved[0]
        ext._workspaces.clear()
        ext._workspaces.update(saved[1])


@pytest.mark.parametrize("mode", ["default", "stream", "neither"])
@pytest.mark.parametrize("M,K,Ns,rank", [(3, 4096, [512, 128, 128], 128), (4, 2048, [300], 64), (4, 5632, [96, 40], 128), (2, 4096, [256], 128)])
def test_small_groups_at_two_to_four_rows(ext, mode, M, K, Ns, rank):
    """Default route limits: a small group at two to four rows runs on the stream-scheduled 4x4x4 matrix-core GEMV; with
    that one switched off on the stream GEMV; with both off, at three or four rows on the skinny MFMA kernel and at two
    rows on the wave-dot GEMV.  All against the oracle, with the shared correction."""
    print(f"case M={M} K={K} Ns={Ns} rank={rank} mode={mode}", flush=True)
    old = {}
    if mode != "default":
        old["qstream_max_m"] = ext.set_tuning("qstream_max_m", 0)
    if mode == "neither":
        old["stream_max_m"] = ext.set_tuning("stream_max_m", 0)
    try:
        # (skinny kernel: 7 is its raw-code form, taken where whole 256-column super-blocks allow it)
        want = {"default": (6,), "stream": (5,), "neither": (0,) if M == 2 else (1, 7)}[mode]
        assert ext.lib.glowq_w4a16_route(M, K, sum(Ns), 128, K // 8) in want
        _small_group_case(ext, M, K, Ns, rank)
    finally:
        for key, value in old.items():
            ext.set_tuning(key, value)


def _small_group_case(ext, M, K, Ns, rank):
    x, members, R = make_group(311 + M + K, M, K, Ns, rank, with_bias=True)
    r = torch.empty(M, rank, dtype=torch.float16, device="cuda")
    mem = [{"qweight": dev(m["qweight"]), "scales": dev(m["scales"]), "qzeros": dev(m["qzeros"]), "L": dev(m["L"]),
            "bias": dev(m["bias"])} for m in members]
    outs = ext.group_forward(dev(x), r, mem, 128, 1.0, R=dev(R))
    torch.cuda.synchronize()
    for i, (m, y) in enumerate(zip(members, outs)):
        want = oracle.corrected_linear_exact(x, m["qweight"], m["qzeros"], m["scales"], 128, R, m["L"], 1.0)
        assert_close(y.cpu().numpy(), want + m["bias"].astype(np.float64)[None, :], f"small group member {i} at M={M}")


@pytest.mark.parametrize("K,k0s", [(256, (0, 64, 192)), (2816, (0, 192, 832, 1728, 2048, 2560, 2752)),
                                   (19456, (0, 2304, 4864, 9984, 19392))])
def test_skinny_identity_block_is_exact(ext, small_m_route, K, k0s):
    """64 rows of the identity select 64 weight columns: the in-register dequantisation, the activation permutation
    and the choice of every super-block's scale and zero-point in the skinny kernel, bit for bit.  The longer rows have
    scales and zero-points fetched in runs of eight super-blocks, with runs that start off a multiple of four."""
    N, gs = 96, 128
    _, (m,), _ = make_group(23, 1, K, [N], 0, group_size=gs)
    want = oracle.dequant(m["qweight"], m["qzeros"], m["scales"], K, gs)
    for k0 in k0s:
        x = np.zeros((64, K), dtype=np.float16)
        x[np.arange(64), k0 + np.arange(64)] = 1.0
        y = ext.w4a16_gemv_forward_cuda(dev(x), dev(m["qweight"]), dev(m["scales"]), dev(m["qzeros"]), gs).cpu().numpy()
        np.testing.assert_array_equal(y.view(np.uint16), np.ascontiguousarray(want[:, k0:k0 + 64].T).view(np.uint16))


@pytest.mark.parametrize("M,K,Ns,rank,alpha", [(8, 4096, [512, 128, 128], 128, 1.0), (16, 1024, [96, 200], 64, 0.5),
                                               (64, 2048, [256], 256, 1.0), (12, 512, [64, 64, 64, 64], 64, 2.0)])
def test_skinny_group_with_correction(ext, small_m_route, M, K, Ns, rank, alpha):
    print(f"case M={M} K={K} Ns={Ns} rank={rank}", flush=True)
    x, members, R = make_group(67 + M, M, K, Ns, rank, with_bias=True)
    r = torch.empty(M, rank, dtype=torch.float16, device="cuda")
    mem = [{"qweight": dev(m["qweight"]), "scales": dev(m["scales"]), "qzeros": dev(m["qzeros"]),
            "L": dev(m["L"]) if i != 1 else None, "bias": dev(m["bias"])} for i, m in enumerate(members)]
    outs = ext.group_forward(dev(x), r, mem, 128, alpha, R=dev(R))
    torch.cuda.synchronize()
    for i, (m, y) in enumerate(zip(members, outs)):
        if i == 1:
            want = oracle.linear_exact(x, m["qweight"], m["qzeros"], m["scales"], 128)
        else:
            want = oracle.corrected_linear_exact(x, m["qweight"], m["qzeros"], m["scales"], 128, R, m["L"], alpha)
        assert_close(y.cpu().numpy(), want + m["bias"].astype(np.float64)[None, :], f"skinny group member {i}")


@pytest.mark.parametrize("M,K,rank", [(64, 14336, 128), (40, 8192, 256), (17, 17408, 256), (130, 18944, 64)])
def test_shared_proj_split_workspace(ext, M, K, rank):
    """Many-row projection with K split over workgroups through a workspace of any contents: same values on every call
    (the partials are added in slice order), smaller workspaces split less, none not at all."""
    g = torch.Generator().manual_seed(M + K + rank)
    x = torch.randn(M, K, generator=g).half()
    R = (torch.randn(rank, K, generator=g) * K ** -0.5).half()
    want = x.numpy().astype(np.float64) @ R.numpy().astype(np.float64).T
    xd, Rd = dev(x.numpy()), dev(R.numpy())
    full = int(ext.lib.glowq_proj_workspace_bytes(M, K, rank))
    assert full > 0
    results = []
    for nbytes in (full, full, full // 3, 2 * 4096 * 4, 0):
        print(f"M={M} K={K} rank={rank} workspace={nbytes}", flush=True)
        ws = torch.full((max(nbytes, 16),), 0xFF, dtype=torch.uint8, device="cuda")  # NaN patterns
        out = torch.full((M, rank), float("nan"), dtype=torch.float16, device="cuda")
        for _ in range(3):  # the same workspace again and again
            rc = ext.lib.glowq_shared_proj_ws(xd.data_ptr(), Rd.data_ptr(), out.data_ptr(), M, K, rank,
                                              ws.data_ptr() if nbytes else None, nbytes, torch.cuda.current_stream().cuda_stream)
            assert rc == 0, ext.lib.glowq_last_error()
            torch.cuda.synchronize()
            assert_close(out.cpu().numpy(), want, f"shared_proj_ws {nbytes} bytes")
            results.append((nbytes, out.clone()))
    first = results[0][1]
    for nbytes, out in results[1:6]:
        assert torch.equal(out, first), "same workspace size, different result"


@pytest.mark.parametrize("M,K,Ns,rank", [(512, 16384, [2048], 64), (1024, 8192, [2048, 1024], 128), (300, 17408, [2000], 0),
                                         (128, 14336, [4096], 128)])
def test_gemm_split_k_through_workspace(ext, M, K, Ns, rank):
    """Tiled GEMM with K split over workgroups (few output tiles, long K): against the oracle, the same bits on every
    call, and with workspaces that hold fewer slices or none."""
    x, members, R = make_group(5 + M + K, M, K, Ns, rank, with_bias=True)
    xd = dev(x)
    mem = [{"qweight": dev(m["qweight"]), "scales": dev(m["scales"]), "qzeros": dev(m["qzeros"]),
            "L": dev(m["L"]) if rank else None, "bias": dev(m["bias"])} for m in members]
    if rank:
        r = ext.shared_proj(xd, dev(R))
        want = [oracle.corrected_linear_exact(x, m["qweight"], m["qzeros"], m["scales"], 128, R, m["L"], 1.0) for m in members]
    else:
        r = None
        want = [oracle.linear_exact(x, m["qweight"], m["qzeros"], m["scales"], 128) for m in members]
    want = [w + m["bias"].astype(np.float64)[None, :] for w, m in zip(want, members)]
    slice_bytes = 4 * ((M + 127) // 128 * 128) * sum((N + 255) // 256 * 256 for N in Ns)
    seen = {}
    for nbytes in (64 << 20, 64 << 20, 2 * slice_bytes, slice_bytes, 0):
        print(f"M={M} K={K} Ns={Ns} rank={rank} workspace={nbytes}", flush=True)
        ext.WORKSPACE_BYTES = max(nbytes, 16)
        ext._workspaces.clear()
        outs = ext.group_forward(xd, r, mem, 128, 1.0)
        torch.cuda.synchronize()
        for i, y in enumerate(outs):
            assert_close(y.cpu().numpy(), want[i], f"member {i}, workspace {nbytes}")
        if nbytes in seen:
            for a, b in zip(outs, seen[nbytes]):
                assert torch.equal(a, b), "same workspace size, different bits"
        seen[nbytes] = [o.clone() for o in outs]
    ext.WORKSPACE_BYTES = 64 << 20
    ext._workspaces.clear()


@pytest.mark.parametrize("M,K,Ns,rank", [(384, 2048, [16384, 5120, 1024], 64), (200, 1024, [40000], 0), (2048, 3584, [3584, 512, 512], 128)])
def test_gemm_tail_tiles_split_along_k(ext, M, K, Ns, rank):
    """More output tiles than CUs, with a partly filled last round: the tiles of that round are cut along K (partials in
    the workspace, summed by a second launch).  Sampled rows and the columns of the first and of the last tiles of every
    member against the oracle; the same bits on a second call; and the unsplit launch (no workspace) within tolerance."""
    print(f"case M={M} K={K} Ns={Ns} rank={rank}", flush=True)
    g = torch.Generator().manual_seed(M + K)
    x = torch.randn(M, K, generator=g).half().numpy()
    R = (torch.randn(rank, K, generator=g) * K ** -0.5).half().numpy() if rank else None
    rows = np.unique(np.concatenate([[0, M - 1], np.random.default_rng(M).integers(0, M, 6)]))
    mem, checks = [], []
    for N in Ns:
        w = (torch.randn(N, K, generator=g) * 0.02).half().numpy()
        qw, qz, sc, _ = oracle.quantize_per_group_w4(w, 128)
        L = (torch.randn(N, rank, generator=g) * 0.01).half().numpy() if rank else None
        bias = (torch.randn(N, generator=g) * 0.1).half().numpy()
        mem.append({"qweight": dev(qw), "scales": dev(sc), "qzeros": dev(qz), "L": dev(L) if rank else None, "bias": dev(bias)})
        cols = np.unique(np.concatenate([np.arange(0, min(N, 300)), np.arange(max(0, N - 600), N)]))
        xs = x[rows]
        if rank:
            want = oracle.corrected_linear_exact(xs, qw[cols], qz[cols], sc[cols], 128, R, L[cols], 1.0)
        else:
            want = oracle.linear_exact(xs, qw[cols], qz[cols], sc[cols], 128)
        checks.append((cols, want + bias[cols].astype(np.float64)[None, :]))
    xd = dev(x)
    r = ext.shared_proj(xd, dev(R)) if rank else None
    outs = ext.group_forward(xd, r, mem, 128, 1.0)
    torch.cuda.synchronize()
    for i, (y, (cols, want)) in enumerate(zip(outs, checks)):
        assert_close(y.cpu().numpy()[np.ix_(rows, cols)], want, f"member {i}")
    again = ext.group_forward(xd, r, mem, 128, 1.0)
    torch.cuda.synchronize()
    assert all(torch.equal(a, b) for a, b in zip(outs, again))
    saved = ext.WORKSPACE_BYTES, dict(ext._workspaces)
    try:
        ext.WORKSPACE_BYTES = 16
        ext._workspaces.clear()
        plain = ext.group_forward(xd, r, mem, 128, 1.0)
        torch.cuda.synchronize()
        for i, (y, (cols, want)) in enumerate(zip(plain, checks)):
            assert_close(y.cpu().numpy()[np.ix_(rows, cols)], want, f"member {i} without a workspace")
    finally:
        ext.WORKSPACE_BYTES = saved[0]
        ext._workspaces.clear()
        ext._workspaces.update(saved[1])
