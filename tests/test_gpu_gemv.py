"""GPU parity of the decode route (wave-dot GEMV and the generic route) through the C ABI."""
import numpy as np
import pytest
import torch

import glowq_oracle as oracle
from helpers import assert_close, dev, make_group

pytestmark = pytest.mark.gpu


def _run_single(ext, x, m, gs=128, entry="gemv"):
    fn = ext.w4a16_gemv_forward_cuda if entry == "gemv" else ext.w4a16_gemm_forward_cuda
    args = (dev(x), dev(m["qweight"]), dev(m["scales"]), dev(m["qzeros"]), gs)
    y = fn(*args) if entry == "gemv" else fn(*args, 1)
    torch.cuda.synchronize()
    return y.cpu().numpy()


@pytest.mark.parametrize("M,K,N,gs", [
    (1, 2048, 2048, 128), (1, 4096, 1024, 128), (2, 4096, 512, 128), (3, 1024, 300, 128), (4, 5120, 256, 128),
    (1, 14336, 128, 128), (1, 3584, 130, 128), (1, 4096, 4096, 128), (1, 256, 7, 64), (1, 512, 33, 32),
    (1, 8192, 96, 256), (1, 6144, 70, 128), (1, 16384, 40, 512), (1, 12288, 37, 128),
])
def test_gemv_matches_oracle(ext, small_m_route, M, K, N, gs):
    print(f"case M={M} K={K} N={N} gs={gs}", flush=True)
    x, (m,), _ = make_group(7 + M + K + N, M, K, [N], 0, group_size=gs)
    got = _run_single(ext, x, m, gs)
    want = oracle.linear_exact(x, m["qweight"], m["qzeros"], m["scales"], gs)
    err = assert_close(got, want, f"gemv M={M} K={K} N={N}")
    # and it is at least as close to the exact value as the reference's own fp16 rounding allows
    ref16 = oracle.gemv_ref(x, m["qweight"], m["qzeros"], m["scales"], gs)
    assert err <= np.abs(ref16.astype(np.float64) - want).max() + 2e-3


@pytest.mark.parametrize("M,K,N,gs", [(1, 200, 5, 40), (2, 72, 9, 8), (5, 136, 17, 8), (6, 4096, 64, 128), (9, 1000, 3, 200)])
def test_generic_route_odd_shapes(ext, M, K, N, gs):
    print(f"case M={M} K={K} N={N} gs={gs}", flush=True)
    x, (m,), _ = make_group(100 + K, M, K, [N], 0, group_size=gs)
    got = _run_single(ext, x, m, gs)
    want = oracle.linear_exact(x, m["qweight"], m["qzeros"], m["scales"], gs)
    assert_close(got, want, f"generic M={M} K={K} N={N}")


def test_one_hot_input_selects_dequantised_column(ext, small_m_route):
    """x = e_k makes y[n] = (code - z) * s for column k: every nibble position, exactly (fp16 of an
    exactly representable product of a 5-bit integer and an fp16 is exact when it fits 11 bits)."""
    K, N, gs = 256, 64, 128
    _, (m,), _ = make_group(3, 1, K, [N], 0, group_size=gs)
    deq = oracle.dequant(m["qweight"], m["qzeros"], m["scales"], K, gs)
    for k in list(range(0, 40)) + [127, 128, 255]:
        x = np.zeros((1, K), dtype=np.float16)
        x[0, k] = 1.0
        got = _run_single(ext, x, m, gs)
        np.testing.assert_array_equal(got[0].view(np.uint16), deq[:, k].view(np.uint16), err_msg=f"column {k}")


def test_dequant_and_unpack_exact(ext):
    for (N, K, gs) in [(48, 256, 128), (40, 1152, 128), (5, 200, 40), (3, 72, 8)]:
        _, (m,), _ = make_group(N + K, 1, K, [N], 0, group_size=gs)
        got = ext.dequant(dev(m["qweight"]), dev(m["scales"]), dev(m["qzeros"]), K, gs).cpu().numpy()
        want = oracle.dequant(m["qweight"], m["qzeros"], m["scales"], K, gs)
        np.testing.assert_array_equal(got.view(np.uint16), want.view(np.uint16))
        codes = ext.unpack_int4(dev(m["qweight"]), K).cpu().numpy()
        np.testing.assert_array_equal(codes, oracle.unpack_int4_i32(m["qweight"], K))


def test_golden_module_vectors(ext, small_m_route, golden):
    """The reference's own dequantised weights and CPU forward outputs (tests/golden)."""
    for name in ("m1", "m2"):
        gs = int(golden[f"{name}_gs"][0])
        x = golden[f"{name}_x"]
        qw, qz, sc = golden[f"{name}_qweight"], golden[f"{name}_qzeros"], golden[f"{name}_scales"]
        K = x.shape[1]
        deq = ext.dequant(dev(qw), dev(sc), dev(qz), K, gs).cpu().numpy()
        np.testing.assert_array_equal(deq.view(np.uint16), golden[f"{name}_deq"].view(np.uint16))
        y = ext.w4a16_gemv_forward_cuda(dev(x), dev(qw), dev(sc), dev(qz), gs).cpu().numpy().astype(np.float32)
        if name == "m2":
            y = y + golden["m2_bias"].astype(np.float32)
        want = golden[f"{name}_y"].astype(np.float64)
        assert np.all(np.abs(y - want) <= 1e-2 + 1e-3 * np.abs(want))


def test_group_forward_with_correction(ext, small_m_route):
    for (M, K, Ns, rank, alpha) in [(1, 2048, [256, 128, 128], 64, 1.0), (2, 4096, [512, 96], 128, 0.5),
                                    (1, 4096, [300], 256, 1.0), (4, 1024, [64, 64, 64, 64], 32, 2.0),
                                    (1, 1024, [128, 64], 37, 1.0)]:
        print(f"case M={M} K={K} Ns={Ns} rank={rank}", flush=True)
        x, members, R = make_group(11 + K + rank, M, K, Ns, rank, with_bias=True)
        r = ext.shared_proj(dev(x), dev(R))
        r_ref = oracle.shared_proj(x, R)
        rerr = np.abs(r.cpu().numpy().astype(np.float64) - r_ref.astype(np.float64))
        assert np.all(rerr <= 1e-2 + 1e-3 * np.abs(r_ref.astype(np.float64)))
        mem = [{"qweight": dev(m["qweight"]), "scales": dev(m["scales"]), "qzeros": dev(m["qzeros"]),
                "L": dev(m["L"]), "bias": dev(m["bias"])} for m in members]
        outs = ext.group_forward(dev(x), r, mem, 128, alpha)
        torch.cuda.synchronize()
        for m, y in zip(members, outs):
            want = oracle.corrected_linear_exact(x, m["qweight"], m["qzeros"], m["scales"], 128, R, m["L"], alpha)
            want = want + m["bias"].astype(np.float64)[None, :]
            assert_close(y.cpu().numpy(), want, f"group K={K} rank={rank}")


def test_selective_members_skip_correction(ext, small_m_route):
    """GlowQ-S: a member without L gets exactly the uncorrected result, the others the corrected one."""
    M, K, Ns, rank = 1, 2048, [128, 64, 192], 64
    x, members, R = make_group(5, M, K, Ns, rank)
    r = ext.shared_proj(dev(x), dev(R))
    mem = [{"qweight": dev(m["qweight"]), "scales": dev(m["scales"]), "qzeros": dev(m["qzeros"]),
            "L": dev(m["L"]) if i != 1 else None} for i, m in enumerate(members)]
    outs = ext.group_forward(dev(x), r, mem, 128, 1.0)
    plain = _run_single(ext, x, members[1])
    np.testing.assert_array_equal(outs[1].cpu().numpy().view(np.uint16), plain.view(np.uint16))
    want0 = oracle.corrected_linear_exact(x, members[0]["qweight"], members[0]["qzeros"], members[0]["scales"], 128, R, members[0]["L"], 1.0)
    assert_close(outs[0].cpu().numpy(), want0, "selected member")
    # alpha = 0 switches the correction off for every member
    outs0 = ext.group_forward(dev(x), r, mem, 128, 0.0)
    plain0 = _run_single(ext, x, members[0])
    np.testing.assert_array_equal(outs0[0].cpu().numpy().view(np.uint16), plain0.view(np.uint16))


# ---------------------------------------------------------------- side streams of the single-token GEMV
def _unpack_side(side, N, K, gs, rank):
    """Host reading of a side stream following its layout description (csrc/side_stream.hpp): per row block of two rows
    and lane, np scale/zero-point dwords then 2 lw dwords of L, in lane-major chunks of four dwords."""
    U = K // 32
    kit = -(-U // 64)
    np_, lw = (kit + 1) // 2, (rank + 127) // 128
    D = np_ + 2 * lw
    upg = (gs // 32).bit_length() - 1
    G = -(-U // (1 << upg))
    blocks = (N + 1) // 2
    raw = side.cpu().numpy().view(np.uint32).reshape(blocks, 64 * D)
    dw = np.zeros((blocks, 64, D), dtype=np.uint32)
    for d in range(D):
        c = d // 4
        size = min(4, D - 4 * c)
        for lane in range(64):
            dw[:, lane, d] = raw[:, (1024 * c + lane * 4 * size + 4 * (d % 4)) // 4]
    return dw, np_, lw, upg, G


@pytest.mark.parametrize("N,K,gs,rank,with_L", [(64, 4096, 128, 128, True), (33, 4096, 128, 128, True), (40, 14336, 128, 128, True),
                                                (24, 5120, 128, 256, True), (16, 8192, 256, 64, True), (10, 4096, 128, 0, False),
                                                (12, 2048, 128, 128, False), (8, 17408, 128, 0, False)])
def test_side_stream_holds_exactly_the_canonical_values(ext, N, K, gs, rank, with_L):
    _, (m,), _ = make_group(N + K, 1, K, [N], rank if with_L else 0, group_size=gs)
    L = dev(m["L"]) if with_L else None
    side = ext.pack_side(dev(m["scales"]), dev(m["qzeros"]), L, K, gs, rank)
    assert side is not None and side.numel() == ext.lib.glowq_side_bytes(N, K, gs, rank)
    dw, np_, lw, upg, G = _unpack_side(side, N, K, gs, rank)
    _, zeros, scales, _ = oracle.codes_and_params(m["qweight"], m["qzeros"], m["scales"], K, gs)
    for b in range((N + 1) // 2):
        for lane in range(64):
            row = 2 * b + lane // 32
            for p in range(np_):
                g = min(((128 * p) >> upg) + lane % 32, G - 1)
                want = (int(scales[row, g].view(np.uint16)) | (int(zeros[row, g]) << 16)) if row < N else 0
                assert int(dw[b, lane, p]) == want, (b, lane, p)
            for j in range(lw):
                for rr in range(2):
                    row, i = 2 * b + rr, lane + 64 * j
                    want = 0
                    if with_L and row < N and i < rank // 2:
                        want = int(m["L"][row, 2 * i:2 * i + 2].view(np.uint32)[0])
                    assert int(dw[b, lane, np_ + 2 * j + rr]) == want, (b, lane, j, rr)


@pytest.mark.parametrize("K,Ns,rank", [(4096, [256, 64, 33], 128), (14336, [96], 128), (5120, [64, 64], 256), (2048, [40], 64),
                                       (8192, [48], 0), (17408, [32], 0)])
def test_single_token_launch_reads_the_same_values_through_side_streams(ext, K, Ns, rank):
    print(f"case K={K} Ns={Ns} rank={rank}", flush=True)
    x, members, R = make_group(3 + K + rank, 1, K, Ns, rank, with_bias=True)
    base = [{"qweight": dev(m["qweight"]), "scales": dev(m["scales"]), "qzeros": dev(m["qzeros"]),
             "L": dev(m["L"]) if rank else None, "bias": dev(m["bias"])} for m in members]
    if rank:
        base[-1]["L"] = None                      # one member of the corrected group without its own L
    xd = dev(x)
    r = ext.shared_proj(xd, dev(R)) if rank else None
    plain = ext.group_forward(xd, r, base, 128, 0.5)
    packed = [dict(m, side=(ext.pack_side(m["scales"], m["qzeros"], m["L"], K, 128, rank), rank)) for m in base]
    assert all(m["side"][0] is not None for m in packed)
    with_side = ext.group_forward(xd, r, packed, 128, 0.5)
    torch.cuda.synchronize()
    for a, b, m in zip(plain, with_side, members):
        assert torch.equal(a, b)
    # and both are right
    for y, m, bm in zip(with_side, members, base):
        want = (oracle.corrected_linear_exact(x, m["qweight"], m["qzeros"], m["scales"], 128, R, m["L"], 0.5) if bm["L"] is not None
                else oracle.linear_exact(x, m["qweight"], m["qzeros"], m["scales"], 128)) + m["bias"].astype(np.float64)[None, :]
        assert_close(y.cpu().numpy(), want, f"side stream K={K}")
    # a stream packed for another rank than the launch applies is ignored, not misread
    other = rank + 2                              # neither the rank of this launch nor 0
    wrong = [dict(m, side=(torch.full_like(p["side"][0], 0x5A), other)) for m, p in zip(base, packed)]
    for a, b in zip(plain, ext.group_forward(xd, r, wrong, 128, 0.5)):
        assert torch.equal(a, b)
    # the prepared group builds its own streams and gives the same bits
    from glowq_amd.kernels import PreparedGroup
    pg = PreparedGroup(ext, base, K, 128, 0.5, R=dev(R) if rank else None, side_streams=True)
    assert all(k[5] is not None for k in pg.keep)
    for a, b in zip(plain, pg.run(xd)):
        assert torch.equal(a, b)
