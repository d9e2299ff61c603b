"""The tiled copy of a member's weights (glowq_pack_tiled / glowq_pack_tiled_left) and the matrix-core kernel that streams
it at 5..64 token rows, through the C ABI: the copy holds exactly the canonical codes, scales and zero-points in the
documented order (checked by undoing the order in numpy), and the kernel's outputs match the oracle's unrounded value
(the arithmetic of the reference's GEMV, src/cuda_w4a16/csrc/gemv_w4a16.cu:96-112, which it uses up to 128 token rows, with
the correction of src/step3_eval_dataset.py:484-511)."""
import numpy as np
import pytest
import torch

import glowq_oracle as oracle
from helpers import assert_close, dev, make_group

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def every_shape_on_the_tiled_route(ext):
    """The library sends short streams to the skinny kernel; these tests want the tiled kernel on small shapes."""
    old = ext.set_tuning("tiled_shape_rule", 0)
    yield
    ext.set_tuning("tiled_shape_rule", old)


def _untile_weights(blob, N, K):
    """Inverse of the tiled order, written from its definition: chunk (rb, sb), the (sb * RB + rb)-th of 4352 bytes, = 4 x 1024 bytes of codes
    (piece j = 2 g + p of lane l = 32 h + c is bytes [64 g + 32 h + 16 p, +16) of the 128-byte segment sb of row
    32 rb + c, nibbles re-ordered inside every word) + per row c the pair (g = 0, 1) of side words: scale bits | fp16(-zero * 2^-16) << 16 of the half's group."""
    SB, RB = K // 256, (N + 31) // 32
    b = blob.reshape(SB, RB, 4352).transpose(1, 0, 2)               # [rb, sb, byte]
    codes = b[:, :, :4096].reshape(RB, SB, 2, 2, 2, 32, 16)          # [rb, sb, g, p, h, c, byte]
    rows = codes.transpose(0, 5, 1, 2, 4, 3, 6).reshape(RB * 32, SB * 128)  # [rb, c, sb, g, h, p, byte] -> row bytes
    side = b[:, :, 4096:].copy().view(np.uint32).reshape(RB, SB, 32, 2)   # [rb, sb, c, g]
    side = side.transpose(0, 2, 1, 3).reshape(RB * 32, SB * 2)            # [row, 128-column half]
    scales = (side & 0xFFFF).astype(np.uint16).view(np.float16)
    zl = (side >> 16).astype(np.uint16).view(np.float16).astype(np.float64)
    # inside a word the code of column k sits in nibble (0,4,1,5,2,6,3,7)[k]
    words = rows.copy().view(np.uint32)
    canon = np.zeros_like(words)
    for k, at in enumerate((0, 4, 1, 5, 2, 6, 3, 7)):
        canon |= ((words >> np.uint32(4 * at)) & np.uint32(0xF)) << np.uint32(4 * k)
    return canon.view(np.int32), scales, (-zl * 65536.0).astype(np.float32)


@pytest.mark.parametrize("N,K,gs", [(64, 512, 128), (40, 1024, 128), (130, 768, 256), (7, 256, 128)])
def test_tiled_weights_hold_the_canonical_buffers(ext, N, K, gs):
    _, (m,), _ = make_group(N + K, 1, K, [N], 0, group_size=gs)
    t = ext.pack_tiled(dev(m["qweight"]), dev(m["scales"]), dev(m["qzeros"]), K, gs)
    assert t is not None and t.numel() == ext.lib.glowq_tiled_bytes(N, K, gs) == ((N + 31) // 32) * (K // 256) * 4352
    qw, sc, z = _untile_weights(t.cpu().numpy(), N, K)
    np.testing.assert_array_equal(qw[:N], m["qweight"])
    assert not qw[N:].any()                                           # rows past N: zero codes
    codes, zeros, scales = oracle.codes_and_params(m["qweight"], m["qzeros"], m["scales"], K, gs)[:3]
    per_half = (np.arange(K // 128) * 128) // gs                      # group of every 128-column half
    np.testing.assert_array_equal(sc[:N].view(np.uint16), np.asarray(scales)[:, per_half].astype(np.float16).view(np.uint16))
    np.testing.assert_array_equal(z[:N], np.asarray(zeros)[:, per_half].astype(np.float32))
    assert not sc[N:].any() and not z[N:].any()


def test_tiled_layout_is_refused_where_it_does_not_apply(ext):
    assert ext.lib.glowq_tiled_bytes(64, 4096 + 128, 128) == 0 and ext.lib.glowq_tiled_bytes(64, 4096, 64) == 0
    assert ext.lib.glowq_tiled_bytes(64, 4096, 96) == 0 and ext.lib.glowq_tiled_left_bytes(64, 12) == 0
    _, (m,), _ = make_group(1, 1, 384, [16], 0, group_size=128)
    assert ext.pack_tiled(dev(m["qweight"]), dev(m["scales"]), dev(m["qzeros"]), 384, 128) is None


@pytest.mark.parametrize("N,rank", [(64, 64), (40, 72), (33, 8), (100, 256)])
def test_tiled_left_factor_holds_L(ext, N, rank):
    L = (torch.randn(N, rank, generator=torch.Generator().manual_seed(N + rank)) * 0.01).half()
    t = ext.pack_tiled_left(L.cuda()).cpu().numpy()
    LB, RB = (rank + 63) // 64, (N + 31) // 32
    # chunk (rb, jb): piece t of lane 32 h + c = L[32 rb + c, 64 jb + 32 h + 8 t + (0..7)], the elements 2, 3, 6, 7 times 16
    b = t.view(np.float16).reshape(RB, LB, 4, 2, 32, 8).copy()        # [rb, jb, t, h, c, e]
    b[..., [2, 3, 6, 7]] /= np.float16(16)
    full = b.transpose(0, 4, 1, 3, 2, 5).reshape(RB * 32, LB * 64)    # [rb, c, jb, h, t, e]
    np.testing.assert_array_equal(full[:N, :rank].view(np.uint16), L.numpy().view(np.uint16))
    assert not full[N:].any() and not full[:, rank:].any()


CASES = [
    # M, K, Ns, rank, gs, alpha, bias, member without L
    (5, 256, [32], 0, 128, 1.0, False, None),
    (8, 512, [64, 40], 64, 128, 1.0, True, None),
    (7, 4096, [300], 128, 128, 0.5, False, None),
    (13, 1024, [128, 64, 96], 72, 128, 1.0, True, 1),
    (16, 2048, [256], 256, 128, 1.0, False, None),
    (17, 768, [130, 31], 8, 256, 2.0, True, None),
    (24, 4096, [512, 128], 128, 128, 1.0, False, 0),
    (32, 1280, [257], 320, 128, 1.0, True, None),
    (33, 512, [64, 64, 64, 64], 64, 128, 1.0, False, None),
    (40, 2560, [384], 128, 128, 1.0, True, None),
    (64, 1024, [200, 56], 128, 512, 1.0, False, None),
    (64, 14336, [160], 128, 128, 1.0, False, None),
    (9, 17408, [96], 256, 128, 1.0, False, None),
]


@pytest.mark.parametrize("M,K,Ns,rank,gs,alpha,bias,bare", CASES)
def test_tiled_kernel_matches_oracle(ext, M, K, Ns, rank, gs, alpha, bias, bare):
    print(f"case M={M} K={K} Ns={Ns} rank={rank} gs={gs}", flush=True)
    x, members, R = make_group(31 + M + K + rank, M, K, Ns, rank, group_size=gs, with_bias=bias)
    mem = [{"qweight": dev(m["qweight"]), "scales": dev(m["scales"]), "qzeros": dev(m["qzeros"]),
            "L": dev(m["L"]) if rank and i != bare else None, "bias": dev(m["bias"]) if bias else None}
           for i, m in enumerate(members)]
    assert ext.route(M, K, sum(Ns), gs, tiled=True) == "skinny_tiled_mfma"
    r = ext.shared_proj(dev(x), dev(R)) if rank else None
    outs = ext.group_forward(dev(x), r, mem, gs, alpha)
    torch.cuda.synchronize()
    assert all(hasattr(m["qweight"], "_glowq_tiled") for m in mem)    # the call built and used the tiled copies
    for i, (m, y) in enumerate(zip(members, outs)):
        if rank and i != bare:
            want = oracle.corrected_linear_exact(x, m["qweight"], m["qzeros"], m["scales"], gs, R, m["L"], alpha)
        else:
            want = oracle.linear_exact(x, m["qweight"], m["qzeros"], m["scales"], gs)
        if bias:
            want = want + m["bias"].astype(np.float64)[None, :]
        assert_close(y.cpu().numpy(), want, f"tiled member {i} M={M} K={K}")


def test_tiled_kernel_is_exact_on_integer_inputs(ext):
    """x in {-2..2}, scales powers of two: every product and sum is exact in fp32 and fits fp16, so the kernel must give
    the integer arithmetic's result bit for bit -- with and without the split of K through the workspace."""
    rng = np.random.default_rng(5)
    M, K, N, gs = 24, 3072, 96, 128
    x = rng.integers(-2, 3, (M, K)).astype(np.float16)
    codes = rng.integers(0, 16, (N, K)).astype(np.uint8)
    zeros = rng.integers(0, 16, (N, K // gs)).astype(np.uint8)
    scales = (2.0 ** rng.integers(-6, -3, (N, K // gs))).astype(np.float16)
    qw = oracle.pack_int4_to_int32(codes.reshape(N, K // 8, 8))
    zfull = np.full((N, 8 * ((K // gs + 7) // 8)), 8, dtype=np.uint8)
    zfull[:, :K // gs] = zeros
    qz = oracle.pack_int4_to_int32(zfull.reshape(N, -1, 8))
    want = (x.astype(np.float64) @ ((codes.astype(np.float64) - np.repeat(zeros, gs, axis=1)) * np.repeat(scales.astype(np.float64), gs, axis=1)).T)
    assert np.abs(want).max() < 60000
    mem = [{"qweight": dev(qw), "scales": dev(scales), "qzeros": dev(qz)}]
    y = ext.group_forward(dev(x), None, mem, gs, 0.0)[0].cpu().numpy()
    np.testing.assert_array_equal(y.astype(np.float64), want.astype(np.float16).astype(np.float64))


def test_tiled_copy_follows_in_place_updates(ext):
    """The copy is kept on the weight tensor: an in-place change of the canonical buffer must rebuild it."""
    M, K, N = 8, 512, 64
    x, (m,), _ = make_group(77, M, K, [N], 0)
    mem = [{"qweight": dev(m["qweight"]), "scales": dev(m["scales"]), "qzeros": dev(m["qzeros"])}]
    y0 = ext.group_forward(dev(x), None, mem, 128, 0.0)[0].clone()
    _, (m2,), _ = make_group(78, M, K, [N], 0)
    mem[0]["qweight"].copy_(dev(m2["qweight"]))
    mem[0]["scales"].copy_(dev(m2["scales"]))
    mem[0]["qzeros"].copy_(dev(m2["qzeros"]))
    y1 = ext.group_forward(dev(x), None, mem, 128, 0.0)[0]
    torch.cuda.synchronize()
    assert not torch.equal(y0, y1)
    assert_close(y1.cpu().numpy(), oracle.linear_exact(x, m2["qweight"], m2["qzeros"], m2["scales"], 128), "after in-place update")


# ---------------------------------------------------------------- the MFMA GEMM on the tiled copy (more than 64 token rows)
GEMM_CASES = [
    # M, K, Ns, rank, alpha, bias
    (65, 512, [96], 0, 0.0, False),
    (128, 1024, [256, 300], 72, 0.5, True),
    (200, 2048, [512], 128, 1.0, False),
    (300, 768, [130, 64, 31], 8, 1.0, True),
    (1000, 3584, [512, 512], 128, 1.0, False),
]


@pytest.mark.parametrize("M,K,Ns,rank,alpha,bias", GEMM_CASES)
def test_gemm_on_the_tiled_copy_matches_oracle(ext, M, K, Ns, rank, alpha, bias):
    """Above 64 token rows the group runs on the MFMA GEMM, which takes its B operand from the tiled copy: the reference's
    dequantise-then-matmul arithmetic (src/cuda_w4a16/csrc/gemm_w4a16.cu:46-49,132), weight rounded to fp16 once."""
    print(f"case M={M} K={K} Ns={Ns} rank={rank}", flush=True)
    x, members, R = make_group(91 + M + K + rank, M, K, Ns, rank, with_bias=bias)
    mem = [{"qweight": dev(m["qweight"]), "scales": dev(m["scales"]), "qzeros": dev(m["qzeros"]),
            "L": dev(m["L"]) if rank else None, "bias": dev(m["bias"]) if bias else None} for m in members]
    assert ext.route(M, K, sum(Ns), 128, tiled=True) == "tiled_mfma_gemm"
    r = ext.shared_proj(dev(x), dev(R)) if rank else None
    outs = ext.group_forward(dev(x), r, mem, 128, alpha)
    torch.cuda.synchronize()
    assert all(hasattr(m["qweight"], "_glowq_tiled") for m in mem)    # the call built the tiled copies
    assert ext.last_launch()["kernel"].startswith("gemm_tiled_kernel")
    for i, (m, y) in enumerate(zip(members, outs)):
        if rank:
            want = oracle.corrected_linear_rounded_exact(x, m["qweight"], m["qzeros"], m["scales"], 128, R, m["L"], alpha)
        else:
            want = oracle.linear_rounded_exact(x, m["qweight"], m["qzeros"], m["scales"], 128)
        if bias:
            want = want + m["bias"].astype(np.float64)[None, :]
        assert_close(y.cpu().numpy(), want, f"tiled GEMM member {i} M={M} K={K}")


def test_gemm_on_the_tiled_copy_dequantises_exactly(ext):
    """Rows of the identity select weight columns: y[m, n] must be the reference's fp16((code - zero) * scale) of column
    m bit for bit -- the lane order of the tiled chunks, the nibble order inside a word, the side words and the swizzled
    LDS slots of the activations, all at once."""
    K, N, gs = 1024, 160, 128
    _, (m,), _ = make_group(404, 1, K, [N], 0, group_size=gs)
    cols = np.concatenate([np.arange(0, 256), np.arange(256, K, 3)])
    x = np.zeros((len(cols), K), dtype=np.float16)
    x[np.arange(len(cols)), cols] = 1.0
    mem = [{"qweight": dev(m["qweight"]), "scales": dev(m["scales"]), "qzeros": dev(m["qzeros"])}]
    y = ext.group_forward(dev(x), None, mem, gs, 0.0)[0].cpu().numpy()
    assert ext.last_launch()["kernel"].startswith("gemm_tiled_kernel")
    w = oracle.dequant(m["qweight"], m["qzeros"], m["scales"], K, gs)          # fp16 [N, K]
    np.testing.assert_array_equal(y.view(np.uint16), np.ascontiguousarray(w[:, cols].T).view(np.uint16))
