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
