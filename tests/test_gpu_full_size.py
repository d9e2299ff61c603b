"""Llama-3.1-8B layer shapes at full size through the C ABI.  The oracle cannot hold a 28672 x 4096 layer in float64
in seconds, so it judges sampled output rows (first, last, member boundaries, random) of the full-size launch on the
same buffers, and size-independent properties cover the rest: one-hot inputs select dequantised columns exactly, a
group launch equals its members launched alone bit for bit, token rows of a batched launch equal single-row launches
within tolerance, and the result is additive in x within tolerance."""
import numpy as np
import pytest
import torch

import glowq_oracle as oracle
from helpers import assert_close

pytestmark = pytest.mark.gpu

GS, RANK = 128, 128
SHAPES = {"qkv": (4096, [4096, 1024, 1024]), "o": (4096, [4096]), "gate_up": (4096, [14336, 14336]), "down": (14336, [4096])}


def _layer(name, M, seed):
    K, Ns = SHAPES[name]
    g = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.randn(M, K, device="cuda", generator=g).half()
    R = (torch.randn(RANK, K, device="cuda", generator=g) * K ** -0.5).half()
    members = []
    for N in Ns:
        members.append({
            "qweight": torch.randint(-2**31, 2**31 - 1, (N, K // 8), device="cuda", generator=g, dtype=torch.int64).to(torch.int32),
            "scales": (torch.rand(N, K // GS, device="cuda", generator=g) * 0.008 + 0.002).half(),
            "qzeros": torch.randint(-2**31, 2**31 - 1, (N, (K // GS + 7) // 8), device="cuda", generator=g, dtype=torch.int64).to(torch.int32),
            "L": (torch.randn(N, RANK, device="cuda", generator=g) * 0.01).half(), "bias": None})
    return x, R, members


def _sample_rows(N, seed):
    rng = np.random.default_rng(seed)
    return np.unique(np.concatenate(([0, 1, 2, 3, N - 4, N - 3, N - 2, N - 1], rng.integers(0, N, 24))))


def _oracle_rows(x, R, mem, rows, alpha=1.0):
    sub = [mem[k][torch.from_numpy(rows).cuda()].cpu().numpy() for k in ("qweight", "qzeros", "scales", "L")]
    return oracle.corrected_linear_exact(x.cpu().numpy(), sub[0], sub[1], sub[2], GS, R.cpu().numpy(), sub[3], alpha)


@pytest.mark.parametrize("name", list(SHAPES))
@pytest.mark.parametrize("M", [1, 4, 16])
def test_full_size_group_sampled_rows_against_oracle(ext, name, M):
    print(f"case {name} M={M}", flush=True)
    x, R, members = _layer(name, M, seed=len(name) + M)
    r = torch.empty(M, RANK, dtype=torch.float16, device="cuda")
    outs = ext.group_forward(x, r, members, GS, 1.0, R=R)
    torch.cuda.synchronize()
    for i, (mem, y) in enumerate(zip(members, outs)):
        rows = _sample_rows(mem["qweight"].size(0), i)
        want = _oracle_rows(x, R, mem, rows)
        assert_close(y[:, torch.from_numpy(rows).cuda()].cpu().numpy(), want, f"{name} member {i} M={M}")
    # the group launch and its members launched alone: the same sums for one token row (a wave owns a whole row there);
    # with more rows the split of K over waves depends on the row count of the launch, so only the tolerance holds
    for mem, y in zip(members, outs):
        alone = ext.group_forward(x, r, [mem], GS, 1.0)[0]
        if M == 1:
            assert torch.equal(alone, y)
        else:
            assert ((alone.float() - y.float()).abs() <= 1e-2 + 1e-3 * y.float().abs()).all()


def test_full_size_one_hot_columns_are_exact(ext):
    K, Ns = SHAPES["gate_up"]
    x, _, members = _layer("gate_up", 1, seed=3)
    mem = members[1]
    deq = ext.dequant(mem["qweight"], mem["scales"], mem["qzeros"], K, GS)
    for k in (0, 5, 127, 128, 2049, K - 1):
        e = torch.zeros(1, K, dtype=torch.float16, device="cuda")
        e[0, k] = 1.0
        y = ext.w4a16_gemv_forward_cuda(e, mem["qweight"], mem["scales"], mem["qzeros"], GS)
        assert torch.equal(y[0], deq[:, k]), k


def test_full_size_batched_rows_match_single_rows_and_add_up(ext):
    x, R, members = _layer("down", 8, seed=9)
    r = torch.empty(8, RANK, dtype=torch.float16, device="cuda")
    batched = ext.group_forward(x, r, members, GS, 1.0, R=R)[0].float()
    r1 = torch.empty(1, RANK, dtype=torch.float16, device="cuda")
    tol = lambda ref: 1e-2 + 1e-3 * ref.abs()
    for m in (0, 3, 7):
        single = ext.group_forward(x[m:m + 1].contiguous(), r1, members, GS, 1.0, R=R)[0].float()
        assert ((batched[m:m + 1] - single).abs() <= 2 * tol(single)).all(), m
    # additivity in x, on inputs whose sum is exact in fp16 (multiples of 1/64 below 4)
    g = torch.Generator(device="cuda").manual_seed(2)
    a = (torch.randint(-128, 128, (1, x.size(1)), device="cuda", generator=g).float() / 64).half()
    b = (torch.randint(-128, 128, (1, x.size(1)), device="cuda", generator=g).float() / 64).half()
    ya, yb, yab = (ext.group_forward(v, r1, members, GS, 1.0, R=R)[0].float() for v in (a, b, (a + b)))
    assert ((yab - (ya + yb)).abs() <= 3 * tol(yab)).all()


def test_full_size_prefill_sampled_against_oracle(ext):
    M = 2048
    x, R, members = _layer("gate_up", M, seed=5)
    r = torch.empty(M, RANK, dtype=torch.float16, device="cuda")
    outs = ext.group_forward(x, r, members, GS, 1.0, R=R)
    torch.cuda.synchronize()
    tok = np.array([0, 1, 31, 32, 777, 2047])
    xs = x[torch.from_numpy(tok).cuda()]
    for i, (mem, y) in enumerate(zip(members, outs)):
        rows = _sample_rows(mem["qweight"].size(0), 10 + i)
        want = _oracle_rows(xs, R, mem, rows)
        got = y[torch.from_numpy(tok).cuda()][:, torch.from_numpy(rows).cuda()].cpu().numpy()
        # the GEMM route rounds the dequantised weight and r to fp16 as the reference does: twice the decode tolerance
        err = np.abs(got.astype(np.float64) - want)
        assert (err <= 2 * (1e-2 + 1e-3 * np.abs(want))).all(), float(err.max())
