"""The chained single-token group launch (glowq_w4a16_group_forward_chained) through the C ABI against the oracle:
RMSNorm + accumulator prologue, accumulator prologue, residual and SwiGLU epilogues, what they leave in the
accumulators, the overflow flag, and a layer's worth of launches handing over to each other."""
import numpy as np
import pytest
import torch

import glowq_oracle as oracle
from glowq_amd.kernels import (CHAIN_ACC_BYTES, CHAIN_EPI_NONE, CHAIN_EPI_RESIDUAL, CHAIN_EPI_SWIGLU, CHAIN_PRO_ACC,
                               CHAIN_PRO_NORM_ACC, CHAIN_PRO_PLAIN, PreparedGroup)
from helpers import ABS_TOL, REL_TOL, assert_close, dev, make_group

pytestmark = pytest.mark.gpu

COPIES, STRIDE = 16, 256


def new_acc():
    return torch.zeros(CHAIN_ACC_BYTES, dtype=torch.uint8, device="cuda")


def acc_values(acc, rank):
    """(P [rank] float64, overflow flag) of an accumulator."""
    words = acc.cpu().numpy().view(np.int64)
    p = words[:COPIES * STRIDE].reshape(COPIES, STRIDE)[:, :rank].sum(axis=0)
    return p.astype(np.float64) * 2.0 ** -32, int(words[COPIES * STRIDE])


def fill_acc(P, seed):
    """An accumulator holding P (float64 [rank]) in fixed point, dealt over the copies at random (sums to P exactly)."""
    rng = np.random.default_rng(seed)
    fixed = np.rint(P * 2.0 ** 32).astype(np.int64)
    words = np.zeros(COPIES * STRIDE + 8, dtype=np.int64)
    view = words[:COPIES * STRIDE].reshape(COPIES, STRIDE)
    parts = rng.integers(-2 ** 40, 2 ** 40, size=(COPIES - 1, len(P)))
    view[:COPIES - 1, :len(P)] = parts
    view[COPIES - 1, :len(P)] = fixed - parts.sum(axis=0)
    return torch.from_numpy(words.view(np.uint8).copy()).cuda()


def prepared(ext, members, K, gs, alpha, with_bias=False):
    mem = [{"qweight": dev(m["qweight"]), "scales": dev(m["scales"]), "qzeros": dev(m["qzeros"]), "L": dev(m["L"]),
            "bias": dev(m["bias"]) if with_bias else None} for m in members]
    return PreparedGroup(ext, mem, K, gs, alpha)


def close(got, want, what, slack=0.0):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    err, bound = np.abs(got - want), ABS_TOL + REL_TOL * np.abs(want) + slack
    assert np.all(err <= bound), f"{what}: max err {err.max():.3e} (bound {bound[np.argmax(err - bound)]:.3e})"


# K, N, rank, group size, bias: o_proj-like and down_proj-like shapes, odd N, a partial last step, large groups
RESIDUAL_CASES = [(4096, 4096, 128, 128, False), (14336, 4096, 128, 128, False), (3584, 301, 64, 128, True),
                  (2048, 1000, 256, 256, True), (18432, 64, 128, 128, False), (512, 130, 6, 128, False)]


@pytest.mark.parametrize("K,N,rank,gs,bias", RESIDUAL_CASES)
@pytest.mark.parametrize("pro", [CHAIN_PRO_PLAIN, CHAIN_PRO_ACC], ids=["r_given", "r_from_accumulator"])
def test_residual_epilogue(ext, pro, K, N, rank, gs, bias):
    print(f"case K={K} N={N} rank={rank} gs={gs} bias={bias} pro={pro}", flush=True)
    x, (m,), R = make_group(500 + N, 1, K, [N], rank, group_size=gs, with_bias=bias)
    g = torch.Generator().manual_seed(N)
    resid = (torch.randn(N, generator=g) * 2).half().numpy()
    next_w = (1 + 0.2 * torch.randn(N, generator=g)).half().numpy()
    next_R = (torch.randn(rank, N, generator=g) * N ** -0.5).half().numpy()
    pg = prepared(ext, [m], K, gs, 0.5, bias)
    r64 = x[0].astype(np.float64) @ R.astype(np.float64).T
    resid_d, acc_out, y = dev(resid), new_acc(), torch.zeros(N, dtype=torch.float16, device="cuda")
    kw = dict(outs=[y], resid=resid_d, next_norm_weight=dev(next_w), next_Rt=dev(np.ascontiguousarray(next_R.T)), acc_out=acc_out)
    if pro == CHAIN_PRO_PLAIN:
        pg.run_chained(dev(x[0]), CHAIN_PRO_PLAIN, CHAIN_EPI_RESIDUAL, r=dev(r64.astype(np.float16)), **kw)
    else:
        pg.run_chained(dev(x[0]), CHAIN_PRO_ACC, CHAIN_EPI_RESIDUAL, acc_in=fill_acc(r64, N), **kw)
    torch.cuda.synchronize()
    want_y = oracle.corrected_linear_exact(x, m["qweight"], m["qzeros"], m["scales"], gs, R, m["L"], 0.5)[0]
    if bias:
        want_y = want_y + m["bias"].astype(np.float64)
    assert_close(y.cpu().numpy(), want_y, "y")
    # the residual stream: exactly the fp16 sum of what was there and the y the launch wrote
    got_resid = resid_d.cpu().numpy()
    np.testing.assert_array_equal(got_resid.view(np.uint16), oracle.residual_add(resid, y.cpu().numpy()).view(np.uint16))
    # the accumulator: next_R (next_w (.) resid) of the launch's own residual stream, to fp32 summation accuracy
    P, flag = acc_values(acc_out, rank)
    c = next_w.astype(np.float64) * got_resid.astype(np.float64)
    want_P = next_R.astype(np.float64) @ c
    assert flag == 0
    np.testing.assert_allclose(P, want_P, rtol=0, atol=2e-6 * (np.abs(next_R.astype(np.float64)) @ np.abs(c)).max() + 1e-6)
    # integer sums: a second run of the producer leaves the same bits
    resid2, acc2 = dev(resid), new_acc()
    kw.update(resid=resid2, acc_out=acc2)
    if pro == CHAIN_PRO_PLAIN:
        pg.run_chained(dev(x[0]), CHAIN_PRO_PLAIN, CHAIN_EPI_RESIDUAL, r=dev(r64.astype(np.float16)), **kw)
    else:
        pg.run_chained(dev(x[0]), CHAIN_PRO_ACC, CHAIN_EPI_RESIDUAL, acc_in=fill_acc(r64, N + 1), **kw)
    torch.cuda.synchronize()
    assert torch.equal(acc2, acc_out) and torch.equal(resid2, resid_d)


@pytest.mark.parametrize("K,Ns,rank,gs", [(4096, [4096, 1024, 1024], 128, 128), (3584, [300, 77], 64, 128), (2048, [512], 256, 256),
                                          (8192, [96, 40, 40, 8], 128, 128), (512, [70], 6, 128)])
def test_norm_prologue(ext, K, Ns, rank, gs):
    """x is the residual stream: the launch norms it itself and takes r = fp16(f P) from the accumulator."""
    print(f"case K={K} Ns={Ns} rank={rank} gs={gs}", flush=True)
    x, members, R = make_group(900 + K, 1, K, Ns, rank, group_size=gs)
    g = torch.Generator().manual_seed(K)
    x_res = (x[0].astype(np.float32) * 3).astype(np.float16)
    w = (1 + 0.2 * torch.randn(K, generator=g)).half().numpy()
    eps = 1e-5
    P = R.astype(np.float64) @ (w.astype(np.float64) * x_res.astype(np.float64))
    pg = prepared(ext, members, K, gs, 1.0)
    outs = [torch.zeros(N, dtype=torch.float16, device="cuda") for N in Ns]
    pg.run_chained(dev(x_res), CHAIN_PRO_NORM_ACC, CHAIN_EPI_NONE, outs=outs, norm_weight=dev(w), eps=eps, acc_in=fill_acc(P, K))
    torch.cuda.synchronize()
    h = oracle.rmsnorm(x_res[None, :], w, eps)
    for m, y in zip(members, outs):
        want = oracle.corrected_linear_exact(h, m["qweight"], m["qzeros"], m["scales"], gs, R, m["L"], 1.0)[0]
        assert_close(y.cpu().numpy(), want, "norm prologue member")


@pytest.mark.parametrize("K,N,rank,gs,bias", [(4096, 14336, 128, 128, False), (3584, 301, 64, 128, True), (2048, 1030, 256, 256, False),
                                              (512, 67, 6, 128, True)])
def test_norm_prologue_with_swiglu_epilogue(ext, K, N, rank, gs, bias):
    print(f"case K={K} N={N} rank={rank} gs={gs} bias={bias}", flush=True)
    x, members, R = make_group(1300 + N, 1, K, [N, N], rank, group_size=gs, with_bias=bias)
    g = torch.Generator().manual_seed(N)
    x_res = (x[0].astype(np.float32) * 2).astype(np.float16)
    w = (1 + 0.2 * torch.randn(K, generator=g)).half().numpy()
    next_R = (torch.randn(rank, N, generator=g) * N ** -0.5).half().numpy()
    eps = 1e-6
    P = R.astype(np.float64) @ (w.astype(np.float64) * x_res.astype(np.float64))
    pg = prepared(ext, members, K, gs, 1.0, bias)
    act, acc_out = torch.zeros(N, dtype=torch.float16, device="cuda"), new_acc()
    gate_y, up_y = (torch.zeros(N, dtype=torch.float16, device="cuda") for _ in range(2))
    pg.run_chained(dev(x_res), CHAIN_PRO_NORM_ACC, CHAIN_EPI_SWIGLU, outs=[gate_y, up_y], norm_weight=dev(w), eps=eps,
                   acc_in=fill_acc(P, N), act=act, next_Rt=dev(np.ascontiguousarray(next_R.T)), acc_out=acc_out)
    torch.cuda.synchronize()
    h = oracle.rmsnorm(x_res[None, :], w, eps)
    want = [oracle.corrected_linear_exact(h, m["qweight"], m["qzeros"], m["scales"], gs, R, m["L"], 1.0)[0]
            + (m["bias"].astype(np.float64) if bias else 0.0) for m in members]
    assert_close(gate_y.cpu().numpy(), want[0], "gate")
    assert_close(up_y.cpu().numpy(), want[1], "up")
    # the gate of the launch's own fp16 outputs, bit for bit up to the hardware exponential (1 ulp of fp16 at most)
    ref_act = oracle.swiglu(gate_y.cpu().numpy(), up_y.cpu().numpy()).astype(np.float64)
    got_act = act.cpu().numpy().astype(np.float64)
    assert np.all(np.abs(got_act - ref_act) <= 2.0 ** -10 * np.abs(ref_act) + 1e-7)
    P2, flag = acc_values(acc_out, rank)
    assert flag == 0
    want_P = next_R.astype(np.float64) @ got_act
    np.testing.assert_allclose(P2, want_P, rtol=0, atol=2e-6 * (np.abs(next_R.astype(np.float64)) @ np.abs(got_act)).max() + 1e-6)
    # outputs nobody reads may be left out
    act2, acc2 = torch.zeros_like(act), new_acc()
    pg.run_chained(dev(x_res), CHAIN_PRO_NORM_ACC, CHAIN_EPI_SWIGLU, outs=[None, None], norm_weight=dev(w), eps=eps,
                   acc_in=fill_acc(P, N), act=act2, next_Rt=dev(np.ascontiguousarray(next_R.T)), acc_out=acc2)
    torch.cuda.synchronize()
    assert torch.equal(act2, act) and torch.equal(acc2, acc_out)


@pytest.mark.parametrize("K,N,rank,gs", [(4096, 2048, 128, 128), (1536, 333, 64, 128)])
def test_swiglu_epilogue_with_r_given(ext, K, N, rank, gs):
    """h and r come from a norm launch of their own; the launch gates its two members and projects the result."""
    print(f"case K={K} N={N} rank={rank}", flush=True)
    x, members, R = make_group(1700 + N, 1, K, [N, N], rank, group_size=gs)
    next_R = (torch.randn(rank, N, generator=torch.Generator().manual_seed(N)) * N ** -0.5).half().numpy()
    pg = prepared(ext, members, K, gs, 1.0)
    r64 = x[0].astype(np.float64) @ R.astype(np.float64).T
    act, acc_out = torch.zeros(N, dtype=torch.float16, device="cuda"), new_acc()
    gate_y, up_y = (torch.zeros(N, dtype=torch.float16, device="cuda") for _ in range(2))
    pg.run_chained(dev(x[0]), CHAIN_PRO_PLAIN, CHAIN_EPI_SWIGLU, r=dev(r64.astype(np.float16)), outs=[gate_y, up_y], act=act,
                   next_Rt=dev(np.ascontiguousarray(next_R.T)), acc_out=acc_out)
    torch.cuda.synchronize()
    want = [oracle.corrected_linear_exact(x, m["qweight"], m["qzeros"], m["scales"], gs, R, m["L"], 1.0)[0] for m in members]
    assert_close(gate_y.cpu().numpy(), want[0], "gate")
    assert_close(up_y.cpu().numpy(), want[1], "up")
    ref_act = oracle.swiglu(gate_y.cpu().numpy(), up_y.cpu().numpy()).astype(np.float64)
    got_act = act.cpu().numpy().astype(np.float64)
    assert np.all(np.abs(got_act - ref_act) <= 2.0 ** -10 * np.abs(ref_act) + 1e-7)
    P, flag = acc_values(acc_out, rank)
    assert flag == 0
    np.testing.assert_allclose(P, next_R.astype(np.float64) @ got_act, rtol=0,
                               atol=2e-6 * (np.abs(next_R.astype(np.float64)) @ np.abs(got_act)).max() + 1e-6)


def test_overflow_raises_the_flag_and_poisons_r(ext):
    """A partial sum beyond the fixed point's range must not wrap silently: the producer sets the flag, the consumer's
    outputs come out NaN."""
    K, N, rank, gs = 512, 256, 64, 128
    x, (m,), R = make_group(77, 1, K, [N], rank, group_size=gs)
    pg = prepared(ext, [m], K, gs, 1.0)
    resid = dev(np.full(N, 60000.0, np.float16))
    next_w = dev(np.full(N, 60000.0, np.float16))
    next_Rt = dev(np.full((N, rank), 8.0, np.float16))
    acc = new_acc()
    r = dev((x[0].astype(np.float64) @ R.astype(np.float64).T).astype(np.float16))
    pg.run_chained(dev(x[0]), CHAIN_PRO_PLAIN, CHAIN_EPI_RESIDUAL, r=r, outs=[None], resid=resid, next_norm_weight=next_w,
                   next_Rt=next_Rt, acc_out=acc)
    torch.cuda.synchronize()
    assert acc_values(acc, rank)[1] != 0
    x2, members2, _ = make_group(78, 1, N, [96], rank, group_size=gs)
    pg2 = prepared(ext, members2, N, gs, 1.0)
    y = torch.zeros(96, dtype=torch.float16, device="cuda")
    pg2.run_chained(dev(x2[0]), CHAIN_PRO_ACC, CHAIN_EPI_RESIDUAL, acc_in=acc, outs=[y], resid=torch.zeros(96, dtype=torch.float16, device="cuda"))
    torch.cuda.synchronize()
    assert torch.isnan(y).all()


def test_bad_arguments_are_refused(ext):
    K, N, rank, gs = 512, 64, 64, 128
    x, members, R = make_group(5, 1, K, [N, N], rank, group_size=gs)
    pg = prepared(ext, members, K, gs, 1.0)
    y = [torch.zeros(N, dtype=torch.float16, device="cuda") for _ in range(2)]
    with pytest.raises(RuntimeError, match="not served"):
        pg.run_chained(dev(x[0]), CHAIN_PRO_ACC, CHAIN_EPI_NONE, outs=y, acc_in=new_acc())
    with pytest.raises(RuntimeError, match="one member"):
        pg.run_chained(dev(x[0]), CHAIN_PRO_ACC, CHAIN_EPI_RESIDUAL, outs=y, acc_in=new_acc(), resid=torch.zeros(2 * N, dtype=torch.float16, device="cuda"))
    with pytest.raises(RuntimeError, match="acc_in"):
        pg.run_chained(dev(x[0]), CHAIN_PRO_NORM_ACC, CHAIN_EPI_NONE, outs=y, norm_weight=dev(np.ones(K, np.float16)))
    bare = PreparedGroup(ext, [{"qweight": dev(members[0]["qweight"]), "scales": dev(members[0]["scales"]), "qzeros": dev(members[0]["qzeros"])}], K, gs, 0.0)
    with pytest.raises(RuntimeError, match="correction"):
        bare.run_chained(dev(x[0]), CHAIN_PRO_PLAIN, CHAIN_EPI_RESIDUAL, outs=[y[0]], resid=torch.zeros(N, dtype=torch.float16, device="cuda"))


def test_a_layer_of_chained_launches_matches_the_separate_kernels(ext):
    """o_proj -> gate|up -> down_proj -> next q|k|v handing over through accumulators, against the same layer run with
    the separate norm / gate / projection launches (same inputs, north-star tolerance on every tensor handed on)."""
    H, I, rank, gs, eps = 1024, 2816, 64, 128, 1e-5
    g = torch.Generator().manual_seed(11)
    _, (o_m,), R_o = make_group(1, 1, H, [H], rank, group_size=gs)
    _, gu_m, R_gu = make_group(2, 1, H, [I, I], rank, group_size=gs)
    _, (dn_m,), R_dn = make_group(3, 1, I, [H], rank, group_size=gs)
    _, qkv_m, R_qkv = make_group(4, 1, H, [H, 256, 256], rank, group_size=gs)
    attn = torch.randn(H, generator=g).half().cuda()
    x_res0 = (torch.randn(H, generator=g) * 2).half().cuda()
    ln2 = (1 + 0.1 * torch.randn(H, generator=g)).half().cuda()
    ln1n = (1 + 0.1 * torch.randn(H, generator=g)).half().cuda()
    pg_o, pg_gu, pg_dn, pg_qkv = (prepared(ext, ms, K, gs, 1.0) for ms, K in (([o_m], H), (gu_m, H), ([dn_m], I), (qkv_m, H)))
    Rd = {k: dev(v) for k, v in (("o", R_o), ("gu", R_gu), ("dn", R_dn), ("qkv", R_qkv))}
    f16 = dict(dtype=torch.float16, device="cuda")

    # separate launches
    r_o = ext.shared_proj(attn[None, :], Rd["o"])
    o_out = pg_o.run(attn[None, :], r=r_o, project=False)[0]
    x1, h, r_gu = torch.zeros(1, H, **f16), torch.zeros(1, H, **f16), torch.zeros(1, rank, **f16)
    ext.add_rmsnorm_proj(x_res0[None, :], o_out, ln2, x1, h, Rd["gu"], r_gu, eps)
    gate, up = pg_gu.run(h, r=r_gu, project=False)
    act, r_dn = torch.zeros(1, I, **f16), torch.zeros(1, rank, **f16)
    ext.silu_mul_proj(gate, up, act, Rd["dn"], r_dn)
    dn_out = pg_dn.run(act, r=r_dn, project=False)[0]
    x2, h2, r_qkv = torch.zeros(1, H, **f16), torch.zeros(1, H, **f16), torch.zeros(1, rank, **f16)
    ext.add_rmsnorm_proj(x1, dn_out, ln1n, x2, h2, Rd["qkv"], r_qkv, eps)
    want_qkv = pg_qkv.run(h2, r=r_qkv, project=False)

    # chained
    acc_o, acc_gu, acc_dn = new_acc(), new_acc(), new_acc()
    xr = x_res0.clone()
    act_c = torch.zeros(I, **f16)
    pg_o.run_chained(attn, CHAIN_PRO_PLAIN, CHAIN_EPI_RESIDUAL, r=r_o[0], outs=[None], resid=xr, next_norm_weight=ln2,
                     next_Rt=Rd["gu"].t().contiguous(), acc_out=acc_o)
    x_after_o = xr.clone()
    pg_gu.run_chained(xr, CHAIN_PRO_NORM_ACC, CHAIN_EPI_SWIGLU, outs=[None, None], norm_weight=ln2, eps=eps, acc_in=acc_o,
                      act=act_c, next_Rt=Rd["dn"].t().contiguous(), acc_out=acc_gu)
    pg_dn.run_chained(act_c, CHAIN_PRO_ACC, CHAIN_EPI_RESIDUAL, acc_in=acc_gu, outs=[None], resid=xr, next_norm_weight=ln1n,
                      next_Rt=Rd["qkv"].t().contiguous(), acc_out=acc_dn)
    got_qkv = [torch.zeros(N, **f16) for N in (H, 256, 256)]
    pg_qkv.run_chained(xr, CHAIN_PRO_NORM_ACC, CHAIN_EPI_NONE, outs=got_qkv, norm_weight=ln1n, eps=eps, acc_in=acc_dn)
    torch.cuda.synchronize()
    assert torch.equal(x_after_o, x1[0])  # same fp16 additions
    close(act_c.cpu().numpy(), act[0].cpu().numpy(), "act")
    close(xr.cpu().numpy(), x2[0].cpu().numpy(), "residual stream after the layer")
    for a, b in zip(got_qkv, want_qkv):
        close(a.cpu().numpy(), b[0].cpu().numpy(), "next q|k|v")
