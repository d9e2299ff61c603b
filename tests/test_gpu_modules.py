"""GPU parity of the drop-in modules: converted linears, the correction wrapper with its fused group launch,
cache behaviour (reuse, miss, out-of-order callers), the selective patcher and the output-dtype knob."""
import numpy as np
import pytest
import torch
import torch.nn as nn

import glowq_oracle as oracle
from glowq_amd import correction as corr
from glowq_amd import linear
from helpers import assert_close
from test_host import Toy, toy_artifacts

pytestmark = pytest.mark.gpu


def _ref(x, mod, L=None, R=None, alpha=1.0):
    """float64 yardstick from the module's own (CPU copy of the) buffers."""
    qw, qz, sc = (t.cpu().numpy() for t in (mod.qweight_i32, mod.qzeros_i32, mod.scales_f16))
    y = oracle.linear_exact(x, qw, qz, sc, mod.group_size)[:, : mod.out_features]
    if L is not None:
        y = y + alpha * (x.astype(np.float64) @ R.cpu().numpy().astype(np.float64).T @ L.cpu().numpy().astype(np.float64).T)
    if mod.bias is not None:
        y = y + mod.bias.detach().cpu().numpy().astype(np.float64)[None, :]
    return y


@pytest.fixture()
def fp16_out(monkeypatch):
    monkeypatch.setenv("W4A16_KERNEL_OUT_DTYPE", "fp16")
    linear.refresh_env_knobs()
    with torch.no_grad():  # inference path: the reference evaluates under no_grad as well
        yield


def test_converted_linear_forward(fp16_out, monkeypatch):
    torch.manual_seed(0)
    lin = nn.Linear(512, 96, bias=True).half()
    lin.weight.data.mul_(0.5)
    mod = linear.CudaW4A16Linear.from_float(lin, 128).cuda()
    for shape in [(1, 512), (2, 3, 512), (5, 512), (200, 512)]:
        x = torch.randn(*shape).half()
        y = mod(x.cuda())
        assert y.shape == (*shape[:-1], 96) and y.dtype == torch.float16
        assert_close(y.cpu().numpy().reshape(-1, 96), _ref(x.numpy().reshape(-1, 512), mod), f"linear {shape}")
    # fp32 inputs are cast; fp32 output is the reference's module default
    monkeypatch.setenv("W4A16_KERNEL_OUT_DTYPE", "fp32")
    x4 = torch.randn(4, 512).half()
    y32 = mod(x4.cuda())                                                # a switch set after import is seen by the next forward
    assert y32.dtype == torch.float32
    # with fp32 output the bias is added in fp32 after the cast of the fp16 kernel output (linear.py:183-186)
    bare = mod._bare_group().run(x4.cuda())[0]
    assert torch.equal(y32, bare.float() + mod.bias.float())
    # forced routes agree with each other within tolerance
    x = torch.randn(3, 512).half()
    monkeypatch.setenv("W4A16_KERNEL_OUT_DTYPE", "fp16")
    monkeypatch.setenv("W4A16_FORCE_GEMM", "1")
    linear.refresh_env_knobs()
    assert linear.KNOBS.force_gemm and not mod._prefer_gemv(1)
    yg = mod(x.cuda()).cpu().numpy()
    monkeypatch.delenv("W4A16_FORCE_GEMM")
    linear.refresh_env_knobs()
    assert_close(yg, _ref(x.numpy(), mod), "forced gemm route")
    w = mod.dequantize().cpu().numpy()
    np.testing.assert_array_equal(w.view(np.uint16), oracle.dequant(mod.qweight_i32.cpu().numpy(), mod.qzeros_i32.cpu().numpy(),
                                                                     mod.scales_f16.cpu().numpy(), 512, 128).view(np.uint16))


def _patched_toy(alpha=1.0, groups=None):
    torch.manual_seed(1)
    model = Toy(n=2, h=256, kv=64, f=512).half()
    for p in model.parameters():
        p.data.mul_(0.3)
    model = linear.convert_to_cuda_w4a16(model, 128).cuda()
    shared, bmap = toy_artifacts(n=2, h=256, kv=64, f=512, rank=32)
    shared = {k: (v * 0.05).cuda() for k, v in shared.items()}
    if groups is None:
        corr.patch_svd_correction_wrappers(model, shared, bmap, alpha_svd=alpha)
    else:
        corr.patch_svd_correction_wrappers_cumulative(model, shared, bmap, groups, alpha_svd=alpha)
    return model, shared


@pytest.mark.parametrize("M", [1, 3, 40])
def test_group_wrappers_match_oracle_and_share_one_launch(fp16_out, M):
    model, shared = _patched_toy(alpha=1.0)
    sa, mlp = model.model.layers[0].self_attn, model.model.layers[0].mlp
    x = torch.randn(M, 256).half()
    xd = x.cuda()
    yq = sa.q_proj(xd)
    cache = sa.q_proj.group_cache
    assert cache.valid and cache.uses_left == 2 and len(cache.outputs) == 2  # k and v are waiting in the cache
    yk, yv = sa.k_proj(xd), sa.v_proj(xd)
    assert not cache.valid and cache.r is None and not cache.outputs
    yo = sa.o_proj(xd)
    yg, yu = mlp.gate_proj(xd), mlp.up_proj(xd)
    torch.cuda.synchronize()
    R = shared["layer0_qkv.B_shared"]
    for w, y, nm in ((sa.q_proj, yq, "q_proj"), (sa.k_proj, yk, "k_proj"), (sa.v_proj, yv, "v_proj")):
        assert_close(y.cpu().numpy(), _ref(x.numpy(), w.inner, shared[f"layer0_qkv.{nm}.A"], R), nm)
    assert_close(yo.cpu().numpy(), _ref(x.numpy(), sa.o_proj.inner, shared["model.layers.0.self_attn.o_proj.A"],
                                        shared["model.layers.0.self_attn.o_proj.B"]), "o_proj")
    Rm = shared["layer0_mlp.B_shared"]
    assert_close(yg.cpu().numpy(), _ref(x.numpy(), mlp.gate_proj.inner, shared["layer0_mlp.gate_proj.A"], Rm), "gate")
    assert_close(yu.cpu().numpy(), _ref(x.numpy(), mlp.up_proj.inner, shared["layer0_mlp.up_proj.A"], Rm), "up")


def test_followers_recompute_on_miss_and_on_a_different_input(fp16_out):
    model, shared = _patched_toy()
    sa = model.model.layers[1].self_attn
    R = shared["layer1_qkv.B_shared"]
    x1, x2 = torch.randn(2, 256).half(), torch.randn(2, 256).half()
    # k before q: nothing cached
    yk = sa.k_proj(x1.cuda())
    assert_close(yk.cpu().numpy(), _ref(x1.numpy(), sa.k_proj.inner, shared["layer1_qkv.k_proj.A"], R), "k on miss")
    # q on x1, then k on ANOTHER input: the cached output must not be returned
    sa.q_proj(x1.cuda())
    yk2 = sa.k_proj(x2.cuda())
    assert_close(yk2.cpu().numpy(), _ref(x2.numpy(), sa.k_proj.inner, shared["layer1_qkv.k_proj.A"], R), "k on other x")
    # calling q twice in a row restarts the cache cleanly
    sa.q_proj(x1.cuda()); sa.q_proj(x2.cuda())
    yv = sa.v_proj(x2.cuda())
    assert_close(yv.cpu().numpy(), _ref(x2.numpy(), sa.v_proj.inner, shared["layer1_qkv.v_proj.A"], R), "v after 2x q")


def test_replaced_buffers_are_picked_up_by_the_next_forward(fp16_out):
    """The group launch runs on descriptors built once from tensor addresses: a follower's factor or a member's weight
    replaced by attribute assignment (re-quantisation, cumulative patching) must rebuild them."""
    model, shared = _patched_toy()
    sa = model.model.layers[0].self_attn
    R = shared["layer0_qkv.B_shared"]
    x = torch.randn(2, 256).half()
    xd = x.cuda()
    sa.q_proj(xd), sa.k_proj(xd), sa.v_proj(xd)  # descriptors of the three-member group exist now
    new_A = (torch.randn_like(sa.k_proj.A_q) * 0.05).contiguous()
    sa.k_proj.A_q = new_A                        # a follower's left factor swapped
    lin = nn.Linear(256, 64, bias=True).half()
    lin.weight.data.mul_(0.3)
    fresh = linear.CudaW4A16Linear.from_float(lin, 128).cuda()
    sa.v_proj.inner.qweight_i32 = fresh.qweight_i32  # a member re-quantised in place
    sa.v_proj.inner.scales_f16 = fresh.scales_f16
    sa.v_proj.inner.qzeros_i32 = fresh.qzeros_i32
    yq, yk, yv = sa.q_proj(xd), sa.k_proj(xd), sa.v_proj(xd)
    torch.cuda.synchronize()
    assert_close(yk.cpu().numpy(), _ref(x.numpy(), sa.k_proj.inner, new_A, R), "k after its factor was replaced")
    assert_close(yv.cpu().numpy(), _ref(x.numpy(), sa.v_proj.inner, shared["layer0_qkv.v_proj.A"], R), "v after re-quantisation")
    assert_close(yq.cpu().numpy(), _ref(x.numpy(), sa.q_proj.inner, shared["layer0_qkv.q_proj.A"], R), "q unchanged")


def test_alpha_switch_and_scaling(fp16_out):
    model, shared = _patched_toy(alpha=0.5)
    sa = model.model.layers[0].self_attn
    x = torch.randn(1, 256).half()
    y = sa.q_proj(x.cuda())
    assert_close(y.cpu().numpy(), _ref(x.numpy(), sa.q_proj.inner, shared["layer0_qkv.q_proj.A"], shared["layer0_qkv.B_shared"], 0.5), "alpha .5")
    for m in model.modules():
        if isinstance(m, corr.AddSVDCorrection):
            m.alpha_svd = 0.0  # how the reference's evaluator turns the correction off
    y0 = sa.q_proj(x.cuda())
    bare = sa.q_proj.inner(x.cuda())
    assert torch.equal(y0, bare)


def test_selective_groups_leave_the_rest_uncorrected(fp16_out):
    model, shared = _patched_toy(groups={"layer0_qkv", "model.layers.0.mlp.down_proj"})
    l0 = model.model.layers[0]
    x = torch.randn(1, 256).half()
    yq = l0.self_attn.q_proj(x.cuda())
    assert_close(yq.cpu().numpy(), _ref(x.numpy(), l0.self_attn.q_proj.inner, shared["layer0_qkv.q_proj.A"], shared["layer0_qkv.B_shared"]), "selected")
    assert isinstance(l0.mlp.gate_proj, linear.CudaW4A16Linear)
    yg = l0.mlp.gate_proj(x.cuda())
    assert_close(yg.cpu().numpy(), _ref(x.numpy(), l0.mlp.gate_proj), "unselected")
    x2 = torch.randn(1, 512).half()
    yd = l0.mlp.down_proj(x2.cuda())
    assert_close(yd.cpu().numpy(), _ref(x2.numpy(), l0.mlp.down_proj.inner, shared["model.layers.0.mlp.down_proj.A"],
                                        shared["model.layers.0.mlp.down_proj.B"]), "selected solo")


def test_state_dict_round_trip_on_device(fp16_out):
    torch.manual_seed(3)
    lin = nn.Linear(256, 32, bias=False).half()
    a = linear.CudaW4A16Linear.from_float(lin, 128).cuda()
    b = linear.CudaW4A16Linear(256, 32, 128).cuda()
    b.load_state_dict(a.state_dict())
    x = torch.randn(2, 256).half().cuda()
    assert torch.equal(a(x), b(x))


def test_dequant_chunk_rows_match_the_reference_vectors(golden):
    """`_dequant_chunk(start, end)` (src/cuda_w4a16/linear.py:248-253): rows of the dequantised weight, bit for bit
    against what the reference's own method returned for the whole matrix."""
    from glowq_amd.linear import CudaW4A16Linear

    gs = int(golden["m2_gs"][0])
    n, k = golden["m2_w"].shape
    mod = CudaW4A16Linear(k, n, gs, bias=False).cuda()
    mod.qweight_i32.copy_(torch.from_numpy(golden["m2_qweight"]))
    mod.scales_f16.copy_(torch.from_numpy(golden["m2_scales"]))
    mod.qzeros_i32.copy_(torch.from_numpy(golden["m2_qzeros"]))
    want = golden["m2_deq"]
    for start, end in ((0, n), (3, 17), (n - 1, n), (5, 5), (30, n + 10)):
        got = mod._dequant_chunk(start, end).cpu().numpy()
        np.testing.assert_array_equal(got.view(np.uint16), want[start:min(end, n)].view(np.uint16))
