"""Host-side logic on CPU: the drop-in module surface, the quantiser against the reference's golden
vectors, model conversion, correction patching (full and selective), and the C ABI's symbols.  No kernel
is launched here."""
import ctypes
import os
import re
import types

import numpy as np
import pytest
import torch
import torch.nn as nn

import glowq_oracle as oracle
from glowq_amd import correction as corr
from glowq_amd import kernels, linear

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ---------------------------------------------------------------- quantiser / packing of the product
@pytest.mark.parametrize("name", list("abcde"))
def test_product_quantizer_matches_reference_golden(golden, name):
    gs, kp = (int(v) for v in golden[f"q_{name}_gs"])
    qw, qz, sc, kp2 = linear._quantize_per_group_w4(torch.from_numpy(golden[f"q_{name}_w"]), gs)
    assert kp2 == kp
    np.testing.assert_array_equal(qw.numpy(), golden[f"q_{name}_qweight"])
    np.testing.assert_array_equal(qz.numpy(), golden[f"q_{name}_qzeros"])
    np.testing.assert_array_equal(sc.numpy().view(np.uint16), golden[f"q_{name}_scales"].view(np.uint16))
    assert qw.dtype == torch.int32 and qz.dtype == torch.int32 and sc.dtype == torch.float16


def test_product_pack_unpack(golden):
    codes = torch.from_numpy(golden["pack_codes"])
    words = linear._pack_int4_to_int32(codes)
    np.testing.assert_array_equal(words.numpy(), golden["pack_words"])
    np.testing.assert_array_equal(linear._unpack_int4_i32(words, 50).numpy(), golden["unpack_vals_50"])
    with pytest.raises(AssertionError):
        linear._pack_int4_to_int32(codes.to(torch.int32))


def test_quantizer_rejects_group_not_multiple_of_8():
    with pytest.raises(ValueError):
        linear._quantize_per_group_w4(torch.zeros(2, 20, dtype=torch.float16), 10)


# ---------------------------------------------------------------- module surface
def test_module_buffers_and_state_dict():
    m = linear.CudaW4A16Linear(300, 40, group_size=64, bias=True)
    assert m.qweight_i32.shape == (40, 38) and m.qweight_i32.dtype == torch.int32
    assert m.qzeros_i32.shape == (40, 1) and m.scales_f16.shape == (40, 5) and m.scales_f16.dtype == torch.float16
    assert m.gid.shape == (300,) and m.gid.dtype == torch.long and int(m.gid[-1]) == 4
    assert sorted(m.state_dict().keys()) == ["bias", "qweight_i32", "qzeros_i32", "scales_f16"]  # gid is not persistent
    assert m.bias.dtype == torch.float16
    assert (m.groups, m.groups_packed, m.in_features, m.out_features, m.group_size) == (5, 1, 300, 40, 64)
    assert "in_features=300" in repr(m) and "bias=True" in repr(m)
    for bad in (0, -8, 12):
        with pytest.raises(ValueError):
            linear.CudaW4A16Linear(8, 8, group_size=bad)


def test_from_float_matches_golden_buffers(golden):
    for name in ("m1", "m2"):
        w = torch.from_numpy(golden[f"{name}_w"])
        has_bias = f"{name}_bias" in golden
        lin = nn.Linear(w.shape[1], w.shape[0], bias=has_bias).half()
        lin.weight.data.copy_(w)
        if has_bias:
            lin.bias.data.copy_(torch.from_numpy(golden[f"{name}_bias"]))
        mod = linear.CudaW4A16Linear.from_float(lin, int(golden[f"{name}_gs"][0]))
        np.testing.assert_array_equal(mod.qweight_i32.numpy(), golden[f"{name}_qweight"])
        np.testing.assert_array_equal(mod.qzeros_i32.numpy(), golden[f"{name}_qzeros"])
        np.testing.assert_array_equal(mod.scales_f16.numpy().view(np.uint16), golden[f"{name}_scales"].view(np.uint16))
        assert sorted(mod.state_dict().keys()) == list(golden[f"{name}_state_keys"])
        # a saved state dict loads back into a fresh module
        fresh = linear.CudaW4A16Linear(w.shape[1], w.shape[0], int(golden[f"{name}_gs"][0]), bias=has_bias)
        fresh.qweight_i32.resize_(mod.qweight_i32.shape)
        fresh.load_state_dict(mod.state_dict())
        assert torch.equal(fresh.qweight_i32, mod.qweight_i32)


def test_forward_errors_on_cpu_and_bad_shapes():
    m = linear.CudaW4A16Linear(64, 8, 32)
    with pytest.raises(ValueError, match="Input dim mismatch"):
        m(torch.zeros(2, 63, dtype=torch.float16))
    with pytest.raises(RuntimeError, match="only on the GPU"):
        m(torch.zeros(2, 64, dtype=torch.float16))  # no CPU route, on purpose


def test_env_knobs(monkeypatch):
    monkeypatch.delenv("W4A16_KERNEL_OUT_DTYPE", raising=False)
    monkeypatch.delenv("MIXED_KERNEL_OUT_DTYPE", raising=False)
    assert linear._get_kernel_out_dtype() == torch.float32  # module default, as in the reference
    monkeypatch.setenv("W4A16_KERNEL_OUT_DTYPE", "fp16")
    assert linear._get_kernel_out_dtype() == torch.float16
    monkeypatch.setenv("W4A16_GEMV_M_MAX", "7")
    m = linear.CudaW4A16Linear(64, 8, 32)
    assert m._gemv_threshold == 7 and m._prefer_gemv(7) and not m._prefer_gemv(8)
    assert not m._prefer_gemv(1000)
    monkeypatch.setenv("W4A16_FORCE_GEMV", "1")
    assert m._prefer_gemv(1000)                # as in the reference, a switch set between two forwards is seen by the next
    monkeypatch.setenv("W4A16_FORCE_GEMM", "true")
    assert not m._prefer_gemv(1)
    monkeypatch.setenv("W4A16_SPLIT_K_ITERS", "4")
    linear.KNOBS.sync()
    assert linear.KNOBS.split_k_iters == 4 and linear.KNOBS.out_dtype == torch.float16
    raw = linear.KNOBS._raw
    linear.KNOBS.sync()                        # nothing changed: nothing is parsed again
    assert linear.KNOBS._raw is raw
    monkeypatch.delenv("W4A16_GEMV_M_MAX")
    monkeypatch.setenv("CUDA_MIXED_GEMV_M_MAX", "3")  # legacy alias
    assert linear.CudaW4A16Linear(64, 8, 32)._gemv_threshold == 3


# ---------------------------------------------------------------- conversion and patching on a toy model
class Attn(nn.Module):
    def __init__(self, h, kv):
        super().__init__()
        self.q_proj, self.k_proj, self.v_proj, self.o_proj = nn.Linear(h, h), nn.Linear(h, kv), nn.Linear(h, kv), nn.Linear(h, h)


class Mlp(nn.Module):
    def __init__(self, h, f):
        super().__init__()
        self.gate_proj, self.up_proj, self.down_proj = nn.Linear(h, f, bias=False), nn.Linear(h, f, bias=False), nn.Linear(f, h, bias=False)


class Layer(nn.Module):
    def __init__(self, h, kv, f):
        super().__init__()
        self.self_attn, self.mlp, self.norm = Attn(h, kv), Mlp(h, f), nn.LayerNorm(h)


class Toy(nn.Module):
    def __init__(self, n=2, h=128, kv=64, f=256):
        super().__init__()
        self.model = nn.Module()
        self.model.layers = nn.ModuleList([Layer(h, kv, f) for _ in range(n)])
        self.lm_head = nn.Linear(h, 50, bias=False)


def toy_artifacts(n=2, h=128, kv=64, f=256, rank=16):
    """`shared` / `bmap` in the artifact key scheme: grouped q/k/v and gate/up, solo o and down."""
    shared, bmap = {}, {}
    for i in range(n):
        pre = f"model.layers.{i}"
        shared[f"layer{i}_qkv.B_shared"] = torch.randn(rank, h).half()
        for s, o in (("q_proj", h), ("k_proj", kv), ("v_proj", kv)):
            shared[f"layer{i}_qkv.{s}.A"] = torch.randn(o, rank).half()
            bmap[f"{pre}.self_attn.{s}.weight"] = f"layer{i}_qkv.B_shared"
        shared[f"layer{i}_mlp.B_shared"] = torch.randn(rank, h).half()
        for s in ("gate_proj", "up_proj"):
            shared[f"layer{i}_mlp.{s}.A"] = torch.randn(f, rank).half()
            bmap[f"{pre}.mlp.{s}.weight"] = f"layer{i}_mlp.B_shared"
        for mod, k, o in ((f"{pre}.self_attn.o_proj", h, h), (f"{pre}.mlp.down_proj", f, h)):
            shared[f"{mod}.A"], shared[f"{mod}.B"] = torch.randn(o, rank).half(), torch.randn(rank, k).half()
            bmap[f"{mod}.weight"] = f"{mod}.B"
    return shared, bmap


def test_convert_replaces_everything_but_lm_head():
    model = linear.convert_to_cuda_w4a16(Toy().half(), group_size=64)
    kinds = {n: type(m).__name__ for n, m in model.named_modules() if isinstance(m, (nn.Linear, linear.CudaW4A16Linear))}
    assert kinds.pop("lm_head") == "Linear"
    assert len(kinds) == 14 and set(kinds.values()) == {"CudaW4A16Linear"}
    q = model.model.layers[0].self_attn.q_proj
    assert q.bias is not None and q.group_size == 64 and q.qweight_i32.shape == (128, 16)
    # a layer that cannot be converted (group size not a multiple of 8) is left alone, silently
    model2 = linear.convert_to_cuda_w4a16(Toy(n=1).half(), group_size=12)
    assert isinstance(model2.model.layers[0].mlp.down_proj, nn.Linear)


def test_patch_wraps_groups_and_solos_with_shared_caches():
    model = linear.convert_to_cuda_w4a16(Toy().half(), 64)
    shared, bmap = toy_artifacts()
    corr.patch_svd_correction_wrappers(model, shared, bmap, alpha_svd=0.75)
    l0 = model.model.layers[0]
    q, k, v, o = l0.self_attn.q_proj, l0.self_attn.k_proj, l0.self_attn.v_proj, l0.self_attn.o_proj
    for w, role in ((q, "q"), (k, "k"), (v, "v"), (l0.mlp.gate_proj, "gate"), (l0.mlp.up_proj, "up"), (o, "solo"), (l0.mlp.down_proj, "solo")):
        assert isinstance(w, corr.AddSVDCorrection) and w.role == role and w.alpha_svd == 0.75
        assert isinstance(w.inner, linear.CudaW4A16Linear)
    assert q.group_cache is k.group_cache is v.group_cache and q.is_group
    assert l0.mlp.gate_proj.group_cache is l0.mlp.up_proj.group_cache is not q.group_cache
    assert o.group_cache is None and not o.is_group
    assert model.model.layers[1].self_attn.q_proj.group_cache is not q.group_cache
    assert [w.role for w in q.group_cache.members] == ["q", "k", "v"]
    assert torch.equal(q.B_q, shared["layer0_qkv.B_shared"]) and torch.equal(k.A_q, shared["layer0_qkv.k_proj.A"])
    assert "A_q" not in q.state_dict() and "inner.qweight_i32" in q.state_dict()  # factors are not persistent
    assert not isinstance(model.lm_head, corr.AddSVDCorrection)


def test_patch_skips_missing_factors_and_unquantised_modules():
    model = linear.convert_to_cuda_w4a16(Toy(n=1).half(), 64)
    shared, bmap = toy_artifacts(n=1)
    del shared["layer0_qkv.k_proj.A"]
    bmap["lm_head.weight"] = "lm_head.B"
    shared["lm_head.A"], shared["lm_head.B"] = torch.zeros(50, 16).half(), torch.zeros(16, 128).half()
    bmap["model.layers.0.nowhere.weight"] = "model.layers.0.self_attn.o_proj.B"
    corr.patch_svd_correction_wrappers(model, shared, bmap)
    sa = model.model.layers[0].self_attn
    assert isinstance(sa.q_proj, corr.AddSVDCorrection) and isinstance(sa.k_proj, linear.CudaW4A16Linear)
    assert isinstance(model.lm_head, nn.Linear)  # not a quantised linear: left bare


def test_selective_patch_only_touches_selected_groups():
    shared, bmap = toy_artifacts()
    model = linear.convert_to_cuda_w4a16(Toy().half(), 64)
    corr.patch_svd_correction_wrappers_cumulative(model, shared, bmap, set())
    assert not any(isinstance(m, corr.AddSVDCorrection) for m in model.modules())
    chosen = {"layer0_qkv", "layer1_mlp", "model.layers.1.self_attn.o_proj"}
    corr.patch_svd_correction_wrappers_cumulative(model, shared, bmap, chosen, alpha_svd=1.0)
    wrapped = sorted(n for n, m in model.named_modules() if isinstance(m, corr.AddSVDCorrection))
    assert wrapped == sorted([
        "model.layers.0.self_attn.q_proj", "model.layers.0.self_attn.k_proj", "model.layers.0.self_attn.v_proj",
        "model.layers.1.mlp.gate_proj", "model.layers.1.mlp.up_proj", "model.layers.1.self_attn.o_proj"])
    assert isinstance(model.model.layers[0].mlp.gate_proj, linear.CudaW4A16Linear)


def test_role_from_suffix_and_parent_lookup():
    assert [corr._role_from_suffix(s) for s in ("q_proj", "k_proj", "v_proj", "gate_proj", "up_proj", "o_proj", "down_proj", "fc1")] == \
        ["q", "k", "v", "gate", "up", "solo", "solo", "solo"]
    model = Toy(n=1)
    parent, leaf = corr.get_parent_module(model, "model.layers.0.mlp.up_proj")
    assert parent is model.model.layers[0].mlp and leaf == "up_proj"


def test_mini_group_cache_matches_oracle_state_machine():
    a, b = corr.MiniGroupCache(), oracle.MiniGroupCacheModel()
    script = [("consume",), ("set", "r1", 2), ("consume",), ("consume",), ("consume",), ("set", "r2", 1), ("clear",),
              ("consume",), ("set", "r3", 1), ("consume",), ("consume",)]
    for op in script:
        if op[0] == "set":
            a.set(op[1], op[2]); b.set(op[1], op[2])
        elif op[0] == "clear":
            a.clear(); b.clear()
        else:
            assert a.consume() == b.consume()
        assert (a.valid, a.uses_left, a.r) == (b.valid, b.uses_left, b.r)


def test_alpha_zero_returns_inner_output_untouched():
    class Probe(nn.Module):
        def forward(self, x):
            return x + 1
    w = corr.AddSVDCorrection(Probe(), torch.zeros(4, 2), torch.zeros(2, 4), "solo", False, None, alpha_svd=0.0)
    x = torch.ones(3, 4)
    assert torch.equal(w(x), x + 1)
    w.alpha_svd = 1.0
    with pytest.raises(RuntimeError):
        w(x)


def test_configure_env(monkeypatch, capsys):
    for k in ("W4A16_KERNEL_OUT_DTYPE", "W4A16_GEMM_CUDA", "W4A16_DEQUANT_CACHE", "W4A16_GEMV_M_MAX", "W4A16_FORCE_GEMM", "W4A16_FORCE_GEMV"):
        monkeypatch.delenv(k, raising=False)
    corr._configure_cuda_w4a16_env(types.SimpleNamespace(use_cuda_w4a16=False))
    assert "W4A16_KERNEL_OUT_DTYPE" not in os.environ
    monkeypatch.setenv("W4A16_FORCE_GEMM", "1")
    corr._configure_cuda_w4a16_env(types.SimpleNamespace(use_cuda_w4a16=True, cuda_w4a16_gemv_m_max=16, cuda_w4a16_force_gemv=True))
    assert os.environ["W4A16_KERNEL_OUT_DTYPE"] == "fp16" and os.environ["W4A16_GEMV_M_MAX"] == "16"
    assert os.environ["W4A16_FORCE_GEMV"] == "1" and "W4A16_FORCE_GEMM" not in os.environ
    assert "[CUDA W4A16] env:" in capsys.readouterr().out
    for k in ("W4A16_KERNEL_OUT_DTYPE", "W4A16_GEMM_CUDA", "W4A16_DEQUANT_CACHE", "W4A16_GEMV_M_MAX", "W4A16_FORCE_GEMV"):
        monkeypatch.delenv(k, raising=False)


def test_reference_import_paths():
    import cuda_w4a16
    from cuda_w4a16.kernels import load_w4a16_extension
    from cuda_w4a16.linear import CudaW4A16Linear, convert_to_cuda_w4a16
    assert cuda_w4a16.CudaW4A16Linear is linear.CudaW4A16Linear is CudaW4A16Linear
    assert convert_to_cuda_w4a16 is linear.convert_to_cuda_w4a16 and load_w4a16_extension is kernels.load_w4a16_extension


# ---------------------------------------------------------------- the C ABI library
def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "glowq_w4a16.h")).read()
    declared = set(re.findall(r"\b(glowq_[a-z0-9_]+)\s*\(", header))
    assert {"glowq_w4a16_gemv_forward", "glowq_w4a16_gemm_forward", "glowq_w4a16_group_forward", "glowq_shared_proj",
            "glowq_w4a16_dequant", "glowq_unpack_int4", "glowq_last_error", "glowq_version"} <= declared
    lib = ctypes.CDLL(kernels.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name
    assert set(kernels._SIGNATURES) == declared
    assert ctypes.sizeof(kernels._Member) == 6 * 8 + 6 * 4 + 8 + 2 * 8 + 2 * 4  # matches glowq_member_t
    assert kernels._Member.side.offset == 72 and kernels._Member.side_rank.offset == 68


def test_abi_rejects_bad_arguments_without_a_gpu():
    ext = kernels.load_w4a16_extension()
    lib = ext.lib
    one = ctypes.c_void_p(16)
    assert lib.glowq_w4a16_gemv_forward(None, one, one, one, one, 1, 64, 8, 32, 8, 2, 1, None) == -1
    assert b"inputs" in lib.glowq_last_error()
    assert lib.glowq_w4a16_gemv_forward(one, one, one, one, one, 1, 64, 8, 12, 8, 6, 1, None) == -1
    assert b"multiple of 8" in lib.glowq_last_error()
    assert lib.glowq_w4a16_gemv_forward(one, one, one, one, one, 1, 64, 8, 32, 7, 2, 1, None) == -2
    assert b"qweight packed cols too small" in lib.glowq_last_error()
    assert lib.glowq_w4a16_gemm_forward(one, one, one, one, one, 1, 64, 8, 32, 1, 8, 1, 1, None) == -2
    assert b"scales groups mismatch" in lib.glowq_last_error()
    assert lib.glowq_w4a16_group_forward(one, None, None, 0, 1, 64, 32, 0, 1.0, None) == -1
    assert lib.glowq_shared_proj(one, one, one, 0, 64, 8, None) == -1
    assert lib.glowq_w4a16_dequant(one, one, one, one, 4, 64, 32, 8, 2, 0, None) == -2
    assert ext.route(2048, 3584, 3584) == "tiled_mfma_gemm"
    # the stream-scheduled 4x4x4 matrix-core GEMV: two to four token rows, groups of 128 columns and up, rows of up to
    # 16384 columns; at two rows not where the last 2048-column slice of a short group's rows is mostly empty
    assert ext.route(2, 4096, 28672) == "quad_stream_gemv" and ext.route(4, 4096, 4096) == "quad_stream_gemv"
    assert ext.route(3, 14336, 4096) == "quad_stream_gemv" and ext.route(4, 8192, 10240) == "quad_stream_gemv"
    assert ext.route(2, 5120, 5120) != "quad_stream_gemv" and ext.route(2, 5120, 34816, tiled=False) == "quad_stream_gemv"
    # with the tiled copy the longest streams (80 MB of codes and more) go to the kernel that streams it from two rows on
    assert ext.route(2, 5120, 34816, tiled=True) == "skinny_tiled_mfma" and ext.route(4, 4096, 28672, tiled=True) == "quad_stream_gemv"
    assert ext.route(4, 5120, 5120) == "quad_stream_gemv" and ext.route(4, 6144, 28672, tiled=False) == "quad_stream_gemv"
    assert ext.route(1, 4096, 4096) != "quad_stream_gemv" and ext.route(5, 4096, 4096) != "quad_stream_gemv"
    assert ext.route(4, 4096, 4096, group_size=64) != "quad_stream_gemv" and ext.route(4, 17408, 5120) != "quad_stream_gemv"
    rule = ext.set_tuning("qstream_shape_rule", 0)
    assert ext.route(2, 5120, 5120) == "quad_stream_gemv"
    ext.set_tuning("qstream_shape_rule", rule)
    qstream = ext.set_tuning("qstream_max_m", 0)                                # the routes behind it
    assert qstream == 4
    # the stream GEMV: one token row always, more rows by the measured shape rule (short K; fewer rows of output the more
    # token rows), never past four
    assert ext.route(1, 4096, 4096) == "stream_gemv" and ext.route(1, 14336, 4096) == "stream_gemv" and ext.route(1, 17408, 5120) == "stream_gemv"
    assert ext.route(2, 4096, 28672) == "stream_gemv" and ext.route(2, 14336, 4096) != "stream_gemv"
    assert ext.route(3, 4096, 6144) == "stream_gemv" and ext.route(3, 4096, 28672) != "stream_gemv"
    assert ext.route(4, 4096, 4096) == "stream_gemv" and ext.route(4, 4096, 6144) != "stream_gemv" and ext.route(5, 4096, 4096) != "stream_gemv"
    assert ext.route(1, 4096, 4096, group_size=64) != "stream_gemv"          # groups below 128 columns stay on the others
    rule = ext.set_tuning("stream_shape_rule", 0)
    assert ext.route(4, 4096, 28672) == "stream_gemv"
    ext.set_tuning("stream_shape_rule", rule)
    stream = ext.set_tuning("stream_max_m", 0)                                  # the routes behind it
    old = ext.set_tuning("quad_max_m", 0)
    assert ext.route(1, 4096, 4096) == "wave_dot_gemv" and ext.route(8, 4096, 4096, tiled=False) == "skinny_codes_mfma"
    # a member that brings the tiled copy of its weights: 33..64 token rows go to the kernel that streams it, 5..32 where
    # the stream is long enough (40 MB of codes and more; 24 MB from 17 rows)
    assert ext.route(64, 4096, 4096, tiled=True) == "skinny_tiled_mfma" and ext.route(64, 14336, 4096, tiled=True) == "skinny_tiled_mfma"
    assert ext.route(8, 4096, 28672, tiled=True) == "skinny_tiled_mfma" and ext.route(8, 4096, 4096, tiled=True) == "skinny_codes_mfma"
    assert ext.route(16, 14336, 4096, tiled=True) == "skinny_mfma" and ext.route(17, 14336, 4096, tiled=True) == "skinny_tiled_mfma"
    assert ext.route(4, 4096, 28672, tiled=True) != "skinny_tiled_mfma" and ext.route(65, 4096, 28672, tiled=True) == "tiled_mfma_gemm"
    rule = ext.set_tuning("tiled_shape_rule", 0)
    assert rule == 1 and ext.route(8, 4096, 4096, tiled=True) == "skinny_tiled_mfma" and ext.route(5, 256, 32, tiled=True) == "skinny_tiled_mfma"
    assert ext.route(8, 4096 + 128, 4096, tiled=True) != "skinny_tiled_mfma"   # K must be whole super-blocks of 256 columns
    assert ext.route(8, 4096, 4096, group_size=64, tiled=True) != "skinny_tiled_mfma"
    tmax = ext.set_tuning("tiled_max_m", 0)
    assert tmax == 64 and ext.route(8, 4096, 4096, tiled=True) == "skinny_codes_mfma"
    ext.set_tuning("tiled_max_m", tmax)
    ext.set_tuning("tiled_shape_rule", rule)
    ext.set_tuning("quad_max_m", 16)
    assert ext.route(8, 4096, 4096, tiled=False) == "quad_mfma_gemv"
    ext.set_tuning("quad_max_m", old)
    # 2..4 rows: small groups stay on the wave-dot GEMV, large ones take the 4x4x4 matrix-core GEMV
    assert ext.route(2, 4096, 4096) == "wave_dot_gemv" and ext.route(2, 4096, 28672) == "quad_mfma_gemv"
    assert ext.route(4, 4096, 4096, tiled=False) == "skinny_codes_mfma" and ext.route(4, 14336, 4096) == "quad_mfma_gemv"
    old = ext.set_tuning("small_group_mb", 0)
    assert ext.route(2, 4096, 4096) == "quad_mfma_gemv"
    ext.set_tuning("small_group_mb", old)
    ext.set_tuning("stream_max_m", stream)
    ext.set_tuning("qstream_max_m", 4)
    with pytest.raises(ValueError):
        ext.set_tuning("no_such_key", 1)
    assert ext.route(1, 100, 8) == "generic"
    # the switch and the poll limit of the group launch that computes r itself: defaults, ranges, round trip
    assert ext.set_tuning("proj_in_launch", 0) == 1 and ext.set_tuning("proj_in_launch", 2) == 0
    assert ext.set_tuning("proj_in_launch", 1) == 2
    assert ext.set_tuning("proj_spin_limit", 0) == 16384 and ext.set_tuning("proj_spin_limit", 16384) == 0
    assert ext.set_tuning("small_rows_in_launch", 0) == 1 and ext.set_tuning("small_rows_in_launch", 1) == 0
    for key, bad in (("proj_in_launch", 3), ("proj_spin_limit", -1), ("proj_spin_limit", (1 << 24) + 1), ("small_rows_in_launch", 2)):
        with pytest.raises(ValueError):
            ext.set_tuning(key, bad)


def test_tensor_front_end_checks():
    ext = kernels.load_w4a16_extension()
    x = torch.zeros(1, 64, dtype=torch.float16)
    qw, sc, qz = torch.zeros(8, 8, dtype=torch.int32), torch.zeros(8, 2, dtype=torch.float16), torch.zeros(8, 1, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="inputs must be CUDA"):
        ext.w4a16_gemv_forward_cuda(x, qw, sc, qz, 32)
    with pytest.raises(RuntimeError, match="inputs must be CUDA"):
        ext.w4a16_gemm_forward_cuda(x, qw, sc, qz, 32, 1)
    assert ext.gemv_w4a16_asym.__func__ is ext.w4a16_gemv_forward_cuda.__func__


def test_missing_library_raises(monkeypatch):
    monkeypatch.setattr(kernels, "_ext", None)
    monkeypatch.setattr(kernels, "LIB_PATH", "/nonexistent/libglowq_w4a16.so")
    monkeypatch.delenv("W4A16_ALLOW_JIT", raising=False)
    with pytest.raises(RuntimeError, match="python -m glowq_amd.build"):
        kernels.load_w4a16_extension()


def test_allow_jit_builds_a_missing_library_once(monkeypatch):
    """W4A16_ALLOW_JIT=1 (src/cuda_w4a16/kernels.py:24-59): a library that does not load is built and loaded again; the
    build itself is stubbed here (it takes a minute), once leaving the library missing and once putting it in place."""
    from glowq_amd import build as build_mod

    real = kernels.LIB_PATH
    calls = []
    monkeypatch.setattr(kernels, "_ext", None)
    monkeypatch.setattr(kernels, "LIB_PATH", "/nonexistent/libglowq_w4a16.so")
    monkeypatch.setenv("W4A16_ALLOW_JIT", "1")
    monkeypatch.setattr(build_mod, "build", lambda verbose=False, extra_flags=(): calls.append("build"))
    with pytest.raises(RuntimeError, match="still does not load"):
        kernels.load_w4a16_extension()
    assert calls == ["build"]

    def fake_build(verbose=False, extra_flags=()):
        calls.append("build")
        monkeypatch.setattr(kernels, "LIB_PATH", real)

    monkeypatch.setattr(build_mod, "build", fake_build)
    monkeypatch.setattr(kernels, "LIB_PATH", "/nonexistent/libglowq_w4a16.so")
    ext = kernels.load_w4a16_extension()
    assert calls == ["build", "build"] and ext.version >= 100
    monkeypatch.setattr(kernels, "_ext", None)
