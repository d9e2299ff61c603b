"""GPU checks of the decode loop over the quantised, corrected linears: the logits of a tiny random-init decoder
against the same network with every quantised module replaced by an fp32 matmul on its effective weight
(dequantised codes + alpha * L R, oracle-dequantised on the host), the HIP-graph replay against the eager loop,
and the artifact loader round trip."""
import json

import numpy as np
import pytest
import torch
import torch.nn as nn

import glowq_oracle as oracle
from glowq_amd import correction as corr
from glowq_amd import decode
from glowq_amd.linear import CudaW4A16Linear

pytestmark = pytest.mark.gpu

TINY = dict(hidden=256, layers=2, heads=4, kv_heads=2, head_dim=64, intermediate=512, vocab=1000, max_len=48,
            group_size=128, rank=64)


@pytest.fixture()
def fp16_out(monkeypatch):
    monkeypatch.setenv("W4A16_KERNEL_OUT_DTYPE", "fp16")
    with torch.no_grad():
        yield


class _RefLinear(nn.Module):
    def __init__(self, w32):
        super().__init__()
        self.w = w32

    def forward(self, x):
        return (x.float() @ self.w.T).to(x.dtype)


def _effective_weight(mod, with_correction=True):
    inner = mod.inner if isinstance(mod, corr.AddSVDCorrection) else mod
    assert isinstance(inner, CudaW4A16Linear)
    w = oracle.dequant(inner.qweight_i32.cpu().numpy(), inner.qzeros_i32.cpu().numpy(), inner.scales_f16.cpu().numpy(),
                       inner.in_features, inner.group_size)[:, : inner.in_features].astype(np.float32)
    w = torch.from_numpy(w).cuda()
    if with_correction and isinstance(mod, corr.AddSVDCorrection):
        w = w + float(mod.alpha_svd) * (mod.A_q.float() @ mod.B_q.float())
    return w


def _swap_in_reference(model, with_correction=True):
    saved = []
    for layer in model.model.layers:
        for owner, names in ((layer.self_attn, ("q_proj", "k_proj", "v_proj", "o_proj")),
                             (layer.mlp, ("gate_proj", "up_proj", "down_proj"))):
            for n in names:
                mod = getattr(owner, n)
                saved.append((owner, n, mod))
                setattr(owner, n, _RefLinear(_effective_weight(mod, with_correction)))
    return saved


def _restore(saved):
    for owner, n, mod in saved:
        setattr(owner, n, mod)


def _logits(model, tokens):
    cfg = model.cfg
    dec = decode.GreedyDecoder(model, use_graph=False)
    pos = torch.arange(tokens.numel(), device="cuda")
    return model.forward_tokens(tokens.cuda(), pos, dec.caches, dec.cos, dec.sin).float().cpu().numpy()


@pytest.mark.parametrize("T", [1, 7, 40])
def test_tiny_decoder_logits_match_effective_weight_network(fp16_out, T):
    model, _, _ = decode.build_decoder(decode.DecoderConfig(**TINY), seed=5)
    n_wrapped = sum(isinstance(m, corr.AddSVDCorrection) for m in model.modules())
    assert n_wrapped == 7 * TINY["layers"]
    tokens = torch.randint(0, TINY["vocab"], (T,), generator=torch.Generator().manual_seed(T))
    got = _logits(model, tokens)
    saved = _swap_in_reference(model)
    want = _logits(model, tokens)
    _restore(saved)
    saved = _swap_in_reference(model, with_correction=False)
    without = _logits(model, tokens)
    _restore(saved)
    err = np.abs(got - want).max()
    # fp16 activations between the linears are common to both networks; what differs is the kernels' arithmetic
    assert err <= 1e-2 + 1e-3 * np.abs(want).max(), err
    # the check discriminates: dropping the correction moves the logits by far more than the tolerance
    assert np.abs(without - want).max() > 10 * max(err, 1e-3)


def test_graph_replay_matches_eager_decode(fp16_out):
    model, _, _ = decode.build_decoder(decode.DecoderConfig(**TINY), seed=6)
    prompt = torch.randint(0, TINY["vocab"], (9,), generator=torch.Generator().manual_seed(1))
    eager = decode.GreedyDecoder(model, use_graph=False)
    want, _, _ = eager.generate(prompt, 12)
    graphed = decode.GreedyDecoder(model, use_graph=True)
    for _ in range(3):  # replays after the first, with eager prefill work and synchronisations in between
        got, ttfb, dt = graphed.generate(prompt, 12)
        assert torch.equal(got, want)
        assert ttfb > 0 and dt > 0
    with pytest.raises(ValueError):
        graphed.generate(prompt, TINY["max_len"])


def test_selective_decoder_and_artifact_round_trip(fp16_out, tmp_path):
    cfg = decode.DecoderConfig(**TINY)
    model, shared, bmap = decode.build_decoder(cfg, seed=7, groups_to_patch={"layer0_qkv", "model.layers.1.mlp.down_proj"})
    wrapped = sorted(n for n, m in model.named_modules() if isinstance(m, corr.AddSVDCorrection))
    assert wrapped == ["model.layers.0.self_attn.k_proj", "model.layers.0.self_attn.q_proj",
                       "model.layers.0.self_attn.v_proj", "model.layers.1.mlp.down_proj"]
    tokens = torch.randint(0, TINY["vocab"], (5,), generator=torch.Generator().manual_seed(2))
    got = _logits(model, tokens)
    saved = _swap_in_reference(model)
    want = _logits(model, tokens)
    _restore(saved)
    assert np.abs(got - want).max() <= 1e-2 + 1e-3 * np.abs(want).max()

    # the files step 2 writes: a dict of fp16 tensors and a json map; read back without executing anything
    torch.save({k: v.cpu() for k, v in shared.items()}, tmp_path / "low_rank_shared.pt")
    (tmp_path / "b_ref_map.json").write_text(json.dumps(bmap))
    shared2, bmap2 = decode.load_glowq_artifacts(str(tmp_path / "low_rank_shared.pt"), str(tmp_path / "b_ref_map.json"))
    assert bmap2 == bmap and set(shared2) == set(shared)
    assert all(torch.equal(shared2[k].cpu(), shared[k].cpu()) for k in shared)
