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
from glowq_amd.linear import CudaW4A16Linear, refresh_env_knobs

pytestmark = pytest.mark.gpu

TINY = dict(hidden=256, layers=2, heads=4, kv_heads=2, head_dim=64, intermediate=512, vocab=1000, max_len=48,
            group_size=128, rank=64)


@pytest.fixture()
def fp16_out(monkeypatch):
    monkeypatch.setenv("W4A16_KERNEL_OUT_DTYPE", "fp16")
    refresh_env_knobs()
    with torch.no_grad():
        yield


class _RefLinear(nn.Module):
    def __init__(self, w32):
        super().__init__()
        self.w = w32

    def forward(self, x):
        return (x.float() @ self.w.T).to(x.dtype)


def _effective_weight(mod, with_correction=True, deq_cache=None):
    inner = mod.inner if isinstance(mod, corr.AddSVDCorrection) else mod
    assert isinstance(inner, CudaW4A16Linear)
    w = deq_cache.get(id(inner)) if deq_cache is not None else None
    if w is None:
        w = oracle.dequant(inner.qweight_i32.cpu().numpy(), inner.qzeros_i32.cpu().numpy(), inner.scales_f16.cpu().numpy(),
                           inner.in_features, inner.group_size)[:, : inner.in_features].astype(np.float32)
        w = torch.from_numpy(w).cuda()
        if deq_cache is not None:
            deq_cache[id(inner)] = w
    if with_correction and isinstance(mod, corr.AddSVDCorrection):
        w = w + float(mod.alpha_svd) * (mod.A_q.float() @ mod.B_q.float())
    return w


def _swap_in_reference(model, with_correction=True, deq_cache=None):
    """`deq_cache` (a dict) keeps the oracle-dequantised weights between calls on the same model."""
    saved = []
    for layer in model.model.layers:
        for owner, names in ((layer.self_attn, ("q_proj", "k_proj", "v_proj", "o_proj")),
                             (layer.mlp, ("gate_proj", "up_proj", "down_proj"))):
            for n in names:
                mod = getattr(owner, n)
                saved.append((owner, n, mod))
                setattr(owner, n, _RefLinear(_effective_weight(mod, with_correction, deq_cache)))
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


def test_prefill_without_mask_matches_masked_path(fp16_out):
    model, _, _ = decode.build_decoder(decode.DecoderConfig(**TINY), seed=12)
    tokens = torch.randint(0, TINY["vocab"], (23,), generator=torch.Generator().manual_seed(3)).cuda()
    pos = torch.arange(23, device="cuda")
    a, b = decode.GreedyDecoder(model, use_graph=False), decode.GreedyDecoder(model, use_graph=False)
    masked = model.forward_tokens(tokens, pos, a.caches, a.cos, a.sin).float()
    causal = model.forward_tokens(tokens, pos, b.caches, b.cos, b.sin, from_empty_cache=True).float()
    assert (masked - causal).abs().max() <= 2e-3 + 2e-3 * masked.abs().max()
    for (ka, va), (kb, vb) in zip(a.caches, b.caches):          # both leave the same cache behind
        assert (ka.float() - kb.float()).abs().max() <= 2e-3 and (va.float() - vb.float()).abs().max() <= 2e-3


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


def test_glue_kernels_match_torch(ext, fp16_out):
    g = torch.Generator(device="cuda").manual_seed(11)
    M, H = 3, 512
    x = torch.randn(M, H, device="cuda", generator=g).half()
    d = torch.randn(M, H, device="cuda", generator=g).half()
    w = (1 + 0.1 * torch.randn(H, device="cuda", generator=g)).half()
    h = torch.empty_like(x)
    want_x = (x + d)
    want_h = torch.nn.functional.rms_norm(want_x.float(), (H,), w.float(), 1e-5)
    x2 = x.clone()
    ext.add_rmsnorm(x2, d, w, h, 1e-5)
    assert torch.equal(x2, want_x)
    assert (h.float() - want_h).abs().max() <= 4e-3 * want_h.abs().max()
    ext.add_rmsnorm(x2, None, w, h, 1e-5)          # no residual: x untouched
    assert torch.equal(x2, want_x)

    gate, up = torch.randn(1, 1024, device="cuda", generator=g).half() * 3, torch.randn(1, 1024, device="cuda", generator=g).half()
    out = torch.empty_like(gate)
    ext.silu_mul(gate, up, out)
    want = torch.nn.functional.silu(gate.float()) * up.float()
    assert (out.float() - want).abs().max() <= 4e-3 * want.abs().max()

    logits = torch.randn(1, 5000, device="cuda", generator=g).half()
    logits[0, 1234] = 9.0
    logits[0, 4321] = 9.0                           # a tie: the first index wins
    nxt, tok, pos = (torch.zeros(1, dtype=torch.long, device="cuda") for _ in range(3))
    pos.fill_(41)
    ext.argmax_advance(logits, nxt, tok, pos)
    assert (int(nxt), int(tok), int(pos)) == (1234, 1234, 42)
    # a vocabulary-sized vector (several batches of pieces per thread, then a tail) with the tie far apart
    big = torch.randn(128256 + 3, device="cuda", generator=g).half()
    big[100003] = 11.0
    big[9001] = 11.0
    big[128258] = 11.0
    ext.argmax_advance(big.reshape(1, -1), nxt, tok, pos)
    assert (int(nxt), int(tok), int(pos)) == (9001, 9001, 43)
    big[9001] = 0.0
    big[100003] = 0.0
    ext.argmax_advance(big.reshape(1, -1), nxt, tok, pos)
    assert (int(nxt), int(pos)) == (128258, 44)      # the maximum in the tail behind the last whole piece


@pytest.mark.parametrize("d,max_len,pos", [(64, 320, 0), (64, 320, 1), (64, 320, 37), (64, 320, 300), (128, 2100, 257),
                                           (128, 2100, 700), (128, 2100, 2047), (64, 1500, 1300)])
def test_rope_attend_matches_torch(ext, fp16_out, d, max_len, pos):
    heads, kvh = 8, 2
    g = torch.Generator(device="cuda").manual_seed(pos)
    q = torch.randn(heads, d, device="cuda", generator=g).half()
    k = torch.randn(kvh, d, device="cuda", generator=g).half()
    v = torch.randn(kvh, d, device="cuda", generator=g).half()
    ck = torch.randn(kvh, max_len, d, device="cuda", generator=g).half()
    cv = torch.randn(kvh, max_len, d, device="cuda", generator=g).half()
    model = decode.Decoder(decode.DecoderConfig(hidden=heads * d, layers=0, heads=heads, kv_heads=kvh, head_dim=d, intermediate=64,
                                                vocab=8, max_len=max_len))
    cos, sin = model.rope_tables("cuda")
    p = torch.tensor([pos], device="cuda")
    # torch yardstick in fp32 on the fp16-rounded tables
    c, s = cos[pos].half().float(), sin[pos].half().float()
    rot = lambda t: torch.cat((-t[..., d // 2:], t[..., :d // 2]), dim=-1)
    qr = (q.float() * c + rot(q.float()) * s).half().float()
    kr = (k.float() * c + rot(k.float()) * s).half()
    K = torch.cat((ck[:, :pos].float(), kr.float()[:, None]), dim=1).repeat_interleave(heads // kvh, dim=0)
    V = torch.cat((cv[:, :pos].float(), v.float()[:, None]), dim=1).repeat_interleave(heads // kvh, dim=0)
    att = torch.softmax(torch.einsum("hd,htd->ht", qr, K) * d ** -0.5, dim=-1)
    want = torch.einsum("ht,htd->hd", att, V)
    ck2, cv2 = ck.clone(), cv.clone()
    out = torch.empty(heads, d, dtype=torch.float16, device="cuda")
    ext.rope_attend(q.reshape(-1), k.reshape(-1), v.reshape(-1), cos, sin, p, ck2, cv2, out, d ** -0.5)
    torch.cuda.synchronize()
    assert (out.float() - want).abs().max() <= 2e-3 + 2e-3 * want.abs().max()
    assert torch.equal(ck2[:, pos], kr) and torch.equal(cv2[:, pos], v)          # appended at pos
    keep = torch.ones(max_len, dtype=torch.bool, device="cuda")
    keep[pos] = False
    assert torch.equal(ck2[:, keep], ck[:, keep]) and torch.equal(cv2[:, keep], cv[:, keep])   # nothing else touched


def test_appended_key_is_bit_identical_to_the_tensor_expression(ext, fp16_out):
    """The rotated key written to the cache equals (k * cos + rotate_half(k) * sin) evaluated op by op in fp32 and
    rounded once to fp16, bit for bit: first on the one input where a fused multiply-add in the kernel's rotary
    embedding once landed an fp16 ulp away (head dim 128, 2 KV heads, 16 heads, position 1645 of 4100, generator seed
    23), then over a seeded sweep of keys and positions; the one-workgroup and the split kernel write the same bits."""
    def run(d, kvh, heads, max_len, pos, seed, splits):
        g = torch.Generator(device="cuda").manual_seed(seed)
        q = torch.randn(heads * d, device="cuda", generator=g).half()
        k = torch.randn(kvh * d, device="cuda", generator=g).half()
        v = torch.randn(kvh * d, device="cuda", generator=g).half()
        ck = torch.randn(kvh, max_len, d, device="cuda", generator=g).half()
        cv = torch.randn(kvh, max_len, d, device="cuda", generator=g).half()
        model = decode.Decoder(decode.DecoderConfig(hidden=heads * d, layers=0, heads=heads, kv_heads=kvh, head_dim=d,
                                                    intermediate=64, vocab=8, max_len=max_len))
        cos, sin = model.rope_tables("cuda")
        c, s = cos[pos].half().float(), sin[pos].half().float()
        kf = k.view(kvh, d).float()
        kr = (kf * c + torch.cat((-kf[..., d // 2:], kf[..., :d // 2]), dim=-1) * s).half()
        p = torch.tensor([pos], device="cuda")
        ck1, cv1, o1 = ck.clone(), cv.clone(), torch.empty(heads * d, dtype=torch.float16, device="cuda")
        ext.rope_attend(q, k, v, cos, sin, p, ck1, cv1, o1, d ** -0.5)
        ck2, cv2 = ck.clone(), cv.clone()
        part = torch.zeros(heads, splits, d + 4, device="cuda")
        ext.rope_attend_split(q, k, v, cos, sin, p, ck2, cv2, part, d ** -0.5)
        torch.cuda.synchronize()
        assert torch.equal(ck1[:, pos], kr), (d, kvh, pos, seed)
        assert torch.equal(ck1, ck2) and torch.equal(cv1, cv2)

    run(128, 2, 16, 4100, 1645, 23, 3)
    rng = np.random.default_rng(8)
    for i in range(48):
        d = int(rng.choice([64, 128]))
        run(d, 8, 8, 200, int(rng.integers(0, 200)), 1000 + i, int(rng.choice([2, 4])))


def test_position_outside_the_cache_touches_no_cache_row_and_poisons_the_output(ext, fp16_out):
    heads, kvh, d, max_len = 8, 2, 64, 96
    g = torch.Generator(device="cuda").manual_seed(1)
    q = torch.randn(heads * d, device="cuda", generator=g).half()
    k = torch.randn(kvh * d, device="cuda", generator=g).half()
    v = torch.randn(kvh * d, device="cuda", generator=g).half()
    ck = torch.randn(kvh, max_len, d, device="cuda", generator=g).half()
    cv = torch.randn(kvh, max_len, d, device="cuda", generator=g).half()
    model = decode.Decoder(decode.DecoderConfig(hidden=heads * d, layers=0, heads=heads, kv_heads=kvh, head_dim=d, intermediate=64,
                                                vocab=8, max_len=max_len))
    cos, sin = model.rope_tables("cuda")
    for bad in (max_len, max_len + 7, -1):
        p = torch.tensor([bad], device="cuda")
        ck2, cv2 = ck.clone(), cv.clone()
        out = torch.full((heads * d,), 7.0, dtype=torch.float16, device="cuda")
        part = torch.full((heads, 4, d + 4), 7.0, device="cuda")
        ext.rope_attend(q, k, v, cos, sin, p, ck2, cv2, out, d ** -0.5)
        ext.rope_attend_split(q, k, v, cos, sin, p, ck2, cv2, part, d ** -0.5)
        torch.cuda.synchronize()
        assert torch.equal(ck2, ck) and torch.equal(cv2, cv)
        # the step is marked, not silently skipped: whatever is computed from it is NaN
        assert torch.isnan(out).all() and torch.isnan(part).all()
        merged = torch.empty(heads * d, dtype=torch.float16, device="cuda")
        ext.attend_combine_proj(part, merged)
        assert torch.isnan(merged).all()


@pytest.mark.parametrize("pos,splits", [(0, 4), (1, 4), (3, 8), (37, 4), (300, 4), (300, 7)])
def test_split_attention_and_merge_match_single_workgroup(ext, fp16_out, pos, splits):
    heads, kvh, d, max_len, rank = 8, 2, 128, 320, 64
    g = torch.Generator(device="cuda").manual_seed(100 + pos)
    q = torch.randn(heads * d, device="cuda", generator=g).half()
    k = torch.randn(kvh * d, device="cuda", generator=g).half()
    v = torch.randn(kvh * d, device="cuda", generator=g).half()
    ck = torch.randn(kvh, max_len, d, device="cuda", generator=g).half()
    cv = torch.randn(kvh, max_len, d, device="cuda", generator=g).half()
    R = (torch.randn(rank, heads * d, device="cuda", generator=g) * (heads * d) ** -0.5).half()
    model = decode.Decoder(decode.DecoderConfig(hidden=heads * d, layers=0, heads=heads, kv_heads=kvh, head_dim=d, intermediate=64,
                                                vocab=8, max_len=max_len))
    cos, sin = model.rope_tables("cuda")
    p = torch.tensor([pos], device="cuda")
    ck1, cv1, want = ck.clone(), cv.clone(), torch.empty(heads * d, dtype=torch.float16, device="cuda")
    ext.rope_attend(q, k, v, cos, sin, p, ck1, cv1, want, d ** -0.5)
    ck2, cv2 = ck.clone(), cv.clone()
    part = torch.full((heads, splits, d + 4), float("nan"), device="cuda")
    got, r = torch.empty_like(want), torch.empty(rank, dtype=torch.float16, device="cuda")
    ext.rope_attend_split(q, k, v, cos, sin, p, ck2, cv2, part, d ** -0.5)
    ext.attend_combine_proj(part, got, R, r)
    torch.cuda.synchronize()
    assert torch.equal(ck1, ck2) and torch.equal(cv1, cv2)
    assert (got.float() - want.float()).abs().max() <= 1e-3 + 2e-3 * want.float().abs().max()
    r_ref = ext.shared_proj(got.reshape(1, -1), R).reshape(-1)
    assert (r.float() - r_ref.float()).abs().max() <= 1e-3 + 2e-3 * r_ref.float().abs().max()
    plain = torch.empty_like(want)
    ext.attend_combine_proj(part, plain)                      # without R: only the merge
    assert torch.equal(plain, got)


@pytest.mark.parametrize("chain", ["full", "mlp", False], ids=["chained", "chained_mlp", "separate_glue"])
def test_fused_step_matches_module_path(fp16_out, chain):
    cfg = decode.DecoderConfig(**TINY)
    model, _, _ = decode.build_decoder(cfg, seed=8)
    prompt = torch.randint(0, cfg.vocab, (11,), generator=torch.Generator().manual_seed(4))
    ref = decode.GreedyDecoder(model, use_graph=False)
    fus = decode.GreedyDecoder(model, use_graph=False, fused=True, chain=chain)
    assert fus.fused.chained == chain
    first = ref.prefill(prompt)
    fus.prefill(prompt)
    tok = first.clone()
    for step in range(6):                                   # teacher forcing: both see the yardstick's tokens
        pos = torch.tensor([prompt.numel() + step], device="cuda")
        want = model.forward_tokens(tok, pos, ref.caches, ref.cos, ref.sin).float()
        fus.tok.copy_(tok), fus.pos.copy_(pos)
        fus.fused.run()
        got = fus.fused.logits.float()
        assert (got - want).abs().max() <= 1e-2 + 1e-2 * want.abs().max(), step
        assert int(fus.pos) == int(pos) + 1 and int(fus.tok) == int(got.argmax())
        tok = want.argmax(-1)
    # without sharing (one projection and one launch per module) the step computes the same tokens
    alone, _, _ = decode.GreedyDecoder(model, use_graph=False, fused=True, share=False).generate(prompt, 10)
    assert torch.equal(alone, decode.GreedyDecoder(model, use_graph=False, fused=True, chain=chain).generate(prompt, 10)[0])
    # the context split over 3 workgroups per head merges to the same logits within tolerance
    spl = decode.GreedyDecoder(model, use_graph=False, fused=True)
    spl.fused = decode.FusedStep(model, spl.caches, spl.cos, spl.sin, spl.tok, spl.pos, spl.next_tok, attention_splits=3)
    spl.prefill(prompt)
    spl.tok.copy_(first), spl.pos.fill_(prompt.numel())
    spl.fused.run()
    one = decode.GreedyDecoder(model, use_graph=False, fused=True)
    one.prefill(prompt)
    one.tok.copy_(first), one.pos.fill_(prompt.numel())
    one.fused.run()
    assert (spl.fused.logits.float() - one.fused.logits.float()).abs().max() <= 1e-2
    # the captured fused step replays to the same tokens as the eager fused step
    eager, _, _ = decode.GreedyDecoder(model, use_graph=False, fused=True, chain=chain).generate(prompt, 10)
    graphed = decode.GreedyDecoder(model, use_graph=True, fused=True, chain=chain)
    for _ in range(3):
        got, _, _ = graphed.generate(prompt, 10)
        assert torch.equal(got, eager)


def test_module_path_with_single_token_glue_matches_torch_expressions(fp16_out):
    """The decoder's modules with the library's glue kernels between the linears (norm + residual add, rotary + cache
    append + attention, gate) against the same modules with torch expressions, teacher forced, and under a graph."""
    cfg = decode.DecoderConfig(**TINY)
    model, _, _ = decode.build_decoder(cfg, seed=8)
    prompt = torch.randint(0, cfg.vocab, (11,), generator=torch.Generator().manual_seed(4))
    ref = decode.GreedyDecoder(model, use_graph=False)
    fast = decode.GreedyDecoder(model, use_graph=False, module_glue=True)
    first = ref.prefill(prompt)
    fast.prefill(prompt)
    tok = first.clone()
    for step in range(5):
        pos = torch.tensor([prompt.numel() + step], device="cuda")
        want = model.forward_tokens(tok, pos, ref.caches, ref.cos, ref.sin).float()
        fast.tok.copy_(tok), fast.pos.copy_(pos)
        fast._step()
        assert all(m.glue is None for m in model.modules() if hasattr(m, "glue"))   # switched back after the step
        assert int(fast.pos) == int(pos) + 1
        for (ka, va), (kb, vb) in zip(ref.caches, fast.caches):
            assert (ka[:, int(pos)].float() - kb[:, int(pos)].float()).abs().max() <= 2e-2
            assert (va[:, int(pos)].float() - vb[:, int(pos)].float()).abs().max() <= 2e-2
        # the step's own logits are not kept: compare the pick, and the logits of a second pass through the glue path
        model.use_single_token_glue(fast.cos, fast.sin, fast.pos)
        fast.pos.copy_(pos)
        got = model.forward_tokens(tok, fast.pos, fast.caches, fast.cos, fast.sin).float()
        model.use_single_token_glue()
        fast.pos.copy_(pos + 1)
        assert (got - want).abs().max() <= 1e-2 + 1e-2 * want.abs().max(), step
        tok = want.argmax(-1)
    eager, _, _ = decode.GreedyDecoder(model, use_graph=False, module_glue=True).generate(prompt, 8)
    graphed = decode.GreedyDecoder(model, use_graph=True, module_glue=True)
    for _ in range(2):
        assert torch.equal(graphed.generate(prompt, 8)[0], eager)


GEOM_8B = dict(hidden=4096, layers=2, heads=32, kv_heads=8, head_dim=128, intermediate=14336, vocab=4096, max_len=640,
               group_size=128, rank=128)


@pytest.mark.parametrize("chain", ["full", "mlp", False], ids=["chained", "chained_mlp", "separate_glue"])
def test_fused_step_at_8b_geometry_matches_effective_weight_network(fp16_out, chain):
    """Two layers of the Llama-3.1-8B geometry (hidden 4096, 32 query / 8 KV heads of 128, SwiGLU 14336, W4A16 g = 128,
    rank 128) with 512 cached positions: the fused single-token step (group launches, attention split over 4 workgroups
    per head, glue kernels that carry the projections) against the same network with every quantised module replaced
    by an fp32 matmul on its effective weight, teacher forced; the cache of both is filled by the yardstick network."""
    cfg = decode.DecoderConfig(**GEOM_8B)
    model, _, _ = decode.build_decoder(cfg, seed=21)
    assert sum(isinstance(m, corr.AddSVDCorrection) for m in model.modules()) == 7 * cfg.layers
    prompt = torch.randint(0, cfg.vocab, (512,), generator=torch.Generator().manual_seed(6))
    deq = {}
    ref = decode.GreedyDecoder(model, use_graph=False)
    fus = decode.GreedyDecoder(model, use_graph=False, fused=True, chain=chain)     # reads the quantised buffers of the modules
    assert fus.fused.chained == chain
    bare = decode.GreedyDecoder(model, use_graph=False)
    saved = _swap_in_reference(model, with_correction=False, deq_cache=deq)
    bare.prefill(prompt)
    _restore(saved)
    saved = _swap_in_reference(model, deq_cache=deq)
    first = ref.prefill(prompt)
    fus.prefill(prompt)
    tok = first.clone()
    worst = 0.0
    for step in range(4):
        print(f"8B-geometry step {step}", flush=True)
        pos = torch.tensor([prompt.numel() + step], device="cuda")
        want = model.forward_tokens(tok, pos, ref.caches, ref.cos, ref.sin).float()
        fus.tok.copy_(tok), fus.pos.copy_(pos)
        fus.fused.run()
        got = fus.fused.logits.float()
        err = float((got - want).abs().max())
        worst = max(worst, err)
        assert err <= 1e-2 + 1e-2 * float(want.abs().max()), (step, err)
        assert int(fus.pos) == int(pos) + 1 and int(fus.tok) == int(got.argmax())
        # the step left the same key / value rows in its cache as the yardstick network
        for (ka, va), (kb, vb) in zip(ref.caches, fus.caches):
            assert (ka[:, int(pos)].float() - kb[:, int(pos)].float()).abs().max() <= 2e-2
            assert (va[:, int(pos)].float() - vb[:, int(pos)].float()).abs().max() <= 2e-2
        tok = want.argmax(-1)
    _restore(saved)
    # the check discriminates: the same step on the network without the correction is much further away
    saved = _swap_in_reference(model, with_correction=False, deq_cache=deq)
    pos = torch.tensor([prompt.numel()], device="cuda")
    without = model.forward_tokens(first, pos, bare.caches, bare.cos, bare.sin).float()
    _restore(saved)
    fus2 = decode.GreedyDecoder(model, use_graph=False, fused=True, chain=chain)
    saved = _swap_in_reference(model, deq_cache=deq)
    fus2.prefill(prompt)
    _restore(saved)
    fus2.tok.copy_(first), fus2.pos.copy_(pos)
    fus2.fused.run()
    assert float((fus2.fused.logits.float() - without).abs().max()) > 5 * max(worst, 1e-3)


def test_fused_step_with_a_factor_pair_per_module(fp16_out):
    """Artifacts whose q / k / v (gate / up) hold different right factors cannot share one group launch: the fused step
    must run them one by one, each with its own r, and still match the module path."""
    cfg = decode.DecoderConfig(**TINY)
    model, _, _ = decode.build_decoder(cfg, seed=13)
    g = torch.Generator(device="cuda").manual_seed(2)
    for layer in model.model.layers:
        for owner, name in ((layer.self_attn, "k_proj"), (layer.mlp, "up_proj")):
            # a solo wrapper with its own R instead of the group's, as the patcher builds for a key without "B_shared"
            old = getattr(owner, name)
            old.group_cache.members.remove(old)
            R = (torch.randn(old.B_q.shape, device="cuda", generator=g) * old.B_q.size(1) ** -0.5).half()
            setattr(owner, name, corr.AddSVDCorrection(old.inner, old.A_q, R, "solo", False, None, 1.0))
    prompt = torch.randint(0, cfg.vocab, (9,), generator=torch.Generator().manual_seed(4))
    ref = decode.GreedyDecoder(model, use_graph=False)
    fus = decode.GreedyDecoder(model, use_graph=False, fused=True)
    assert fus.fused.plan[0]["qkv"]["per_member"] is not None and fus.fused.plan[0]["o"]["per_member"] is None
    assert not fus.fused.chained  # the chained launches need one shared factor per group
    first = ref.prefill(prompt)
    fus.prefill(prompt)
    pos = torch.tensor([prompt.numel()], device="cuda")
    want = model.forward_tokens(first, pos, ref.caches, ref.cos, ref.sin).float()
    fus.tok.copy_(first), fus.pos.copy_(pos)
    fus.fused.run()
    assert (fus.fused.logits.float() - want).abs().max() <= 1e-2 + 1e-2 * want.abs().max()


def test_perplexity_windows_and_effective_weight_network(fp16_out, tmp_path):
    from glowq_amd import evaluate
    cfg = decode.DecoderConfig(**TINY)
    model, _, _ = decode.build_decoder(cfg, seed=9)
    ids = torch.randint(0, cfg.vocab, (131,), generator=torch.Generator().manual_seed(5))
    np.save(tmp_path / "ids.npy", ids.numpy().astype(np.int32))
    assert torch.equal(evaluate.load_local_tokens(str(tmp_path / "ids.npy"), cfg.vocab), ids)
    (tmp_path / "raw.bin").write_bytes(bytes([1, 2, 250]))
    assert evaluate.load_local_tokens(str(tmp_path / "raw.bin"), cfg.vocab).tolist() == [1, 2, 250]
    with pytest.raises(ValueError):
        evaluate.load_local_tokens(str(tmp_path / "raw.bin"), 200)
    ppl, secs = evaluate.evaluate_token_ids(model, ids, seq_len=40)
    # the same windows by hand on the effective-weight network: 40+40+40+11 tokens -> 39+39+39+10 predictions
    saved = _swap_in_reference(model)
    tot, cnt = 0.0, 0
    for b in range(0, 131, 40):
        w = ids[b:b + 40]
        lg = torch.from_numpy(_logits(model, w))
        lp = torch.log_softmax(lg[:-1].double(), dim=-1)
        tot += float(-lp[torch.arange(w.numel() - 1), w[1:]].sum())
        cnt += w.numel() - 1
    _restore(saved)
    assert cnt == 127
    want = float(np.exp(tot / cnt))
    assert abs(ppl - want) <= 5e-3 * want and secs > 0
    # a window of one token is skipped; uniform logits give PPL = vocab whatever the windows are
    model.lm_head.weight.zero_()
    ppl0, _ = evaluate.evaluate_token_ids(model, ids[:41], seq_len=40)
    assert abs(ppl0 - cfg.vocab) <= 1e-3 * cfg.vocab
    with pytest.raises(ValueError):
        evaluate.evaluate_token_ids(model, ids, seq_len=cfg.max_len + 1)


def test_glue_with_projection_matches_separate_launches(ext, fp16_out):
    g = torch.Generator(device="cuda").manual_seed(21)
    H, rank = 1024, 64
    x = torch.randn(1, H, device="cuda", generator=g).half()
    d = torch.randn(1, H, device="cuda", generator=g).half()
    w = (1 + 0.1 * torch.randn(H, device="cuda", generator=g)).half()
    R = (torch.randn(rank, H, device="cuda", generator=g) * H ** -0.5).half()
    x_ref, h_ref = x.clone(), torch.empty_like(x)
    ext.add_rmsnorm(x_ref, d, w, h_ref, 1e-5)
    r_ref = ext.shared_proj(h_ref, R)
    x_out, h, r = torch.empty_like(x), torch.empty_like(x), torch.empty(1, rank, dtype=torch.float16, device="cuda")
    ext.add_rmsnorm_proj(x, d, w, x_out, h, R, r, 1e-5)
    assert torch.equal(x_out, x_ref) and torch.equal(h, h_ref)
    assert (r.float() - r_ref.float()).abs().max() <= 2e-3 * r_ref.float().abs().max() + 1e-3
    with pytest.raises(RuntimeError):
        ext.add_rmsnorm_proj(x, d, w, x, h, R, r, 1e-5)           # in place is refused: other workgroups still read x

    n = 2048
    gate, up = torch.randn(1, n, device="cuda", generator=g).half() * 2, torch.randn(1, n, device="cuda", generator=g).half()
    R2 = (torch.randn(rank, n, device="cuda", generator=g) * n ** -0.5).half()
    act_ref = torch.empty_like(gate)
    ext.silu_mul(gate, up, act_ref)
    r2_ref = ext.shared_proj(act_ref, R2)
    act, r2 = torch.empty_like(gate), torch.empty(1, rank, dtype=torch.float16, device="cuda")
    ext.silu_mul_proj(gate, up, act, R2, r2)
    assert torch.equal(act, act_ref)
    assert (r2.float() - r2_ref.float()).abs().max() <= 2e-3 * r2_ref.float().abs().max() + 1e-3
