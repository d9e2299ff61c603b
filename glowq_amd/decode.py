"""Minimal Llama-style decoder over the W4A16 + GlowQ linears, with a HIP-graph-captured decode step.

The counterpart of what the reference measures with `generate()` (`measure_generation_metrics`,
src/step3_eval_dataset.py:705-798: TTFB = wall of a 1-token generate, tok/s = new tokens / wall) and of the manual
greedy loop with a KV cache in test/step3_1_layerwise.py:181-210 -- without Hugging Face: random-init weights of
the named architecture (RMSNorm, RoPE, grouped-query attention, SwiGLU), HF-style module names
(`model.layers.N.self_attn.{q,k,v,o}_proj`, `model.layers.N.mlp.{gate,up,down}_proj`) so that
`convert_to_cuda_w4a16` and `patch_svd_correction_wrappers` apply unchanged, and the artifact key scheme of
src/step2_rsvd.py:487-527 for the low-rank factors.

    python -m glowq_amd.decode --layers 32 --prompt 512 --new 256        # Llama-3.1-8B shape, batch 1

Two ways to run a token: the module path (`Decoder.forward_tokens`: the patched linears inside plain torch norms, RoPE
and attention; used for prefill and as the yardstick) and `FusedStep` (single-token decode as a fixed chain of this
library's launches: add+RMSNorm, group linears, RoPE+cache append+attention, SwiGLU gating, greedy pick; only the
lm_head matmul and the embedding lookup stay torch ops).
"""
from __future__ import annotations

import argparse
import json
import time
from dataclasses import dataclass
from typing import Dict, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from .correction import AddSVDCorrection, patch_svd_correction_wrappers, patch_svd_correction_wrappers_cumulative
from .kernels import (CHAIN_ACC_BYTES, CHAIN_EPI_NONE, CHAIN_EPI_RESIDUAL, CHAIN_EPI_SWIGLU, CHAIN_PRO_ACC, CHAIN_PRO_NORM_ACC,
                      CHAIN_PRO_PLAIN, PreparedGroup, load_w4a16_extension)
from .linear import CudaW4A16Linear, convert_to_cuda_w4a16, refresh_env_knobs


@dataclass
class DecoderConfig:
    hidden: int = 4096
    layers: int = 32
    heads: int = 32
    kv_heads: int = 8
    head_dim: int = 128
    intermediate: int = 14336
    vocab: int = 128256
    rope_theta: float = 500000.0
    rms_eps: float = 1e-5
    max_len: int = 1024
    group_size: int = 128
    rank: int = 128


class _Glue:
    """What the modules need to run a single token through the library's glue kernels instead of torch expressions
    (`Decoder.use_single_token_glue`): the extension, the rotary tables [max_len, head_dim] fp32 and the device tensor
    holding the token's position."""

    def __init__(self, ext, cos_t, sin_t, pos):
        self.ext, self.cos_t, self.sin_t, self.pos = ext, cos_t, sin_t, pos


class RMSNorm(nn.Module):
    def __init__(self, dim: int, eps: float):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim, dtype=torch.float16))
        self.eps = eps
        self.glue: Optional[_Glue] = None

    def forward(self, x, delta=None):
        """rmsnorm(x) * weight; with `delta` (single-token glue only) x += delta first, in place."""
        if self.glue is not None and x.dim() == 2 and x.size(0) == 1 and x.dtype == torch.float16:
            h = torch.empty_like(x)
            self.glue.ext.add_rmsnorm(x, delta, self.weight, h, self.eps)
            return h
        if delta is not None:
            x.add_(delta)
        return F.rms_norm(x, (x.size(-1),), self.weight, self.eps)


class Attention(nn.Module):
    def __init__(self, cfg: DecoderConfig):
        super().__init__()
        self.cfg = cfg
        h, d = cfg.hidden, cfg.head_dim
        self.q_proj = nn.Linear(h, cfg.heads * d, bias=False)
        self.k_proj = nn.Linear(h, cfg.kv_heads * d, bias=False)
        self.v_proj = nn.Linear(h, cfg.kv_heads * d, bias=False)
        self.o_proj = nn.Linear(cfg.heads * d, h, bias=False)
        self.glue: Optional[_Glue] = None

    def forward(self, x, cos, sin, cache_k, cache_v, pos_idx, mask):
        """x [T, hidden]; cos/sin [T, head_dim]; caches [kv_heads, max_len, head_dim]; pos_idx [T] (device,
        positions of the T tokens); mask [T, max_len] additive, or None when the T tokens are positions 0..T-1 of an
        empty cache (prefill): attention then runs causally over the new keys alone."""
        cfg = self.cfg
        T = x.size(0)
        if self.glue is not None and T == 1 and mask is not None and pos_idx is self.glue.pos:
            # one launch: rotary embedding, cache append and attention of the one query over the cache
            q, k, v = self.q_proj(x), self.k_proj(x), self.v_proj(x)
            if q.dtype == k.dtype == v.dtype == torch.float16:
                out = torch.empty_like(q)
                self.glue.ext.rope_attend(q[0], k[0], v[0], self.glue.cos_t, self.glue.sin_t, pos_idx, cache_k, cache_v, out[0],
                                          cfg.head_dim ** -0.5)
                return self.o_proj(out)
        q = self.q_proj(x).view(T, cfg.heads, cfg.head_dim).transpose(0, 1)      # [H, T, d]
        k = self.k_proj(x).view(T, cfg.kv_heads, cfg.head_dim).transpose(0, 1)   # [KV, T, d]
        v = self.v_proj(x).view(T, cfg.kv_heads, cfg.head_dim).transpose(0, 1)
        q, k = _rope(q, cos, sin), _rope(k, cos, sin)
        cache_k.index_copy_(1, pos_idx, k.to(cache_k.dtype))
        cache_v.index_copy_(1, pos_idx, v.to(cache_v.dtype))
        if mask is None:
            out = F.scaled_dot_product_attention(q.unsqueeze(0), k.unsqueeze(0), v.unsqueeze(0), is_causal=True, enable_gqa=True)
        else:
            out = F.scaled_dot_product_attention(q.to(cache_k.dtype).unsqueeze(0), cache_k.unsqueeze(0), cache_v.unsqueeze(0),
                                                 attn_mask=mask.unsqueeze(0).unsqueeze(0), enable_gqa=True)
        out = out.squeeze(0).transpose(0, 1).reshape(T, cfg.heads * cfg.head_dim)
        return self.o_proj(out)


def _rope(t, cos, sin):
    d = t.size(-1) // 2
    rot = torch.cat((-t[..., d:], t[..., :d]), dim=-1)
    return t * cos + rot * sin


class MLP(nn.Module):
    def __init__(self, cfg: DecoderConfig):
        super().__init__()
        self.gate_proj = nn.Linear(cfg.hidden, cfg.intermediate, bias=False)
        self.up_proj = nn.Linear(cfg.hidden, cfg.intermediate, bias=False)
        self.down_proj = nn.Linear(cfg.intermediate, cfg.hidden, bias=False)
        self.glue: Optional[_Glue] = None

    def forward(self, x):
        gate, up = self.gate_proj(x), self.up_proj(x)
        if self.glue is not None and x.size(0) == 1 and gate.dtype == up.dtype == torch.float16:
            act = torch.empty_like(gate)
            self.glue.ext.silu_mul(gate, up, act)
            return self.down_proj(act)
        return self.down_proj(F.silu(gate) * up)


class DecoderLayer(nn.Module):
    def __init__(self, cfg: DecoderConfig):
        super().__init__()
        self.self_attn = Attention(cfg)
        self.mlp = MLP(cfg)
        self.input_layernorm = RMSNorm(cfg.hidden, cfg.rms_eps)
        self.post_attention_layernorm = RMSNorm(cfg.hidden, cfg.rms_eps)

    def forward(self, x, cos, sin, cache_k, cache_v, pos_idx, mask):
        if self.input_layernorm.glue is not None and x.size(0) == 1 and x.dtype == torch.float16:
            # single-token glue: the residual add rides on the norm launch that follows it (x is updated in place)
            attn = self.self_attn(self.input_layernorm(x), cos, sin, cache_k, cache_v, pos_idx, mask)
            h = self.post_attention_layernorm(x, delta=attn.to(x.dtype))
            return x.add_(self.mlp(h).to(x.dtype))
        x = x + self.self_attn(self.input_layernorm(x), cos, sin, cache_k, cache_v, pos_idx, mask)
        return x + self.mlp(self.post_attention_layernorm(x))


class _Body(nn.Module):
    def __init__(self):
        super().__init__()


class Decoder(nn.Module):
    """`model.embed_tokens`, `model.layers`, `model.norm`, `lm_head`: the attribute layout HF Llama uses."""

    def __init__(self, cfg: DecoderConfig):
        super().__init__()
        self.cfg = cfg
        self.model = _Body()
        self.model.embed_tokens = nn.Embedding(cfg.vocab, cfg.hidden)
        self.model.layers = nn.ModuleList()
        self.model.norm = RMSNorm(cfg.hidden, cfg.rms_eps)
        self.lm_head = nn.Linear(cfg.hidden, cfg.vocab, bias=False)

    def use_single_token_glue(self, cos_t=None, sin_t=None, pos=None) -> None:
        """Switches the modules' single-token path to the library's glue kernels (one launch each for norm + residual
        add, rotary + cache append + attention, and the gate), or back to torch expressions when called without
        arguments.  `cos_t` / `sin_t` are the tables of `rope_tables`, `pos` the int64 device tensor the decode loop
        passes as `pos_idx` for its one token (the attention kernel reads the position from it on the device)."""
        glue = _Glue(load_w4a16_extension(), cos_t, sin_t, pos) if cos_t is not None else None
        for mod in self.modules():
            if isinstance(mod, (RMSNorm, Attention, MLP)):
                mod.glue = glue

    def rope_tables(self, device):
        cfg = self.cfg
        inv = 1.0 / (cfg.rope_theta ** (torch.arange(0, cfg.head_dim, 2, dtype=torch.float32, device=device) / cfg.head_dim))
        ang = torch.arange(cfg.max_len, dtype=torch.float32, device=device)[:, None] * inv[None, :]
        ang = torch.cat((ang, ang), dim=-1)
        return ang.cos(), ang.sin()

    def forward_tokens(self, tokens, pos_idx, caches, cos_t, sin_t, from_empty_cache: bool = False):
        """tokens [T] (device), pos_idx [T] (device): logits [T, vocab] after writing the KV cache at pos_idx.
        `from_empty_cache`: pos_idx is 0..T-1 and nothing older is cached, so attention needs no mask over the cache."""
        cfg = self.cfg
        x = self.model.embed_tokens(tokens)
        cos, sin = cos_t.index_select(0, pos_idx).to(x.dtype), sin_t.index_select(0, pos_idx).to(x.dtype)
        mask = None
        if not from_empty_cache:
            col = torch.arange(cfg.max_len, device=tokens.device)
            mask = torch.where(col[None, :] <= pos_idx[:, None], 0.0, float("-inf")).to(torch.float16)
        for layer, (ck, cv) in zip(self.model.layers, caches):
            x = layer(x, cos, sin, ck, cv, pos_idx, mask)
        return self.lm_head(self.model.norm(x))


def build_decoder(cfg: DecoderConfig, device="cuda", seed: int = 3, with_correction: bool = True,
                  groups_to_patch: Optional[set] = None) -> Tuple[Decoder, Dict[str, torch.Tensor], Dict[str, str]]:
    """Random-init weights ~ N(0, 0.02) layer by layer on the device, each layer quantised as soon as it exists
    (an 8B model never holds more than one layer in fp16), then synthetic low-rank factors in the artifact key
    scheme (R ~ N(0, 1/K), L ~ N(0, 0.01^2)) patched in with the reference's patcher."""
    g = torch.Generator(device=device).manual_seed(seed)
    model = Decoder(cfg).half()
    model.model.embed_tokens.to(device)
    model.model.norm.to(device)
    model.lm_head.to(device)
    with torch.no_grad():
        model.model.embed_tokens.weight.normal_(0, 0.02, generator=g)
        model.lm_head.weight.normal_(0, 0.02, generator=g)
    for _ in range(cfg.layers):
        layer = DecoderLayer(cfg).half().to(device)
        with torch.no_grad():
            for mod in layer.modules():
                if isinstance(mod, nn.Linear):
                    mod.weight.normal_(0, 0.02, generator=g)
        convert_to_cuda_w4a16(layer, cfg.group_size)
        model.model.layers.append(layer)
    shared: Dict[str, torch.Tensor] = {}
    bmap: Dict[str, str] = {}
    if with_correction:
        def rnd(*shape, std):
            return (torch.randn(*shape, device=device, generator=g) * std).half()

        for i, layer in enumerate(model.model.layers):
            pre = f"model.layers.{i}"
            for gname, sub, members in (("qkv", "self_attn", ("q_proj", "k_proj", "v_proj")), ("mlp", "mlp", ("gate_proj", "up_proj"))):
                K = getattr(getattr(layer, sub), members[0]).in_features
                shared[f"layer{i}_{gname}.B_shared"] = rnd(cfg.rank, K, std=K ** -0.5)
                for mname in members:
                    N = getattr(getattr(layer, sub), mname).out_features
                    shared[f"layer{i}_{gname}.{mname}.A"] = rnd(N, cfg.rank, std=0.01)
                    bmap[f"{pre}.{sub}.{mname}.weight"] = f"layer{i}_{gname}.B_shared"
            for sub, mname in (("self_attn", "o_proj"), ("mlp", "down_proj")):
                lin = getattr(getattr(layer, sub), mname)
                mod = f"{pre}.{sub}.{mname}"
                shared[f"{mod}.A"] = rnd(lin.out_features, cfg.rank, std=0.01)
                shared[f"{mod}.B"] = rnd(cfg.rank, lin.in_features, std=lin.in_features ** -0.5)
                bmap[f"{mod}.weight"] = f"{mod}.B"
        if groups_to_patch is None:
            patch_svd_correction_wrappers(model, shared, bmap, alpha_svd=1.0)
        else:
            patch_svd_correction_wrappers_cumulative(model, shared, bmap, groups_to_patch, alpha_svd=1.0)
    return model.eval(), shared, bmap


def load_glowq_artifacts(shared_path: str, bmap_path: str, device="cuda"):
    """`low_rank_shared.pt` (dict name -> fp16 tensor) and `b_ref_map.json` (weight name -> key of its right factor)
    as written by the reference's step 2 (src/step2_rsvd.py:519-527; consumer src/step3_eval_dataset.py:1077-1080).
    Loaded with `weights_only=True`: nothing from the file is executed."""
    shared = torch.load(shared_path, map_location=device, weights_only=True)
    with open(bmap_path) as f:
        bmap = json.load(f)
    return shared, bmap


# How much of the work between the linears the fused step folds into the group launches by default (FusedStep).
DEFAULT_CHAIN = "mlp"


class FusedStep:
    """One decode token as a fixed chain of launches on static buffers, ready for HIP-graph capture.  Reads the
    quantised buffers and low-rank factors straight out of the model's modules.
    Without `chain` a layer is nine launches: q|k|v, attention, merge of its splits, o_proj, gate|up, down_proj and,
    between them, two norm launches and a gate launch that also produce the projections r = x R^T.
    `chain` (for a model whose four groups per layer all carry a shared correction of one rank) moves that work into
    the group launches on either side of it (glowq_w4a16_group_forward_chained): "mlp" folds the gate into gate|up and
    the residual add, the next layer's norm and its projection into down_proj and q|k|v (seven launches per layer);
    "full" also folds the norm in front of gate|up into o_proj and gate|up (six)."""

    def __init__(self, model: Decoder, caches, cos, sin, tok, pos, next_tok, share: bool = True, attention_splits: int = 4,
                 chain=DEFAULT_CHAIN):
        cfg = model.cfg
        self.share = share  # False: every module projects x on R by itself and launches alone (the no-sharing comparator)
        self.model, self.cfg = model, cfg
        self.ext = load_w4a16_extension()
        dev = model.lm_head.weight.device
        self.caches, self.cos, self.sin = caches, cos, sin
        self.tok, self.pos, self.next_tok = tok, pos, next_tok
        f16 = dict(dtype=torch.float16, device=dev)
        qd, kd = cfg.heads * cfg.head_dim, cfg.kv_heads * cfg.head_dim
        self.x = torch.zeros(1, cfg.hidden, **f16)
        self.x_alt = torch.zeros(1, cfg.hidden, **f16)   # the residual stream alternates between the two
        self.h = torch.zeros(1, cfg.hidden, **f16)
        self.qkv = torch.zeros(1, qd + 2 * kd, **f16)
        self.attn = torch.zeros(1, qd, **f16)
        self.o = torch.zeros(1, cfg.hidden, **f16)
        self.gu = torch.zeros(1, 2 * cfg.intermediate, **f16)
        self.act = torch.zeros(1, cfg.intermediate, **f16)
        self.dn = torch.zeros(1, cfg.hidden, **f16)
        self.logits = torch.zeros(1, cfg.vocab, **f16)
        # cached positions dealt to several workgroups per head; the merge kernel also produces o_proj's projection, so the
        # launch count is the same as with one workgroup per head (2.36 ms per token at 4 or 8 splits, 2.40 ms at 1, with
        # 512..768 cached tokens)
        self.splits = attention_splits
        self.partials = torch.zeros(cfg.heads, attention_splits, cfg.head_dim + 4, dtype=torch.float32, device=dev)
        self.scale = cfg.head_dim ** -0.5
        self.plan = []
        for layer in model.model.layers:
            at, mlp = layer.self_attn, layer.mlp
            self.plan.append({
                "ln1": layer.input_layernorm, "ln2": layer.post_attention_layernorm,
                "qkv": self._group([at.q_proj, at.k_proj, at.v_proj],
                                   [self.qkv[:, :qd], self.qkv[:, qd:qd + kd], self.qkv[:, qd + kd:]], f16),
                "o": self._group([at.o_proj], [self.o], f16),
                "gu": self._group([mlp.gate_proj, mlp.up_proj],
                                  [self.gu[:, :cfg.intermediate], self.gu[:, cfg.intermediate:]], f16),
                "down": self._group([mlp.down_proj], [self.dn], f16),
            })
        self.q_view, self.k_view, self.v_view = self.qkv[0, :qd], self.qkv[0, qd:qd + kd], self.qkv[0, qd + kd:]
        if chain is True:
            chain = "full"
        if chain not in (False, None, "full", "mlp"):
            raise ValueError("chain must be False, 'mlp' or 'full'")
        self.chained = chain if (chain and share and attention_splits > 1 and self._chainable()) else False
        if self.chained:
            # the next group's right factor transposed (rows = the producing group's output rows), and one accumulator
            # per hand-over, all cleared by one fill at the head of the step
            n = len(self.plan)
            self.acc = torch.zeros(n, 3, CHAIN_ACC_BYTES, dtype=torch.uint8, device=dev)
            for i, lay in enumerate(self.plan):
                lay["Rt_gu"] = lay["gu"]["R"].t().contiguous()
                lay["Rt_down"] = lay["down"]["R"].t().contiguous()
                lay["Rt_next"] = self.plan[i + 1]["qkv"]["R"].t().contiguous() if i + 1 < n else None
                lay["ln1_next"] = self.plan[i + 1]["ln1"] if i + 1 < n else None

    def _chainable(self) -> bool:
        """Every group of every layer: one launch with a shared right factor, one rank throughout, shapes the chained
        launch takes; o_proj and down_proj alone in their groups, gate and up of equal width."""
        ranks = set()
        for lay in self.plan:
            for name in ("qkv", "o", "gu", "down"):
                grp = lay[name]
                if grp["per_member"] is not None or grp["R"] is None or any(m["L"] is None for m in grp["members"]):
                    return False
                K, gs, rank = grp["call"].K, grp["gs"], grp["R"].size(0)
                ranks.add(rank)
                if K % 32 or K > 9 * 2048 or gs < 128 or gs & (gs - 1) or rank % 2 or not 2 <= rank <= 256:
                    return False
            if len(lay["o"]["members"]) != 1 or len(lay["down"]["members"]) != 1 or len(lay["gu"]["members"]) != 2:
                return False
            if lay["gu"]["members"][0]["qweight"].size(0) != lay["gu"]["members"][1]["qweight"].size(0):
                return False
        return len(ranks) == 1

    @staticmethod
    def _group(mods, outs, f16):
        """Launch description of a group.  The corrected members of one launch must share one right factor and one
        alpha (the group kernel applies a single r and a single alpha); artifacts with a factor pair per module
        (layer-wise, non-shared correction) get `per_member` instead: one projection and one launch per module."""
        members, factors, gs = [], [], None
        for mod in mods:
            inner = mod.inner if isinstance(mod, AddSVDCorrection) else mod
            if not isinstance(inner, CudaW4A16Linear):
                raise TypeError("FusedStep needs every projection converted to CudaW4A16Linear")
            L = None
            if isinstance(mod, AddSVDCorrection) and mod.alpha_svd != 0.0:
                L = mod.A_q
                factors.append((mod.B_q, float(mod.alpha_svd)))
            else:
                factors.append(None)
            gs = inner.group_size
            members.append({"qweight": inner.qweight_i32, "scales": inner.scales_f16, "qzeros": inner.qzeros_i32, "L": L,
                            "bias": inner.bias})
        corrected = [f for f in factors if f is not None]
        R, alpha = (corrected[0] if corrected else (None, 1.0))
        shared = all(a == alpha and (B.data_ptr() == R.data_ptr() or (B.shape == R.shape and bool(torch.equal(B, R))))
                     for B, a in corrected)
        ext = load_w4a16_extension()
        K = mods[0].inner.in_features if isinstance(mods[0], AddSVDCorrection) else mods[0].in_features

        def single(mem, Ri, ai, out):
            return {"members": [mem], "R": Ri, "r": torch.zeros(1, Ri.size(0), **f16) if Ri is not None else None,
                    "alpha": ai, "gs": gs, "outs": [out], "per_member": None,
                    "call": PreparedGroup(ext, [mem], K, gs, ai if Ri is not None else 0.0, R=Ri)}

        # the no-sharing comparator and artifacts with a factor pair per module: one projection and one launch per module
        per_member = [single(mem, *(f if f is not None else (None, 1.0)), out) for mem, f, out in zip(members, factors, outs)]
        if shared:
            r = torch.zeros(1, R.size(0), **f16) if R is not None else None
            return {"members": members, "R": R, "r": r, "alpha": alpha, "gs": gs, "outs": outs, "per_member": None,
                    "alone": per_member, "call": PreparedGroup(ext, members, K, gs, alpha if R is not None else 0.0, R=R)}
        return {"members": members, "R": None, "r": None, "alpha": 1.0, "gs": gs, "outs": outs, "per_member": per_member}

    def _norm(self, x, delta, ln, grp):
        """Residual add + RMSNorm into self.h; with a shared group behind it the projection r = h R^T comes out of the same
        launch.  Returns (residual stream after the add, whether r is already computed)."""
        if self.share and grp["R"] is not None:
            nxt = self.x_alt if x is self.x else self.x
            self.ext.add_rmsnorm_proj(x, delta, ln.weight, nxt, self.h, grp["R"], grp["r"], ln.eps)
            return nxt, True
        self.ext.add_rmsnorm(x, delta, ln.weight, self.h, ln.eps)
        return x, False

    def _linear(self, x, grp, r_ready=False):
        if grp["per_member"] is not None:
            for sub in grp["per_member"]:
                sub["call"].run(x, r=sub["r"], outs=sub["outs"])
            return
        if self.share:
            grp["call"].run(x, r=grp["r"], outs=grp["outs"], project=not r_ready)
            return
        # layer-wise correction without sharing (test/step3_1_layerwise.py:133-153): one projection and one launch per module
        for sub in grp["alone"]:
            sub["call"].run(x, r=sub["r"], outs=sub["outs"])

    @torch.no_grad()
    def _run_chained(self):
        ext, cfg = self.ext, self.cfg
        x = self.x  # the residual stream, updated in place by the o_proj and down_proj launches
        self.acc.zero_()
        for i, (lay, (ck, cv)) in enumerate(zip(self.plan, self.caches)):
            qkv, o, gu, down = lay["qkv"], lay["o"], lay["gu"], lay["down"]
            outs = [self.q_view, self.k_view, self.v_view]
            if i == 0:
                torch.index_select(self.model.model.embed_tokens.weight, 0, self.tok, out=self.x_alt)
                ext.add_rmsnorm_proj(self.x_alt, None, lay["ln1"].weight, x, self.h, qkv["R"], qkv["r"], lay["ln1"].eps)
                qkv["call"].run(self.h, r=qkv["r"], outs=qkv["outs"], project=False)
            else:
                qkv["call"].run_chained(x[0], CHAIN_PRO_NORM_ACC, CHAIN_EPI_NONE, outs=outs, norm_weight=lay["ln1"].weight,
                                        eps=lay["ln1"].eps, acc_in=self.acc[i - 1, 2])
            ext.rope_attend_split(self.q_view, self.k_view, self.v_view, self.cos, self.sin, self.pos, ck, cv, self.partials, self.scale)
            ext.attend_combine_proj(self.partials, self.attn, o["R"], o["r"])
            o["call"].run_chained(self.attn[0], CHAIN_PRO_PLAIN, CHAIN_EPI_RESIDUAL, r=o["r"][0], outs=[None], resid=x[0],
                                  next_norm_weight=lay["ln2"].weight, next_Rt=lay["Rt_gu"], acc_out=self.acc[i, 0])
            gu["call"].run_chained(x[0], CHAIN_PRO_NORM_ACC, CHAIN_EPI_SWIGLU, outs=[None, None], norm_weight=lay["ln2"].weight,
                                   eps=lay["ln2"].eps, acc_in=self.acc[i, 0], act=self.act[0], next_Rt=lay["Rt_down"],
                                   acc_out=self.acc[i, 1])
            nxt = lay["ln1_next"]
            down["call"].run_chained(self.act[0], CHAIN_PRO_ACC, CHAIN_EPI_RESIDUAL, acc_in=self.acc[i, 1], outs=[None], resid=x[0],
                                     next_norm_weight=nxt.weight if nxt is not None else None, next_Rt=lay["Rt_next"],
                                     acc_out=self.acc[i, 2] if nxt is not None else None)
        norm = self.model.model.norm
        ext.add_rmsnorm(x, None, norm.weight, self.h, norm.eps)
        torch.mm(self.h, self.model.lm_head.weight.t(), out=self.logits)
        ext.argmax_advance(self.logits, self.next_tok, self.tok, self.pos)

    @torch.no_grad()
    def _run_chained_mlp(self):
        """Seven launches per layer: the norm in front of gate|up stays a launch of its own (it also adds o_proj's output
        to the residual stream and projects on gate|up's right factor); the residual stream moves to the other of the
        two buffers there."""
        ext = self.ext
        cur = self.x
        self.acc.zero_()
        for i, (lay, (ck, cv)) in enumerate(zip(self.plan, self.caches)):
            qkv, o, gu, down = lay["qkv"], lay["o"], lay["gu"], lay["down"]
            if i == 0:
                torch.index_select(self.model.model.embed_tokens.weight, 0, self.tok, out=self.x_alt)
                ext.add_rmsnorm_proj(self.x_alt, None, lay["ln1"].weight, cur, self.h, qkv["R"], qkv["r"], lay["ln1"].eps)
                qkv["call"].run(self.h, r=qkv["r"], outs=qkv["outs"], project=False)
            else:
                qkv["call"].run_chained(cur[0], CHAIN_PRO_NORM_ACC, CHAIN_EPI_NONE, outs=[self.q_view, self.k_view, self.v_view],
                                        norm_weight=lay["ln1"].weight, eps=lay["ln1"].eps, acc_in=self.acc[i - 1, 2])
            ext.rope_attend_split(self.q_view, self.k_view, self.v_view, self.cos, self.sin, self.pos, ck, cv, self.partials, self.scale)
            ext.attend_combine_proj(self.partials, self.attn, o["R"], o["r"])
            o["call"].run(self.attn, r=o["r"], outs=o["outs"], project=False)
            nxt_buf = self.x_alt if cur is self.x else self.x
            ext.add_rmsnorm_proj(cur, self.o, lay["ln2"].weight, nxt_buf, self.h, gu["R"], gu["r"], lay["ln2"].eps)
            cur = nxt_buf
            gu["call"].run_chained(self.h[0], CHAIN_PRO_PLAIN, CHAIN_EPI_SWIGLU, r=gu["r"][0], outs=[None, None], act=self.act[0],
                                   next_Rt=lay["Rt_down"], acc_out=self.acc[i, 1])
            nxt = lay["ln1_next"]
            down["call"].run_chained(self.act[0], CHAIN_PRO_ACC, CHAIN_EPI_RESIDUAL, acc_in=self.acc[i, 1], outs=[None], resid=cur[0],
                                     next_norm_weight=nxt.weight if nxt is not None else None, next_Rt=lay["Rt_next"],
                                     acc_out=self.acc[i, 2] if nxt is not None else None)
        norm = self.model.model.norm
        ext.add_rmsnorm(cur, None, norm.weight, self.h, norm.eps)
        torch.mm(self.h, self.model.lm_head.weight.t(), out=self.logits)
        ext.argmax_advance(self.logits, self.next_tok, self.tok, self.pos)

    @torch.no_grad()
    def run(self):
        if self.chained == "full":
            return self._run_chained()
        if self.chained == "mlp":
            return self._run_chained_mlp()
        ext, cfg = self.ext, self.cfg
        x = self.x
        torch.index_select(self.model.model.embed_tokens.weight, 0, self.tok, out=x)
        delta = None
        for lay, (ck, cv) in zip(self.plan, self.caches):
            x, ready = self._norm(x, delta, lay["ln1"], lay["qkv"])
            self._linear(self.h, lay["qkv"], ready)
            o = lay["o"]
            if self.splits > 1:
                # the context split over several workgroups per head; the merge also projects the result on o_proj's R
                ext.rope_attend_split(self.q_view, self.k_view, self.v_view, self.cos, self.sin, self.pos, ck, cv, self.partials, self.scale)
                ready = self.share and o["R"] is not None
                ext.attend_combine_proj(self.partials, self.attn, o["R"] if ready else None, o["r"] if ready else None)
                self._linear(self.attn, o, ready)
            else:
                ext.rope_attend(self.q_view, self.k_view, self.v_view, self.cos, self.sin, self.pos, ck, cv, self.attn, self.scale)
                self._linear(self.attn, o)
            x, ready = self._norm(x, self.o, lay["ln2"], lay["gu"])
            self._linear(self.h, lay["gu"], ready)
            gate, up, down = self.gu[:, :cfg.intermediate], self.gu[:, cfg.intermediate:], lay["down"]
            if self.share and down["R"] is not None:
                ext.silu_mul_proj(gate, up, self.act, down["R"], down["r"])
                self._linear(self.act, down, True)
            else:
                ext.silu_mul(gate, up, self.act)
                self._linear(self.act, down)
            delta = self.dn
        norm = self.model.model.norm
        ext.add_rmsnorm(x, delta, norm.weight, self.h, norm.eps)
        torch.mm(self.h, self.model.lm_head.weight.t(), out=self.logits)
        ext.argmax_advance(self.logits, self.next_tok, self.tok, self.pos)


class GreedyDecoder:
    """Prefill + greedy decode at batch 1 with a static KV cache; the one-token step is captured as a HIP graph."""

    def __init__(self, model: Decoder, use_graph: bool = True, fused: bool = False, share: bool = True,
                 attention_splits: int = 0, chain=DEFAULT_CHAIN, module_glue: bool = False):
        self.model = model
        cfg = model.cfg
        if attention_splits <= 0:
            # workgroups per head in the fused step's attention: 4 up to 2048 positions of cache, 8 beyond
            # (measured at 32 heads: 2.34 -> 2.28 ms per token at 3.6k tokens of context, 2.73 -> 2.57 at 7.7k;
            # 16 is slower than either, and at 0.5k to 0.8k tokens 4 beats 8)
            attention_splits = 4 if cfg.max_len <= 2048 else 8
        dev = model.lm_head.weight.device
        self.dev = dev
        self.caches = [(torch.zeros(cfg.kv_heads, cfg.max_len, cfg.head_dim, dtype=torch.float16, device=dev),
                        torch.zeros(cfg.kv_heads, cfg.max_len, cfg.head_dim, dtype=torch.float16, device=dev))
                       for _ in range(cfg.layers)]
        self.cos, self.sin = model.rope_tables(dev)
        self.tok = torch.zeros(1, dtype=torch.long, device=dev)
        self.pos = torch.zeros(1, dtype=torch.long, device=dev)
        self.next_tok = torch.zeros(1, dtype=torch.long, device=dev)
        self.use_graph = use_graph
        self.graph = None
        self.fused = FusedStep(model, self.caches, self.cos, self.sin, self.tok, self.pos, self.next_tok, share,
                               attention_splits, chain) if fused else None
        # module path: torch expressions between the linears (the default, what an unmodified model does) or the
        # library's single-token glue kernels
        self.module_glue = bool(module_glue) and not fused

    @torch.no_grad()
    def _step(self):
        """One token: logits of `tok` at `pos`, greedy pick, then advance `tok` and `pos` on the device (so a
        replayed graph needs no host-side update between tokens)."""
        if self.fused is not None:
            self.fused.run()
            return
        if self.module_glue:
            self.model.use_single_token_glue(self.cos, self.sin, self.pos)
        try:
            logits = self.model.forward_tokens(self.tok, self.pos, self.caches, self.cos, self.sin)
        finally:
            if self.module_glue:
                self.model.use_single_token_glue()
        self.next_tok.copy_(logits.argmax(-1))
        self.tok.copy_(self.next_tok)
        self.pos.add_(1)

    @torch.no_grad()
    def prefill(self, prompt: torch.Tensor) -> torch.Tensor:
        T = prompt.numel()
        pos = torch.arange(T, device=self.dev)
        logits = self.model.forward_tokens(prompt.to(self.dev), pos, self.caches, self.cos, self.sin, from_empty_cache=True)
        return logits[-1].argmax().reshape(1)

    @torch.no_grad()
    def capture(self):
        """Captures `_step`.  Its warm-up and the capture pass itself write the KV cache at `pos`, which the caller
        must treat as scratch (generate() points `pos` at the last cache slot meanwhile)."""
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            self._step()  # outside the capture: lazy initialisation, kernel attributes
            torch.cuda.synchronize()
            self.pos.sub_(1)
            self.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self.graph, stream=side):
                self._step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()

    @torch.no_grad()
    def generate(self, prompt: torch.Tensor, new_tokens: int):
        """Returns (tokens [new_tokens] on the host, ttfb_s, decode_s): TTFB = prefill + first token,
        decode_s = wall of the remaining new_tokens - 1 steps."""
        cfg = self.model.cfg
        if prompt.numel() + new_tokens > cfg.max_len - 1:
            raise ValueError("prompt + new tokens exceed the KV cache (the last slot is kept as capture scratch)")
        if self.use_graph and self.graph is None:
            self.tok.zero_()
            self.pos.fill_(cfg.max_len - 1)
            self.capture()
        out = torch.zeros(new_tokens, dtype=torch.long, device=self.dev)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        first = self.prefill(prompt)
        out[0:1].copy_(first)
        torch.cuda.synchronize()
        ttfb = time.perf_counter() - t0
        self.tok.copy_(first)
        self.pos.fill_(prompt.numel())
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for i in range(1, new_tokens):
            if self.graph is not None:
                self.graph.replay()
            else:
                self._step()
            out[i:i + 1].copy_(self.next_tok)
        torch.cuda.synchronize()
        decode_s = time.perf_counter() - t1
        return out.cpu(), ttfb, decode_s


def measure(layers: int = 32, prompt_tokens: int = 512, new_tokens: int = 256, vocab: int = 128256, graph: bool = True,
            fused: bool = True, share: bool = True, correction: bool = True, attention_splits: int = 0,
            chain=DEFAULT_CHAIN, module_glue: bool = True, model: Optional[Decoder] = None) -> dict:
    """Greedy decode of a random-init Llama-3.1-8B-shaped model at batch 1: time to the first token and tokens per
    second over the decode phase, the counterpart of `measure_generation_metrics` (src/step3_eval_dataset.py:705-798).
    `fused=False` decodes through the torch modules (CudaW4A16Linear / AddSVDCorrection inside the decoder's layers),
    with the library's single-token glue kernels between them (`module_glue`) or torch expressions."""
    import os

    os.environ.setdefault("W4A16_KERNEL_OUT_DTYPE", "fp16")
    refresh_env_knobs()
    t0 = time.perf_counter()
    if model is None:  # (a caller that measures several paths builds the model once and hands it in)
        cfg = DecoderConfig(layers=layers, vocab=vocab, max_len=max(1024, prompt_tokens + new_tokens + 8))
        model, _, _ = build_decoder(cfg, with_correction=correction)
        torch.cuda.synchronize()
    cfg = model.cfg
    build_s = time.perf_counter() - t0
    dec = GreedyDecoder(model, use_graph=graph, fused=fused, share=share, attention_splits=attention_splits, chain=chain,
                        module_glue=module_glue)
    chained = dec.fused.chained if dec.fused is not None else False
    g = torch.Generator().manual_seed(3)
    prompt = torch.randint(0, cfg.vocab, (prompt_tokens,), generator=g)
    dec.generate(prompt, 4)  # warm-up (also captures the graph)
    _, ttfb, decode_s = dec.generate(prompt, new_tokens)
    return {
        "workload": f"random-init Llama-style decoder, {cfg.layers} layers, hidden {cfg.hidden}, GQA {cfg.heads}/{cfg.kv_heads}x{cfg.head_dim}, "
                    f"SwiGLU {cfg.intermediate}, W4A16 g={cfg.group_size}" + (f" + GlowQ r={cfg.rank}" if correction else ""),
        "prompt_tokens": prompt_tokens, "new_tokens": new_tokens, "graph": graph, "fused_step": fused, "group_sharing": share,
        "chained_launches": chained, "module_glue": dec.module_glue,
        "launches_per_token": ({"full": 6 * cfg.layers + 6, "mlp": 7 * cfg.layers + 6, False: 9 * cfg.layers + 5}[chained]
                               if (fused and share and correction) else None),
        "ttfb_ms": round(ttfb * 1e3, 2), "decode_tok_per_s": round((new_tokens - 1) / decode_s, 1),
        "ms_per_token": round(decode_s * 1e3 / (new_tokens - 1), 3), "build_s": round(build_s, 1)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--prompt", type=int, default=512)
    ap.add_argument("--new", type=int, default=256)
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--no-sharing", action="store_true", help="fused step with one projection and one launch per module")
    ap.add_argument("--module-path", action="store_true", help="decode through the torch modules instead of the fused step")
    ap.add_argument("--torch-glue", action="store_true",
                    help="with --module-path: torch expressions between the linears instead of the library's single-token glue kernels")
    ap.add_argument("--no-correction", action="store_true")
    ap.add_argument("--chain", choices=["off", "mlp", "full"], default=None,
                    help="fused step: how much of the work between the linears the group launches take over (9 / 7 / 6 launches per layer)")
    ap.add_argument("--vocab", type=int, default=128256)
    ap.add_argument("--attention-splits", type=int, default=0,
                    help="workgroups per head in the fused step's attention (0: by the cache length)")
    args = ap.parse_args()
    print(json.dumps(measure(args.layers, args.prompt, args.new, vocab=args.vocab, graph=not args.no_graph,
                             fused=not args.module_path, share=not args.no_sharing, correction=not args.no_correction,
                             attention_splits=args.attention_splits,
                             chain={None: DEFAULT_CHAIN, "off": False, "mlp": "mlp", "full": "full"}[args.chain],
                             module_glue=not args.torch_glue)))


if __name__ == "__main__":
    main()
