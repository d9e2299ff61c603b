"""Perplexity of a decoder over a local file of token ids, window by window.

The counterpart of `evaluate` in the reference (src/step3_eval_dataset.py:802-866) without its tokenizer and dataset
download: the same non-overlapping windows of `seq_len` tokens, the mean next-token cross entropy of each window
weighted by its number of predicted tokens, PPL = exp(total / tokens); windows of fewer than two tokens are skipped.
Every window is one prefill pass (M = window length) through the patched linears, i.e. the tiled MFMA route.

    python -m glowq_amd.evaluate --tokens ids.npy --layers 2 --seq-len 2048     # random-init decoder: PPL ~ vocab
"""
from __future__ import annotations

import argparse
import json
import math
import os
import time
from typing import Tuple

import numpy as np
import torch
import torch.nn.functional as F

from .decode import Decoder, DecoderConfig, GreedyDecoder, build_decoder
from .linear import refresh_env_knobs


def load_local_tokens(path: str, vocab: int) -> torch.Tensor:
    """Token ids from a local file: `.npy` (any integer dtype), `.pt` (a 1-D integer tensor, loaded with
    weights_only=True), or any other file read as raw bytes (byte-level ids, needs vocab >= 256)."""
    ext = os.path.splitext(path)[1].lower()
    if ext == ".npy":
        ids = torch.from_numpy(np.load(path, allow_pickle=False).astype(np.int64).reshape(-1))
    elif ext == ".pt":
        ids = torch.load(path, map_location="cpu", weights_only=True).to(torch.int64).reshape(-1)
    else:
        with open(path, "rb") as f:
            ids = torch.from_numpy(np.frombuffer(f.read(), dtype=np.uint8).astype(np.int64))
    if ids.numel() and (int(ids.min()) < 0 or int(ids.max()) >= vocab):
        raise ValueError(f"token ids must lie in [0, {vocab})")
    return ids


@torch.no_grad()
def evaluate_token_ids(model: Decoder, input_ids: torch.Tensor, seq_len: int = 2048) -> Tuple[float, float]:
    """(ppl, seconds) over `input_ids` (1-D int64)."""
    cfg = model.cfg
    if seq_len > cfg.max_len:
        raise ValueError(f"seq_len {seq_len} exceeds the decoder's max_len {cfg.max_len}")
    dec = GreedyDecoder(model, use_graph=False)
    dev = dec.dev
    total_loss, total_tokens = 0.0, 0
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for begin in range(0, input_ids.numel(), seq_len):
        end = min(begin + seq_len, input_ids.numel())
        if end - begin <= 1:
            continue
        window = input_ids[begin:end].to(dev)
        pos = torch.arange(end - begin, device=dev)
        logits = model.forward_tokens(window, pos, dec.caches, dec.cos, dec.sin, from_empty_cache=True)
        loss = F.cross_entropy(logits[:-1].float(), window[1:])
        n = end - begin - 1
        total_loss += float(loss) * n
        total_tokens += n
    torch.cuda.synchronize()
    if total_tokens == 0:
        raise ValueError("need at least two tokens")
    return math.exp(total_loss / total_tokens), time.perf_counter() - t0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--tokens", help="local token-id file (.npy, .pt, or raw bytes); default: 8192 seeded random ids")
    ap.add_argument("--layers", type=int, default=2)
    ap.add_argument("--seq-len", type=int, default=2048)
    ap.add_argument("--vocab", type=int, default=128256)
    args = ap.parse_args()
    os.environ.setdefault("W4A16_KERNEL_OUT_DTYPE", "fp16")
    refresh_env_knobs()
    cfg = DecoderConfig(layers=args.layers, vocab=args.vocab, max_len=args.seq_len)
    model, _, _ = build_decoder(cfg)
    if args.tokens:
        ids = load_local_tokens(args.tokens, cfg.vocab)
    else:
        ids = torch.randint(0, cfg.vocab, (8192,), generator=torch.Generator().manual_seed(0))
    ppl, secs = evaluate_token_ids(model, ids, args.seq_len)
    print(json.dumps({"ppl": round(ppl, 3), "seconds": round(secs, 3), "tokens": int(ids.numel()), "seq_len": args.seq_len,
                      "tokens_per_s": round(ids.numel() / secs, 1), "layers": cfg.layers, "vocab": cfg.vocab}))


if __name__ == "__main__":
    main()
