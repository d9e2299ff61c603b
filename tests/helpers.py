"""Seeded synthetic inputs for the parity tests and the tolerance they are judged with."""
import contextlib

import numpy as np
import torch

import glowq_oracle as oracle

ABS_TOL = 1e-2   # north-star tolerance: |a - b| <= 1e-2 + 1e-3 * |b| against the fp32-accumulate result
REL_TOL = 1e-3


def make_group(seed, M, K, Ns, rank, group_size=128, w_std=0.02, with_bias=False):
    """x ~ N(0,1) [M,K]; W_i ~ N(0, w_std^2); R ~ N(0, 1/K) [rank,K]; L_i ~ N(0, 0.01^2) [N_i, rank];
    drawn in fp32 from one seeded generator in this fixed order, then rounded to fp16."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g).half().numpy()
    members = []
    for N in Ns:
        w = (torch.randn(N, K, generator=g) * w_std).half().numpy()
        qw, qz, sc, _ = oracle.quantize_per_group_w4(w, group_size)
        members.append({"qweight": qw, "qzeros": qz, "scales": sc, "group_size": group_size, "w": w})
    R = None
    if rank:
        R = (torch.randn(rank, K, generator=g) * K ** -0.5).half().numpy()
        for m, N in zip(members, Ns):
            m["L"] = (torch.randn(N, rank, generator=g) * 0.01).half().numpy()
    if with_bias:
        for m, N in zip(members, Ns):
            m["bias"] = (torch.randn(N, generator=g) * 0.1).half().numpy()
    return x, members, R


def outlier_activations(x, seed, scale=4.0, fraction=0.01, factor=200.0):
    """x scaled by `scale`, with a seeded `fraction` of its channels (columns) another `factor` times larger, rounded
    to fp16: a few channels in the thousands among values of order one."""
    rng = np.random.default_rng(seed)
    K = x.shape[1]
    cols = rng.choice(K, size=max(1, int(K * fraction)), replace=False)
    out = x.astype(np.float32)
    out[:, cols] *= factor
    return (out * scale).astype(np.float16)


def dev(a, device="cuda"):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def assert_close(got, want64, what=""):
    """`got` fp16 array vs float64 yardstick, north-star tolerance plus half an fp16 ulp of the
    yardstick (the output itself is rounded to fp16)."""
    got = np.asarray(got, dtype=np.float64)
    want64 = np.asarray(want64, dtype=np.float64)
    err = np.abs(got - want64)
    bound = ABS_TOL + REL_TOL * np.abs(want64)
    worst = np.unravel_index(np.argmax(err - bound), err.shape)
    assert np.all(err <= bound), f"{what}: max err {err.max():.3e} at {worst} (got {got[worst]}, want {want64[worst]})"
    return float(err.max())


@contextlib.contextmanager
def tuning(ext, **limits):
    """Route limits of the library set for the body of a `with` and put back afterwards."""
    old = {key: ext.set_tuning(key, value) for key, value in limits.items()}
    try:
        yield
    finally:
        for key, value in old.items():
            ext.set_tuning(key, value)
