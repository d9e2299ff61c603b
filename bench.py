#!/usr/bin/env python3
"""Benchmark of the GlowQ Step-3 hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload (the headline configuration of the benchmark): the decode linears of a Llama-3.1-8B-shaped model at batch 1 --
per layer the QKV group (N = 4096+1024+1024, K = 4096), o_proj (4096x4096), the gate|up group
(N = 2 x 14336, K = 4096) and down_proj (K = 14336, N = 4096); int4 codes, asymmetric per-group scale and
zero-point (g = 128), fp16 activations ~ N(0,1), shared rank-128 correction on every group.  One STEP is
one pass of all four groups over 32 layers of DISTINCT weight buffers (4.2 GB, far beyond the 256 MB
last-level cache): per group one library call that computes the shared projection r = x R^T and runs the group on it
-- one launch where the group launch computes r itself (groups whose whole grid is on the chip at once: q|k|v, o_proj,
down_proj), else the projection launch and the group launch (gate|up); 160 launches, replayed as a HIP graph so that the
host is not in the timed path.  Inputs are resident in HBM before
the timed region starts.  Every timed region follows about 30 ms of untimed replays of the same graph (the clocks
ramp for 10-20 ms after an idle gap), then the W warm-up steps.

Prints ONE JSON line: the metric (microseconds per layer), the roofline of the dominant kernel (the
gate|up group GEMV, priced on algorithmic bytes against 8 TB/s) and the CPU baseline (the oracle's
restatement of the reference's torch path, timed on this box's host cores on a bounded sample).  Next to the
metric: the same step with r given (the decode loop's launch structure), every group at 2 / 4 / 8 token rows, the
prefill configuration (MFMA-bound), the GlowQ-S configuration and the whole decode loop.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
LAYERS = 32
RANK = 128
GROUP_SIZE = 128
M_TOKENS = 1
# name -> (K, member widths)
GROUPS = {
    "qkv": (4096, [4096, 1024, 1024]),
    "o_proj": (4096, [4096]),
    "gate_up": (4096, [14336, 14336]),
    "down_proj": (14336, [4096]),
}
# the prefill configuration of the same benchmark: Qwen2.5-7B-shaped layer at 2048 tokens (MFMA-bound)
PREFILL_TOKENS = 2048
PREFILL_GROUPS = {
    "qkv": (3584, [3584, 512, 512]),
    "o_proj": (3584, [3584]),
    "gate_up": (3584, [18944, 18944]),
    "down_proj": (18944, [3584]),
}
MFMA_FP16_PEAK_TFLOPS = 2516.6
# the selective configuration (GlowQ-S): Qwen3-14B-shaped layer, rank 256, correction on a seeded half of the groups
SELECTIVE_RANK = 256
SELECTIVE_LAYERS = 24
SELECTIVE_GROUPS = {
    "qkv": (5120, [5120, 1024, 1024]),
    "o_proj": (5120, [5120]),
    "gate_up": (5120, [17408, 17408]),
    "down_proj": (17408, [5120]),
}
DOMINANT = "gate_up"
# HBM bytes per launch of the dominant kernel as counted by rocprofv3 (FETCH_SIZE + WRITE_SIZE, scaled by the same
# counters on a copy of known size): written by `python bench.py --summarize-pmc FETCH_CSV WRITE_CSV` from the counter
# files of two profiling runs of this script, read back here for `roofline.traffic` (null when the file is missing)
TRAFFIC_SIDECAR = os.path.join(ROOT, "profiles", "decode_gemv_gate_up_llama8b_hbm_traffic.json")


def algorithmic_bytes(M, K, N, rank, gs=GROUP_SIZE):
    G = -(-K // gs)
    b = N * K // 2 + 2 * N * G + 4 * N * (-(-G // 8)) + 2 * M * K + 2 * M * N
    if rank:
        b += 2 * rank * K + 2 * N * rank
    return b


def make_layer(torch, dev, seed, groups=None, rank=RANK):
    """Random codes / zero-point nibbles (any bit pattern is a valid quantised weight), scales in the
    range a N(0, 0.02) weight produces, R ~ N(0, 1/K), L ~ N(0, 0.01^2)."""
    g = torch.Generator(device=dev).manual_seed(seed)
    layer = {}
    for name, (K, Ns) in (groups or GROUPS).items():
        G = K // GROUP_SIZE
        members = []
        for N in Ns:
            members.append({
                "qweight": torch.randint(-2**31, 2**31 - 1, (N, K // 8), dtype=torch.int32, device=dev, generator=g),
                "scales": (torch.rand(N, G, device=dev, generator=g) * 0.004 + 0.006).half(),
                "qzeros": torch.randint(-2**31, 2**31 - 1, (N, (G + 7) // 8), dtype=torch.int32, device=dev, generator=g),
                "L": (torch.randn(N, rank, device=dev, generator=g) * 0.01).half(),
                "bias": None,
            })
        R = (torch.randn(rank, K, device=dev, generator=g) * K ** -0.5).half()
        layer[name] = (members, R)
    return layer


def settle(torch, graph, busy_ms=30.0):
    """Untimed replays until the card has been busy for about `busy_ms`: after an idle gap the first 10-20 ms run at
    ramping clocks (the step reads 47.5 us per layer in the first 7 ms after two idle seconds, 45.0 from then on)."""
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    graph.replay()
    b.record()
    torch.cuda.synchronize()
    for _ in range(max(1, min(2000, int(busy_ms / max(a.elapsed_time(b), 1e-3))))):
        graph.replay()
    torch.cuda.synchronize()


def timed_replays(torch, graph, reps):
    """Milliseconds per replay over `reps` replays, HIP events on the launch stream, after settle()."""
    settle(torch, graph)
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        graph.replay()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / reps


def cpu_baseline(torch, budget_s=18.0):
    """The reference's torch CPU path (oracle/torch_cpu_path.py) on one layer of the same workload,
    repeated until about `budget_s` seconds of CPU work are spent."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import torch_cpu_path as tp

    cores = os.cpu_count() or 1
    env_threads = int(os.environ.get("OMP_NUM_THREADS", "0") or 0)
    if env_threads > 0:
        cores = min(cores, env_threads)
    torch.set_num_threads(cores)
    layer = make_layer(torch, "cpu", 1)
    for members, _ in layer.values():
        for m in members:
            m["group_size"] = GROUP_SIZE
    g = torch.Generator().manual_seed(1)
    xs = {name: torch.randn(M_TOKENS, K, generator=g).half() for name, (K, _) in GROUPS.items()}

    def one_layer():
        for name, (members, R) in layer.items():
            tp.corrected_group(xs[name], members, R, 1.0)

    one_layer()  # warm-up
    times = []
    t_start = time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_start < budget_s and len(times) < 50):
        t0 = time.perf_counter()
        one_layer()
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]

    # the same layer with the weights dequantised once beforehand and fp32 matmuls: the CPU figure without the
    # Python dequantisation cost (the reference's optional dequant cache, src/cuda_w4a16/linear.py:212-227)
    dense = {}
    for name, (members, R) in layer.items():
        K_in = xs[name].size(1)
        gid = torch.arange(K_in, dtype=torch.long) // GROUP_SIZE
        dense[name] = [{"w_f32": tp.dequant_chunk(m["qweight"], m["qzeros"], m["scales"], gid, K_in, -(-K_in // GROUP_SIZE),
                                                  0, m["qweight"].size(0)).float(), "L": m.get("L")} for m in members]

    def one_layer_cached():
        for name, (members, R) in layer.items():
            tp.cached_dequant_group(xs[name], dense[name], R, 1.0)

    one_layer_cached()
    cached = []
    for _ in range(7):
        t0 = time.perf_counter()
        one_layer_cached()
        cached.append(time.perf_counter() - t0)
    cached.sort()
    return {
        "cached_dequant_value": cached[len(cached) // 2] * 1e6,
        "value": med * 1e6,
        "unit": "us/layer",
        "cores": int(torch.get_num_threads()),
        "kind": "port",
        "sample": f"1 layer (4 groups, M=1, rank 128) x {len(times)} repeats, median; torch fp16 CPU path "
                  f"(512-row chunked dequant + matmul + shared-r correction); cached_dequant_value: the same layer, "
                  f"us/layer, weights dequantised once beforehand, fp32 matmuls, median of 7",
    }


def prefill_leg(torch, ext, dev):
    """Every group of a Qwen2.5-7B-shaped layer at 2048 tokens: projection launch + group launch as in decode,
    algorithmic flops 2 M N K + 2 M r K + 2 M N r against the dense fp16 MFMA peak."""
    g = torch.Generator(device=dev).manual_seed(11)
    prefill = {"workload": f"Qwen2.5-7B-shaped layer, M={PREFILL_TOKENS}, int4 g=128 asym, shared rank-{RANK} correction",
               "per_group": {}}
    pl = make_layer(torch, dev, 7, PREFILL_GROUPS)
    tot_us, tot_fl, tot_vus, tot_vfl = 0.0, 0.0, 0.0, 0.0
    for name, (K, Ns) in PREFILL_GROUPS.items():
        members, R = pl[name]
        xp = torch.randn(PREFILL_TOKENS, K, device=dev, generator=g).half()
        rp = torch.empty(PREFILL_TOKENS, RANK, dtype=torch.float16, device=dev)
        op = [torch.empty(PREFILL_TOKENS, N, dtype=torch.float16, device=dev) for N in Ns]
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < 0.03:  # untimed: first call of a route, then the clock ramp
            ext.group_forward(xp, rp, members, GROUP_SIZE, 1.0, outs=op, R=R)
            torch.cuda.synchronize()
        ts = []
        for _ in range(5):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(4):
                ext.group_forward(xp, rp, members, GROUP_SIZE, 1.0, outs=op, R=R)
            b.record()
            torch.cuda.synchronize()
            ts.append(a.elapsed_time(b) * 1e3 / 4)
        us = sorted(ts)[len(ts) // 2]
        N = sum(Ns)
        fl = 2.0 * PREFILL_TOKENS * (N * K + RANK * K + N * RANK)
        # yardstick: the vendor library's plain fp16 GEMM of the same M x N x K on weights that are already fp16 (no
        # dequantisation, no correction): what the matrix cores sustain on this shape under their power limit
        wd = torch.randn(N, K, device=dev, generator=g).half().mul_(0.02)
        yd = torch.empty(PREFILL_TOKENS, N, dtype=torch.float16, device=dev)
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < 0.03:
            torch.mm(xp, wd.t(), out=yd)
            torch.cuda.synchronize()
        tv = []
        for _ in range(5):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(4):
                torch.mm(xp, wd.t(), out=yd)
            b.record()
            torch.cuda.synchronize()
            tv.append(a.elapsed_time(b) * 1e3 / 4)
        vus = sorted(tv)[len(tv) // 2]
        vfl = 2.0 * PREFILL_TOKENS * N * K
        prefill["per_group"][name] = {"us": round(us, 1), "TFLOPs": round(fl / us / 1e6, 1),
                                      "frac_mfma_peak": round(fl / us / 1e6 / MFMA_FP16_PEAK_TFLOPS, 4),
                                      "vendor_fp16_gemm_us": round(vus, 1),
                                      "vendor_fp16_gemm_frac_mfma_peak": round(vfl / vus / 1e6 / MFMA_FP16_PEAK_TFLOPS, 4)}
        tot_us += us
        tot_fl += fl
        tot_vus += vus
        tot_vfl += vfl
        del xp, rp, op, wd, yd
    prefill["us_per_layer"] = round(tot_us, 1)
    prefill["TFLOPs"] = round(tot_fl / tot_us / 1e6, 1)
    prefill["frac_mfma_peak"] = round(tot_fl / tot_us / 1e6 / MFMA_FP16_PEAK_TFLOPS, 4)
    prefill["vendor_fp16_gemm_us_per_layer"] = round(tot_vus, 1)
    prefill["vendor_fp16_gemm_frac_mfma_peak"] = round(tot_vfl / tot_vus / 1e6 / MFMA_FP16_PEAK_TFLOPS, 4)
    return prefill


def selective_leg(torch, ext, dev):
    """GlowQ-S on a Qwen3-14B-shaped layer (rank 256) across the switch from the GEMV kernels to the MFMA kernels:
    per token-row count the time of every group with its correction (projection + group launch) and without (the bare
    quantised group: what an unselected group costs), the kernel route taken, and the layer with a seeded random half
    of its groups selected.  24 layers of distinct weights (4 GB; every single group kind alone is more than the
    256 MB last-level cache holds) per replay."""
    g = torch.Generator(device=dev).manual_seed(21)
    layers = [make_layer(torch, dev, 300 + i, SELECTIVE_GROUPS, SELECTIVE_RANK) for i in range(SELECTIVE_LAYERS)]
    names = list(SELECTIVE_GROUPS)
    pick = torch.randperm(SELECTIVE_LAYERS * len(names), generator=torch.Generator().manual_seed(1234))
    selected = set(int(i) for i in pick[: SELECTIVE_LAYERS * len(names) // 2])  # groups enumerated layer-major
    side = torch.cuda.Stream()
    out = {"workload": f"Qwen3-14B-shaped layer, int4 g=128 asym, rank {SELECTIVE_RANK}, {SELECTIVE_LAYERS} layers of "
                       f"distinct weights, correction on a seeded half of the groups", "rows": {}}

    def timed(run):
        with torch.cuda.stream(side):
            run()  # outside the capture first: kernel attributes
            torch.cuda.synchronize()
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr, stream=side):
                run()
        torch.cuda.synchronize()
        return timed_replays(torch, gr, 20) * 1e3

    for rows in (1, 4, 16, 64):
        xs = {n: torch.randn(rows, K, device=dev, generator=g).half() for n, (K, _) in SELECTIVE_GROUPS.items()}
        rb = torch.empty(rows, SELECTIVE_RANK, dtype=torch.float16, device=dev)
        ob = {n: [torch.empty(rows, N, dtype=torch.float16, device=dev) for N in Ns] for n, (_, Ns) in SELECTIVE_GROUPS.items()}
        bare = [{n: [dict(m, L=None) for m in layer[n][0]] for n in names} for layer in layers]

        def corrected(n, layer):
            ext.group_forward(xs[n], rb, layer[n][0], GROUP_SIZE, 1.0, outs=ob[n], R=layer[n][1])

        def plain(n, li):
            ext.group_forward(xs[n], None, bare[li][n], GROUP_SIZE, 0.0, outs=ob[n])

        entry = {"route": {n: ext.route(rows, K, sum(Ns), GROUP_SIZE) for n, (K, Ns) in SELECTIVE_GROUPS.items()},
                 "corrected_us": {}, "plain_us": {}}
        for n in names:
            entry["corrected_us"][n] = round(timed(lambda: [corrected(n, layer) for layer in layers]) / SELECTIVE_LAYERS, 2)
            entry["plain_us"][n] = round(timed(lambda: [plain(n, li) for li in range(SELECTIVE_LAYERS)]) / SELECTIVE_LAYERS, 2)

        def half():
            for li, layer in enumerate(layers):
                for gi, n in enumerate(names):
                    if li * len(names) + gi in selected:
                        corrected(n, layer)
                    else:
                        plain(n, li)

        # fraction of the HBM peak per group: algorithmic bytes of the call (with R, L and r where corrected) over its time
        entry["corrected_pct_hbm_peak"] = {n: round(100.0 * algorithmic_bytes(rows, K, sum(Ns), SELECTIVE_RANK) / entry["corrected_us"][n] / 1e6 / (HBM_PEAK_GBPS / 1e3), 1)
                                           for n, (K, Ns) in SELECTIVE_GROUPS.items()}
        entry["plain_pct_hbm_peak"] = {n: round(100.0 * algorithmic_bytes(rows, K, sum(Ns), 0) / entry["plain_us"][n] / 1e6 / (HBM_PEAK_GBPS / 1e3), 1)
                                       for n, (K, Ns) in SELECTIVE_GROUPS.items()}
        entry["all_corrected_us_per_layer"] = round(sum(entry["corrected_us"].values()), 2)
        entry["none_corrected_us_per_layer"] = round(sum(entry["plain_us"].values()), 2)
        entry["half_selected_us_per_layer"] = round(timed(half) / SELECTIVE_LAYERS, 2)
        out["rows"][str(rows)] = entry
    return out


def stream_read_probe(torch, ext, capture, pool, sink, nbytes, launch):
    """GB/s of the library's bare streaming-read kernel over `nbytes` per launch, launched with the grid and workgroup
    size of `launch` on the buffers of `pool` in turn (None where the launch record holds no grid)."""
    if not launch["grid"][0] or not launch["block"]:
        return None
    nbytes = nbytes // 16 * 16
    dev = pool[0].device
    gr = capture(lambda: [ext.lib.glowq_probe_stream_read(b.data_ptr(), nbytes, sink.data_ptr(), launch["grid"][0] * max(1, launch["grid"][1]),
                                                          launch["block"], ext._stream(dev)) for b in pool])
    us = timed_replays(torch, gr, 20) * 1e3 / len(pool)
    return round(nbytes / us / 1e3, 1)


def module_eager_leg(torch, model, iters=300):
    """Host cost of the torch modules outside a graph: wall time per module-group forward at one token (the q|k|v
    wrappers fuse into one library call on the lead's forward, gate|up likewise), launches queued without waiting for
    the GPU, on the first layer of the decode loop's model."""
    layer = model.model.layers[0]
    attn, mlp = layer.self_attn, layer.mlp
    dev = next(model.parameters()).device
    cfg = model.cfg
    x = torch.randn(1, cfg.hidden, device=dev).half()
    a = torch.randn(1, cfg.heads * cfg.head_dim, device=dev).half()
    h = torch.randn(1, cfg.intermediate, device=dev).half()
    groups = {
        "qkv": lambda: (attn.q_proj(x), attn.k_proj(x), attn.v_proj(x)),
        "o_proj": lambda: attn.o_proj(a),
        "gate_up": lambda: (mlp.gate_proj(x), mlp.up_proj(x)),
        "down_proj": lambda: mlp.down_proj(h),
    }
    out = {}
    with torch.no_grad():
        for name, fn in groups.items():
            for _ in range(20):
                fn()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(iters):
                fn()
            host = time.perf_counter() - t0   # the queue is not waited for: host time per call unless the GPU is slower
            torch.cuda.synchronize()
            total = time.perf_counter() - t0
            out[name] = {"host_us_per_group_forward": round(host / iters * 1e6, 2), "with_gpu_drain_us": round(total / iters * 1e6, 2)}
    out["sum_host_us_per_layer"] = round(sum(v["host_us_per_group_forward"] for v in out.values()), 2)
    return out


def calibrate_copy(torch, dev, graph):
    """Eight plain device copies of 256 MiB each from cold sources (the kernel shows up in a profile as a copy kernel):
    262144 KiB read and 262144 KiB written per copy, the yardstick the FETCH_SIZE / WRITE_SIZE counts are scaled by."""
    srcs = [torch.full((128 * 1024 * 1024,), float(i), dtype=torch.float16, device=dev) for i in range(8)]
    dst = torch.empty_like(srcs[0])
    if graph is not None:
        graph.replay()  # push the sources out of the last-level cache
    torch.cuda.synchronize()
    for s_ in srcs:
        dst.copy_(s_)
    torch.cuda.synchronize()


def summarize_pmc(fetch_csv, write_csv):
    """Reads the per-dispatch counter files of two rocprofv3 --pmc runs of `bench.py --groups-only --calibrate-copy`
    (FETCH_SIZE, then WRITE_SIZE) and writes the traffic sidecar: bytes per launch of every group's GEMV launch, each
    counter scaled by what it reads for the 256 MiB device copies of the same run.  The only writer of that file."""
    import csv

    def per_kernel(path, counter):
        per = {}
        with open(path, newline="") as f:
            for row in csv.DictReader(f):
                if row.get("Counter_Name") == counter:
                    per.setdefault((row["Kernel_Name"], int(row.get("Grid_Size", 0) or 0)), []).append(float(row["Counter_Value"]))
        return per

    # a stream GEMV launch is one wave per two output rows: threads = 32 N; its first template argument is ceil(K / 2048)
    label = {(-(-K // 2048), 32 * sum(Ns)): name for name, (K, Ns) in GROUPS.items()}
    out = {"kernel": None, "command": "rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE --output-format csv -- python3 bench.py "
                                      "--groups-only --calibrate-copy", "copy_bytes_each_way": 256 << 20, "groups": {}}
    for path, counter in ((fetch_csv, "FETCH_SIZE"), (write_csv, "WRITE_SIZE")):
        per = per_kernel(path, counter)
        # the 256 MiB copies are the largest dispatches of any copy kernel in the run (smaller ones move parameters)
        copies = [v for (k, _), vs in per.items() if "copy" in k.lower() for v in vs]
        gemv = {key: vs for key, vs in per.items() if "gemv_stream_kernel" in key[0] or "gemv_wave_dot_kernel" in key[0]}
        if not copies or not gemv:
            raise SystemExit(f"{path}: need the copy kernel and the GEMV kernels in the counter file, found {sorted(k for k, _ in per)}")
        big = [v for v in copies if v >= 0.5 * max(copies)]
        per_copy = sum(big) / len(big)
        factor = (256 << 20) / 1024.0 / per_copy          # KiB per count
        out[counter + "_KiB_per_count"] = round(factor, 4)
        out[counter + "_count_per_copy"] = round(per_copy, 1)
        for (kname, threads), vs in gemv.items():
            targs = template_args(kname) or [0]
            name = label.get((targs[0], threads), f"{threads} threads")
            entry = out["groups"].setdefault(name, {"kernel": kname[:140], "launches_counted": len(vs)})
            entry[counter + "_KiB_per_launch"] = round(sum(vs) / len(vs) * factor, 1)
    for name, entry in out["groups"].items():
        K, Ns = GROUPS.get(name, (0, [0]))
        entry["algorithmic_KiB_per_launch"] = round((algorithmic_bytes(M_TOKENS, K, sum(Ns), RANK) - 2 * RANK * K) / 1024.0, 1) if K else None
        entry["traffic_bytes_per_launch"] = int(round((entry.get("FETCH_SIZE_KiB_per_launch", 0) + entry.get("WRITE_SIZE_KiB_per_launch", 0)) * 1024))
    if DOMINANT not in out["groups"]:
        raise SystemExit(f"no launch of the {DOMINANT} group in the counter files: {sorted(out['groups'])}")
    out["kernel"] = out["groups"][DOMINANT]["kernel"]
    out["traffic_bytes_per_launch"] = out["groups"][DOMINANT]["traffic_bytes_per_launch"]
    with open(TRAFFIC_SIDECAR, "w") as f:
        json.dump(out, f, indent=1)
        f.write("\n")
    print(json.dumps(out))


def template_args(kernel_name):
    """The integer template arguments of a kernel name, from the mangled symbol a counter file holds (...ILi2ELi1ELb0E...)
    or from the library's launch record (name<2,1,0,...>)."""
    import re
    m = re.search(r"<([0-9, ]+)>", kernel_name)
    if m:
        return [int(t) for t in m.group(1).split(",")]
    m = re.search(r"kernelI((?:L[ib]\d+E)+)E", kernel_name)
    return [int(t) for t in re.findall(r"L[ib](\d+)E", m.group(1))] if m else None


def read_traffic_sidecar(launched_kernel):
    """Traffic of the dominant launch from the counter file, if that file was taken on the instantiation this run
    launched (same kernel, same template arguments); else (None, why)."""
    try:
        with open(TRAFFIC_SIDECAR) as f:
            d = json.load(f)
        counted = d["kernel"]
        base = launched_kernel.split("<")[0]
        if base not in counted or template_args(counted) != template_args(launched_kernel):
            return None, f"{os.path.relpath(TRAFFIC_SIDECAR, ROOT)} was counted on {counted[:100]}, this run launched {launched_kernel}"
        return int(d["traffic_bytes_per_launch"]), os.path.relpath(TRAFFIC_SIDECAR, ROOT)
    except (OSError, ValueError, KeyError):
        return None, None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the CPU leg (profiling runs)")
    ap.add_argument("--prefill-only", action="store_true", help="run only the prefill leg and print it (profiling runs)")
    ap.add_argument("--selective-only", action="store_true", help="run only the GlowQ-S leg and print it")
    ap.add_argument("--no-decode-loop", action="store_true", help="skip the full decode loop leg (profiling runs)")
    ap.add_argument("--dominant-only", action="store_true",
                    help="run only the graph of the dominant kernel (32 launches per replay) and print its timing (profiling runs)")
    ap.add_argument("--groups-only", action="store_true",
                    help="run only the graph of the four group launches per layer on a given r and print its timing (profiling runs)")
    ap.add_argument("--summarize-pmc", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"),
                    help="no GPU work: turn the counter files of two --pmc runs into the traffic sidecar under profiles/")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run plain device copies of known size (256 MiB read + 256 MiB written each) so that "
                         "FETCH_SIZE / WRITE_SIZE counters of a profiling run can be scaled")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU execution (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    if args.summarize_pmc:
        summarize_pmc(*args.summarize_pmc)
        return

    import torch
    from glowq_amd.kernels import load_w4a16_extension

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    ext = load_w4a16_extension()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.prefill_only:
        print(json.dumps({"prefill": prefill_leg(torch, ext, dev)}))
        return

    if args.selective_only:
        print(json.dumps({"selective": selective_leg(torch, ext, dev)}))
        if args.calibrate_copy:
            calibrate_copy(torch, dev, None)
        return

    from glowq_amd.kernels import PreparedGroup

    layers = [make_layer(torch, dev, 100 + i) for i in range(LAYERS)]
    g = torch.Generator(device=dev).manual_seed(1)
    xs = {name: torch.randn(M_TOKENS, K, device=dev, generator=g).half() for name, (K, _) in GROUPS.items()}
    rbuf = torch.empty(M_TOKENS, RANK, dtype=torch.float16, device=dev)
    outs = {name: [torch.empty(M_TOKENS, N, dtype=torch.float16, device=dev) for N in Ns] for name, (_, Ns) in GROUPS.items()}
    # every group validated once, descriptors built once: a call is one library call
    calls = [{name: PreparedGroup(ext, layer[name][0], GROUPS[name][0], GROUP_SIZE, 1.0, R=layer[name][1]) for name in GROUPS}
             for layer in layers]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())

    def capture(run):
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            run()  # outside the capture first: kernel attributes of the routes these shapes take
            torch.cuda.synchronize()
            with torch.cuda.graph(gr, stream=side):
                run()
        torch.cuda.synchronize()
        return gr

    def run_group(li, name, project=True, x=None, r=None, o=None):
        # project: one call = the shared-projection launch (r = x R^T left in the r buffer) + the fused group launch;
        # otherwise the group launch alone on an r that is already there (what a decode loop does, whose glue kernels
        # produce r together with x)
        calls[li][name].run(xs[name] if x is None else x, r=rbuf if r is None else r, outs=outs[name] if o is None else o,
                            project=project)

    # dominant kernel: the gate|up group launch alone (r given), 32 layers of distinct weights back to back in one
    # graph, HIP events around the replays on the launch stream
    K_d, Ns_d = GROUPS[DOMINANT]
    # the group kernel's own bytes: the group total minus R, which the projection launch reads
    dom_bytes = algorithmic_bytes(M_TOKENS, K_d, sum(Ns_d), RANK) - 2 * RANK * K_d
    gdom = capture(lambda: [run_group(li, DOMINANT, project=False) for li in range(LAYERS)])
    dom_launch = ext.last_launch()  # the instantiation, grid and workgroup size the library used for it
    if args.groups_only:
        gg_ = capture(lambda: [run_group(li, name, project=False) for li in range(LAYERS) for name in GROUPS])
        us = timed_replays(torch, gg_, max(10, min(args.steps, 50))) * 1e3 / LAYERS
        if args.calibrate_copy:
            calibrate_copy(torch, dev, gg_)
        print(json.dumps({"r_given_us_per_layer": round(us, 3), "dominant_launch": dom_launch}))
        return
    if args.dominant_only:
        dom_us = timed_replays(torch, gdom, max(10, min(args.steps, 50))) * 1e3 / LAYERS
        if args.calibrate_copy:
            calibrate_copy(torch, dev, gdom)
        print(json.dumps({"dominant_kernel_us": round(dom_us, 3), "GBps": round(dom_bytes / dom_us / 1e3, 1),
                          "algorithmic_bytes_per_launch": dom_bytes}))
        return

    graph = capture(lambda: [run_group(li, name) for li in range(LAYERS) for name in GROUPS])
    settle(torch, graph)  # clock ramp after the idle gap of the capture, before the warm-up steps
    for _ in range(args.warmup):
        graph.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t_wall0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        graph.replay()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t_wall0) * 1e3
    ms_per_step = e0.elapsed_time(e1) / args.steps

    bytes_layer = sum(algorithmic_bytes(M_TOKENS, K, sum(Ns), RANK) for K, Ns in GROUPS.values())
    us_per_layer = ms_per_step * 1e3 / LAYERS
    gbps = bytes_layer / (us_per_layer * 1e-6) / 1e9

    dom_us = timed_replays(torch, gdom, max(10, min(args.steps, 50))) * 1e3 / LAYERS
    achieved = dom_bytes / (dom_us * 1e-6) / 1e9

    # the same step with r given: 4 group launches per layer, the structure of the decode loop (its glue kernels produce
    # r together with the activations); the bytes of R belong to those kernels and are left out of this figure's bytes
    g_given = capture(lambda: [run_group(li, name, project=False) for li in range(LAYERS) for name in GROUPS])
    given_us = timed_replays(torch, g_given, max(10, min(args.steps, 50))) * 1e3 / LAYERS
    given_bytes = sum(algorithmic_bytes(M_TOKENS, K, sum(Ns), RANK) - 2 * RANK * K for K, Ns in GROUPS.values())

    # what the memory system gives a kernel of the same launch shape that only reads: 32 cold buffers of the launch's
    # algorithmic bytes each, back to back in one graph like the launches themselves; and the cost of launching nothing
    pool = [torch.full(((dom_bytes + 15) // 16 * 16,), 1 + i, dtype=torch.uint8, device=dev) for i in range(LAYERS)]
    sink = torch.zeros(4, dtype=torch.uint8, device=dev)
    stream_read = stream_read_probe(torch, ext, capture, pool, sink, dom_bytes, dom_launch)
    g_empty = capture(lambda: [ext.lib.glowq_probe_empty_launch(dom_launch["grid"][0], dom_launch["block"],
                                                                 ext._stream(dev)) for _ in range(LAYERS)])
    empty_us = timed_replays(torch, g_empty, 20) * 1e3 / LAYERS

    # per-group split of the step, from graphs of one group kind each (reported, not the metric)
    per_group = {}
    for name in GROUPS:
        K, Ns = GROUPS[name]
        by = algorithmic_bytes(M_TOKENS, K, sum(Ns), RANK)
        us = timed_replays(torch, capture(lambda: [run_group(li, name) for li in range(LAYERS)]), 10) * 1e3 / LAYERS
        projecting = ext.last_launch()["kernel"]  # prologue 3 of the stream GEMV: the launch computes r itself
        in_launch = projecting.startswith("gemv_stream_kernel<") and template_args(projecting)[4] == 3
        us_g = timed_replays(torch, capture(lambda: [run_group(li, name, project=False) for li in range(LAYERS)]), 10) * 1e3 / LAYERS
        launch = ext.last_launch()
        read_gbps = stream_read_probe(torch, ext, capture, pool, sink, by - 2 * RANK * K, launch)
        per_group[name] = {"launch": launch, "launch_with_projection": projecting, "launches_per_call": 1 if in_launch else 2,
                           "stream_read_GBps": read_gbps,
                           "frac_of_stream_read": round((by - 2 * RANK * K) / us_g / 1e3 / read_gbps, 4) if read_gbps else None,"us": round(us, 3), "GBps": round(by / us / 1e3, 1), "pct_hbm_peak": round(by / us / 1e3 / HBM_PEAK_GBPS * 100, 2),
                           "group_launch_only_us": round(us_g, 3),
                           "group_launch_only_pct_hbm_peak": round((by - 2 * RANK * K) / us_g / 1e3 / HBM_PEAK_GBPS * 100, 2)}

    # the same layers at more token rows per call (the batch sizes of the configuration, then 16 and 64): projection +
    # group launch per group as in the step; 8 layers of distinct weights (1 GB) per replay keep the last-level cache
    # out of the picture.  Fractions are algorithmic bytes at that row count over the time, against the HBM peak.
    batched, batched_groups = {}, {}
    for rows in (2, 4, 8, 16, 64):
        xb = {name: torch.randn(rows, K, device=dev, generator=g).half() for name, (K, _) in GROUPS.items()}
        rb = torch.empty(rows, RANK, dtype=torch.float16, device=dev)
        ob = {name: [torch.empty(rows, N, dtype=torch.float16, device=dev) for N in Ns] for name, (_, Ns) in GROUPS.items()}
        gb = capture(lambda: [run_group(li, name, x=xb[name], r=rb, o=ob[name]) for li in range(8) for name in GROUPS])
        batched[str(rows)] = round(timed_replays(torch, gb, 10) * 1e3 / 8, 2)
        if rows <= 8:
            entry = {}
            for name, (K, Ns) in GROUPS.items():
                gg = capture(lambda: [run_group(li, name, x=xb[name], r=rb, o=ob[name]) for li in range(8)])
                us = timed_replays(torch, gg, 10) * 1e3 / 8
                by = algorithmic_bytes(rows, K, sum(Ns), RANK)
                entry[name] = {"us": round(us, 2), "route": ext.route(rows, K, sum(Ns), GROUP_SIZE),
                               "pct_hbm_peak": round(by / us / 1e3 / HBM_PEAK_GBPS * 100, 2)}
            batched_groups[str(rows)] = entry

    prefill = prefill_leg(torch, ext, dev)

    if args.calibrate_copy:
        calibrate_copy(torch, dev, graph)

    del layers, calls, graph, gdom, g_given, pool, g_empty
    torch.cuda.empty_cache()
    selective = selective_leg(torch, ext, dev)
    # the whole decode loop of the same benchmark (32-layer random-init model, 512-token prompt, 256 new tokens, greedy)
    torch.cuda.empty_cache()
    decode, module_eager = None, None
    if not args.no_decode_loop:
        import contextlib
        from glowq_amd import decode as decode_loop
        with contextlib.redirect_stdout(sys.stderr):  # the patcher reports what it wrapped; stdout carries the JSON line only
            cfg = decode_loop.DecoderConfig(layers=32, max_len=1024)
            model, _, _ = decode_loop.build_decoder(cfg)
            decode = decode_loop.measure(32, 512, 256, model=model)
            # the same model through its torch modules (CudaW4A16Linear / AddSVDCorrection), single-token glue kernels
            # between them, under a graph
            mod = decode_loop.measure(32, 512, 64, fused=False, model=model)
            decode["module_path"] = {k: mod[k] for k in ("new_tokens", "graph", "module_glue", "decode_tok_per_s", "ms_per_token")}
            module_eager = module_eager_leg(torch, model)
            del model

    traffic, traffic_source = read_traffic_sidecar(dom_launch["kernel"])
    result = {
        "metric": "W4A16+GlowQ decode linears, microseconds per layer (Llama-3.1-8B shape, batch 1)",
        "value": round(us_per_layer, 3),
        "unit": "us/layer",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "settle_ms_before_warmup": 30,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int4 weights x fp16 activations, fp32 accumulate",
        "data": "synthetic",
        "config": {
            "workload": "Llama-3.1-8B decode linears (qkv 6144x4096, o 4096x4096, gate|up 28672x4096, "
                        "down 4096x14336), int4 g=128 asym, shared rank-128 correction, batch tokens 1, 32 layers of distinct weights",
            "tokens": M_TOKENS, "rank": RANK, "group_size": GROUP_SIZE, "layers": LAYERS,
            "launches_per_step": sum(v["launches_per_call"] for v in per_group.values()) * LAYERS, "execution": "HIP graph replay",
            "structure": "per group one library call that computes r = x R^T and runs the group on it: one launch where "
                         "the group launch computes r itself (per_group.*.launches_per_call = 1), else the shared-projection "
                         "launch + the group launch; the figure under r_given is the same step with the 4 group launches "
                         "alone on an r that is there",
        },
        "hbm_GBps": round(gbps, 1),
        "pct_hbm_peak": round(gbps / HBM_PEAK_GBPS * 100, 2),
        "decode_tok_per_s_linears_only": round(1e3 / ms_per_step, 1),
        "algorithmic_bytes_per_layer": bytes_layer,
        "r_given": {
            "structure": "4 group launches per layer on an r that is already there, as in the decode loop, whose glue "
                         "kernels (norm, attention merge, gating) produce r together with the activations",
            "us_per_layer": round(given_us, 3), "launches_per_step": len(GROUPS) * LAYERS,
            "algorithmic_bytes_per_layer": given_bytes,
            "hbm_GBps": round(given_bytes / given_us / 1e3, 1),
            "pct_hbm_peak": round(given_bytes / given_us / 1e3 / HBM_PEAK_GBPS * 100, 2),
        },
        "per_group": per_group,
        "batched_rows_us_per_layer": batched,
        "batched_rows_per_group": batched_groups,
        "prefill": prefill,
        "selective": selective,
        "decode_loop": decode,
        "module_forward_eager_us": module_eager,
        "wall_ms_timed_region": round(wall_ms, 2),
        "roofline": {
            "bound": "hbm",
            "kernel": f"{dom_launch['kernel']} (gate|up group launch, N=28672, K=4096, M=1, rank 128, r given; grid "
                      f"{dom_launch['grid'][0]} x {dom_launch['block']} threads)",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "avg_launch_us": round(dom_us, 3),
            "algorithmic_bytes_per_launch": dom_bytes,
            # the same group with its projection launch: all of the group's bytes over the time of both launches
            "frac_with_projection_launch": round(per_group[DOMINANT]["pct_hbm_peak"] / 100, 4),
            # a kernel of the same grid that only reads the launch's algorithmic bytes (glowq_probe_stream_read), and one
            # that does nothing (back-to-back launches in a graph): what the memory system and the launch path leave
            "stream_read_GBps": stream_read,
            "frac_of_stream_read": round(achieved / stream_read, 4) if stream_read else None,
            "empty_launch_us": round(empty_us, 3),
            # HBM bytes per launch counted by rocprofv3 (FETCH_SIZE + WRITE_SIZE scaled on a copy of known size) in an
            # earlier profiling run of this script: read from the file named next to it, null without that file
            "traffic": traffic,
            "traffic_source": traffic_source,
        },
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(torch)
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result))


if __name__ == "__main__":
    main()
