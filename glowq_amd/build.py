"""Builds libglowq_w4a16.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

    python -m glowq_amd.build            # compile every source, link the shared library

The library has no dependency on torch: it is plain HIP behind `extern "C"` entry points
(include/glowq_w4a16.h).  Objects are compiled in parallel, one hipcc process per source.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libglowq_w4a16.so")
SOURCES = ["abi.hip", "gemv.hip", "gemv_stream.hip", "gemv_chain.hip", "gemv_quad.hip", "gemv_qstream.hip", "skinny.hip", "skinny_tiled.hip", "gemm.hip", "misc.hip", "decode_glue.hip"]
ARCH = "gfx950"

HIPCC_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    "-Wall",
    "-Wno-unused-function",
    # keep hipcc from forming packed-fp32 instructions out of scalar float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the first kernel arguments arrive in scalar registers with the wave instead of through a load from the argument
    # buffer (a memory round trip at the head of every wave; kernels keep a prologue for firmware without the feature)
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


# Sources whose kernels keep loads in flight that the compiler does not track (inline assembly with hand-placed waits):
# a register spilled there would be stored before its load has returned, so these must compile without scratch memory,
# and their assembly must not touch a register of a load that is still outstanding (isa_lint.py).
NO_SCRATCH = {"gemv_stream.hip": "gemv_stream_kernel", "gemv_chain.hip": "gemv_stream_kernel",
              "gemv_qstream.hip": "gemv_qstream_kernel"}


def _check_no_scratch(src: str, kernel: str, remarks: str) -> None:
    name = None
    for line in remarks.splitlines():
        if "Function Name:" in line:
            name = line.split("Function Name:")[1].split()[0]
        elif "ScratchSize" in line and name and kernel in name:
            size = int(line.split("ScratchSize [bytes/lane]:")[1].split()[0])
            if size:
                raise RuntimeError(f"{src}: {name} spills {size} bytes per lane to scratch memory; its in-flight loads "
                                   "must stay in registers")


def _check_in_flight_registers(src: str, kernel: str, asm_dir: str) -> None:
    """The device assembly the compile left in `asm_dir` through the lint of isa_lint.py."""
    from .isa_lint import lint

    stem = os.path.splitext(src)[0]
    listings = [f for f in os.listdir(asm_dir) if f.startswith(stem + "-hip-amdgcn") and f.endswith(".s")]
    if not listings:
        raise RuntimeError(f"{src}: the compile left no device assembly to check")
    for f in listings:
        with open(os.path.join(asm_dir, f)) as fh:
            found = lint(fh.read(), kernel)
        if found:
            raise RuntimeError(f"{src}: registers of loads in flight are touched before their wait "
                               f"({len(found)} places), first:\n  " + "\n  ".join(found[:3]))


def _compile(src: str, obj_dir: str, extra) -> str:
    obj = os.path.join(obj_dir, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    if src in NO_SCRATCH:
        cmd.insert(1, "-Rpass-analysis=kernel-resource-usage")
        cmd.insert(1, "-save-temps=obj")  # keeps the device assembly beside the object
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    if src in NO_SCRATCH and res.returncode == 0:
        _check_no_scratch(src, NO_SCRATCH[src], res.stderr)
        _check_in_flight_registers(src, NO_SCRATCH[src], obj_dir)
        kept, skip = [], 0
        for l in res.stderr.splitlines():  # a remark is its own line plus the source line and the caret under it
            if "-Rpass-analysis=kernel-resource-usage" in l:
                skip = 2
            elif skip:
                skip -= 1
            elif "remarks generated" not in l and not l.startswith("In file included from"):
                kept.append(l)
        res.stderr = "\n".join(kept)
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose: bool = False, extra_flags=()) -> str:
    obj_dir = os.path.join(PKG_DIR, "build")
    os.makedirs(obj_dir, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(lambda s: _compile(s, obj_dir, list(extra_flags)), SOURCES))
    tmp = LIB_PATH + ".tmp"
    cmd = [_hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-fno-gpu-rdc", "-o", tmp, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print("built", LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    build(verbose=True, extra_flags=sys.argv[1:])
