"""Writes the golden vectors in this folder by running the reference's own Python functions once.

Run in the build container only (the reference checkout is not available anywhere else):

    python tests/golden/make_golden.py [/root/reference]

Covers the functions whose bit-exact behaviour depends on per-op fp16 rounding of torch CPU ops
and so cannot be fixed by mathematics alone:
  _pack_int4_to_int32, _unpack_int4_i32, _quantize_per_group_w4, CudaW4A16Linear._dequant_chunk and
  the CPU chunked forward (src/cuda_w4a16/linear.py:42-88,229-253).
and the quantiser of step 1's layer, TritonTrue4BitLinear.from_float with dequantize_from_triton_layer
(src/step1_quantize.py:215-290), on CPU tensors (its Triton kernel is never launched).
Outputs are plain ``.npz`` arrays (inputs and expected outputs only).
"""
import os
import sys

import numpy as np
import torch


def main(ref_root: str) -> None:
    sys.path.insert(0, os.path.join(ref_root, "src"))
    from cuda_w4a16 import linear as ref  # noqa: E402

    here = os.path.dirname(os.path.abspath(__file__))
    out = {}

    # ---- pack / unpack -------------------------------------------------------------
    g = torch.Generator().manual_seed(100)
    codes = torch.randint(0, 16, (5, 7, 8), generator=g, dtype=torch.uint8)
    codes[0, 0] = 15  # all nibbles set: sign bit of the int32
    codes[0, 1] = torch.tensor([0, 0, 0, 0, 0, 0, 0, 8], dtype=torch.uint8)  # only the sign bit
    packed = ref._pack_int4_to_int32(codes)
    out["pack_codes"] = codes.numpy()
    out["pack_words"] = packed.numpy()
    out["unpack_vals_50"] = ref._unpack_int4_i32(packed, 50).numpy()
    out["unpack_vals_56"] = ref._unpack_int4_i32(packed, 56).numpy()

    # ---- quantiser -----------------------------------------------------------------
    cases = {
        # name: (N, K, group_size, std, seed)
        "a": (8, 256, 128, 0.02, 0),
        "b": (16, 384, 128, 0.02, 1),     # 3 groups -> zero-point word padded with code 8
        "c": (4, 200, 64, 1.0, 2),        # K not a multiple of the group: zero padding
        "d": (6, 1152, 128, 0.05, 3),     # 9 groups -> two zero-point words
        "e": (4, 64, 32, 0.02, 4),
    }
    for name, (n, k, gs, std, seed) in cases.items():
        g = torch.Generator().manual_seed(seed)
        w = (torch.randn(n, k, generator=g) * std).half()
        if name == "a":
            # ties and clipping: positive-only group (zero-point clamps to 0), negative-only
            # group (zero-point clamps to 15), and exact half-way values.
            w[0, :128] = w[0, :128].abs() + 0.01
            w[1, :128] = -w[1, :128].abs() - 0.01
            w[2, :128] = torch.linspace(-0.75, 0.75, 128).half()
            w[3, 128:] = (torch.arange(128) % 16).half() * 0.5 - 3.75
        qw, qz, sc, kp = ref._quantize_per_group_w4(w, gs)
        out[f"q_{name}_w"] = w.numpy()
        out[f"q_{name}_gs"] = np.array([gs, kp], dtype=np.int64)
        out[f"q_{name}_qweight"] = qw.numpy()
        out[f"q_{name}_qzeros"] = qz.numpy()
        out[f"q_{name}_scales"] = sc.numpy()

    # ---- module: from_float, dequant chunk, CPU chunked forward --------------------------
    os.environ["W4A16_KERNEL_OUT_DTYPE"] = "fp16"
    # CPU tensors + forced GEMM route = the 512-row chunked torch branch; the reference's
    # prebuilt extension is never imported.
    os.environ["W4A16_FORCE_GEMM"] = "1"
    for name, (n, k, gs, m, bias, seed) in {
        "m1": (48, 256, 128, 3, False, 10),
        "m2": (40, 1152, 128, 5, True, 11),
    }.items():
        g = torch.Generator().manual_seed(seed)
        lin = torch.nn.Linear(k, n, bias=bias).half()
        with torch.no_grad():
            lin.weight.copy_((torch.randn(n, k, generator=g) * 0.02).half())
            if bias:
                lin.bias.copy_((torch.randn(n, generator=g) * 0.1).half())
        x = torch.randn(m, k, generator=g).half()
        mod = ref.CudaW4A16Linear.from_float(lin, gs)
        deq = mod._dequant_chunk(0, n)
        y = mod(x)  # CPU tensors: 512-row chunked dequant + matmul branch
        out[f"{name}_w"] = lin.weight.detach().numpy()
        if bias:
            out[f"{name}_bias"] = lin.bias.detach().numpy()
        out[f"{name}_x"] = x.numpy()
        out[f"{name}_gs"] = np.array([gs], dtype=np.int64)
        out[f"{name}_qweight"] = mod.qweight_i32.numpy()
        out[f"{name}_qzeros"] = mod.qzeros_i32.numpy()
        out[f"{name}_scales"] = mod.scales_f16.numpy()
        out[f"{name}_deq"] = deq.numpy()
        out[f"{name}_y"] = y.detach().numpy()
        out[f"{name}_state_keys"] = np.array(sorted(mod.state_dict().keys()))

    np.savez_compressed(os.path.join(here, "w4a16_golden.npz"), **out)
    print("wrote", os.path.join(here, "w4a16_golden.npz"), len(out), "arrays")


def step1(ref_root: str) -> None:
    """Step 1's quantiser: in-range groups, one-sided groups (zero-point outside [0, 15]), two group sizes."""
    sys.path.insert(0, os.path.join(ref_root, "src"))
    import step1_quantize as ref  # noqa: E402  (imports transformers / datasets / triton; runs nothing of them)

    here = os.path.dirname(os.path.abspath(__file__))
    out = {}
    cases = {
        # name: (N, K, group_size, std, seed, one-sided rows)
        "in_range": (8, 512, 128, 0.02, 20, False),
        "many_groups": (6, 1024, 128, 0.05, 21, False),   # (an odd number of groups raises in the reference: its
                                                           #  zero-point buffer holds G // 2 bytes, from_float packs ceil)
        "small_groups": (4, 256, 64, 1.0, 22, False),      # (K not a multiple of the group size raises as well: the code
                                                           #  buffer holds K // 2 bytes, from_float packs the padded row)
        "one_sided": (8, 256, 128, 0.02, 23, True),
    }
    for name, (n, k, gs, std, seed, one_sided) in cases.items():
        g = torch.Generator().manual_seed(seed)
        w = (torch.randn(n, k, generator=g) * std).half()
        if one_sided:
            w[0, :128] = w[0, :128].abs() + 0.05          # all positive, far from zero: zero-point below 0
            w[1, 128:] = -w[1, 128:].abs() - 0.05         # all negative: zero-point above 15
            w[2, :128] = w[2, :128].abs() + 0.001         # all positive, touching zero: zero-point 0 or -1
        lin = torch.nn.Linear(k, n, bias=False).half()
        with torch.no_grad():
            lin.weight.copy_(w)
        layer = ref.TritonTrue4BitLinear.from_float(lin, gs)
        out[f"{name}_w"] = w.numpy()
        out[f"{name}_gs"] = np.array([gs], dtype=np.int64)
        out[f"{name}_qweight"] = layer.qweight.numpy()
        out[f"{name}_qzeros"] = layer.qzeros.numpy()
        out[f"{name}_scales"] = layer.scales.numpy()
        out[f"{name}_deq"] = ref.dequantize_from_triton_layer(layer).numpy()
    np.savez_compressed(os.path.join(here, "step1_golden.npz"), **out)
    print("wrote", os.path.join(here, "step1_golden.npz"), len(out), "arrays")


if __name__ == "__main__":
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    main(root)
    step1(root)
