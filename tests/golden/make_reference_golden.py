"""Writes tests/golden/reference_golden.npz: input/output vectors of the reference's OWN PyTorch
quantizer, so that the CPU oracle and the kernels are checked against the reference's code and not
only against this repository's reading of it.

It runs in the build container only (the reference checkout is needed, default /root/reference or
$FPQ_REFERENCE); only the .npz it writes is committed.  The four torch-only leaf modules of the
reference are loaded by file path under a private package name -- `import src.quantization` itself
fails in this image because src/quantization/__init__.py pulls in modules that need
fast_hadamard_transform:

    src/quantization/quant_args.py   (enums)
    src/quantization/quant_ops.py    (cast_to_fp4, cast_to_eBm0, pack_fp4_to_uint8, cast_scales_to_eXmY)
    src/quantization/quantizer.py    (Quantizer.get_quantization_params / quantize)
    src/helpers.py                   (split_dim)

Per case the script does what the reference's exporter does for a weight (src/quantization/rtn.py:172-188):
    scales, zeros = quantizer.get_quantization_params(x)
    q             = quantizer.quantize(x, scales, zeros)
    codes         = pack_fp4_to_uint8(q)
    scale bytes   = cast_scales_to_eXmY(scales * quantizer.global_scale, precision)
on fp32 inputs whose values are bf16-representable (the kernels take bf16), without rotation (the
rotation is not part of these modules; the tests use the identity rotation).

Run from the repository root:  python tests/golden/make_reference_golden.py
"""
import importlib.util
import os
import sys
import types

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
REFERENCE = os.environ.get("FPQ_REFERENCE", "/root/reference")


def load_reference_modules():
    pkg = "_fpq_reference_src"
    for name, path in ((pkg, os.path.join(REFERENCE, "src")),
                       (pkg + ".quantization", os.path.join(REFERENCE, "src", "quantization"))):
        mod = types.ModuleType(name)
        mod.__path__ = [path]          # a namespace: submodules resolve, no __init__.py is executed
        sys.modules[name] = mod
    loaded = {}
    for name, rel in ((pkg + ".helpers", "src/helpers.py"),
                      (pkg + ".quantization.quant_args", "src/quantization/quant_args.py"),
                      (pkg + ".quantization.quant_ops", "src/quantization/quant_ops.py"),
                      (pkg + ".quantization.quantizer", "src/quantization/quantizer.py")):
        spec = importlib.util.spec_from_file_location(name, os.path.join(REFERENCE, rel))
        mod = importlib.util.module_from_spec(spec)
        sys.modules[name] = mod
        spec.loader.exec_module(mod)
        loaded[name.rsplit(".", 1)[1]] = mod
    return loaded


def inputs(fmt: str) -> torch.Tensor:
    """64 x 256 fp32, every value bf16-representable: Gaussian rows with outliers, rows made of E2M1
    decision points (ties) at several scales, zero rows and zero groups, tiny and huge magnitudes,
    powers of two and their bf16 neighbours as group maxima.  The NVFP4 input keeps its extremes
    within what one fp32 global scale and E4M3 group scales can span (2^-10 .. 3e4)."""
    gen = torch.Generator().manual_seed(4242)
    x = torch.randn(64, 256, generator=gen)
    x = torch.where(torch.rand(64, 256, generator=gen) < 0.01, x * 25.0, x)
    ties = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0, -0.25, -0.75, -1.25, -1.75, -2.5, -3.5, -5.0, -6.0])
    x[3] = 0.0                                    # an all-zero row
    x[4, :64] = 0.0                               # zero groups inside a row
    x[5] *= 2.0 ** -60 if fmt == "mxfp" else 2.0 ** -10
    x[6] *= 2.0 ** 40 if fmt == "mxfp" else 2.0 ** 6
    x[7] = ties.repeat(16)                        # maximum 6: scaled values sit exactly on the ties
    x[8] = (ties * 2.0 ** -7).repeat(16)
    x[9] = (ties * 3.0).repeat(16)                # maximum 18: ties after a non-trivial division
    x[10] = 2.0                                   # constant groups
    x[11] = -0.0                                  # negative zeros
    x[12, ::2] = 0.0                              # zeros next to values (zero nibble beside a code)
    for i, top in enumerate((1.0, 0.99609375, 1.0078125, 4.0, 3.984375, 448.0, 0.0078125, 1.9921875)):
        x[13 + i] = x[13 + i].clamp(-0.9, 0.9) * top     # group maxima around binade borders
        x[13 + i, ::16] = top
    x[21] *= 2.0 ** -20 if fmt == "mxfp" else 2.0 ** -6
    x[22, 5] = 3.0e4                              # one large outlier: the tracked NVFP4 global scale follows it
    return x.to(torch.bfloat16).to(torch.float32)


def run_case(ref, x, fmt, global_scale):
    """(packed codes uint8 [R, C/2], scale bytes uint8 [R, C/group], global scale used)."""
    Quantizer = ref["quantizer"].Quantizer
    ops = ref["quant_ops"]
    if fmt == "mxfp":
        q = Quantizer(bits=4, symmetric=True, format="mxfp", granularity="group", observer="minmax",
                      group_size=32, scale_precision="e8m0")
        precision = "e8m0"
    else:
        q = Quantizer(bits=4, symmetric=True, format="nvfp", granularity="group", observer="minmax",
                      group_size=16, scale_precision="e4m3")
        precision = "e4m3"
        if global_scale is not None:              # a static scale, as FPQuantLinear's buffers hold at inference
            q.global_scale = torch.tensor([global_scale], dtype=torch.float32)
            q._track_global_scale = False
    scales, zeros = q.get_quantization_params(x.clone())
    qx = q.quantize(x.clone(), scales, zeros)
    codes = ops.pack_fp4_to_uint8(qx)
    sbytes = ops.cast_scales_to_eXmY(scales * q.global_scale, precision)
    return codes.numpy(), sbytes.contiguous().numpy(), float(q.global_scale)


def main():
    ref = load_reference_modules()
    x = inputs("mxfp")
    out = {"mx_x_bits": x.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)}
    out["mx_codes"], out["mx_scales"], gs = run_case(ref, x, "mxfp", None)
    assert gs == 3.0
    x = inputs("nvfp")
    out["nv_x_bits"] = x.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    for tag, gs_in in (("tracked", None), ("gs3", 3.0), ("gs10", 10.0)):
        c, s, gs = run_case(ref, x, "nvfp", gs_in)
        out[f"nv_{tag}_codes"], out[f"nv_{tag}_scales"] = c, s
        out[f"nv_{tag}_global_scale"] = np.array([gs], dtype=np.float32)
    # the packing function alone, on every E2M1 grid value and both zeros in both nibble positions
    grid = torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])
    vals = torch.cat([grid, -grid])
    pairs = torch.stack([vals.repeat_interleave(16), vals.repeat(16)], dim=1).reshape(1, -1)
    out["pack_values"] = pairs.numpy()
    out["pack_bytes"] = ref["quant_ops"].pack_fp4_to_uint8(pairs).numpy()
    # cast_to_fp4 on every bf16 bit pattern in [-8, 8] (decision points included)
    bits = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).to(torch.float32)
    bits = bits[bits.abs() <= 8.0]
    out["fp4_in"] = bits.numpy()
    out["fp4_out"] = ref["quant_ops"].cast_to_fp4(bits.clone()).numpy()
    path = os.path.join(ROOT, "tests", "golden", "reference_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
