#!/usr/bin/env python3
"""Benchmark of the FP4 quantized-linear hot path on one MI355X.

python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

Prints ONE JSON line.  A step is one pass of the workload's kernel(s) over one synthetic batch
resident in HBM; buffers rotate through more than the 256 MB last-level cache so that the
HBM-bound kernels are measured against HBM, not cache.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "fp-quant_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

METRIC = "W4A4 FP4 GEMM TFLOPS + fused quantize GB/s (% roofline), 1 MI355X"
HBM_PEAK_GBS = 8000.0
FP4_PEAK_TFLOPS = 10100.0
BF16_PEAK_TFLOPS = 2500.0


def student_t(torch, rows, cols, seed, df=3):
    gen = torch.Generator().manual_seed(seed)
    z = torch.randn(rows, cols, generator=gen)
    chi = torch.randn(df, rows, cols, generator=gen).pow(2).sum(0)
    return (z / torch.sqrt(chi / df)).to(torch.bfloat16)


def outlier_normal(torch, rows, cols, seed, frac=0.005, mult=25.0):
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, cols, generator=gen)
    mask = torch.rand(rows, cols, generator=gen) < frac
    return torch.where(mask, x * mult, x).to(torch.bfloat16)


SETTLE_MS = 30.0        # untimed GPU work before any timed region, so that short runs see settled clocks
BLOCK_MIN_MS = 50.0     # GPU time a block-median measurement covers at least, per leg
BLOCK_MIN_COUNT = 9


def _settle(torch, fn, n_variants, chunk):
    """Untimed launches until SETTLE_MS of GPU time have passed (the part's clock moves with load: the
    first milliseconds after an idle period run at another frequency than a sustained loop)."""
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    spent, i = 0.0, 0
    while spent < SETTLE_MS:
        e0.record()
        for _ in range(chunk):
            fn(i % n_variants)
            i += 1
        e1.record()
        torch.cuda.synchronize()
        spent += e0.elapsed_time(e1)


def time_kernel(torch, fn, n_variants, steps, warmup):
    """Runs fn(i % n_variants) warmup+steps times on the current stream (plus the untimed settling
    launches above, before the timed region).  Returns (wall ms per step, event ms per step) over
    EXACTLY `steps` timed steps."""
    for i in range(warmup):
        fn(i % n_variants)
    torch.cuda.synchronize()
    _settle(torch, fn, n_variants, max(4, min(steps, 64)))
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for i in range(steps):
        fn(i % n_variants)
    e1.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    return wall, e0.elapsed_time(e1) / steps


def time_blocks(torch, legs, n_variants, block):
    """Interleaved block timing of several legs (name -> fn): blocks of `block` launches of each leg
    in turn, HIP events around every block, until every leg has BLOCK_MIN_MS of GPU time and
    BLOCK_MIN_COUNT blocks.  Returns name -> (median ms per launch, min, max, blocks).  Interleaving
    makes the legs see the same clocks, the median discards the blocks a frequency change fell into."""
    names = list(legs)
    for nm in names:
        _settle(torch, legs[nm], n_variants, block)
    per = {nm: [] for nm in names}
    total = {nm: 0.0 for nm in names}
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    i = 0
    while min(total.values()) < BLOCK_MIN_MS or len(per[names[0]]) < BLOCK_MIN_COUNT:
        for nm in names:
            fn = legs[nm]
            e0.record()
            for _ in range(block):
                fn(i % n_variants)
                i += 1
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1)
            per[nm].append(ms / block)
            total[nm] += ms
        if len(per[names[0]]) >= 400:
            break
    out = {}
    for nm in names:
        v = sorted(per[nm])
        out[nm] = (v[len(v) // 2], v[0], v[-1], len(v))
    return out


def bench_quantize(torch, fmt, rows, cols, g, steps, warmup, seed, packed=False):
    """Fused rotate+quantize on rotating input buffers through the C ABI (packed: MXFP4 written in the
    packed GEMM operand layout, same bytes in another order)."""
    from fp_quant import _engine
    lib = _engine.lib()
    dev = torch.device("cuda:0")
    group = 32 if fmt == "mxfp4" else 16
    x_cpu = outlier_normal(torch, rows, cols, seed) if fmt == "mxfp4" else student_t(torch, rows, cols, seed)
    in_bytes = rows * cols * 2
    n_buf = max(2, int(640e6 // in_bytes) + 1)
    xs = [x_cpu.to(dev) if i == 0 else x_cpu.to(dev).roll(i, 0).contiguous() for i in range(n_buf)]
    codes = [torch.empty(rows, cols // 2, dtype=torch.uint8, device=dev) for _ in range(n_buf)]
    scales = [torch.empty(rows, cols // group, dtype=torch.uint8, device=dev) for _ in range(n_buf)]
    norm = float(torch.tensor(g ** -0.5, dtype=torch.bfloat16))
    gs = torch.tensor([1.0], dtype=torch.float32, device=dev)
    if fmt == "nvfp4":
        # the tracked global scale of the configuration: 2688 * fl(1 / max|rotated x|), two fp32 roundings as
        # src/quantization/quantizer.py:145-150 writes it (outside the timed region)
        amax = torch.zeros(1, dtype=torch.float32, device=dev)
        _engine.check(lib.fpq_rotated_absmax(xs[0].data_ptr(), rows, cols, 0, g, norm, None, amax.data_ptr(),
                                             torch.cuda.current_stream().cuda_stream), "fpq_rotated_absmax")
        gs.copy_(torch.tensor(2688.0, dtype=torch.float32, device=dev) * (1.0 / amax))
    stream = torch.cuda.current_stream().cuda_stream
    ptrs = [(xs[i].data_ptr(), codes[i].data_ptr(), scales[i].data_ptr()) for i in range(n_buf)]

    def run(i):
        xp, cp, sp = ptrs[i]
        if fmt == "mxfp4" and packed:
            st = lib.fpq_quantize_mx_packed(xp, rows, cols, 0, g, norm, cp, sp, 0, stream)
        elif fmt == "mxfp4":
            st = lib.fpq_quantize_mx(xp, rows, cols, 0, g, norm, None, cp, sp, rows, cols // group, 0, stream)
        else:
            st = lib.fpq_quantize_nv(xp, rows, cols, 0, g, norm, None, gs.data_ptr(), cp, sp, rows,
                                     cols // group, 0, stream)
        if st != 0:
            _engine.check(st, "bench quantize")

    wall, ev_steps = time_kernel(torch, run, n_buf, steps, warmup)
    ev, ev_min, ev_max, blocks = time_blocks(torch, {"q": run}, n_buf, max(20, min(steps, 100)))["q"]
    algo_bytes = rows * cols * (2 + 0.5 + 1.0 / group)
    return {
        "workload": f"{fmt}_quantize_{rows}x{cols}_had{g}" + ("_packed" if packed else ""),
        "ms_per_step": wall,
        "kernel_ms": ev,
        "kernel_ms_min": ev_min,
        "kernel_ms_over_steps": ev_steps,
        "blocks": blocks,
        "algo_bytes": algo_bytes,
        "gbps": algo_bytes / (ev * 1e-3) / 1e9,
        "buffers": n_buf,
    }


def bench_fused_producers(torch, steps, warmup):
    """The quantizers fused with the producer of their input at Llama-3.1-8B prefill sizes (8192 tokens), MXFP4
    Hadamard-128, packed output, through the C ABI: RMSNorm (row statistic + fused kernel, with the bf16
    by-product) over [8192, 4096] and SiLU(gate)*up over [8192, 14336].  Algorithmic bytes: inputs once, codes,
    scales, by-product."""
    from fp_quant import _engine
    lib = _engine.lib()
    dev = torch.device("cuda:0")
    norm = float(torch.tensor(128 ** -0.5, dtype=torch.bfloat16))
    stream = torch.cuda.current_stream().cuda_stream
    out = {}

    def packed(rows, cols):
        return (torch.empty(lib.fpq_packed_codes_bytes(rows, cols), dtype=torch.uint8, device=dev),
                torch.empty(lib.fpq_packed_scales_bytes(rows, cols), dtype=torch.uint8, device=dev))

    rows, cols = 8192, 4096
    n_buf = 8
    xs = [outlier_normal(torch, rows, cols, 10 + i).to(dev) for i in range(2)]
    xs = [xs[i % 2].roll(i, 0).contiguous() for i in range(n_buf)]
    w = (1 + 0.1 * torch.randn(cols)).to(torch.bfloat16).to(dev)
    inv = torch.empty(rows, dtype=torch.float32, device=dev)
    y = torch.empty(rows, cols, dtype=torch.bfloat16, device=dev)
    pc, ps = packed(rows, cols)

    def run_norm(i):
        st = lib.fpq_row_inv_rms(xs[i].data_ptr(), cols, rows, cols, 1e-5, inv.data_ptr(), stream)
        st = st or lib.fpq_rmsnorm_quantize_mx_packed(xs[i].data_ptr(), cols, inv.data_ptr(), w.data_ptr(), rows, cols,
                                                      0, 128, norm, y.data_ptr(), pc.data_ptr(), ps.data_ptr(), 0, stream)
        if st != 0:
            _engine.check(st, "bench rmsnorm_quantize")

    wall, ev = time_kernel(torch, run_norm, n_buf, steps, warmup)
    algo = rows * cols * (2 + 2 + 0.5 + 1.0 / 32)
    out["rmsnorm_quantize"] = {"workload": f"rmsnorm_quantize_mx_packed_{rows}x{cols}_had128 (+ bf16 by-product)",
                               "kernels_us": round(ev * 1e3, 2), "GB/s": round(algo / (ev * 1e-3) / 1e9, 1),
                               "hbm_frac": round(algo / (ev * 1e-3) / 8e12, 4)}
    del xs, y

    cols = 14336
    n_buf = 3
    g0 = student_t(torch, rows, cols, 20).to(dev)
    gates = [g0.roll(i, 0).contiguous() for i in range(n_buf)]
    ups = [g0.roll(i + 1, 1).contiguous() for i in range(n_buf)]
    pc, ps = packed(rows, cols)

    def run_silu(i):
        st = lib.fpq_silu_mul_quantize_mx_packed(gates[i].data_ptr(), cols, ups[i].data_ptr(), cols, rows, cols, 0, 128,
                                                 norm, None, pc.data_ptr(), ps.data_ptr(), 0, stream)
        if st != 0:
            _engine.check(st, "bench silu_mul_quantize")

    wall, ev = time_kernel(torch, run_silu, n_buf, steps, warmup)
    algo = rows * cols * (2 + 2 + 0.5 + 1.0 / 32)
    out["silu_mul_quantize"] = {"workload": f"silu_mul_quantize_mx_packed_{rows}x{cols}_had128",
                                "kernel_us": round(ev * 1e3, 2), "GB/s": round(algo / (ev * 1e-3) / 1e9, 1),
                                "hbm_frac": round(algo / (ev * 1e-3) / 8e12, 4)}
    return out


def bench_hbm_probe(torch, steps, warmup):
    """What plain data movement reaches on this GPU, for judging the HBM-bound kernels: a device-to-device copy
    (bytes read + bytes written per second) moving as many bytes as the NVFP4 quantize workload (86 MB) and at
    256 MiB."""
    dev = torch.device("cuda:0")
    out = {}
    for name, nbytes in (("copy_43MB", 43 << 20), ("copy_256MiB", 256 << 20)):
        n_buf = max(2, (640 << 20) // nbytes)
        src = [torch.empty(nbytes, dtype=torch.uint8, device=dev).random_(0, 256) for _ in range(n_buf)]
        dst = [torch.empty_like(b) for b in src]
        wall, ev = time_kernel(torch, lambda i: dst[i].copy_(src[i]), n_buf, steps, warmup)
        out[name] = {"us": round(ev * 1e3, 2), "GB/s": round(2 * nbytes / (ev * 1e-3) / 1e9, 1)}
        del src, dst
    return out


def check_linear_output(torch, x, y, w, wq, ws, m, n, k, g, alpha, rows=48, cols=192):
    """Outside every timed region: a seeded sample of the output the timed kernels just wrote against the
    CPU oracle (quantize the sampled activation rows, dequantize, fp64 matmul against the sampled weight
    rows), with the tolerance of the GEMM tests.  The oracle is the checker here, never the thing timed."""
    from oracle import fpq_oracle as O
    gen = torch.Generator().manual_seed(m + n)
    ri = torch.randperm(m, generator=gen)[:min(rows, m)].sort().values
    ci = torch.randperm(n, generator=gen)[:min(cols, n)].sort().values
    xq, xs, _ = O.quantize_mx(x[ri.to(x.device)].cpu(), O.ROT_HADAMARD, g)
    wq_s, ws_s = wq[ci.to(wq.device)].cpu(), ws[ci.to(ws.device)].cpu()
    wq_o, ws_o, _ = O.quantize_mx(w[ci.to(w.device)].cpu(), O.ROT_HADAMARD, g)
    if not (torch.equal(wq_o, wq_s) and torch.equal(ws_o, ws_s)):
        raise RuntimeError("bench: quantized weights differ from the oracle's")
    ref, mag = O.gemm_ref(xq, xs, wq_s, ws_s, alpha, "mxfp4")
    got = y[ri.to(y.device)][:, ci.to(y.device)].cpu()
    tol = 2.0 ** -8 * ref.abs() + 1e-5 * mag + 1e-6
    ok = bool(((got.double() - ref).abs() <= tol).all())
    exact = float((got == ref.to(torch.bfloat16)).float().mean())
    if not ok:
        raise RuntimeError("bench: the timed MXFP4 linear's output differs from the oracle beyond the tolerance")
    return {"sample": f"{len(ri)}x{len(ci)} outputs", "within_tolerance": ok, "equal_to_bf16_of_fp64": round(exact, 4)}


def bench_linear(torch, fmt, m, n, k, g, steps, warmup, seed, check=False):
    """Quantize activations + W4A4 GEMM (the body of FPQuantLinear.forward) through the C ABI.
    Weights are quantized once outside the timed region; activations rotate through buffers."""
    from fp_quant import _engine
    lib = _engine.lib()
    dev = torch.device("cuda:0")
    group = 32 if fmt == "mxfp4" else 16
    gen = torch.Generator().manual_seed(seed)
    w = (torch.randn(n, k, generator=gen) * 0.02).to(torch.bfloat16).to(dev)
    norm = float(torch.tensor(g ** -0.5, dtype=torch.bfloat16))
    gs = torch.tensor([3.0], dtype=torch.float32, device=dev)
    alpha = torch.tensor([float((1.0 / (torch.tensor([3.0], dtype=torch.bfloat16) ** 2)).float())],
                         dtype=torch.float32, device=dev)
    stream = torch.cuda.current_stream().cuda_stream

    def quant(src, rows, codes, scales):
        if fmt == "mxfp4":
            return lib.fpq_quantize_mx(src, rows, k, 0, g, norm, None, codes, scales, rows, k // group, 0, stream)
        return lib.fpq_quantize_nv(src, rows, k, 0, g, norm, None, gs.data_ptr(), codes, scales, rows,
                                   k // group, 0, stream)

    wq = torch.empty(n, k // 2, dtype=torch.uint8, device=dev)
    ws = torch.empty(n, k // group, dtype=torch.uint8, device=dev)
    _engine.check(quant(w.data_ptr(), n, wq.data_ptr(), ws.data_ptr()), "weight quantize")
    n_buf = max(2, min(64, int(320e6 // max(1, m * k * 2 + m * n * 2)) + 1))
    xs_ = [torch.randn(m, k, generator=gen).to(torch.bfloat16).to(dev) for _ in range(min(n_buf, 4))]
    xs_ = [xs_[i % len(xs_)].clone() for i in range(n_buf)]
    xq = [torch.empty(m, k // 2, dtype=torch.uint8, device=dev) for _ in range(n_buf)]
    xsc = [torch.empty(m, k // group, dtype=torch.uint8, device=dev) for _ in range(n_buf)]
    ys = [torch.empty(m, n, dtype=torch.bfloat16, device=dev) for _ in range(n_buf)]
    gemm = lib.fpq_gemm_mxf4 if fmt == "mxfp4" else lib.fpq_gemm_nvf4
    p = [(xs_[i].data_ptr(), xq[i].data_ptr(), xsc[i].data_ptr(), ys[i].data_ptr()) for i in range(n_buf)]

    from fp_quant.module import hip_ops
    nv_packed = fmt == "nvfp4" and hip_ops.nv_packed_eligible(m, n, k, fused_linear=True)
    if (fmt == "mxfp4" and hip_ops.packed_linear_eligible(m, k, "abs_max")) or nv_packed:
        # what FPQuantLinear.forward runs for this many rows: activations quantized straight into the
        # packed operand layout, weights re-tiled once (outside the timed region, like their quantization)
        wp, wsp = (hip_ops.pack_nvf4 if nv_packed else hip_ops.pack_mxf4)(wq, ws, n, k)
        scales_bytes = lib.fpq_packed_scales_bytes_nv if nv_packed else lib.fpq_packed_scales_bytes
        gemm_packed = lib.fpq_gemm_nvf4_packed if nv_packed else lib.fpq_gemm_mxf4_packed

        def quant_packed(src, codes, scales):
            if nv_packed:
                return lib.fpq_quantize_nv_packed(src, m, k, 0, g, norm, gs.data_ptr(), codes, scales, 0, stream)
            return lib.fpq_quantize_mx_packed(src, m, k, 0, g, norm, codes, scales, 0, stream)

        # Up to 128 rows the GEMM streams the weights (HBM-bound): they rotate through enough copies to
        # exceed the 256 MB last-level cache, so that every launch reads them from HBM as a decode step
        # does; the figure with one resident copy is reported beside it.
        n_w = 1 if m > 128 else int(640e6 // (wp.numel() + wsp.numel())) + 1
        wps = [(wp, wsp)] + [(wp.clone(), wsp.clone()) for _ in range(n_w - 1)]
        wptr = [(a.data_ptr(), b.data_ptr()) for a, b in wps]
        xp = [torch.empty(lib.fpq_packed_codes_bytes(m, k), dtype=torch.uint8, device=dev) for _ in range(n_buf)]
        xsp = [torch.empty(scales_bytes(m, k), dtype=torch.uint8, device=dev) for _ in range(n_buf)]
        pp = [(xs_[i].data_ptr(), xp[i].data_ptr(), xsp[i].data_ptr(), ys[i].data_ptr()) for i in range(n_buf)]

        def run_linear(i):
            a, b, c, d = pp[i]
            wc, wsc = wptr[i % n_w]
            st = quant_packed(a, b, c)
            st = st or gemm_packed(b, c, wc, wsc, alpha.data_ptr(), None, d, m, n, k, stream)
            if st != 0:
                _engine.check(st, "bench packed linear")

        def run_gemm(i):
            a, b, c, d = pp[i]
            wc, wsc = wptr[i % n_w]
            st = gemm_packed(b, c, wc, wsc, alpha.data_ptr(), None, d, m, n, k, stream)
            if st != 0:
                _engine.check(st, "bench packed gemm")

        def run_gemm_resident(i):
            a, b, c, d = pp[i]
            st = gemm_packed(b, c, wptr[0][0], wptr[0][1], alpha.data_ptr(), None, d, m, n, k, stream)
            if st != 0:
                _engine.check(st, "bench packed gemm")

        res = _time_linear(torch, run_linear, run_gemm, fmt, m, n, k, g, group, n_buf, steps, warmup, "packed",
                           run_gemm_resident if n_w > 1 else None)
        res["weight_copies"] = n_w
        if check and fmt == "mxfp4":
            run_linear(0)
            res["output_check"] = check_linear_output(torch, xs_[0], ys[0], w, wq, ws, m, n, k, g, float(alpha))
        return res

    def run_linear(i):
        a, b, c, d = p[i]
        st = quant(a, m, b, c)
        st = st or gemm(b, c, k // group, wq.data_ptr(), ws.data_ptr(), k // group, alpha.data_ptr(), None,
                        d, m, n, k, stream)
        if st != 0:
            _engine.check(st, "bench linear")

    def run_gemm(i):
        a, b, c, d = p[i]
        st = gemm(b, c, k // group, wq.data_ptr(), ws.data_ptr(), k // group, alpha.data_ptr(), None,
                  d, m, n, k, stream)
        if st != 0:
            _engine.check(st, "bench gemm")

    res = _time_linear(torch, run_linear, run_gemm, fmt, m, n, k, g, group, n_buf, steps, warmup, "row-major")
    if check and fmt == "mxfp4":
        run_linear(0)
        res["output_check"] = check_linear_output(torch, xs_[0], ys[0], w, wq, ws, m, n, k, g, float(alpha))
    return res


def _time_linear(torch, run_linear, run_gemm, fmt, m, n, k, g, group, n_buf, steps, warmup, layout,
                 run_gemm_resident=None):
    wall, ev_steps = time_kernel(torch, run_linear, n_buf, steps, warmup)
    block = max(10, min(steps, 100))
    consistent = False
    legs = {"linear": run_linear, "gemm": run_gemm}
    if run_gemm_resident is not None:
        legs["gemm_resident"] = run_gemm_resident
    for _ in range(3):   # the GEMM alone cannot take longer than quantize + the same GEMM
        t = time_blocks(torch, legs, n_buf, block)
        ev, ev_gemm = t["linear"][0], t["gemm"][0]
        if ev_gemm <= ev * 1.01:
            consistent = True
            break
    flops = 2.0 * m * n * k
    gemm_bytes = n * k / 2 + n * k / group + m * k / 2 + m * k / group + 2.0 * m * n
    return {
        "workload": f"{fmt}_linear_M{m}_N{n}_K{k}_had{g}",
        "ms_per_step": wall,
        "linear_ms_over_steps": ev_steps,
        "linear_ms": ev,
        "gemm_ms": ev_gemm,
        "gemm_ms_min": t["gemm"][1],
        "gemm_ms_max": t["gemm"][2],
        "blocks": t["gemm"][3],
        "block_launches": block,
        "timing_consistent": consistent,
        "gemm_ms_cache_resident": t["gemm_resident"][0] if run_gemm_resident is not None else None,
        "flops": flops,
        "gemm_bytes": gemm_bytes,
        "linear_tflops": flops / (ev * 1e-3) / 1e12,
        "linear_tflops_over_steps": flops / (ev_steps * 1e-3) / 1e12,
        "gemm_tflops": flops / (ev_gemm * 1e-3) / 1e12,
        "gemm_gbps": gemm_bytes / (ev_gemm * 1e-3) / 1e9,
        "buffers": n_buf,
        "operand_layout": layout,
    }


def bench_vendor_gemm(torch, steps, warmup, shapes=((2048, 14336, 4096), (8192, 14336, 4096), (8192, 4096, 14336))):
    """The library GEMMs PyTorch-ROCm reaches (hipBLASLt) next to this repository's packed MXFP4 kernel, same
    process, same shapes, operands of uniformly random codes (every kernel sees the same bytes): MXFP4 through
    torch._scaled_mm (float4_e2m1fn_x2 operands, float8_e8m0fnu scales per 32), fp8 through torch._scaled_mm,
    bf16 through F.linear.  Only timings are compared; the scale layouts the library kernels expect are not
    reproduced, so their numerical results are not."""
    from fp_quant import _engine
    lib = _engine.lib()
    dev = torch.device("cuda:0")

    def timed(fn):
        for _ in range(max(3, warmup)):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        best = None
        for _ in range(3):
            e0.record()
            for _ in range(steps):
                fn()
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / steps
            best = us if best is None else min(best, us)
        return best

    out = {}
    for m, n, k in shapes:
        gen = torch.Generator(device=dev).manual_seed(m + n + k)
        xq = torch.randint(0, 256, (m, k // 2), dtype=torch.uint8, device=dev, generator=gen)
        wq = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device=dev, generator=gen)
        xs = torch.randint(118, 130, (m, k // 32), dtype=torch.uint8, device=dev, generator=gen)
        ws = torch.randint(118, 130, (n, k // 32), dtype=torch.uint8, device=dev, generator=gen)
        flops = 2.0 * m * n * k
        res = {}
        stream = torch.cuda.current_stream().cuda_stream
        xp = torch.empty(lib.fpq_packed_codes_bytes(m, k), dtype=torch.uint8, device=dev)
        xsp = torch.empty(lib.fpq_packed_scales_bytes(m, k), dtype=torch.uint8, device=dev)
        wp = torch.empty(lib.fpq_packed_codes_bytes(n, k), dtype=torch.uint8, device=dev)
        wsp = torch.empty(lib.fpq_packed_scales_bytes(n, k), dtype=torch.uint8, device=dev)
        _engine.check(lib.fpq_pack_mxf4(xq.data_ptr(), xs.data_ptr(), k // 32, m, k, xp.data_ptr(), xsp.data_ptr(), stream), "pack")
        _engine.check(lib.fpq_pack_mxf4(wq.data_ptr(), ws.data_ptr(), k // 32, n, k, wp.data_ptr(), wsp.data_ptr(), stream), "pack")
        alpha = torch.tensor([1e-3], dtype=torch.float32, device=dev)
        y = torch.empty(m, n, dtype=torch.bfloat16, device=dev)
        us = timed(lambda: lib.fpq_gemm_mxf4_packed(xp.data_ptr(), xsp.data_ptr(), wp.data_ptr(), wsp.data_ptr(),
                                                    alpha.data_ptr(), None, y.data_ptr(), m, n, k, stream))
        res["this_repo_mxfp4_packed"] = {"us": round(us, 2), "TFLOP/s": round(flops / us / 1e6, 1)}
        try:
            a4, b4 = xq.view(torch.float4_e2m1fn_x2), wq.view(torch.float4_e2m1fn_x2)
            sa, sb = xs.view(torch.float8_e8m0fnu), ws.view(torch.float8_e8m0fnu)
            us = timed(lambda: torch._scaled_mm(a4, b4.t(), scale_a=sa, scale_b=sb, out_dtype=torch.bfloat16))
            res["hipblaslt_mxfp4_scaled_mm"] = {"us": round(us, 2), "TFLOP/s": round(flops / us / 1e6, 1)}
        except Exception as e:   # not every PyTorch-ROCm build has the MXFP4 path
            res["hipblaslt_mxfp4_scaled_mm"] = {"error": f"{type(e).__name__}: {str(e)[:160]}"}
        xb = torch.randn(m, k, device=dev, dtype=torch.bfloat16, generator=gen)
        wb = torch.randn(n, k, device=dev, dtype=torch.bfloat16, generator=gen)
        try:
            x8, w8 = xb.to(torch.float8_e4m3fn), wb.to(torch.float8_e4m3fn)
            one = torch.ones((), device=dev)
            us = timed(lambda: torch._scaled_mm(x8, w8.t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16))
            res["hipblaslt_fp8_scaled_mm"] = {"us": round(us, 2), "TFLOP/s": round(flops / us / 1e6, 1)}
        except Exception as e:
            res["hipblaslt_fp8_scaled_mm"] = {"error": f"{type(e).__name__}: {str(e)[:160]}"}
        us = timed(lambda: torch.nn.functional.linear(xb, wb))
        res["hipblaslt_bf16_linear"] = {"us": round(us, 2), "TFLOP/s": round(flops / us / 1e6, 1)}
        out[f"M{m}_N{n}_K{k}"] = res
    return out


def bench_mfma_ceiling(torch, seed=4, iters=192):
    """Register-resident FP4 MFMA loop (no memory system): the matrix throughput and clock the chip
    sustains for all-zero operands and for operands with the bit statistics of quantized data, over
    about the duration of the M=2048 GEMM.  The second number is the practical ceiling of that GEMM."""
    from fp_quant import _engine
    from fp_quant.module import hip_ops
    lib = _engine.lib()
    dev = torch.device("cuda:0")
    blocks = torch.cuda.get_device_properties(0).multi_processor_count
    n_words = blocks * 256 * 32
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(n_words * 4 * 2 // 4096, 4096, generator=gen).to(torch.bfloat16).to(dev)
    from fp_quant.module.linear import get_hadamard_matrix
    h = get_hadamard_matrix(128, torch.bfloat16, dev)
    codes, _, _ = hip_ops.fused_quantize_mx_op(x, h, "abs_max", False)
    words = {"zeros": torch.zeros(n_words, dtype=torch.int32, device=dev),
             "quantized": codes.view(-1).view(torch.int32)[:n_words].contiguous()}
    sink = torch.empty(blocks * 256, dtype=torch.float32, device=dev)
    clocks = torch.empty(blocks * 2, dtype=torch.int64, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    out = {"iters": iters, "workgroups": blocks}
    for name, w in words.items():
        best = None
        for rep in range(6):
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record()
            st = lib.fpq_test_mfma_rate(w.data_ptr(), blocks, iters, sink.data_ptr(), clocks.data_ptr(), stream)
            e1.record()
            torch.cuda.synchronize()
            if st != 0:
                _engine.check(st, "fpq_test_mfma_rate")
            c = clocks.view(blocks, 2).double().cpu()
            us = float(c[:, 1].mean()) * 1e-2  # 100 MHz ticks -> us, inside the kernel (no launch overhead)
            ghz = float(c[:, 0].sum() / (c[:, 1].sum() * 10.0))
            if rep > 0 and (best is None or us < best[0]):
                best = (us, ghz)
        flops = blocks * 4 * iters * 16 * 131072.0
        out[name] = {"TFLOP/s": round(flops / (best[0] * 1e-6) / 1e12, 1), "clock_GHz": round(best[1], 3),
                     "loop_us": round(best[0], 1)}
    return out


def bench_power(torch, seconds=3.0):
    """Socket power and per-XCD clocks (amd-smi) while one kernel runs back to back for `seconds`: the packed
    MXFP4 GEMM at M=2048 N=14336 K=4096 on quantized Gaussian data, the register-resident MFMA loop on the same
    operand bits and on zeros, and a plain 256 MiB copy.  Shows which limit the GEMM runs at: the package power
    cap (the clock the firmware grants falls) or the matrix pipes' own throttle (power below the cap)."""
    import re
    import subprocess
    import threading
    from fp_quant import _engine
    lib = _engine.lib()
    dev = torch.device("cuda:0")
    st = torch.cuda.current_stream().cuda_stream
    norm = float(torch.tensor(128 ** -0.5, dtype=torch.bfloat16))
    m, n, k = 2048, 14336, 4096
    gen = torch.Generator().manual_seed(2)
    w = (torch.randn(n, k, generator=gen) * 0.02).to(torch.bfloat16).to(dev)
    x = torch.randn(m, k, generator=gen).to(torch.bfloat16).to(dev)

    def quantize(t, rows):
        pc = torch.empty(lib.fpq_packed_codes_bytes(rows, k), dtype=torch.uint8, device=dev)
        ps = torch.empty(lib.fpq_packed_scales_bytes(rows, k), dtype=torch.uint8, device=dev)
        _engine.check(lib.fpq_quantize_mx_packed(t.data_ptr(), rows, k, 0, 128, norm, pc.data_ptr(), ps.data_ptr(), 0, st),
                      "quantize")
        return pc, ps

    wp, ws = quantize(w, n)
    xp, xs = quantize(x, m)
    alpha = torch.tensor([0.111328125], device=dev)
    y = torch.empty(m, n, dtype=torch.bfloat16, device=dev)
    blocks = torch.cuda.get_device_properties(0).multi_processor_count
    words = wp.view(torch.int32)[:blocks * 256 * 32].contiguous()
    zeros = torch.zeros_like(words)
    sink = torch.empty(blocks * 256, dtype=torch.float32, device=dev)
    clocks = torch.empty(blocks * 2, dtype=torch.int64, device=dev)
    src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 256)
    dst = torch.empty_like(src)
    # the NVFP4 large-M GEMM (row-major operands, fp16 matrix path after in-register dequantization)
    nm, nn = 4096, 24576
    gen_d = torch.Generator(device=dev).manual_seed(3)
    nxq = torch.randint(0, 256, (nm, k // 2), dtype=torch.uint8, device=dev, generator=gen_d)
    nwq = torch.randint(0, 256, (nn, k // 2), dtype=torch.uint8, device=dev, generator=gen_d)
    nxs = torch.randint(40, 72, (nm, k // 16), dtype=torch.uint8, device=dev, generator=gen_d)
    nws = torch.randint(40, 72, (nn, k // 16), dtype=torch.uint8, device=dev, generator=gen_d)
    ny = torch.empty(nm, nn, dtype=torch.bfloat16, device=dev)
    legs = {
        "nvfp4_gemm_M4096_gate_up": lambda: lib.fpq_gemm_nvf4(nxq.data_ptr(), nxs.data_ptr(), k // 16, nwq.data_ptr(),
                                                              nws.data_ptr(), k // 16, alpha.data_ptr(), None,
                                                              ny.data_ptr(), nm, nn, k, st),
        "mxfp4_gemm_M2048": lambda: lib.fpq_gemm_mxf4_packed(xp.data_ptr(), xs.data_ptr(), wp.data_ptr(), ws.data_ptr(),
                                                             alpha.data_ptr(), None, y.data_ptr(), m, n, k, st),
        "mfma_only_quantized_bits": lambda: lib.fpq_test_mfma_rate(words.data_ptr(), blocks, 192, sink.data_ptr(),
                                                                   clocks.data_ptr(), st),
        "mfma_only_zeros": lambda: lib.fpq_test_mfma_rate(zeros.data_ptr(), blocks, 192, sink.data_ptr(),
                                                          clocks.data_ptr(), st),
        "copy_256MiB": lambda: dst.copy_(src),
    }

    def sample():
        try:
            out = subprocess.run(["amd-smi", "metric", "-p", "-c"], capture_output=True, text=True, timeout=20).stdout
        except Exception as e:  # noqa: BLE001
            return {"error": f"{type(e).__name__}: {e}"}
        watts = re.search(r"SOCKET_POWER:\s*(\d+)\s*W", out)
        clk = [int(v) for v in re.findall(r"GFX_\d+:\s*CLK:\s*(\d+)\s*MHz", out)]
        return {"socket_power_W": int(watts.group(1)) if watts else None,
                "xcd_clock_MHz_min_max": [min(clk), max(clk)] if clk else None}

    res = {}
    for name, fn in legs.items():
        got = []

        def sampler():
            time.sleep(seconds * 0.5)
            got.append(sample())

        th = threading.Thread(target=sampler)
        th.start()
        launches, t0 = 0, time.perf_counter()
        while th.is_alive() or time.perf_counter() - t0 < seconds:
            for _ in range(200):
                fn()
            torch.cuda.synchronize()
            launches += 200
        th.join()
        res[name] = dict(got[0], us_per_launch=round((time.perf_counter() - t0) / launches * 1e6, 2))
    return res


def bench_e2e_llama(torch, layers=32, prefill_batch=4, seq=2048, decode_batches=(1, 32, 64), decode_steps=8,
                    fmt="mxfp4", compiled_decode=False, compact=False):
    """Forward passes of a random-weight Llama-3.1-8B-architecture model (transformers' LlamaForCausalLM) whose
    linears (all but lm_head) were replaced by MXFP4 FPQuantLinear with Hadamard-128: prefill tokens/s, decode
    tokens/s against a `seq`-token bf16 KV cache, and the share of GPU time spent inside the quantized linears
    (HIP events around every FPQuantLinear.forward)."""
    import fp_quant
    from transformers import LlamaConfig, LlamaForCausalLM
    dev = torch.device("cuda:0")
    cfg = LlamaConfig(hidden_size=4096, intermediate_size=14336, num_hidden_layers=layers, num_attention_heads=32,
                      num_key_value_heads=8, vocab_size=128256, max_position_embeddings=8192, rms_norm_eps=1e-5,
                      rope_theta=500000.0, attn_implementation="sdpa")
    old_dtype = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        with dev:
            model = LlamaForCausalLM(cfg)
    finally:
        torch.set_default_dtype(old_dtype)
    model.eval()
    sweep = ((1, 32), (8, 128), (16, 128), (64, 128), (prefill_batch, seq))   # (batch, sequence) prefill points

    def prefill_sweep():
        """Best-of-3 prefill milliseconds per (batch, seq) point: the reference's end-to-end plot is the ratio
        of these between the bf16 and the MXFP4 model (assets/inference_speedup_*.png, batch x seq sweep)."""
        res = {}
        with torch.no_grad():
            for b, sl in sweep:
                ids = torch.randint(0, cfg.vocab_size, (b, sl), generator=torch.Generator().manual_seed(b * sl)).to(dev)
                best = None
                for rep in range(4):
                    e0 = torch.cuda.Event(enable_timing=True)
                    e1 = torch.cuda.Event(enable_timing=True)
                    e0.record()
                    model(input_ids=ids, use_cache=False, logits_to_keep=1)
                    e1.record()
                    torch.cuda.synchronize()
                    if rep:
                        best = e0.elapsed_time(e1) if best is None else min(best, e0.elapsed_time(e1))
                res[f"{b}x{sl}"] = round(best, 3)
        return res

    bf16_ms = None if compact else prefill_sweep()   # the unquantized model: nn.Linear in bf16 (hipBLASLt)
    qcfg = fp_quant.FPQuantConfig(forward_dtype=fp_quant.FPQuantDtype(fmt), forward_method="abs_max",
                                  backward_dtype=fp_quant.FPQuantDtype.BF16,
                                  hadamard_group_size=128 if fmt == "mxfp4" else 16)
    fp_quant.replace_quantize_with_fp_quant_linear(model, qcfg)
    qlinears = [m for m in model.modules() if isinstance(m, fp_quant.FPQuantLinear)]
    spans = []

    def pre(mod, args):
        e = torch.cuda.Event(enable_timing=True)
        e.record()
        mod._bench_e0 = e

    def post(mod, args, out):
        e = torch.cuda.Event(enable_timing=True)
        e.record()
        spans.append((mod._bench_e0, e))

    gen = torch.Generator().manual_seed(7)

    def timed(fn, reps, with_hooks):
        handles = []
        if with_hooks:
            for m in qlinears:
                handles += [m.register_forward_pre_hook(pre), m.register_forward_hook(post)]
        best, share = None, None
        for _ in range(reps):
            spans.clear()
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record()
            fn()
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1)
            if best is None or ms < best:
                best = ms
                share = sum(a.elapsed_time(b) for a, b in spans) / ms if with_hooks else None
        for h in handles:
            h.remove()
        return best, share

    out = {"model": f"Llama-3.1-8B architecture, {layers} layers, random weights, "
                    + ("MXFP4 W4A4 Hadamard-128" if fmt == "mxfp4" else "NVFP4 W4A4 Hadamard-16"),
           "quantized_linears": len(qlinears)}

    def measure(out, with_share):
        with torch.no_grad():
            ids = torch.randint(0, cfg.vocab_size, (prefill_batch, seq), generator=gen).to(dev)
            run = lambda: model(input_ids=ids, use_cache=False, logits_to_keep=1)
            run()
            ms, _ = timed(run, 3, False)
            _, share = timed(run, 2, True) if with_share else (None, None)
            out["prefill"] = {"batch": prefill_batch, "seq": seq, "ms": round(ms, 2),
                              "tokens_per_s": round(prefill_batch * seq / (ms * 1e-3), 1),
                              "linear_time_share": round(share, 3) if share is not None else None}
            out["decode"] = {}
            for b in decode_batches:
                ids = torch.randint(0, cfg.vocab_size, (b, seq), generator=gen).to(dev)
                cache = model(input_ids=ids, use_cache=True, logits_to_keep=1).past_key_values
                tok = torch.randint(0, cfg.vocab_size, (b, 1), generator=gen).to(dev)
                state = {"cache": cache}

                def step():
                    for _ in range(decode_steps):
                        r = model(input_ids=tok, past_key_values=state["cache"], use_cache=True)
                        state["cache"] = r.past_key_values

                step()
                ms, _ = timed(step, 2, False)
                _, share = timed(step, 1, True) if with_share else (None, None)
                out["decode"][f"batch{b}"] = {"kv_tokens": seq, "ms_per_step": round(ms / decode_steps, 3),
                                              "tokens_per_s": round(b * decode_steps / (ms * 1e-3), 1),
                                              "linear_time_share": round(share, 3) if share is not None else None}
                del cache, state
                torch.cuda.empty_cache()

    measure(out, True)
    mx_ms = None if compact else prefill_sweep()
    if compiled_decode:
        out["decode_compiled"] = compiled_decode_ms(torch, model, cfg, seq, decode_batches, decode_steps, gen)
    # the same model with the RMSNorms and the SiLU*up of every block fused into the quantizers that consume
    # them (one fused kernel instead of PyTorch's elementwise operators followed by a quantizer)
    from fp_quant.utils import fuse_producers
    fused = {"patched_modules": fuse_producers(model)}
    measure(fused, False)
    if compiled_decode:   # the traced attention and MLP modules now call the group operators
        fused["decode_compiled"] = compiled_decode_ms(torch, model, cfg, seq, decode_batches, decode_steps, gen)
    elif compact:
        # batch 1 is host-bound in eager mode: the step as the reference's README runs it for speed (README.md:39),
        # compiled and replayed as one HIP graph
        try:
            fused["decode_compiled"] = compiled_decode_ms(torch, model, cfg, seq, decode_batches[:1], decode_steps, gen)
        except Exception as e:  # noqa: BLE001  (a compiler problem must not take the eager figures with it)
            fused["decode_compiled"] = {"error": f"{type(e).__name__}: {str(e)[:200]}"}
    out["fused_producers"] = fused
    if fmt == "mxfp4":
        # what holding the 4-bit weights once (packed layout only) gives back; nothing is timed on it: the
        # kernels read the same buffers either way
        from fp_quant.utils import release_row_major_weights
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        layers = release_row_major_weights(model)
        torch.cuda.synchronize()
        out["weights_held_once"] = {"layers": layers, "freed_GB": round((before - torch.cuda.memory_allocated()) / 1e9, 3)}
    if compact:
        del model
        torch.cuda.empty_cache()
        return out
    fused_ms = prefill_sweep()
    out["prefill_sweep_ms"] = {"bf16": bf16_ms, fmt: mx_ms, fmt + "_fused_producers": fused_ms,
                               "speedup_vs_bf16": {k: round(bf16_ms[k] / mx_ms[k], 2) for k in bf16_ms},
                               "speedup_vs_bf16_fused": {k: round(bf16_ms[k] / fused_ms[k], 2) for k in bf16_ms}}
    return out


def compiled_decode_ms(torch, model, cfg, seq, batches, steps, gen):
    """Decode the way the reference's README recommends for speed (README.md:39): the model's forward under
    torch.compile(mode="reduce-overhead", fullgraph=True), i.e. replayed as one HIP graph per step, over
    transformers' StaticCache holding `seq` tokens.  The quantize / GEMM operators enter the graph as
    custom operators; the prefill stays eager."""
    from transformers import StaticCache
    dev = torch.device("cuda:0")
    res = {}
    with torch.no_grad():
        for b in batches:
            ids = torch.randint(0, cfg.vocab_size, (b, seq), generator=gen).to(dev)
            tok = torch.randint(0, cfg.vocab_size, (b, 1), generator=gen).to(dev)
            cache = StaticCache(config=cfg, max_cache_len=seq + 4 * steps + 16)
            model(input_ids=ids, past_key_values=cache, use_cache=True, logits_to_keep=1)
            torch._dynamo.reset()
            fwd = torch.compile(model.forward, mode="reduce-overhead", fullgraph=True)
            for _ in range(4):                       # compile, graph warm-up, capture, first replay
                fwd(input_ids=tok, past_key_values=cache, use_cache=True)
            best = None
            for _ in range(2):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(steps):
                    fwd(input_ids=tok, past_key_values=cache, use_cache=True)
                torch.cuda.synchronize()
                ms = (time.perf_counter() - t0) * 1e3 / steps
                best = ms if best is None else min(best, ms)
            res[f"batch{b}"] = {"kv_tokens": seq, "ms_per_step": round(best, 3),
                                "tokens_per_s": round(b / (best * 1e-3), 1)}
            del cache, fwd
            torch._dynamo.reset()
            torch.cuda.empty_cache()
    return res


def cpu_baseline_quantize(torch, fmt, rows, cols, g, seed, sample_rows):
    """The oracle (a torch-CPU restatement of the reference's PyTorch quantizer path) timed
    on a bounded row sample of the same workload."""
    from oracle import fpq_oracle as O
    cores = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    x = (outlier_normal(torch, sample_rows, cols, seed) if fmt == "mxfp4"
         else student_t(torch, sample_rows, cols, seed))
    group = 32 if fmt == "mxfp4" else 16
    best = None
    for _ in range(3):
        t0 = time.perf_counter()
        if fmt == "mxfp4":
            O.quantize_mx(x, O.ROT_HADAMARD, g)
        else:
            O.quantize_nv(x, 10.0, O.ROT_HADAMARD, g)
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    algo_bytes = sample_rows * cols * (2 + 0.5 + 1.0 / group)
    return {
        "value": algo_bytes / best / 1e9,
        "unit": "GB/s",
        "cores": cores,
        "kind": "port",
        "sample": f"{sample_rows}x{cols} rows of the same {fmt} quantize workload, best of 3, torch CPU oracle",
    }


def cpu_baseline_linear(torch, m_sample, n, k, g, seed):
    """The oracle's MXFP4 linear (quantize activations, dequantize both operands, fp32 matmul:
    the reference's CPU pseudo-quant path) on a bounded sample of activation rows; weights are
    quantized once outside the timed region, as on the GPU."""
    from oracle import fpq_oracle as O
    cores = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    gen = torch.Generator().manual_seed(seed)
    w = (torch.randn(n, k, generator=gen) * 0.02).to(torch.bfloat16)
    x = torch.randn(m_sample, k, generator=gen).to(torch.bfloat16)
    wq, ws, _ = O.quantize_mx(w, O.ROT_HADAMARD, g)
    dw = O.dequantize(wq, ws, "mxfp4").float()
    best = None
    for _ in range(3):
        t0 = time.perf_counter()
        xq, xs, _ = O.quantize_mx(x, O.ROT_HADAMARD, g)
        dx = O.dequantize(xq, xs, "mxfp4").float()
        y = (torch.nn.functional.linear(dx, dw) * 0.111328125).to(torch.bfloat16)
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    del y
    return {
        "value": 2.0 * m_sample * n * k / best / 1e12,
        "unit": "TFLOP/s",
        "cores": cores,
        "kind": "port",
        "sample": f"{m_sample} activation rows of the M=2048 N={n} K={k} MXFP4 linear (quantize + dequant + "
                  "fp32 matmul), best of 3, torch CPU oracle",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-e2e", action="store_true", help="skip the compact whole-model leg of the default run")
    ap.add_argument("--only", default="", help="comma list of workloads to run (for profiling one kernel): "
                    "nvfp4_quantize, mxfp4_quantize, mxfp4_linear_M2048, mxfp4_linear_M128, mxfp4_linear_M16, "
                    "mxfp4_linear_M1, nvfp4_linear, mfma_ceiling, hbm_probe, vendor_gemm, fused_producers, power (socket power and clocks by "
                    "kernel), e2e_llama (whole-model forward); from hbm_probe on they are not part of the default run")
    ap.add_argument("--e2e-layers", type=int, default=32, help="decoder layers of the --only e2e_llama model")
    ap.add_argument("--e2e-format", default="mxfp4", choices=("mxfp4", "nvfp4"), help="format of the --only e2e_llama model")
    ap.add_argument("--e2e-compiled-decode", action="store_true",
                    help="--only e2e_llama: also time decode under torch.compile(mode='reduce-overhead') with a static cache")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a plain 256 MiB device copy (known traffic) to scale rocprofv3 byte counters")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path uses no collectives; run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from fp_quant import _engine

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (the HIP engine has no CPU path)", file=sys.stderr)
        sys.exit(2)
    _engine.lib()

    only = [w for w in args.only.split(",") if w]
    if args.copy_probe:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda:0").random_(0, 256)
        dst = torch.empty_like(src)
        for _ in range(max(3, args.steps // 10)):
            dst.copy_(src)  # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
    if only:
        out = {}
        if "nvfp4_quantize" in only:
            out["nvfp4_quantize"] = bench_quantize(torch, "nvfp4", 8192, 4096, 16, args.steps, args.warmup, seed=1)
        if "mxfp4_quantize" in only:
            out["mxfp4_quantize"] = bench_quantize(torch, "mxfp4", 2048, 4096, 128, args.steps, args.warmup, seed=0)
            out["mxfp4_quantize_packed"] = bench_quantize(torch, "mxfp4", 2048, 4096, 128, args.steps, args.warmup,
                                                          seed=0, packed=True)
        for m in (2048, 128, 16, 1):
            if f"mxfp4_linear_M{m}" in only:
                out[f"mxfp4_linear_M{m}"] = bench_linear(torch, "mxfp4", m, 14336, 4096, 128, args.steps,
                                                          args.warmup, seed=2)
        if "nvfp4_linear" in only:
            out["nvfp4_linear"] = bench_linear(torch, "nvfp4", 4096, 24576, 4096, 16, max(10, args.steps // 10),
                                               max(2, args.warmup // 10), seed=3)
        if "e2e_llama" in only:
            out["e2e_llama"] = bench_e2e_llama(torch, layers=args.e2e_layers, fmt=args.e2e_format,
                                               compiled_decode=args.e2e_compiled_decode)
        if "mfma_ceiling" in only:
            out["mfma_ceiling"] = bench_mfma_ceiling(torch)
        if "power" in only:
            out["power"] = bench_power(torch)
        if "hbm_probe" in only:
            out["hbm_probe"] = bench_hbm_probe(torch, args.steps, args.warmup)
        if "vendor_gemm" in only:
            out["vendor_gemm"] = bench_vendor_gemm(torch, max(10, args.steps // 4), args.warmup)
        if "fused_producers" in only:
            out["fused_producers"] = bench_fused_producers(torch, args.steps, args.warmup)
        print(json.dumps({"only": only, "steps": args.steps, "results": out}))
        return

    results = {}
    results["nvfp4_quantize"] = bench_quantize(torch, "nvfp4", 8192, 4096, 16, args.steps, args.warmup, seed=1)
    results["mxfp4_quantize"] = bench_quantize(torch, "mxfp4", 2048, 4096, 128, args.steps, args.warmup, seed=0)
    results["mxfp4_quantize_packed"] = bench_quantize(torch, "mxfp4", 2048, 4096, 128, args.steps, args.warmup,
                                                      seed=0, packed=True)

    linears = {}
    for m in (2048, 128, 16, 1):
        linears[m] = bench_linear(torch, "mxfp4", m, 14336, 4096, 128, args.steps, args.warmup, seed=2, check=True)
    nv = bench_linear(torch, "nvfp4", 4096, 24576, 4096, 16, max(10, args.steps // 10), max(2, args.warmup // 10), seed=3)

    nv64 = bench_linear(torch, "nvfp4", 64, 24576, 4096, 16, args.steps, args.warmup, seed=3)

    ceiling = bench_mfma_ceiling(torch)
    quant = results["nvfp4_quantize"]
    head = linears[2048]
    kernels = {
        k: {"workload": v["workload"], "kernel_us": round(v["kernel_ms"] * 1e3, 3),
            "GB/s": round(v["gbps"], 2), "hbm_frac": round(v["gbps"] / HBM_PEAK_GBS, 4)}
        for k, v in results.items()
    }
    for m, v in linears.items():
        kernels[f"mxfp4_gemm_M{m}"] = {
            "workload": v["workload"], "gemm_us": round(v["gemm_ms"] * 1e3, 3),
            "linear_us": round(v["linear_ms"] * 1e3, 3), "gemm_TFLOP/s": round(v["gemm_tflops"], 2),
            "mfma_frac": round(v["gemm_tflops"] / FP4_PEAK_TFLOPS, 4),
            "gemm_GB/s": round(v["gemm_gbps"], 2), "hbm_frac": round(v["gemm_gbps"] / HBM_PEAK_GBS, 4),
            "operand_layout": v["operand_layout"], "output_check": v.get("output_check", {}).get("within_tolerance")}
        if v.get("gemm_ms_cache_resident") is not None:
            # gemm_us streams the weights from HBM (they rotate through `weight_copies` buffers, more than the
            # last-level cache holds); this is the same kernel with one copy that stays in the caches
            kernels[f"mxfp4_gemm_M{m}"]["gemm_us_cache_resident"] = round(v["gemm_ms_cache_resident"] * 1e3, 3)
            kernels[f"mxfp4_gemm_M{m}"]["weight_copies"] = v["weight_copies"]
    kernels["nvfp4_gemm_M4096_gate_up"] = {
        "workload": nv["workload"], "gemm_us": round(nv["gemm_ms"] * 1e3, 3),
        "gemm_TFLOP/s": round(nv["gemm_tflops"], 2),
        "mfma_frac_of_f16_peak": round(nv["gemm_tflops"] / BF16_PEAK_TFLOPS, 4)}
    kernels["nvfp4_gemm_M64_gate_up"] = {
        "workload": nv64["workload"], "gemm_us": round(nv64["gemm_ms"] * 1e3, 3),
        "linear_us": round(nv64["linear_ms"] * 1e3, 3), "gemm_GB/s": round(nv64["gemm_gbps"], 2),
        "hbm_frac": round(nv64["gemm_gbps"] / HBM_PEAK_GBS, 4), "operand_layout": nv64["operand_layout"],
        "gemm_us_cache_resident": round(nv64["gemm_ms_cache_resident"] * 1e3, 3)
        if nv64.get("gemm_ms_cache_resident") is not None else None,
        "weight_copies": nv64.get("weight_copies")}
    traffic = {}
    tpath = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(tpath):
        with open(tpath) as f:
            traffic = json.load(f)  # HBM bytes per launch from an earlier rocprofv3 --pmc run (see profiles/)
    traffic_source = ("profiles/traffic.json: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this command, run by the "
                      "builder on the library built from commit " + str(traffic.get("source_commit", "?")) +
                      " and scaled by a 256 MiB copy; a constant, not measured in this run")
    line = {
        "metric": METRIC,
        "value": round(head["linear_tflops_over_steps"], 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(head["ms_per_step"], 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp4",
        "data": "synthetic",
        "config": {"workload": head["workload"] + " (activation rotate+quantize then W4A4 GEMM)",
                   "rotating_buffers": head["buffers"],
                   "timing": f"value and ms_per_step: exactly --steps timed steps after --warmup steps and {SETTLE_MS:.0f} ms "
                             f"of untimed settling launches; kernel figures: median of interleaved blocks of "
                             f"{head['block_launches']} launches covering at least {BLOCK_MIN_MS:.0f} ms per leg",
                   "value_median_blocks": round(head["linear_tflops"], 2),
                   "output_check": head.get("output_check")},
        "roofline": {
            "kernel": "MXFP4 W4A4 GEMM, M=2048 N=14336 K=4096",
            "bound": "mfma",
            "achieved": round(head["gemm_tflops"], 2),
            "peak": FP4_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(head["gemm_tflops"] / FP4_PEAK_TFLOPS, 4),
            "traffic": traffic.get("mxfp4_gemm_M2048"),
            "traffic_source": traffic_source,
            "kernel_us": round(head["gemm_ms"] * 1e3, 3),
            "kernel_us_min_max": [round(head["gemm_ms_min"] * 1e3, 3), round(head["gemm_ms_max"] * 1e3, 3)],
            "linear_us": round(head["linear_ms"] * 1e3, 3),
            "timing_consistent": head["timing_consistent"],
            "algorithmic_flops_per_launch": int(head["flops"]),
            "operand_layout": head["operand_layout"],
            # what the matrix pipes alone sustain (register-resident operands): the clock drops with
            # non-zero operand bits, so this, not `peak`, is what the kernel can approach
            "sustained_mfma_only": ceiling,
            "frac_of_sustained": round(head["gemm_tflops"] / ceiling["quantized"]["TFLOP/s"], 4),
        },
        "roofline_quantize": {
            "kernel": "NVFP4 fused rotate+quantize, bf16 [8192, 4096], Hadamard 16",
            "bound": "hbm",
            "achieved": round(quant["gbps"], 2),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(quant["gbps"] / HBM_PEAK_GBS, 4),
            "traffic": traffic.get("nvfp4_quantize"),
            "traffic_source": traffic_source,
            "kernel_us": round(quant["kernel_ms"] * 1e3, 3),
            "algorithmic_bytes_per_launch": int(quant["algo_bytes"]),
        },
        "kernels": kernels,
    }
    if not args.no_e2e:
        # the end-to-end configuration in compact form: the whole-model forward (see bench_e2e_llama); an error here
        # (e.g. a transformers version without the model class) is recorded, the kernel figures stand
        try:
            e2e = bench_e2e_llama(torch, compact=True)
            line["e2e"] = {
                "model": e2e["model"],
                "prefill_4x2048_tokens_per_s": e2e["prefill"]["tokens_per_s"],
                "prefill_linear_time_share": e2e["prefill"]["linear_time_share"],
                "decode_tokens_per_s": {k: v["tokens_per_s"] for k, v in e2e["decode"].items()},
                "decode_linear_time_share": {k: v["linear_time_share"] for k, v in e2e["decode"].items()},
                "fused_producers": {"prefill_4x2048_tokens_per_s": e2e["fused_producers"]["prefill"]["tokens_per_s"],
                                    "decode_tokens_per_s": {k: v["tokens_per_s"] for k, v in
                                                            e2e["fused_producers"]["decode"].items()},
                                    "decode_compiled_tokens_per_s": {
                                        k: (v.get("tokens_per_s") if isinstance(v, dict) else v)
                                        for k, v in e2e["fused_producers"].get("decode_compiled", {}).items()}},
                "weights_held_once": e2e.get("weights_held_once"),
                "note": "eager PyTorch model, bf16 KV cache of 2048 tokens, everything outside the linears is stock "
                        "PyTorch-ROCm; decode_compiled: torch.compile(mode='reduce-overhead', fullgraph=True) over a static "
                        "cache; python bench.py --only e2e_llama adds the bf16 comparison and the batch sweep",
            }
        except Exception as e:  # noqa: BLE001
            line["e2e"] = {"error": f"{type(e).__name__}: {str(e)[:300]}"}
        torch.cuda.empty_cache()
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline_linear(torch, 2048, 14336, 4096, 128, seed=2)
        line["cpu_baseline_quantize"] = cpu_baseline_quantize(torch, "nvfp4", 8192, 4096, 16, 1, 8192)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
