"""Thin test helper: call the C ABI of libfpq_hip.so on torch CUDA tensors."""
import ctypes

import torch

from fp_quant import _engine

ROT = {"hadamard": _engine.ROT_HADAMARD, "identity": _engine.ROT_IDENTITY, "gsr": _engine.ROT_GSR,
       "general": _engine.ROT_GENERAL}


def _padded(rows, groups, pad):
    if not pad:
        return rows, groups
    return (rows + 127) // 128 * 128, (groups + 3) // 4 * 4


def quantize(x_bf16, fmt, rot="hadamard", g=128, norm=None, h=None, global_scale=None,
             zero_policy=_engine.ZERO_REFERENCE, pad=False, fill=0xCD):
    """Run fpq_quantize_mx / fpq_quantize_nv on `x_bf16` (CPU or CUDA); returns CPU uint8
    (codes [R, C/2], scales [scale_rows, scale_stride]) and raises on a non-zero status."""
    lib = _engine.lib()
    x = x_bf16.to("cuda").contiguous()
    rows, cols = x.shape
    group = 32 if fmt == "mxfp4" else 16
    srow, scol = _padded(rows, cols // group, pad)
    codes = torch.full((rows, cols // 2), fill, dtype=torch.uint8, device="cuda")
    scales = torch.full((srow, scol), fill, dtype=torch.uint8, device="cuda")
    if norm is None:
        norm = float(torch.tensor(g ** -0.5, dtype=torch.bfloat16))
    h_dev = h.to(device="cuda", dtype=torch.bfloat16).contiguous() if h is not None else None  # keep alive
    hp = h_dev.data_ptr() if h_dev is not None else None
    stream = torch.cuda.current_stream().cuda_stream
    if fmt == "mxfp4":
        st = lib.fpq_quantize_mx(x.data_ptr(), rows, cols, ROT[rot], g, norm, hp, codes.data_ptr(),
                                 scales.data_ptr(), srow, scol, zero_policy, stream)
    else:
        gs = torch.tensor([global_scale], dtype=torch.float32, device="cuda")
        st = lib.fpq_quantize_nv(x.data_ptr(), rows, cols, ROT[rot], g, norm, hp, gs.data_ptr(),
                                 codes.data_ptr(), scales.data_ptr(), srow, scol, zero_policy, stream)
    _engine.check(st, "fpq_quantize")
    torch.cuda.synchronize()
    return codes.cpu(), scales.cpu()


def gemm(xq, xs, wq, ws, alpha, fmt, bias=None):
    """Run fpq_gemm_mxf4 / fpq_gemm_nvf4 on packed operands (CPU or CUDA uint8 tensors);
    returns the bf16 [M, N] result on the CPU."""
    lib = _engine.lib()
    xq, xs, wq, ws = (t.to("cuda").contiguous() for t in (xq, xs, wq, ws))
    m, n, k = xq.shape[0], wq.shape[0], xq.shape[1] * 2
    y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    a = torch.tensor([alpha], dtype=torch.float32, device="cuda")
    b = bias.to("cuda").contiguous() if bias is not None else None
    fn = lib.fpq_gemm_mxf4 if fmt == "mxfp4" else lib.fpq_gemm_nvf4
    st = fn(xq.data_ptr(), xs.data_ptr(), xs.shape[1], wq.data_ptr(), ws.data_ptr(), ws.shape[1],
            a.data_ptr(), b.data_ptr() if b is not None else None, y.data_ptr(), m, n, k,
            torch.cuda.current_stream().cuda_stream)
    _engine.check(st, "fpq_gemm")
    torch.cuda.synchronize()
    return y.cpu()


def packed_sizes(rows, k):
    lib = _engine.lib()
    return lib.fpq_packed_codes_bytes(rows, k), lib.fpq_packed_scales_bytes(rows, k)


def pack(codes, scales, fill=0xCD):
    """fpq_pack_mxf4 on row-major codes [R, K/2] and E8M0 scales [>=R, >=K/32]; CPU uint8 results."""
    lib = _engine.lib()
    codes, scales = codes.to("cuda").contiguous(), scales.to("cuda").contiguous()
    rows, k = codes.shape[0], codes.shape[1] * 2
    nc, ns = packed_sizes(rows, k)
    pc = torch.full((nc,), fill, dtype=torch.uint8, device="cuda")
    ps = torch.full((ns,), fill, dtype=torch.uint8, device="cuda")
    st = lib.fpq_pack_mxf4(codes.data_ptr(), scales.data_ptr(), scales.shape[1], rows, k, pc.data_ptr(),
                           ps.data_ptr(), torch.cuda.current_stream().cuda_stream)
    _engine.check(st, "fpq_pack_mxf4")
    torch.cuda.synchronize()
    return pc.cpu(), ps.cpu()


def unpack(pc, ps, rows, k, scale_pad=0, fill=0xCD, nv=False):
    """fpq_unpack_mxf4 (nv: fpq_unpack_nvf4): CPU uint8 row-major codes [rows, k/2] and scales
    [rows, k/group + scale_pad] (entries past k/group keep `fill`)."""
    lib = _engine.lib()
    pc, ps = pc.to("cuda").contiguous(), ps.to("cuda").contiguous()
    group = 16 if nv else 32
    codes = torch.full((rows, k // 2), fill, dtype=torch.uint8, device="cuda")
    scales = torch.full((rows, k // group + scale_pad), fill, dtype=torch.uint8, device="cuda")
    entry = lib.fpq_unpack_nvf4 if nv else lib.fpq_unpack_mxf4
    st = entry(pc.data_ptr(), ps.data_ptr(), rows, k, codes.data_ptr(), scales.data_ptr(),
               scales.shape[1], torch.cuda.current_stream().cuda_stream)
    _engine.check(st, "fpq_unpack")
    torch.cuda.synchronize()
    return codes.cpu(), scales.cpu()


def quantize_packed(x_bf16, rot="hadamard", g=128, norm=None, zero_policy=_engine.ZERO_REFERENCE, fill=0xCD):
    """fpq_quantize_mx_packed; CPU uint8 (packed codes, packed scales)."""
    lib = _engine.lib()
    x = x_bf16.to("cuda").contiguous()
    rows, cols = x.shape
    nc, ns = packed_sizes(rows, cols)
    pc = torch.full((nc,), fill, dtype=torch.uint8, device="cuda")
    ps = torch.full((ns,), fill, dtype=torch.uint8, device="cuda")
    if norm is None:
        norm = float(torch.tensor(g ** -0.5, dtype=torch.bfloat16))
    st = lib.fpq_quantize_mx_packed(x.data_ptr(), rows, cols, ROT[rot], g, norm, pc.data_ptr(), ps.data_ptr(),
                                    zero_policy, torch.cuda.current_stream().cuda_stream)
    _engine.check(st, "fpq_quantize_mx_packed")
    torch.cuda.synchronize()
    return pc.cpu(), ps.cpu()


def gemm_packed_splitk(xp, xsp, wp, wsp, m, n, k, alpha, bias=None, residual=None, workspace=None, calls=1, nv=False):
    """fpq_gemm_mxf4_packed_splitk (nv: fpq_gemm_nvf4_packed_splitk) on packed operands with `workspace` (a CUDA
    uint8 tensor whose first 16 KB are zero, or None), `calls` times in a row on the same buffers; bf16 [M, N]
    on the CPU."""
    lib = _engine.lib()
    entry = lib.fpq_gemm_nvf4_packed_splitk if nv else lib.fpq_gemm_mxf4_packed_splitk
    xp, xsp, wp, wsp = (t.to("cuda").contiguous() for t in (xp, xsp, wp, wsp))
    a = torch.tensor([alpha], dtype=torch.float32, device="cuda")
    b = bias.to("cuda").contiguous() if bias is not None else None
    r = residual.to("cuda").contiguous() if residual is not None else None
    stream = torch.cuda.current_stream().cuda_stream
    for _ in range(calls):
        y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        st = entry(xp.data_ptr(), xsp.data_ptr(), wp.data_ptr(), wsp.data_ptr(),
                   a.data_ptr(), b.data_ptr() if b is not None else None,
                   r.data_ptr() if r is not None else None, y.data_ptr(), m, n, k,
                   workspace.data_ptr() if workspace is not None else None,
                   workspace.numel() if workspace is not None else 0, stream)
        _engine.check(st, "fpq_gemm_packed_splitk")
    torch.cuda.synchronize()
    return y.cpu()


def gemm_packed_multi(xp, xsp, wp, wsp, m, splits, k, alpha, bias=None, nv=False):
    """fpq_gemm_mxf4_packed_multi (nv: fpq_gemm_nvf4_packed_multi) on packed operands (the weights of
    len(splits) layers end to end); a list of bf16 [M, splits[i]] on the CPU."""
    lib = _engine.lib()
    xp, xsp, wp, wsp = (t.to("cuda").contiguous() for t in (xp, xsp, wp, wsp))
    outs = [torch.full((m, s), float("nan"), dtype=torch.bfloat16, device="cuda") for s in splits]
    a = torch.tensor([alpha], dtype=torch.float32, device="cuda")
    b = bias.to("cuda").contiguous() if bias is not None else None
    ys = (ctypes.c_void_p * len(splits))(*[o.data_ptr() for o in outs])
    ns = (ctypes.c_int64 * len(splits))(*splits)
    entry = lib.fpq_gemm_nvf4_packed_multi if nv else lib.fpq_gemm_mxf4_packed_multi
    st = entry(xp.data_ptr(), xsp.data_ptr(), wp.data_ptr(), wsp.data_ptr(), a.data_ptr(),
               b.data_ptr() if b is not None else None, ys, ns, len(splits), m, k,
               torch.cuda.current_stream().cuda_stream)
    _engine.check(st, "fpq_gemm_packed_multi")
    torch.cuda.synchronize()
    return [o.cpu() for o in outs]


def gemm_packed(xp, xsp, wp, wsp, m, n, k, alpha, bias=None, residual=None, in_place=False):
    """fpq_gemm_mxf4_packed (with `residual`: fpq_gemm_mxf4_packed_residual, `in_place`: writing over
    the residual tensor) on packed operands; bf16 [M, N] on the CPU."""
    lib = _engine.lib()
    xp, xsp, wp, wsp = (t.to("cuda").contiguous() for t in (xp, xsp, wp, wsp))
    y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    a = torch.tensor([alpha], dtype=torch.float32, device="cuda")
    b = bias.to("cuda").contiguous() if bias is not None else None
    bp = b.data_ptr() if b is not None else None
    stream = torch.cuda.current_stream().cuda_stream
    if residual is None:
        st = lib.fpq_gemm_mxf4_packed(xp.data_ptr(), xsp.data_ptr(), wp.data_ptr(), wsp.data_ptr(), a.data_ptr(),
                                      bp, y.data_ptr(), m, n, k, stream)
    else:
        r = residual.to("cuda").contiguous().clone()
        if in_place:
            y = r
        st = lib.fpq_gemm_mxf4_packed_residual(xp.data_ptr(), xsp.data_ptr(), wp.data_ptr(), wsp.data_ptr(),
                                               a.data_ptr(), bp, r.data_ptr(), y.data_ptr(), m, n, k, stream)
    _engine.check(st, "fpq_gemm_mxf4_packed")
    torch.cuda.synchronize()
    return y.cpu()


def quantize_quest(x_bf16, rot="hadamard", g=128, norm=None, h=None, zero_policy=_engine.ZERO_REFERENCE,
                   want_mask=True, pad=False, fill=0xCD):
    """fpq_quantize_mx_quest; CPU uint8 (codes [R, C/2], scales, mask [R, C/8] or None)."""
    lib = _engine.lib()
    x = x_bf16.to("cuda").contiguous()
    rows, cols = x.shape
    srow, scol = _padded(rows, cols // 32, pad)
    codes = torch.full((rows, cols // 2), fill, dtype=torch.uint8, device="cuda")
    scales = torch.full((srow, scol), fill, dtype=torch.uint8, device="cuda")
    mask = torch.full((rows, cols // 8), fill, dtype=torch.uint8, device="cuda") if want_mask else None
    if norm is None:
        norm = float(torch.tensor(g ** -0.5, dtype=torch.bfloat16))
    h_dev = h.to(device="cuda", dtype=torch.bfloat16).contiguous() if h is not None else None
    st = lib.fpq_quantize_mx_quest(x.data_ptr(), rows, cols, ROT[rot], g, norm,
                                   h_dev.data_ptr() if h_dev is not None else None, codes.data_ptr(),
                                   scales.data_ptr(), srow, scol, mask.data_ptr() if want_mask else None,
                                   zero_policy, torch.cuda.current_stream().cuda_stream)
    _engine.check(st, "fpq_quantize_mx_quest")
    torch.cuda.synchronize()
    return codes.cpu(), scales.cpu(), (mask.cpu() if want_mask else None)


def quantize_quest_packed(x_bf16, rot="hadamard", g=128, norm=None, zero_policy=_engine.ZERO_REFERENCE, fill=0xCD):
    """fpq_quantize_mx_quest_packed; CPU uint8 (packed codes, packed scales)."""
    lib = _engine.lib()
    x = x_bf16.to("cuda").contiguous()
    rows, cols = x.shape
    nc, ns = packed_sizes(rows, cols)
    pc = torch.full((nc,), fill, dtype=torch.uint8, device="cuda")
    ps = torch.full((ns,), fill, dtype=torch.uint8, device="cuda")
    if norm is None:
        norm = float(torch.tensor(g ** -0.5, dtype=torch.bfloat16))
    st = lib.fpq_quantize_mx_quest_packed(x.data_ptr(), rows, cols, ROT[rot], g, norm, pc.data_ptr(), ps.data_ptr(),
                                          zero_policy, torch.cuda.current_stream().cuda_stream)
    _engine.check(st, "fpq_quantize_mx_quest_packed")
    torch.cuda.synchronize()
    return pc.cpu(), ps.cpu()


def pack_nv(codes, scales, fill=0xCD):
    """fpq_pack_nvf4 on row-major codes [R, K/2] and E4M3 scales [>=R, >=K/16]; CPU uint8 results."""
    lib = _engine.lib()
    codes, scales = codes.to("cuda").contiguous(), scales.to("cuda").contiguous()
    rows, k = codes.shape[0], codes.shape[1] * 2
    pc = torch.full((lib.fpq_packed_codes_bytes(rows, k),), fill, dtype=torch.uint8, device="cuda")
    ps = torch.full((lib.fpq_packed_scales_bytes_nv(rows, k),), fill, dtype=torch.uint8, device="cuda")
    st = lib.fpq_pack_nvf4(codes.data_ptr(), scales.data_ptr(), scales.shape[1], rows, k, pc.data_ptr(),
                           ps.data_ptr(), torch.cuda.current_stream().cuda_stream)
    _engine.check(st, "fpq_pack_nvf4")
    torch.cuda.synchronize()
    return pc.cpu(), ps.cpu()


def gemm_nv_packed(xp, xsp, wp, wsp, m, n, k, alpha, bias=None, residual=None, in_place=False):
    """fpq_gemm_nvf4_packed (with `residual`: fpq_gemm_nvf4_packed_residual, `in_place`: writing over the
    residual tensor) on packed operands; bf16 [M, N] on the CPU."""
    lib = _engine.lib()
    xp, xsp, wp, wsp = (t.to("cuda").contiguous() for t in (xp, xsp, wp, wsp))
    y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    a = torch.tensor([alpha], dtype=torch.float32, device="cuda")
    b = bias.to("cuda").contiguous() if bias is not None else None
    bp = b.data_ptr() if b is not None else None
    stream = torch.cuda.current_stream().cuda_stream
    if residual is not None:
        r = residual.to("cuda").contiguous().clone()
        if in_place:
            y = r
        st = lib.fpq_gemm_nvf4_packed_residual(xp.data_ptr(), xsp.data_ptr(), wp.data_ptr(), wsp.data_ptr(),
                                               a.data_ptr(), bp, r.data_ptr(), y.data_ptr(), m, n, k, stream)
    else:
        st = lib.fpq_gemm_nvf4_packed(xp.data_ptr(), xsp.data_ptr(), wp.data_ptr(), wsp.data_ptr(), a.data_ptr(),
                                      bp, y.data_ptr(), m, n, k, stream)
    _engine.check(st, "fpq_gemm_nvf4_packed")
    torch.cuda.synchronize()
    return y.cpu()


def rotated_absmax(x_bf16, rot="hadamard", g=128, norm=None, h=None, start=0.0):
    """Run fpq_rotated_absmax on `x_bf16` with *amax preset to `start`; returns the fp32 value."""
    lib = _engine.lib()
    x = x_bf16.to("cuda").contiguous()
    rows, cols = x.shape
    if norm is None:
        norm = float(torch.tensor(g ** -0.5, dtype=torch.bfloat16))
    h_dev = h.to(device="cuda", dtype=torch.bfloat16).contiguous() if h is not None else None  # keep alive
    amax = torch.tensor([start], dtype=torch.float32, device="cuda")
    st = lib.fpq_rotated_absmax(x.data_ptr(), rows, cols, ROT[rot], g, norm,
                                h_dev.data_ptr() if h_dev is not None else None, amax.data_ptr(),
                                torch.cuda.current_stream().cuda_stream)
    _engine.check(st, "fpq_rotated_absmax")
    torch.cuda.synchronize()
    return float(amax.cpu())


def row_inv_rms(x_bf16, eps, ld=None):
    """Run fpq_row_inv_rms; `ld` > cols places the rows in a wider buffer.  Returns CPU fp32 [rows]."""
    lib = _engine.lib()
    rows, cols = x_bf16.shape
    ld = cols if ld is None else ld
    buf = torch.full((rows, ld), 7.0, dtype=torch.bfloat16, device="cuda")
    buf[:, :cols] = x_bf16.to("cuda")
    out = torch.full((rows,), float("nan"), dtype=torch.float32, device="cuda")
    st = lib.fpq_row_inv_rms(buf.data_ptr(), ld, rows, cols, eps, out.data_ptr(), torch.cuda.current_stream().cuda_stream)
    _engine.check(st, "fpq_row_inv_rms")
    torch.cuda.synchronize()
    return out.cpu()


def _strided(t_bf16, ld):
    rows, cols = t_bf16.shape
    buf = torch.full((rows, ld), -3.0, dtype=torch.bfloat16, device="cuda")
    buf[:, :cols] = t_bf16.to("cuda")
    return buf


def fused_quantize(kind, fmt, a, b, g=128, rot="hadamard", norm=None, global_scale=None, eps=1e-5,
                   want_out=True, ld_a=None, ld_b=None, zero_policy=_engine.ZERO_REFERENCE, fill=0xCD):
    """Run fpq_rmsnorm_quantize_* (kind "rmsnorm": a = x [R, C], b = weight [C]) or
    fpq_silu_mul_quantize_* (kind "silu_mul": a = gate, b = up).  Returns CPU (codes, scales, out or None)."""
    lib = _engine.lib()
    rows, cols = a.shape
    ld_a = cols if ld_a is None else ld_a
    ld_b = cols if ld_b is None else ld_b
    group = 32 if fmt == "mxfp4" else 16
    a_dev = _strided(a, ld_a)
    codes = torch.full((rows, cols // 2), fill, dtype=torch.uint8, device="cuda")
    scales = torch.full((rows, cols // group), fill, dtype=torch.uint8, device="cuda")
    out = torch.full((rows, cols), float("nan"), dtype=torch.bfloat16, device="cuda") if want_out else None
    optr = out.data_ptr() if out is not None else None
    if norm is None:
        norm = float(torch.tensor(g ** -0.5, dtype=torch.bfloat16))
    stream = torch.cuda.current_stream().cuda_stream
    gs = torch.tensor([global_scale if global_scale is not None else 1.0], dtype=torch.float32, device="cuda")
    tail = (codes.data_ptr(), scales.data_ptr(), rows, cols // group, zero_policy, stream)
    if kind == "rmsnorm":
        w = b.to("cuda").contiguous()
        inv = torch.empty(rows, dtype=torch.float32, device="cuda")
        _engine.check(lib.fpq_row_inv_rms(a_dev.data_ptr(), ld_a, rows, cols, eps, inv.data_ptr(), stream), "fpq_row_inv_rms")
        head = (a_dev.data_ptr(), ld_a, inv.data_ptr(), w.data_ptr(), rows, cols, ROT[rot], g, norm)
        if fmt == "mxfp4":
            st = lib.fpq_rmsnorm_quantize_mx(*head, optr, *tail)
        else:
            st = lib.fpq_rmsnorm_quantize_nv(*head, gs.data_ptr(), optr, *tail)
    else:
        b_dev = _strided(b, ld_b)
        head = (a_dev.data_ptr(), ld_a, b_dev.data_ptr(), ld_b, rows, cols, ROT[rot], g, norm)
        if fmt == "mxfp4":
            st = lib.fpq_silu_mul_quantize_mx(*head, optr, *tail)
        else:
            st = lib.fpq_silu_mul_quantize_nv(*head, gs.data_ptr(), optr, *tail)
    _engine.check(st, f"fpq_{kind}_quantize")
    torch.cuda.synchronize()
    return codes.cpu(), scales.cpu(), (out.cpu() if out is not None else None)


def fused_quantize_packed(kind, a, b, g=128, rot="hadamard", norm=None, eps=1e-5, want_out=True, ld_a=None,
                          ld_b=None, zero_policy=_engine.ZERO_REFERENCE, fill=0xCD, global_scale=None):
    """fused_quantize with the packed operand layout as output (NVFP4 when `global_scale` is given: a few
    rows only).  Returns CPU (packed codes, packed scales, out or None)."""
    lib = _engine.lib()
    rows, cols = a.shape
    ld_a = cols if ld_a is None else ld_a
    ld_b = cols if ld_b is None else ld_b
    a_dev = _strided(a, ld_a)
    cb, sb = packed_sizes(rows, cols)
    if global_scale is not None:
        sb = lib.fpq_packed_scales_bytes_nv(rows, cols)
        gs = torch.tensor([global_scale], dtype=torch.float32, device="cuda")
    pc = torch.full((cb,), fill, dtype=torch.uint8, device="cuda")
    ps = torch.full((sb,), fill, dtype=torch.uint8, device="cuda")
    out = torch.full((rows, cols), float("nan"), dtype=torch.bfloat16, device="cuda") if want_out else None
    optr = out.data_ptr() if out is not None else None
    if norm is None:
        norm = float(torch.tensor(g ** -0.5, dtype=torch.bfloat16))
    stream = torch.cuda.current_stream().cuda_stream
    if kind == "rmsnorm":
        w = b.to("cuda").contiguous()
        inv = torch.empty(rows, dtype=torch.float32, device="cuda")
        _engine.check(lib.fpq_row_inv_rms(a_dev.data_ptr(), ld_a, rows, cols, eps, inv.data_ptr(), stream), "fpq_row_inv_rms")
        head = (a_dev.data_ptr(), ld_a, inv.data_ptr(), w.data_ptr(), rows, cols, ROT[rot], g, norm)
    else:
        b_dev = _strided(b, ld_b)
        head = (a_dev.data_ptr(), ld_a, b_dev.data_ptr(), ld_b, rows, cols, ROT[rot], g, norm)
    tail = (optr, pc.data_ptr(), ps.data_ptr(), zero_policy, stream)
    if global_scale is not None:
        st = getattr(lib, f"fpq_{kind}_quantize_nv_packed")(*head, gs.data_ptr(), *tail)
    else:
        st = getattr(lib, f"fpq_{kind}_quantize_mx_packed")(*head, *tail)
    _engine.check(st, f"fpq_{kind}_quantize_packed")
    torch.cuda.synchronize()
    return pc.cpu(), ps.cpu(), (out.cpu() if out is not None else None)


def rmsnorm_rows_quantize_packed(x, w, g=128, rot="hadamard", norm=None, eps=1e-5, want_out=True, want_inv=True,
                                 ld=None, zero_policy=_engine.ZERO_REFERENCE, fill=0xCD, global_scale=None):
    """fpq_rmsnorm_rows_quantize_{mx,nv}_packed (row statistic + RMSNorm + rotate + quantize of a few rows in
    one launch; NVFP4 when `global_scale` is given).  Returns CPU (packed codes, packed scales, normed or None,
    inv_rms or None)."""
    lib = _engine.lib()
    rows, cols = x.shape
    ld = cols if ld is None else ld
    x_dev = _strided(x, ld)
    cb, sb = packed_sizes(rows, cols)
    if global_scale is not None:
        sb = lib.fpq_packed_scales_bytes_nv(rows, cols)
        gs = torch.tensor([global_scale], dtype=torch.float32, device="cuda")
    pc = torch.full((cb,), fill, dtype=torch.uint8, device="cuda")
    ps = torch.full((sb,), fill, dtype=torch.uint8, device="cuda")
    out = torch.full((rows, cols), float("nan"), dtype=torch.bfloat16, device="cuda") if want_out else None
    inv = torch.full((rows,), float("nan"), dtype=torch.float32, device="cuda") if want_inv else None
    if norm is None:
        norm = float(torch.tensor(g ** -0.5, dtype=torch.bfloat16))
    wd = w.to("cuda").contiguous()
    head = (x_dev.data_ptr(), ld, wd.data_ptr(), rows, cols, eps, ROT[rot], g, norm)
    tail = (inv.data_ptr() if inv is not None else None, out.data_ptr() if out is not None else None, pc.data_ptr(),
            ps.data_ptr(), zero_policy, torch.cuda.current_stream().cuda_stream)
    if global_scale is not None:
        st = lib.fpq_rmsnorm_rows_quantize_nv_packed(*head, gs.data_ptr(), *tail)
    else:
        st = lib.fpq_rmsnorm_rows_quantize_mx_packed(*head, *tail)
    _engine.check(st, "fpq_rmsnorm_rows_quantize_packed")
    torch.cuda.synchronize()
    return pc.cpu(), ps.cpu(), (out.cpu() if out is not None else None), (inv.cpu() if inv is not None else None)


def quantize_nv_packed(x_bf16, global_scale, rot="hadamard", g=16, norm=None, zero_policy=_engine.ZERO_REFERENCE,
                       fill=0xCD):
    """Run fpq_quantize_nv_packed; returns CPU uint8 (packed codes, packed scales)."""
    lib = _engine.lib()
    x = x_bf16.to("cuda").contiguous()
    rows, cols = x.shape
    pc = torch.full((lib.fpq_packed_codes_bytes(rows, cols),), fill, dtype=torch.uint8, device="cuda")
    ps = torch.full((lib.fpq_packed_scales_bytes_nv(rows, cols),), fill, dtype=torch.uint8, device="cuda")
    if norm is None:
        norm = float(torch.tensor(g ** -0.5, dtype=torch.bfloat16))
    gs = torch.tensor([global_scale], dtype=torch.float32, device="cuda")
    st = lib.fpq_quantize_nv_packed(x.data_ptr(), rows, cols, ROT[rot], g, norm, gs.data_ptr(), pc.data_ptr(),
                                    ps.data_ptr(), zero_policy, torch.cuda.current_stream().cuda_stream)
    _engine.check(st, "fpq_quantize_nv_packed")
    torch.cuda.synchronize()
    return pc.cpu(), ps.cpu()
