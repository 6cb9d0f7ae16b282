"""CPU-side checks of the C ABI: the library loads, exports every symbol include/fpq.h
declares, and rejects bad arguments before touching a device."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "fpq.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fpq_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported():
    from fp_quant import _engine
    lib = ctypes.CDLL(_engine.library_path())
    names = _declared()
    assert "fpq_quantize_mx" in names and "fpq_gemm_mxf4" in names
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/fpq.h but not exported"
    assert sorted(_engine._SIGNATURES) == names


def test_version_and_status_strings():
    from fp_quant import _engine
    lib = _engine.lib()
    assert lib.fpq_version() == 1
    assert lib.fpq_status_string(0) == b"ok"
    for code in range(-6, 0):
        assert len(lib.fpq_status_string(code)) > 3


def test_argument_validation_needs_no_device():
    from fp_quant import _engine
    lib = _engine.lib()
    # null pointers and bad shapes are rejected before any HIP call
    assert lib.fpq_quantize_mx(None, 4, 128, 0, 128, 0.088, None, None, None, 4, 4, 0, None) == -1
    assert lib.fpq_quantize_mx(16, 4, 100, 0, 128, 0.088, None, 16, 16, 4, 4, 0, None) == -2
    assert lib.fpq_quantize_mx(16, 4, 128, 0, 48, 0.088, None, 16, 16, 4, 4, 0, None) == -3
    assert lib.fpq_quantize_mx(8, 4, 128, 0, 128, 0.088, None, 16, 16, 4, 4, 0, None) == -4
    assert lib.fpq_quantize_mx(16, 4, 128, 0, 128, 0.088, None, 16, 16, 4, 4, 9, None) == -5
    assert lib.fpq_quantize_nv(16, 4, 128, 0, 16, 0.25, None, None, 16, 16, 4, 8, 0, None) == -1
    # the multi-output GEMM: 1..4 layers, output features in multiples of 256, aligned outputs
    ys, ns = (ctypes.c_void_p * 2)(256, 512), (ctypes.c_int64 * 2)(256, 512)
    args = (16, 16, 16, 16, 16, None)
    assert lib.fpq_gemm_mxf4_packed_multi(*args, ys, ns, 0, 4, 256, None) == -2
    assert lib.fpq_gemm_mxf4_packed_multi(*args, ys, ns, 5, 4, 256, None) == -2
    assert lib.fpq_gemm_mxf4_packed_multi(*args, None, ns, 2, 4, 256, None) == -1
    assert lib.fpq_gemm_mxf4_packed_multi(*args, ys, (ctypes.c_int64 * 2)(256, 100), 2, 4, 256, None) == -2
    assert lib.fpq_gemm_mxf4_packed_multi(*args, (ctypes.c_void_p * 2)(256, 8), ns, 2, 4, 256, None) == -4
    assert lib.fpq_gemm_mxf4_packed_multi(*args, (ctypes.c_void_p * 2)(256, None), ns, 2, 4, 256, None) == -1
    assert lib.fpq_gemm_mxf4_packed_multi(*args, ys, ns, 2, 4, 100, None) == -2
    assert lib.fpq_gemm_mxf4_packed_multi(*args, ys, ns, 2, 0, 256, None) == 0
    with pytest.raises(ValueError):
        _engine.check(-2, "x")


def test_split_k_workspace_sizes_are_host_arithmetic():
    """fpq_gemm_mxf4_packed_workspace_bytes needs no device: 16 KB of counters plus 4 KB per part, weight tile
    and activation row tile where K is split (few weight tiles, parts of at least 4096 of K), else 0."""
    from fp_quant import _engine
    need = _engine.lib().fpq_gemm_mxf4_packed_workspace_bytes
    assert need(16, 4096, 14336) == 16384 + 2 * 128 * 4096
    assert need(16, 1024, 14336) == 16384 + 3 * 32 * 4096
    assert need(64, 4096, 14336) == 16384 + 2 * 128 * 2 * 4096
    assert need(128, 4096, 8192) == 16384 + 2 * 128 * 4 * 4096 == 4210688   # the most a split ever needs
    assert need(16, 4096, 4096) == need(16, 14336, 4096) == need(129, 4096, 14336) == need(16, 4096, 256) == 0
    assert need(0, 4096, 14336) == need(16, 4096, 100) == 0                 # shapes the kernel does not take
    assert _engine.lib().fpq_gemm_mxf4_packed_noalloc_max_rows() == 128
