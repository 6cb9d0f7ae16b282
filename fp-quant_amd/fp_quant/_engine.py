"""ctypes binding of libfpq_hip.so (the C ABI declared in include/fpq.h).

There is no fallback: if the library is missing or fails to load, every call raises.
"""
import ctypes
import os
import threading

# FPQ_LIBRARY_PATH lets a developer point the binding at another build of the same C ABI.
_LIB_PATH = os.environ.get("FPQ_LIBRARY_PATH") or os.path.join(
    os.path.dirname(os.path.abspath(__file__)), "_lib", "libfpq_hip.so")
_lock = threading.Lock()
_lib = None

ROT_HADAMARD, ROT_IDENTITY, ROT_GSR, ROT_GENERAL = 0, 1, 2, 3
ZERO_REFERENCE, ZERO_SIGNED = 0, 1
E_UNSUPPORTED = -6

_P, _I64, _I, _F = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float

_SIGNATURES = {
    "fpq_version": ([], _I),
    "fpq_status_string": ([_I], ctypes.c_char_p),
    "fpq_device_supported": ([_I], _I),
    "fpq_stream_capture_id": ([_P, ctypes.POINTER(ctypes.c_ulonglong)], _I),
    "fpq_quantize_mx": ([_P, _I64, _I64, _I, _I, _F, _P, _P, _P, _I64, _I64, _I, _P], _I),
    "fpq_quantize_nv": ([_P, _I64, _I64, _I, _I, _F, _P, _P, _P, _P, _I64, _I64, _I, _P], _I),
    "fpq_gemm_mxf4": ([_P, _P, _I64, _P, _P, _I64, _P, _P, _P, _I64, _I64, _I64, _P], _I),
    "fpq_gemm_nvf4": ([_P, _P, _I64, _P, _P, _I64, _P, _P, _P, _I64, _I64, _I64, _P], _I),
    "fpq_test_e2m1": ([_P, _P, _I64, _I, _P], _I),
    "fpq_test_mfma_rate": ([_P, _I, _I, _P, _P, _P], _I),
    "fpq_packed_codes_bytes": ([_I64, _I64], _I64),
    "fpq_packed_scales_bytes": ([_I64, _I64], _I64),
    "fpq_pack_mxf4": ([_P, _P, _I64, _I64, _I64, _P, _P, _P], _I),
    "fpq_quantize_mx_quest": ([_P, _I64, _I64, _I, _I, _F, _P, _P, _P, _I64, _I64, _P, _I, _P], _I),
    "fpq_quantize_mx_packed": ([_P, _I64, _I64, _I, _I, _F, _P, _P, _I, _P], _I),
    "fpq_quantize_nv_packed": ([_P, _I64, _I64, _I, _I, _F, _P, _P, _P, _I, _P], _I),
    "fpq_rotated_absmax": ([_P, _I64, _I64, _I, _I, _F, _P, _P, _P], _I),
    "fpq_row_inv_rms": ([_P, _I64, _I64, _I64, _F, _P, _P], _I),
    "fpq_rmsnorm_quantize_mx": ([_P, _I64, _P, _P, _I64, _I64, _I, _I, _F, _P, _P, _P, _I64, _I64, _I, _P], _I),
    "fpq_rmsnorm_quantize_nv": ([_P, _I64, _P, _P, _I64, _I64, _I, _I, _F, _P, _P, _P, _P, _I64, _I64, _I, _P], _I),
    "fpq_silu_mul_quantize_mx": ([_P, _I64, _P, _I64, _I64, _I64, _I, _I, _F, _P, _P, _P, _I64, _I64, _I, _P], _I),
    "fpq_rmsnorm_quantize_mx_packed": ([_P, _I64, _P, _P, _I64, _I64, _I, _I, _F, _P, _P, _P, _I, _P], _I),
    "fpq_silu_mul_quantize_mx_packed": ([_P, _I64, _P, _I64, _I64, _I64, _I, _I, _F, _P, _P, _P, _I, _P], _I),
    "fpq_silu_mul_quantize_nv": ([_P, _I64, _P, _I64, _I64, _I64, _I, _I, _F, _P, _P, _P, _P, _I64, _I64, _I, _P], _I),
    "fpq_packed_scales_bytes_nv": ([_I64, _I64], _I64),
    "fpq_pack_nvf4": ([_P, _P, _I64, _I64, _I64, _P, _P, _P], _I),
    "fpq_gemm_nvf4_packed": ([_P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _P], _I),
    "fpq_gemm_mxf4_packed": ([_P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _P], _I),
    "fpq_gemm_mxf4_packed_workspace_bytes": ([_I64, _I64, _I64], _I64),
    "fpq_gemm_mxf4_packed_splitk": ([_P, _P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _P, _I64, _P], _I),
    "fpq_gemm_mxf4_packed_residual": ([_P, _P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _P], _I),
    "fpq_gemm_mxf4_packed_noalloc_max_rows": ([], _I64),
    "fpq_gemm_mxf4_packed_noalloc": ([_P, _P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _P], _I),
}


class FPQEngineError(RuntimeError):
    pass


def library_path() -> str:
    return _LIB_PATH


def available() -> bool:
    """True if the HIP library is present and loads (says nothing about a GPU being there)."""
    try:
        lib()
        return True
    except FPQEngineError:
        return False


def lib():
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(_LIB_PATH):
                raise FPQEngineError(
                    f"{_LIB_PATH} is missing: build it with `python fp-quant_amd/build.py` "
                    "(hipcc, gfx950). This package has no other backend."
                )
            try:
                handle = ctypes.CDLL(_LIB_PATH)
            except OSError as exc:
                raise FPQEngineError(f"cannot load {_LIB_PATH}: {exc}") from exc
            for name, (argtypes, restype) in _SIGNATURES.items():
                fn = getattr(handle, name)
                fn.argtypes = argtypes
                fn.restype = restype
            _lib = handle
    return _lib


def check(status: int, what: str) -> None:
    """Turn a status of the C ABI into the exception the reference surface would raise."""
    if status == 0:
        return
    msg = lib().fpq_status_string(status).decode()
    if status < 0:
        raise ValueError(f"{what}: {msg} (fpq status {status})")
    raise RuntimeError(f"{what}: HIP error {status}: {msg}")
