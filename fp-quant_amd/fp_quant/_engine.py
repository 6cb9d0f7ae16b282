"""ctypes binding of libfpq_hip.so (the C ABI declared in include/fpq.h).

There is no fallback: if the library is missing or fails to load, every call raises.
"""
import contextlib
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
E_LIMIT = -7

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
    "fpq_quantize_mx_quest_packed": ([_P, _I64, _I64, _I, _I, _F, _P, _P, _I, _P], _I),
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
    "fpq_gemm_nvf4_packed_workspace_bytes": ([_I64, _I64, _I64], _I64),
    "fpq_gemm_mxf4_packed_splitk": ([_P, _P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _P, _I64, _P], _I),
    "fpq_gemm_nvf4_packed_splitk": ([_P, _P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _P, _I64, _P], _I),
    "fpq_gemm_mxf4_packed_residual": ([_P, _P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _P], _I),
    "fpq_gemm_nvf4_packed_residual": ([_P, _P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _P], _I),
    "fpq_gemm_mxf4_packed_multi": ([_P, _P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _P], _I),
    "fpq_gemm_nvf4_packed_multi": ([_P, _P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _P], _I),
    "fpq_unpack_mxf4": ([_P, _P, _I64, _I64, _P, _P, _I64, _P], _I),
    "fpq_unpack_nvf4": ([_P, _P, _I64, _I64, _P, _P, _I64, _P], _I),
    "fpq_rmsnorm_rows_max_rows": ([], _I64),
    "fpq_rmsnorm_rows_quantize_mx_packed": ([_P, _I64, _P, _I64, _I64, _F, _I, _I, _F, _P, _P, _P, _P, _I, _P], _I),
    "fpq_rmsnorm_rows_quantize_nv_packed": ([_P, _I64, _P, _I64, _I64, _F, _I, _I, _F, _P, _P, _P, _P, _P, _I, _P], _I),
    "fpq_rmsnorm_quantize_nv_packed": ([_P, _I64, _P, _P, _I64, _I64, _I, _I, _F, _P, _P, _P, _P, _I, _P], _I),
    "fpq_silu_mul_quantize_nv_packed": ([_P, _I64, _P, _I64, _I64, _I64, _I, _I, _F, _P, _P, _P, _P, _I, _P], _I),
    "fpq_prepare_device": ([_P], _I),
    "fpq_gemm_mxf4_packed_noalloc_max_rows": ([], _I64),
    "fpq_test_noalloc_counters": ([_P, _I64, _P], _I),
    "fpq_compute_units": ([], _I),
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


# ---- rotation matrices: shared by the fp_quant operators and the qutlass stand-in -------------------------
_SAME_DEVICE = contextlib.nullcontext()


def on_device(dev):
    """`with on_device(dev):` -- torch.cuda.device(dev) when another GPU is current, else a context that does
    nothing (entering the real one costs several microseconds of host time per call)."""
    import torch
    return _SAME_DEVICE if torch.cuda.current_device() == dev.index else torch.cuda.device(dev)


def tensor_version(t):
    """The tensor's in-place modification counter, or None for tensors created under
    torch.inference_mode(), which have none."""
    try:
        return t._version
    except RuntimeError:
        return None


def sylvester_signs(g: int):
    """+-1 entries of the Sylvester Hadamard matrix of size g (scipy.linalg.hadamard order)."""
    import torch
    idx = torch.arange(g)
    anded = idx[:, None] & idx[None, :]
    pop = torch.zeros_like(anded)
    for b in range(8):
        pop += (anded >> b) & 1
    return (1 - 2 * (pop & 1)).to(torch.float32)


def classify_rotation(h):
    """(rotation kind, norm) of a [g, g] matrix: the Hadamard / identity / sequency-ordered matrices the
    reference builds (inference_lib/src/fp_quant/module/linear.py:24-41) are applied as butterflies,
    anything else as a matrix product.  The result is remembered on the tensor object itself, keyed by
    its storage address and modification counter, so the one device->host copy it needs happens once
    per matrix; a tensor without a counter (made under torch.inference_mode()) is classified on every call."""
    import torch
    version = tensor_version(h)
    key = (h.data_ptr(), version)
    hit = getattr(h, "_fpq_rotation", None)
    if version is not None and hit is not None and hit[0] == key:
        return hit[1], hit[2]
    g = h.shape[0]
    if h.dim() != 2 or h.shape[1] != g:
        raise ValueError(f"rotation matrix must be square, got {tuple(h.shape)}")
    hf = h.detach().to(device="cpu", dtype=torch.float32)
    kind, norm = ROT_GENERAL, 0.0
    if torch.equal(hf, torch.eye(g)):
        kind, norm = ROT_IDENTITY, 1.0
    elif g in (16, 32, 64, 128) and float(hf[0, 0]) != 0.0:
        n = float(hf[0, 0])
        signed = sylvester_signs(g) * n
        if torch.equal(hf, signed):
            kind, norm = ROT_HADAMARD, n
        else:
            changes = torch.diff(signed, dim=0).ne(0).sum(dim=0)
            if torch.equal(hf, signed[:, torch.argsort(changes)]):
                kind, norm = ROT_GSR, n
    if version is not None:
        try:
            h._fpq_rotation = (key, kind, norm)
        except AttributeError:  # objects that refuse attributes: classify again next time
            pass
    return kind, norm
