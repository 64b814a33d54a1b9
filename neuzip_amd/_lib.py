"""ctypes binding of libneuzip_hip.so (declared in include/neuzip_hip.h).

Stands where the reference imports its pybind11 extension
(``import neuzip._cuda``, neuzip/binding.py:15-20) and, like the reference,
fails loudly when the native library is missing: there is no Python or CPU
fallback for the codec.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# NEUZIP_HIP_LIB points at an alternative build of the library (development aid)
LIB_PATH = os.environ.get("NEUZIP_HIP_LIB") or os.path.join(_HERE, "libneuzip_hip.so")

OK = 0
ERR_ARG, ERR_DTYPE, ERR_NOT_FOUND, ERR_HIP, ERR_CAPACITY, ERR_CORRUPT, ERR_ALIGN, ERR_ALGO = range(-1, -9, -1)
DTYPE_BF16, DTYPE_F16, DTYPE_F32 = 0, 1, 2
ALGO_ANS = 0
DEFAULT_CHUNK = 131072
DEFAULT_LANE_SYMS = 256
DEFAULT_SIZE_BUDGET = 1.01
LANE_SYMS_AUTO = 0xFFFFFFFF
DECODE_CHECK, DECODE_STREAM_OUT, DECODE_RESIDENT_OUT = 1, 2, 4  # nz_decode flags

EXPORTS = [
    "nz_abi_version", "nz_last_error", "nz_packed_bytes", "nz_packed_stored_bytes", "nz_exp_bound_bytes",
    "nz_encode_workspace_bytes", "nz_norm_bytes", "nz_split", "nz_encode", "nz_encode_static", "nz_decode",
    "nz_manager_create", "nz_manager_destroy", "nz_manager_set_size_budget", "nz_manager_size_budget", "nz_estimated_size_ratio", "nz_manager_in_budget", "nz_manager_write", "nz_manager_write_batch",
    "nz_manager_read", "nz_manager_read_batch", "nz_manager_gemv_batch", "nz_manager_gemv_rows_batch", "nz_manager_gather_rows",
    "nz_manager_meta", "nz_manager_geometry", "nz_manager_size", "nz_manager_size_reference", "nz_manager_exp_bytes", "nz_manager_packed_bytes",
    "nz_manager_norm_bytes", "nz_manager_buffers", "nz_manager_erase", "nz_manager_check",
    "nz_manager_export", "nz_manager_import", "nz_manager_trim", "nz_manager_rewrite_stats", "nz_set_lookback_spins", "nz_manager_geometry_hint",
]

_lib = None


def load() -> ctypes.CDLL:
    """Load the native library; raise ImportError (as the reference does) if absent."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"The HIP extension is not built ({LIB_PATH} missing). "
            "Run `python -c 'import __graft_entry__ as g; g.build()'` or `python neuzip_amd/_build.py`."
        )
    L = ctypes.CDLL(LIB_PATH)
    vp, u64, u32, i32 = ctypes.c_void_p, ctypes.c_uint64, ctypes.c_uint32, ctypes.c_int
    L.nz_abi_version.restype = i32
    L.nz_abi_version.argtypes = []
    L.nz_last_error.restype = ctypes.c_char_p
    L.nz_last_error.argtypes = []
    L.nz_packed_bytes.restype = u64
    L.nz_packed_bytes.argtypes = [u64, i32]
    L.nz_packed_stored_bytes.restype = u64
    L.nz_packed_stored_bytes.argtypes = [u64, i32, u32, u32]
    L.nz_exp_bound_bytes.restype = u64
    L.nz_exp_bound_bytes.argtypes = [u64, u32, u32]
    L.nz_encode_workspace_bytes.restype = u64
    L.nz_encode_workspace_bytes.argtypes = [u64, u32, u32]
    L.nz_split.restype = i32
    L.nz_norm_bytes.restype = u64
    L.nz_norm_bytes.argtypes = [u64, u32]
    L.nz_split.argtypes = [vp, u64, vp, vp, u32, vp, vp]
    L.nz_encode.restype = i32
    L.nz_encode.argtypes = [vp, u64, i32, u32, u32, vp, vp, u64, vp, u64, vp, vp,
                            ctypes.POINTER(u64), u32, vp, vp]
    L.nz_encode_static.restype = i32
    L.nz_encode_static.argtypes = [vp, u64, i32, u32, u32, vp, vp, u64, vp, vp, u32, vp, vp]
    L.nz_decode.restype = i32
    L.nz_decode.argtypes = [vp, u64, vp, u64, i32, u32, u32, vp, vp, i32, u32, vp, vp]
    L.nz_manager_create.restype = i32
    L.nz_manager_create.argtypes = [i32, i32, i32, u32, u32, ctypes.POINTER(vp)]
    L.nz_manager_destroy.restype = None
    L.nz_manager_destroy.argtypes = [vp]
    L.nz_manager_set_size_budget.restype = i32
    L.nz_manager_set_size_budget.argtypes = [vp, ctypes.c_double]
    L.nz_manager_size_budget.restype = ctypes.c_double
    L.nz_manager_size_budget.argtypes = [vp]
    L.nz_manager_in_budget.restype = i32
    L.nz_manager_in_budget.argtypes = [vp, u64, u32, u32]
    L.nz_estimated_size_ratio.restype = ctypes.c_double
    L.nz_estimated_size_ratio.argtypes = [u64, u32, u32]
    L.nz_manager_write.restype = i32
    L.nz_manager_write.argtypes = [vp, ctypes.c_char_p, vp, u64, i32, vp]
    L.nz_manager_write_batch.restype = i32
    L.nz_manager_write_batch.argtypes = [vp, ctypes.POINTER(ctypes.c_char_p), ctypes.POINTER(vp), ctypes.POINTER(u64),
                                         u32, i32, vp]
    L.nz_manager_read.restype = i32
    L.nz_manager_read.argtypes = [vp, ctypes.c_char_p, vp, u64, vp]
    L.nz_manager_rewrite_stats.restype = i32
    L.nz_manager_rewrite_stats.argtypes = [vp, ctypes.POINTER(u64), ctypes.POINTER(u64), ctypes.POINTER(u64)]
    L.nz_manager_geometry_hint.restype = i32
    L.nz_manager_geometry_hint.argtypes = [vp, ctypes.c_char_p, ctypes.c_uint32, ctypes.c_uint32]
    L.nz_set_lookback_spins.restype = None
    L.nz_set_lookback_spins.argtypes = [ctypes.c_uint32]
    L.nz_manager_trim.restype = i32
    L.nz_manager_trim.argtypes = [vp]
    L.nz_manager_export.restype = i32
    L.nz_manager_export.argtypes = [vp, ctypes.c_char_p, vp, u64, vp, u64, vp, u64, vp]
    L.nz_manager_import.restype = i32
    L.nz_manager_import.argtypes = [vp, ctypes.c_char_p, vp, u64, vp, u64, vp, u64, vp]
    L.nz_manager_gather_rows.restype = i32
    L.nz_manager_gather_rows.argtypes = [vp, ctypes.c_char_p, vp, u64, u32, vp, vp]
    L.nz_manager_gemv_batch.restype = i32
    L.nz_manager_gemv_batch.argtypes = [vp, ctypes.POINTER(ctypes.c_char_p), u32, vp, u32, ctypes.POINTER(vp),
                                        ctypes.POINTER(vp), vp]
    L.nz_manager_gemv_rows_batch.restype = i32
    L.nz_manager_gemv_rows_batch.argtypes = [vp, ctypes.POINTER(ctypes.c_char_p), u32, vp, u32, u32,
                                             ctypes.POINTER(vp), ctypes.POINTER(vp), vp]
    L.nz_manager_read_batch.restype = i32
    L.nz_manager_read_batch.argtypes = [vp, ctypes.POINTER(ctypes.c_char_p), ctypes.POINTER(vp),
                                        ctypes.POINTER(u64), u32, vp]
    L.nz_manager_geometry.restype = i32
    L.nz_manager_geometry.argtypes = [vp, ctypes.c_char_p, ctypes.POINTER(u32), ctypes.POINTER(u32)]
    L.nz_manager_meta.restype = i32
    L.nz_manager_meta.argtypes = [vp, ctypes.c_char_p, ctypes.POINTER(u64), ctypes.POINTER(i32)]
    for name in ("nz_manager_size", "nz_manager_size_reference", "nz_manager_exp_bytes", "nz_manager_packed_bytes", "nz_manager_norm_bytes"):
        fn = getattr(L, name)
        fn.restype = u64
        fn.argtypes = [vp, ctypes.c_char_p]
    L.nz_manager_buffers.restype = i32
    L.nz_manager_buffers.argtypes = [vp, ctypes.c_char_p, ctypes.POINTER(vp), ctypes.POINTER(u64),
                                     ctypes.POINTER(vp), ctypes.POINTER(u64)]
    L.nz_manager_erase.restype = i32
    L.nz_manager_erase.argtypes = [vp, ctypes.c_char_p]
    L.nz_manager_check.restype = i32
    L.nz_manager_check.argtypes = [vp, vp]
    _lib = L
    return L


def last_error() -> str:
    msg = load().nz_last_error()
    return msg.decode() if msg else ""


def raise_for(code: int) -> None:
    """Map a C-ABI error code to the exception type the reference raises."""
    if code == OK:
        return
    msg = last_error() or f"libneuzip_hip error {code}"
    if code in (ERR_DTYPE, ERR_NOT_FOUND, ERR_ALGO, ERR_HIP, ERR_CORRUPT, ERR_CAPACITY):
        # std::runtime_error -> RuntimeError (cuda/high_level.cu:67,160,225)
        raise RuntimeError(msg)
    raise ValueError(msg)
