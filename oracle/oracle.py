"""ctypes wrapper around the CPU oracle (``libnz_oracle.so``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, the smoke check and the
``cpu_baseline`` leg of ``bench.py``.  The shipped package never imports it.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libnz_oracle.so")

OK, ERR_ARG, ERR_CAP, ERR_CORRUPT = 0, -1, -2, -3


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (a couple of seconds)."""
    src = os.path.join(_HERE, "nz_oracle.c")
    stale = (not os.path.exists(_LIB_PATH)) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src)
    if force or stale:
        subprocess.check_call(["make", "-B", "-C", _HERE, "libnz_oracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        u8p = ctypes.POINTER(ctypes.c_uint8)
        u16p = ctypes.POINTER(ctypes.c_uint16)
        u32p = ctypes.POINTER(ctypes.c_uint32)
        L.nzo_packed_bytes.restype = ctypes.c_size_t
        L.nzo_packed_bytes.argtypes = [ctypes.c_uint64, ctypes.c_int]
        L.nzo_split_bf16.restype = None
        L.nzo_split_bf16.argtypes = [u16p, ctypes.c_uint64, ctypes.c_int, u8p, u8p]
        L.nzo_merge_bf16.restype = None
        L.nzo_merge_bf16.argtypes = [u8p, u8p, ctypes.c_uint64, ctypes.c_int, u16p]
        L.nzo_merge_bf16_float.restype = None
        L.nzo_merge_bf16_float.argtypes = [u8p, u8p, ctypes.c_uint64, ctypes.c_int, u16p]
        L.nzo_recon_closed_form.restype = ctypes.c_uint16
        L.nzo_recon_closed_form.argtypes = [ctypes.c_uint16, ctypes.c_int]
        L.nzo_norm_count.restype = ctypes.c_size_t
        L.nzo_norm_count.argtypes = [ctypes.c_uint64, ctypes.c_uint32]
        L.nzo_block_normalize.restype = None
        L.nzo_block_normalize.argtypes = [u16p, ctypes.c_uint64, ctypes.c_uint32, u8p, u16p]
        L.nzo_block_denormalize.restype = None
        L.nzo_block_denormalize.argtypes = [u16p, ctypes.c_uint64, ctypes.c_uint32, u8p, u16p]
        L.nzo_normalize_freqs.restype = ctypes.c_int
        L.nzo_normalize_freqs.argtypes = [u32p, ctypes.c_uint64, u16p]
        L.nzo_table_serialize.restype = ctypes.c_size_t
        L.nzo_table_serialize.argtypes = [u16p, u8p]
        L.nzo_table_parse.restype = ctypes.c_int
        L.nzo_table_parse.argtypes = [u8p, ctypes.c_size_t, u16p, ctypes.POINTER(ctypes.c_size_t)]
        L.nzo_check_geometry.restype = ctypes.c_int
        L.nzo_check_geometry.argtypes = [ctypes.c_uint32, ctypes.c_uint32]
        L.nzo_exp_bound.restype = ctypes.c_size_t
        L.nzo_exp_bound.argtypes = [ctypes.c_uint64, ctypes.c_uint32, ctypes.c_uint32]
        L.nzo_exp_encode.restype = ctypes.c_int64
        L.nzo_exp_encode.argtypes = [u8p, ctypes.c_uint64, ctypes.c_uint32, ctypes.c_uint32, u16p, u8p,
                                     ctypes.c_size_t, ctypes.c_int]
        L.nzo_exp_decode.restype = ctypes.c_int
        L.nzo_exp_decode.argtypes = [u8p, ctypes.c_size_t, ctypes.c_uint64, u8p, u16p, ctypes.c_int]
        L.nzo_packed_stored_bytes.restype = ctypes.c_size_t
        L.nzo_packed_stored_bytes.argtypes = [ctypes.c_uint64, ctypes.c_int, ctypes.c_uint32, ctypes.c_uint32]
        L.nzo_compress_bf16.restype = ctypes.c_int64
        L.nzo_compress_bf16.argtypes = [u16p, ctypes.c_uint64, ctypes.c_int, ctypes.c_uint32,
                                        ctypes.c_uint32, u8p, u8p, ctypes.c_size_t, ctypes.c_int]
        L.nzo_decompress_bf16.restype = ctypes.c_int
        L.nzo_decompress_bf16.argtypes = [u8p, ctypes.c_size_t, u8p, ctypes.c_uint64, ctypes.c_int,
                                          u16p, ctypes.c_int]
        _lib = L
    return _lib


def _p(a: np.ndarray, ct):
    return a.ctypes.data_as(ctypes.POINTER(ct))


def _u16(a) -> np.ndarray:
    a = np.ascontiguousarray(a)
    assert a.dtype == np.uint16
    return a.reshape(-1)


def _u8(a) -> np.ndarray:
    a = np.ascontiguousarray(a)
    assert a.dtype == np.uint8
    return a.reshape(-1)


def packed_bytes(n: int, s: int) -> int:
    return int(lib().nzo_packed_bytes(n, s))


def split(bits: np.ndarray, s: int):
    """uint16 bf16 bit patterns -> (exponent bytes, packed sign+mantissa bytes)."""
    bits = _u16(bits)
    n = bits.size
    exps = np.empty(n, np.uint8)
    frac = np.zeros(packed_bytes(n, s), np.uint8)
    lib().nzo_split_bf16(_p(bits, ctypes.c_uint16), n, s, _p(exps, ctypes.c_uint8), _p(frac, ctypes.c_uint8))
    return exps, frac


def merge(exps: np.ndarray, frac: np.ndarray, s: int, literal_float: bool = False) -> np.ndarray:
    exps, frac = _u8(exps), _u8(frac)
    n = exps.size
    assert frac.size >= packed_bytes(n, s)
    out = np.empty(n, np.uint16)
    fn = lib().nzo_merge_bf16_float if literal_float else lib().nzo_merge_bf16
    fn(_p(exps, ctypes.c_uint8), _p(frac, ctypes.c_uint8), n, s, _p(out, ctypes.c_uint16))
    return out


def reconstruct(bits: np.ndarray, s: int) -> np.ndarray:
    """merge(split(x)) — the tensor the reference would hand back for x."""
    e, f = split(bits, s)
    return merge(e, f, s)


def block_normalize(bits: np.ndarray, norm_size: int):
    """-> (one byte per group of norm_size elements, the normalized tensor as bf16 bits)"""
    bits = _u16(bits)
    n = bits.size
    norm = np.zeros(lib().nzo_norm_count(n, norm_size), np.uint8)
    scaled = np.empty(n, np.uint16)
    if n:
        lib().nzo_block_normalize(_p(bits, ctypes.c_uint16), n, norm_size, _p(norm, ctypes.c_uint8),
                                  _p(scaled, ctypes.c_uint16))
    return norm, scaled


def block_denormalize(scaled: np.ndarray, norm_size: int, norm: np.ndarray) -> np.ndarray:
    scaled, norm = _u16(scaled), _u8(norm)
    out = np.empty(scaled.size, np.uint16)
    if scaled.size:
        lib().nzo_block_denormalize(_p(scaled, ctypes.c_uint16), scaled.size, norm_size,
                                    _p(norm, ctypes.c_uint8), _p(out, ctypes.c_uint16))
    return out


def reconstruct_normalized(bits: np.ndarray, s: int, norm_size: int) -> np.ndarray:
    """What the reference hands back for x with block normalizers of norm_size."""
    if not norm_size:
        return reconstruct(bits, s)
    norm, scaled = block_normalize(bits, norm_size)
    return block_denormalize(reconstruct(scaled, s), norm_size, norm)


def recon_closed_form(v: int, s: int) -> int:
    return int(lib().nzo_recon_closed_form(v, s))


def normalize_freqs(cnt: np.ndarray, n: int):
    cnt = np.ascontiguousarray(cnt, dtype=np.uint32)
    freq = np.zeros(256, np.uint16)
    pad = lib().nzo_normalize_freqs(_p(cnt, ctypes.c_uint32), n, _p(freq, ctypes.c_uint16))
    return freq, int(pad)


def table_serialize(freq: np.ndarray) -> np.ndarray:
    freq = np.ascontiguousarray(freq, dtype=np.uint16)
    out = np.zeros(424, np.uint8)
    nb = lib().nzo_table_serialize(_p(freq, ctypes.c_uint16), _p(out, ctypes.c_uint8))
    return out[:nb].copy()


def table_parse(buf: np.ndarray):
    buf = _u8(buf)
    freq = np.zeros(256, np.uint16)
    used = ctypes.c_size_t(0)
    rc = lib().nzo_table_parse(_p(buf, ctypes.c_uint8), buf.size, _p(freq, ctypes.c_uint16), ctypes.byref(used))
    return rc, freq, int(used.value)


def check_geometry(chunk_syms: int, lane_syms: int) -> int:
    return int(lib().nzo_check_geometry(chunk_syms, lane_syms))


def exp_bound(n: int, chunk_syms: int, lane_syms: int) -> int:
    return int(lib().nzo_exp_bound(n, chunk_syms, lane_syms))


def packed_stored_bytes(n: int, s: int, lane_syms: int, chunk_syms: int = 65536) -> int:
    return int(lib().nzo_packed_stored_bytes(n, s, chunk_syms, lane_syms))


def segment_count(n: int, chunk_syms: int, lane_syms: int) -> int:
    """Segments of the container: chunk c owns indices c*spc .. c*spc + spc - 1."""
    seg = 64 * lane_syms
    spc = -(-chunk_syms // seg)
    return (n // chunk_syms) * spc + -(-(n % chunk_syms) // seg)


def exp_encode(syms: np.ndarray, chunk_syms: int = 65536, lane_syms: int = 512, threads: int = 1,
               seeds: np.ndarray | None = None) -> np.ndarray:
    """Entropy-code a byte stream; `seeds` (uint16, 64 per full segment) is the
    payload carried in the coder's start states."""
    syms = _u8(syms)
    cap = exp_bound(syms.size, chunk_syms, lane_syms)
    if cap == 0:
        raise ValueError("unsupported geometry")
    out = np.zeros(cap, np.uint8)
    sp = None
    if seeds is not None:
        seeds = np.ascontiguousarray(seeds, dtype=np.uint16).reshape(-1)
        assert seeds.size >= 64 * segment_count(syms.size, chunk_syms, lane_syms)
        sp = _p(seeds, ctypes.c_uint16)
    r = lib().nzo_exp_encode(_p(syms, ctypes.c_uint8), syms.size, chunk_syms, lane_syms, sp,
                             _p(out, ctypes.c_uint8), cap, threads)
    if r < 0:
        raise RuntimeError(f"nzo_exp_encode failed: {r}")
    return out[:r].copy()


def exp_decode(comp: np.ndarray, n: int, threads: int = 1, lane_syms: int | None = None,
               chunk_syms: int = 65536):
    """Returns (rc, symbols) or, with lane_syms given, (rc, symbols, seeds) where
    seeds holds 64 values per segment (meaningful for full segments only)."""
    comp = _u8(comp)
    out = np.zeros(n, np.uint8)
    if lane_syms is None:
        rc = lib().nzo_exp_decode(_p(comp, ctypes.c_uint8), comp.size, n, _p(out, ctypes.c_uint8), None, threads)
        return int(rc), out
    nseg = segment_count(n, chunk_syms, lane_syms)
    seeds = np.zeros(64 * nseg + 64, np.uint16)
    rc = lib().nzo_exp_decode(_p(comp, ctypes.c_uint8), comp.size, n, _p(out, ctypes.c_uint8),
                              _p(seeds, ctypes.c_uint16), threads)
    return int(rc), out, seeds[: 64 * nseg]


def compress_bf16(bits: np.ndarray, s: int, chunk_syms: int = 65536, lane_syms: int = 512, threads: int = 1):
    bits = _u16(bits)
    n = bits.size
    cap = exp_bound(n, chunk_syms, lane_syms)
    if cap == 0:
        raise ValueError("unsupported geometry")
    comp = np.zeros(cap, np.uint8)
    frac = np.zeros(packed_stored_bytes(n, s, lane_syms, chunk_syms), np.uint8)
    r = lib().nzo_compress_bf16(_p(bits, ctypes.c_uint16), n, s, chunk_syms, lane_syms,
                                _p(frac, ctypes.c_uint8), _p(comp, ctypes.c_uint8), cap, threads)
    if r < 0:
        raise RuntimeError(f"nzo_compress_bf16 failed: {r}")
    return comp[:r].copy(), frac


def decompress_bf16(comp: np.ndarray, frac: np.ndarray, n: int, s: int, threads: int = 1):
    comp, frac = _u8(comp), _u8(frac)
    out = np.zeros(n, np.uint16)
    rc = lib().nzo_decompress_bf16(_p(comp, ctypes.c_uint8), comp.size, _p(frac, ctypes.c_uint8), n, s,
                                   _p(out, ctypes.c_uint16), threads)
    return int(rc), out
