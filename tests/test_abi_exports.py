"""CPU: the C-ABI library loads and exports every symbol include/neuzip_hip.h
declares; size helpers agree with the oracle (no kernel is launched)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "neuzip_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nz_[a-z_0-9]+)\s*\(", text)))


def test_header_symbols_are_exported():
    from neuzip_amd import _lib

    L = _lib.load()
    names = declared_symbols()
    assert len(names) >= 18
    for name in names:
        assert hasattr(L, name), f"{name} declared in include/neuzip_hip.h but not exported"
    assert sorted(_lib.EXPORTS) == names  # the ctypes binding covers the whole header
    assert L.nz_abi_version() == 4


def test_size_helpers_match_oracle(oracle):
    from neuzip_amd import _lib

    L = _lib.load()
    for n in (0, 1, 7, 8, 9, 32767, 32768, 65536, 1_000_003):
        for s in (7, 3, 1, 0):
            assert L.nz_packed_bytes(n, s) == oracle.packed_bytes(n, s) == (n * (s + 1) + 7) // 8
            for lane in (16, 128, 344, 512, 1024):
                assert L.nz_packed_stored_bytes(n, s, 65536, lane) == oracle.packed_stored_bytes(n, s, lane, 65536)
        for lane, chunk in ((512, 65536), (344, 65536), (128, 65536), (1024, 65536), (16, 1024), (2048, 1 << 20)):
            assert L.nz_exp_bound_bytes(n, chunk, lane) == oracle.exp_bound(n, chunk, lane)
            assert L.nz_encode_workspace_bytes(n, chunk, lane) > n
    assert L.nz_exp_bound_bytes(1000, 65536, 100) == 0  # unsupported geometry
    assert L.nz_exp_bound_bytes(1000, 65536, 64) == 0


def test_argument_errors_without_a_gpu():
    from neuzip_amd import _lib

    L = _lib.load()
    # precision / geometry / null checks happen before any HIP call
    assert L.nz_decode(None, 0, None, 16, 5, 65536, 512, None, None, 0, 0, None, None) == _lib.ERR_ARG
    assert "precision" in _lib.last_error()
    assert L.nz_decode(None, 0, None, 16, 7, 65536, 100, None, None, 0, 0, None, None) == _lib.ERR_ARG
    assert L.nz_decode(None, 0, None, 16, 7, 65536, 512, None, None, 0, 0, None, None) == _lib.ERR_ARG
    assert L.nz_decode(None, 0, None, 0, 7, 65536, 512, None, None, 0, 0, None, None) == _lib.OK  # empty tensor
    h = ctypes.c_void_p()
    assert L.nz_manager_create(3, 7, 0, 65536, 0, ctypes.byref(h)) == _lib.ERR_ALGO
    assert _lib.last_error() == "Unsupported algorithm"  # cuda/high_level.cu:67
    assert L.nz_manager_create(0, 5, 0, 65536, 0, ctypes.byref(h)) == _lib.ERR_ARG
    assert L.nz_manager_create(0, 7, 33, 65536, 0, ctypes.byref(h)) == _lib.ERR_ARG  # not a power of two
    with pytest.raises(RuntimeError):
        _lib.raise_for(_lib.ERR_ALGO)
