import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _has_gpu() -> bool:
    try:
        import torch

        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _has_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as O

    O.build()
    return O


def bf16_bits_normal(n: int, seed: int, scale: float = 0.02) -> np.ndarray:
    """bf16 bit patterns of N(0, scale) values (round-to-nearest-even from fp32)."""
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal(n, dtype=np.float32) * np.float32(scale)).view(np.uint32)
    r = ((x + 0x7FFF + ((x >> 16) & 1)) >> 16).astype(np.uint16)
    return r


def stress_bits(rows: int, cols: int, seed: int) -> np.ndarray:
    """Student-t(3) * 0.02 with 1% exact zeros, 0.1% subnormals and 16 outlier
    columns at 50x (the stress configuration), as bf16 bit patterns."""
    rng = np.random.default_rng(seed)
    x = (rng.standard_t(3, size=(rows, cols)).astype(np.float32) * np.float32(0.02))
    out_cols = rng.choice(cols, size=min(16, cols), replace=False)
    x[:, out_cols] *= np.float32(50.0)
    u = x.view(np.uint32)
    bits = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16).reshape(-1)
    n = bits.size
    zeros = rng.random(n) < 0.01
    bits[zeros] = 0
    sub = rng.random(n) < 0.001
    bits[sub] = (rng.integers(0, 2, sub.sum()).astype(np.uint16) << 15) | rng.integers(1, 128, sub.sum()).astype(np.uint16)
    return bits


def closed_form_recon(bits: np.ndarray, s: int) -> np.ndarray:
    """Independent statement of what the reference returns for `bits` at
    precision s: round-half-up of the 15-bit magnitude to a multiple of
    2^(7-s), modulo 2^15; sign untouched."""
    bits = bits.astype(np.uint32)
    if s == 7:
        return bits.astype(np.uint16)
    a = bits & 0x7FFF
    r = ((a + (1 << (6 - s))) & 0x7FFF) & (0x7FFF ^ ((1 << (7 - s)) - 1))
    return ((bits & 0x8000) | r).astype(np.uint16)


def chunk_entropy_bytes(exps: np.ndarray, chunk: int = 65536) -> float:
    """Sum over chunks of n_chunk * H_chunk / 8 (order-0 Shannon bound)."""
    total = 0.0
    for c in range(0, exps.size, chunk):
        cnt = np.bincount(exps[c:c + chunk], minlength=256).astype(np.float64)
        nz = cnt[cnt > 0]
        total += -(nz * np.log2(nz / nz.sum())).sum()
    return total / 8.0
