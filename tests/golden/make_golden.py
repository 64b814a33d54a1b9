"""Writes the golden fixtures of this directory from the CPU oracle.

The reference holds no vectors of its own for this path (it has no tests), so
the fixtures pin THIS build's semantics against accidental change:

  recon_tables.npz  merge(split(v)) for all 65 536 bf16 patterns and every
                    precision, cross-checked here against the independent
                    closed form before being written
  containers.npz    container + stored packed bytes of three seeded inputs
  normalizers.npz   group bytes and reconstruction of two seeded inputs stored
                    with block normalizers

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from conftest import bf16_bits_normal, closed_form_recon, stress_bits  # noqa: E402
from oracle import oracle as O  # noqa: E402

CASES = {
    # name: (generator, n, seed, precision, chunk, lane)
    "normal_1000_s7": ("normal", 1000, 11, 7, 1024, 16),
    "normal_70000_s7": ("normal", 70000, 12, 7, 65536, 512),
    "stress_70000_s3": ("stress", 70000, 13, 3, 65536, 512),
}


NORM_CASES = {
    # name: (generator, n, seed, precision, normalizer_size)
    "stress_5000_s3_n512": ("stress", 5000, 21, 3, 512),
    "normal_3000_s0_n8": ("normal", 3000, 22, 0, 8),
}


def finite(bits):
    return np.where((bits & 0x7F80) == 0x7F80, np.uint16(0x3F80) | (bits & 0x8000), bits).astype(np.uint16)


def make_bits(kind, n, seed):
    return bf16_bits_normal(n, seed) if kind == "normal" else stress_bits(1, n, seed)


def main():
    O.build()
    allv = np.arange(65536, dtype=np.uint16)
    tables = {}
    for s in (7, 3, 1, 0):
        rec = O.reconstruct(allv, s)
        assert np.array_equal(rec, closed_form_recon(allv, s))
        exps, packed = O.split(allv, s)
        tables[f"recon_s{s}"] = rec
        tables[f"exp_s{s}"] = exps
        tables[f"packed_s{s}"] = packed
    np.savez_compressed(os.path.join(HERE, "recon_tables.npz"), **tables)

    cont = {}
    for name, (kind, n, seed, s, chunk, lane) in CASES.items():
        bits = make_bits(kind, n, seed)
        comp, packed = O.compress_bf16(bits, s, chunk, lane)
        rc, out = O.decompress_bf16(comp, packed, n, s)
        assert rc == 0 and np.array_equal(out, closed_form_recon(bits, s))
        cont[name + "_bits"] = bits
        cont[name + "_comp"] = comp
        cont[name + "_packed"] = packed
    np.savez_compressed(os.path.join(HERE, "containers.npz"), **cont)
    nrm = {}
    for name, (kind, n, seed, s, ns) in NORM_CASES.items():
        bits = finite(make_bits(kind, n, seed))
        norm, scaled = O.block_normalize(bits, ns)
        nrm[name + "_bits"] = bits
        nrm[name + "_norm"] = norm
        nrm[name + "_scaled"] = scaled
        nrm[name + "_recon"] = O.reconstruct_normalized(bits, s, ns)
    np.savez_compressed(os.path.join(HERE, "normalizers.npz"), **nrm)
    for f in ("recon_tables.npz", "containers.npz", "normalizers.npz"):
        print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    main()
