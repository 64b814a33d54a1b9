"""Committed fixtures (tests/golden, written by tests/golden/make_golden.py):
the oracle on the CPU, the HIP path on the GPU."""
import os

import numpy as np
import pytest

from conftest import closed_form_recon

HERE = os.path.dirname(os.path.abspath(__file__))
sys_path_golden = os.path.join(HERE, "golden")


def _load(name):
    return np.load(os.path.join(sys_path_golden, name))


def _cases(which="CASES"):
    import importlib.util

    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(sys_path_golden, "make_golden.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return getattr(mod, which)


def test_oracle_matches_recon_tables(oracle):
    t = _load("recon_tables.npz")
    allv = np.arange(65536, dtype=np.uint16)
    for s in (7, 3, 1, 0):
        exps, packed = oracle.split(allv, s)
        assert np.array_equal(exps, t[f"exp_s{s}"])
        assert np.array_equal(packed, t[f"packed_s{s}"])
        assert np.array_equal(oracle.merge(exps, packed, s), t[f"recon_s{s}"])
        assert np.array_equal(t[f"recon_s{s}"], closed_form_recon(allv, s))


def test_oracle_matches_containers(oracle):
    c = _load("containers.npz")
    for name, (kind, n, seed, s, chunk, lane) in _cases().items():
        bits = c[name + "_bits"]
        comp, packed = oracle.compress_bf16(bits, s, chunk, lane)
        assert np.array_equal(comp, c[name + "_comp"]), name
        assert np.array_equal(packed, c[name + "_packed"]), name
        rc, out = oracle.decompress_bf16(c[name + "_comp"], c[name + "_packed"], n, s)
        assert rc == 0 and np.array_equal(out, closed_form_recon(bits, s))


@pytest.mark.gpu
def test_gpu_matches_recon_tables():
    from test_gpu_parity import gpu_decode, gpu_encode

    t = _load("recon_tables.npz")
    allv = np.arange(65536, dtype=np.uint16)
    for s in (7, 3, 1, 0):
        print(f"case golden table s={s}", flush=True)
        comp, packed = gpu_encode(allv, s)
        rc, out = gpu_decode(comp, packed, allv.size, s)
        assert rc == 0 and np.array_equal(out, t[f"recon_s{s}"])


@pytest.mark.gpu
def test_gpu_matches_containers():
    import torch

    from test_gpu_parity import gpu_decode, gpu_encode

    c = _load("containers.npz")
    for name, (kind, n, seed, s, chunk, lane) in _cases().items():
        print(f"case golden container {name}", flush=True)
        bits = c[name + "_bits"]
        comp, packed = gpu_encode(bits, s, chunk, lane)
        assert np.array_equal(comp.cpu().numpy(), c[name + "_comp"]), name
        assert np.array_equal(packed.cpu().numpy(), c[name + "_packed"]), name
        rc, out = gpu_decode(torch.from_numpy(c[name + "_comp"]).cuda(), torch.from_numpy(c[name + "_packed"]).cuda(),
                             n, s, chunk, lane)
        assert rc == 0 and np.array_equal(out, closed_form_recon(bits, s))


def test_oracle_matches_normalizer_fixtures(oracle):
    c = _load("normalizers.npz")
    for name, (kind, n, seed, s, ns) in _cases("NORM_CASES").items():
        bits = c[name + "_bits"]
        norm, scaled = oracle.block_normalize(bits, ns)
        assert np.array_equal(norm, c[name + "_norm"]) and np.array_equal(scaled, c[name + "_scaled"]), name
        assert np.array_equal(oracle.reconstruct_normalized(bits, s, ns), c[name + "_recon"]), name


@pytest.mark.gpu
def test_gpu_matches_normalizer_fixtures():
    from test_gpu_parity import gpu_decode, gpu_encode

    c = _load("normalizers.npz")
    for name, (kind, n, seed, s, ns) in _cases("NORM_CASES").items():
        print(f"case golden normalizer {name}", flush=True)
        bits = c[name + "_bits"]
        comp, packed, nb = gpu_encode(bits, s, norm_size=ns)
        assert np.array_equal(nb.cpu().numpy(), c[name + "_norm"]), name
        rc, out = gpu_decode(comp, packed, n, s, norm_size=ns, norm=nb)
        assert rc == 0 and np.array_equal(out, c[name + "_recon"]), name
