"""Seeded differential run of the HIP codec against the oracle over random sizes,
geometries, precisions and kinds of data (weights, all bit patterns -> raw
chunks, sparse alphabets -> bitmap tables, one exponent, one dominant symbol):
container and packed stream byte-identical, decode output bit-exact."""
import numpy as np
import pytest

from test_gpu_parity import gpu_decode, gpu_encode

pytestmark = pytest.mark.gpu

GEOMETRIES = [(131072, 256), (65536, 344), (65536, 128), (32768, 64), (155648, 304), (65536, 176),
              (16384, 32), (8192, 16), (262144, 512), (2048, 16), (1024, 16)]


def _data(rng, n, kind):
    if kind == 0:  # weights
        x = (rng.standard_normal(n) * 0.02).astype(np.float32)
        return (x.view(np.uint32) >> 16).astype(np.uint16)
    if kind == 1:  # every bit pattern: chunks that are stored raw
        return rng.integers(0, 65536, n, dtype=np.uint16)
    if kind == 2:  # a sparse alphabet with gaps: bitmap tables
        syms = rng.choice(256, size=int(rng.integers(17, 60)), replace=False)
        e = rng.choice(syms, size=n).astype(np.uint16)
        return (e << 7) | rng.integers(0, 128, n, dtype=np.uint16) | (rng.integers(0, 2, n, dtype=np.uint16) << 15)
    if kind == 3:  # a single exponent
        return np.full(n, (int(rng.integers(0, 256)) << 7) | 5, dtype=np.uint16)
    e = np.where(rng.random(n) < 0.97, 120, rng.integers(0, 256, n)).astype(np.uint16)  # one dominant symbol
    return (e << 7) | rng.integers(0, 128, n, dtype=np.uint16)


@pytest.mark.parametrize("seed", range(6))
def test_random_cases_match_the_oracle(oracle, seed):
    rng = np.random.default_rng(1000 + seed)
    for it in range(8):
        chunk, lane = GEOMETRIES[int(rng.integers(len(GEOMETRIES)))]
        s = [7, 3, 1, 0][int(rng.integers(4))]
        n = int(rng.choice([rng.integers(1, 3000), rng.integers(3000, 400_000), rng.integers(400_000, 2_000_000)]))
        kind = int(rng.integers(5))
        bits = _data(rng, n, kind)
        print(f"case seed={seed} #{it}: n={n} kind={kind} s={s} chunk={chunk} lane={lane}", flush=True)
        comp, packed = gpu_encode(bits, s, chunk, lane)
        o_comp, o_packed = oracle.compress_bf16(bits, s, chunk, lane, threads=8)
        assert np.array_equal(comp.cpu().numpy(), o_comp)
        assert np.array_equal(packed.cpu().numpy(), o_packed)
        rc, out = gpu_decode(comp, packed, n, s, chunk, lane)
        assert rc == 0
        assert np.array_equal(out, oracle.reconstruct(bits, s))


@pytest.mark.parametrize("chunk,lane", [(135168, 264), (143360, 280), (147456, 288), (151552, 296)])
def test_segments_between_256_and_288_symbols_per_lane(oracle, chunk, lane):
    """The geometries a manager picks for tensors of one to a few million elements
    under its size budget: up to 288 symbols per lane are coded from registers
    (nz_encode_kernel<S, 36>), 296 by the kernel for longer segments; both give
    the oracle's bytes, for every precision and kind of data, ragged ends included."""
    rng = np.random.default_rng(chunk)
    for s in (7, 3, 1, 0):
        for kind, n in ((0, 3 * chunk + 12345), (1, chunk + 7), (2, 2 * chunk), (3, chunk - 1), (4, 1_000_003)):
            bits = _data(rng, n, kind)
            print(f"case chunk={chunk} lane={lane} s={s} kind={kind} n={n}", flush=True)
            comp, packed = gpu_encode(bits, s, chunk, lane)
            o_comp, o_packed = oracle.compress_bf16(bits, s, chunk, lane, threads=8)
            assert np.array_equal(comp.cpu().numpy(), o_comp)
            assert np.array_equal(packed.cpu().numpy(), o_packed)
            rc, out = gpu_decode(comp, packed, n, s, chunk, lane)
            assert rc == 0
            assert np.array_equal(out, oracle.reconstruct(bits, s))
