"""CPU: the rANS container of the oracle — identity on arbitrary bytes, size
against the Shannon bound, table round trips, corruption detection, and an
independent pure-Python decoder of the same byte format."""
import numpy as np
import pytest
from hypothesis import given, settings, strategies as st

import pyref
from conftest import bf16_bits_normal, chunk_entropy_bytes, closed_form_recon, stress_bits

GEOMS = ((16, 1024), (16, 8192), (24, 2560), (64, 4096), (128, 65536), (344, 65536), (512, 65536),
         (1024, 65536), (2048, 1 << 20), (256, 131072), (344, 131072), (512, 262144))


def roundtrip(oracle, syms, lane, chunk, seeds=None):
    comp = oracle.exp_encode(syms, chunk, lane, seeds=seeds)
    rc, out, sd = oracle.exp_decode(comp, syms.size, lane_syms=lane, chunk_syms=chunk)
    assert rc == 0
    assert np.array_equal(out, syms)
    return comp, sd


@pytest.mark.parametrize("n", list(range(0, 131)) + [511, 512, 513, 1023, 1024, 1025, 2047, 2049])
def test_every_small_length(oracle, n):
    rng = np.random.default_rng(n)
    syms = rng.choice(np.array([120, 121, 122, 123, 7], np.uint8), size=n, p=[.5, .25, .15, .07, .03])
    roundtrip(oracle, syms, 16, 1024)


@pytest.mark.parametrize("lane,chunk", GEOMS)
def test_chunk_and_segment_boundaries(oracle, lane, chunk):
    rng = np.random.default_rng(lane)
    seg = 64 * lane
    for n in (seg - 1, seg, seg + 1, chunk - 1, chunk, chunk + 1, 2 * chunk + seg + 5):
        syms = np.clip(rng.normal(118, 2.5, n), 0, 255).astype(np.uint8)
        nseg = oracle.segment_count(n, chunk, lane)
        seeds = rng.integers(0, 65536, 64 * nseg).astype(np.uint16)
        comp, sd = roundtrip(oracle, syms, lane, chunk, seeds)
        # the carried bits of every full segment come back from the final states
        spc = -(-chunk // seg)
        for k in range(nseg):
            cpos, kk = divmod(k, spc)
            nom = seg if kk + 1 < spc else chunk - (spc - 1) * seg
            if cpos * chunk + kk * seg + nom <= n:
                assert np.array_equal(sd[64 * k: 64 * k + 64], seeds[64 * k: 64 * k + 64])
        assert comp.size <= oracle.exp_bound(n, chunk, lane)


def test_single_symbol_and_full_alphabet(oracle):
    roundtrip(oracle, np.full(70_000, 200, np.uint8), 512, 65536)
    roundtrip(oracle, np.zeros(5, np.uint8), 512, 65536)
    roundtrip(oracle, np.arange(256, dtype=np.uint8).repeat(300), 512, 65536)
    rng = np.random.default_rng(0)
    comp, _ = roundtrip(oracle, rng.integers(0, 256, 200_000).astype(np.uint8), 512, 65536)
    assert comp.size <= oracle.exp_bound(200_000, 65536, 512)  # incompressible -> raw chunks


@settings(max_examples=60, deadline=None)
@given(st.binary(min_size=0, max_size=5000), st.sampled_from([(16, 1024), (16, 2048), (24, 1536)]))
def test_identity_on_arbitrary_bytes(data, geom):
    from oracle import oracle as O

    syms = np.frombuffer(data, np.uint8)
    lane, chunk = geom
    comp = O.exp_encode(syms, chunk, lane)
    rc, out = O.exp_decode(comp, syms.size)
    assert rc == 0 and np.array_equal(out, syms)


@settings(max_examples=25, deadline=None)
@given(st.lists(st.integers(0, 255), min_size=1, max_size=6), st.integers(1, 4000), st.integers(0, 2**31))
def test_python_decoder_agrees(alphabet, n, seed):
    """Two independent readers of the same bytes: the C oracle and pyref."""
    from oracle import oracle as O

    rng = np.random.default_rng(seed)
    syms = rng.choice(np.array(alphabet, np.uint8), size=n)
    seeds = rng.integers(0, 65536, 64 * O.segment_count(n, 2048, 16)).astype(np.uint16)
    comp = O.exp_encode(syms, 2048, 16, seeds=seeds)
    out, carried = pyref.decode_container(comp.tobytes(), n)
    assert np.array_equal(out, syms)
    full = 64 * (n // 1024)  # every 1024-symbol segment the stream does not end inside
    assert np.array_equal(carried[:full], seeds[:full])


def test_size_against_shannon_bound(oracle):
    """Stored bytes beyond the raw sign|mantissa bits stay within 1% of the
    per-64KiB-chunk order-0 entropy of the exponents (header included)."""
    for name, bits in (("normal", bf16_bits_normal(4 * 1024 * 1024, 1)), ("stress", stress_bits(1024, 4096, 2))):
        exps, _ = oracle.split(bits, 7)
        bound = chunk_entropy_bytes(exps)
        comp, packed = oracle.compress_bf16(bits, 7, 65536, 512)
        effective = comp.size + packed.size - bits.size
        assert effective >= bound  # no order-0 coder beats it
        assert effective <= 1.01 * bound, (name, effective / bound)


def test_frequency_normalisation(oracle):
    rng = np.random.default_rng(4)
    for trial in range(200):
        k = int(rng.integers(1, 257))
        cnt = np.zeros(256, np.uint32)
        live = rng.choice(256, k, replace=False)
        cnt[live] = rng.integers(1, 5000, k) ** int(rng.integers(1, 3))
        n = int(cnt.sum())
        freq, pad = oracle.normalize_freqs(cnt, n)
        assert int(freq.sum()) == 4096
        assert np.all(freq[cnt > 0] >= 1) and freq.max() <= 4095
        if k > 1:
            assert np.all(freq[cnt == 0] == 0)
        assert cnt[pad] == cnt.max() and pad == int(np.argmax(cnt))
        # serialise / parse round trip, runs and bitmap forms
        ser = oracle.table_serialize(freq)
        rc, back, used = oracle.table_parse(ser)
        assert rc == 0 and used == ser.size and np.array_equal(back, freq)
        assert ser.size % 4 == 0 and ser.size <= 420


def test_quantisation_loss_is_small(oracle):
    bits = bf16_bits_normal(1 << 20, 9)
    exps, _ = oracle.split(bits, 7)
    cnt = np.bincount(exps, minlength=256).astype(np.uint32)
    freq, _ = oracle.normalize_freqs(cnt, exps.size)
    p = cnt[cnt > 0] / exps.size
    h = -(p * np.log2(p)).sum()
    cross = -(p * np.log2(freq[cnt > 0] / 4096.0)).sum()
    assert cross - h < 0.004  # bits per symbol (0.16% of 2.55)


def test_corruption_is_detected(oracle):
    bits = bf16_bits_normal(150_000, 3)
    comp, packed = oracle.compress_bf16(bits, 7, 65536, 512)
    rc, _ = oracle.decompress_bf16(comp, packed, bits.size, 7)
    assert rc == 0
    for off in (0, 4, 8, 20, 64, 70):  # header and directory fields
        bad = comp.copy()
        bad[off] ^= 0xFF
        rc, _ = oracle.decompress_bf16(bad, packed, bits.size, 7)
        assert rc == oracle.ERR_CORRUPT, off
    rc, _ = oracle.decompress_bf16(comp[: comp.size // 2], packed, bits.size, 7)  # truncated
    assert rc == oracle.ERR_CORRUPT
    rc, _ = oracle.decompress_bf16(comp, packed, bits.size - 1, 7)  # wrong length
    assert rc == oracle.ERR_CORRUPT
    hits = 0
    rng = np.random.default_rng(0)
    for _ in range(20):  # flipped bits in the word stream end in a wrong final state
        bad = comp.copy()
        bad[int(rng.integers(comp.size // 4, comp.size))] ^= 1 << int(rng.integers(0, 8))
        rc, out = oracle.decompress_bf16(bad, packed, bits.size, 7)
        hits += rc == oracle.ERR_CORRUPT or not np.array_equal(out, bits)
    assert hits == 20


def test_geometry_validation(oracle):
    assert oracle.check_geometry(65536, 512) == 0
    assert oracle.check_geometry(65536, 1024) == 0
    assert oracle.check_geometry(65536, 344) == 0  # 2 x 22016 + 21504: a ragged last segment
    assert oracle.check_geometry(65536, 64) != 0  # more than 8 segments per chunk
    assert oracle.check_geometry(65536, 8) != 0  # below the 16-symbol minimum
    assert oracle.check_geometry(65536, 100) != 0  # not a multiple of 8
    assert oracle.check_geometry(60000, 512) != 0  # chunk not a multiple of 512
    assert oracle.check_geometry(65536, 1016) != 0  # would leave a 512-symbol last segment
    assert oracle.exp_bound(1000, 65536, 100) == 0


@pytest.mark.parametrize("s", (7, 3, 1, 0))
def test_whole_tensor_with_carry(oracle, s):
    """Packed stream stored with the carried bytes taken out, all precisions."""
    for n in (32768, 32768 * 3 + 17, 65536 * 2):
        bits = stress_bits(1, n, seed=n + s)
        comp, packed = oracle.compress_bf16(bits, s, 65536, 512)
        assert packed.size == oracle.packed_bytes(n, s) - 128 * (n // 32768) == oracle.packed_stored_bytes(n, s, 512)
        rc, out = oracle.decompress_bf16(comp, packed, n, s)
        assert rc == 0 and np.array_equal(out, closed_form_recon(bits, s))


def test_plumbing_case_4096x4096(oracle):
    """One 4096 x 4096 weight from N(0, 0.02), lossless: split, entropy-code,
    exact round trip, stored size about (8 + 2.546) / 16 of dense."""
    n = 4096 * 4096
    bits = bf16_bits_normal(n, 0)
    comp, packed = oracle.compress_bf16(bits, 7, 65536, 344, threads=4)
    rc, out = oracle.decompress_bf16(comp, packed, n, 7, threads=4)
    assert rc == 0 and np.array_equal(out, bits)
    assert abs((comp.size + packed.size) / (2.0 * n) - 0.659) < 0.004
    exps = ((bits >> 7) & 0xFF).astype(np.uint8)
    effective = comp.size + packed.size - n
    assert effective <= 1.01 * chunk_entropy_bytes(exps)
