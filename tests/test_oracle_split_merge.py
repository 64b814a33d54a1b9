"""CPU: the oracle's split/merge against an independent closed form and the
invariants that follow from the reference kernel text
(cuda/kernels.cuh:120-155 split, :197-216 merge)."""
import numpy as np
import pytest

from conftest import bf16_bits_normal, closed_form_recon, stress_bits

ALL = np.arange(65536, dtype=np.uint16)
PRECISIONS = (7, 3, 1, 0)


@pytest.mark.parametrize("s", PRECISIONS)
def test_all_patterns_match_closed_form(oracle, s):
    rec = oracle.reconstruct(ALL, s)
    assert np.array_equal(rec, closed_form_recon(ALL, s))
    # the C closed form agrees too
    assert all(oracle.recon_closed_form(int(v), s) == int(rec[v]) for v in range(0, 65536, 97))


@pytest.mark.parametrize("s", PRECISIONS)
def test_split_fields_line_by_line(oracle, s):
    """exponent and packed field against a direct numpy reading of kernels.cuh:122-137,153."""
    v = ALL.astype(np.uint32)
    sign = v >> 15
    m = v & 0x7F
    e = (v >> 7) & 0xFF
    carry = ((m >> (6 - s)) & 1) if s < 7 else np.zeros_like(m)
    r = m >> (7 - s)
    popc = np.array([bin(int(t)).count("1") for t in range(128)])[r]
    overflow = ((popc == s) & (carry == 1)).astype(np.uint32)
    repr_ = (sign << s) | (((1 << s) - 1) & (r + carry))
    exps, packed = oracle.split(ALL, s)
    assert np.array_equal(exps, ((e + overflow) & 0xFF).astype(np.uint8))
    # MSB-first packing: byte = idx*(s+1)/8, shift = 7 - s - (idx*(s+1) & 7)
    idx = np.arange(65536, dtype=np.uint64)
    bit = idx * (s + 1)
    shift = 7 - s - (bit & 7)
    want = np.zeros(oracle.packed_bytes(65536, s), np.uint8)
    np.bitwise_or.at(want, (bit >> 3).astype(np.int64), (repr_ << shift).astype(np.uint8))
    assert np.array_equal(packed, want)


def test_lossless_is_identity(oracle):
    assert np.array_equal(oracle.reconstruct(ALL, 7), ALL)


@pytest.mark.parametrize("s", (3, 1, 0))
def test_lossy_invariants(oracle, s):
    rec = oracle.reconstruct(ALL, s)
    # idempotent
    assert np.array_equal(oracle.reconstruct(rec, s), rec)
    # dropped mantissa bits are zero, sign preserved (incl. -0)
    assert not np.any(rec & ((1 << (7 - s)) - 1))
    assert np.array_equal(rec & 0x8000, ALL & 0x8000)
    # |recon - a| <= half a step in magnitude units, except the wrap of 0x7FFF.. -> 0
    a = (ALL & 0x7FFF).astype(np.int64)
    r = (rec & 0x7FFF).astype(np.int64)
    wrap = a + (1 << (6 - s)) >= 0x8000
    assert np.all(np.abs(r - a)[~wrap] <= (1 << (6 - s)))
    assert np.all(r[wrap] == 0)
    # monotone non-decreasing in the magnitude outside the wrap
    pos = rec[:0x8000].astype(np.int64) & 0x7FFF
    keep = ~wrap[:0x8000]
    assert np.all(np.diff(pos[keep]) >= 0)


@pytest.mark.parametrize("s,count", ((3, 16), (1, 64), (0, 128)))
def test_enumerated_special_cases(oracle, s, count):
    rec = oracle.reconstruct(ALL, s)
    finite254 = (ALL & 0x7F80) == 0x7F00
    to_inf = finite254 & ((rec & 0x7FFF) == 0x7F80)
    assert to_inf.sum() == count  # 2^(6-s) mantissas per sign round up to +-Inf
    exp255 = (ALL & 0x7F80) == 0x7F80
    wrapped = exp255 & ((rec & 0x7F80) == 0)
    assert wrapped.sum() == count  # same mantissas at exponent 255: the byte 255 + 1 wraps to 0
    # subnormals keep exponent 0 unless they round up into the first normal
    sub = (ALL & 0x7F80) == 0
    assert np.all(((rec[sub] & 0x7F80) >> 7) <= 1)


@pytest.mark.parametrize("s", PRECISIONS)
def test_float_path_agrees_on_non_nan(oracle, s):
    """kernels.cuh:213-216 multiplies through fp32; identical for every non-NaN result."""
    e, f = oracle.split(ALL, s)
    bits = oracle.merge(e, f, s)
    lit = oracle.merge(e, f, s, literal_float=True)
    nan = (bits & 0x7FFF) > 0x7F80
    assert np.array_equal(bits[~nan], lit[~nan])
    assert np.all((lit[nan] & 0x7FFF) > 0x7F80)  # NaN stays NaN; payload is unpinned


@pytest.mark.parametrize("s", PRECISIONS)
@pytest.mark.parametrize("n", (0, 1, 2, 7, 8, 9, 15, 17, 1023, 1025))
def test_ragged_lengths_and_tail_padding(oracle, n, s):
    bits = stress_bits(5, 205, seed=n)[:n] if n else np.zeros(0, np.uint16)
    e, f = oracle.split(bits, s)
    assert f.size == (n * (s + 1) + 7) // 8  # cuda/high_level.cu:81-83
    if n and (n * (s + 1)) % 8:
        used = (n * (s + 1)) % 8
        assert f[-1] & ((1 << (8 - used)) - 1) == 0  # missing elements contribute zero bits
    assert np.array_equal(oracle.merge(e, f, s), closed_form_recon(bits, s))


def test_config1_plumbing_4096x4096(oracle):
    """BASELINE config 1: one 4096x4096 N(0,0.02) weight, lossless, on the CPU."""
    n = 4096 * 4096
    bits = bf16_bits_normal(n, seed=0)
    comp, packed = oracle.compress_bf16(bits, 7, 65536, 512, threads=8)
    rc, out = oracle.decompress_bf16(comp, packed, n, 7, threads=8)
    assert rc == 0 and np.array_equal(out, bits)
    stored = comp.size + packed.size
    assert 0.655 < stored / (2 * n) < 0.665  # (8 + ~2.55) / 16
