"""Block normalizers of the oracle against an exact rational-arithmetic model.

The oracle follows the reference's float code (divide in fp32, cast to bf16);
the model below never touches floating point: it divides integers and rounds
to the bf16 grid (nearest, ties to even, gradual underflow, overflow to
infinity).  Agreement over every pair of 7-bit mantissas at exponents chosen
around the subnormal, normal and overflow ranges pins the arithmetic."""
import numpy as np
import pytest

from conftest import bf16_bits_normal, closed_form_recon, stress_bits


def _value(bits: int):
    """bf16 pattern -> (sign, integer significand, power of two)."""
    e, m = (bits >> 7) & 0xFF, bits & 0x7F
    return (bits >> 15, m, -133) if e == 0 else (bits >> 15, 128 + m, e - 134)


def _round_bf16(sign: int, num: int, den: int, e2: int) -> int:
    """Nearest bf16 pattern (ties to even) of (-1)^sign * num / den * 2^e2, in integers only."""
    sign <<= 15
    if num == 0:
        return sign
    e = num.bit_length() - den.bit_length()  # floor(log2(num / den)) or one more
    if (num if e >= 0 else num << -e) < (den << e if e >= 0 else den):
        e -= 1
    E = max(e + e2, -126)  # below 2^-126 the grid stays that of the smallest normal exponent
    shift = e2 - E + 7
    a, b = (num << shift, den) if shift >= 0 else (num, den << -shift)
    k, r = divmod(a, b)
    if 2 * r > b or (2 * r == b and (k & 1)):
        k += 1
    if k >= 256:
        k, E = 128, E + 1
    if k < 128:  # subnormal result
        return sign | k
    if E + 127 >= 255:
        return sign | 0x7F80
    return sign | ((E + 127) << 7) | (k - 128)


def _model_normalize(bits, n):
    norm, out = [], []
    for g0 in range(0, len(bits), n):
        grp = [int(b) for b in bits[g0:g0 + n]]
        mant = max(b & 0x7FFF for b in grp) & 0x7F  # the raw low 7 bits, also for a subnormal maximum
        norm.append(mant << 1)
        for b in grp:
            sg, sig, e2 = _value(b)
            out.append(_round_bf16(sg, sig * 128, 128 + mant, e2))  # x / (1 + mant/128)
    return np.array(norm, np.uint8), np.array(out, np.uint16)


def _model_denormalize(scaled, n, norm):
    out = []
    for i, v in enumerate(scaled):
        sg, sig, e2 = _value(int(v))
        out.append(_round_bf16(sg, sig * (256 + int(norm[i // n])), 256, e2))
    return np.array(out, np.uint16)


def test_round_model_is_the_identity_on_representable_values():
    for bits in list(range(0, 0x7F81, 97)) + [1, 0x7F, 0x80, 0x7F7F, 0x7F80, 0x8001, 0xFF7F]:
        sg, sig, e2 = _value(bits)
        assert _round_bf16(sg, sig, 1, e2) == bits


@pytest.mark.parametrize("e_big,e_x", [(1, 0), (1, 1), (2, 0), (3, 1), (100, 100), (127, 120), (140, 139),
                                       (254, 254), (254, 200), (9, 1), (8, 0)])
def test_every_mantissa_pair(oracle, e_big, e_x):
    """Groups of two: [largest element with mantissa mb, element with mantissa mx]."""
    mb, mx = np.meshgrid(np.arange(128), np.arange(128), indexing="ij")
    big = ((e_big << 7) | mb).astype(np.uint16).reshape(-1)
    x = ((e_x << 7) | mx).astype(np.uint16).reshape(-1)
    x = np.where((x & 0x7FFF) > (big & 0x7FFF), big, x)  # keep `big` the maximum
    x ^= np.uint16(0x8000) * (np.arange(x.size) % 2).astype(np.uint16)
    data = np.stack([big, x], axis=1).reshape(-1)
    norm, scaled = oracle.block_normalize(data, 2)
    m_norm, m_scaled = _model_normalize(data, 2)
    assert np.array_equal(norm, m_norm)
    assert np.array_equal(scaled, m_scaled)
    # the largest element of a group becomes a power of two
    assert np.all((scaled[0::2] & 0x7F) == 0)
    back = oracle.block_denormalize(scaled, 2, norm)
    assert np.array_equal(back, _model_denormalize(scaled, 2, norm))
    # without truncation the round trip stays within one unit in the last place
    # of the bf16 pattern (two roundings), and is exact for the largest element
    mag = lambda a: (a & 0x7FFF).astype(np.int32)
    finite = (scaled & 0x7F80) != 0x7F80
    assert np.all(np.abs(mag(back) - mag(data))[finite] <= 1)
    assert np.array_equal(back[0::2], data[0::2])
    assert np.array_equal(back & 0x8000, data & 0x8000)


@pytest.mark.parametrize("n", [1, 2, 4, 8, 16, 64, 512, 1024])
def test_group_sizes_and_ragged_tail(oracle, n):
    bits = stress_bits(3, 1000 + 7, seed=n)
    bits = bits[(bits & 0x7F80) != 0x7F80]  # NaN / Inf are outside what the reference defines
    norm, scaled = oracle.block_normalize(bits, n)
    assert norm.size == (bits.size + n - 1) // n
    sub = slice(0, 4096 + 3 if n > 8 else 1200)
    m_norm, m_scaled = _model_normalize(bits[sub], n)
    k = m_norm.size - (1 if (sub.stop % n and sub.stop < bits.size) else 0)  # last model group may be cut short
    assert np.array_equal(norm[:k], m_norm[:k])
    assert np.array_equal(scaled[: k * n][: sub.stop], m_scaled[: k * n][: sub.stop])
    # the byte is the mantissa of the group's largest magnitude
    for g in range(min(norm.size, 50)):
        grp = bits[g * n:(g + 1) * n]
        assert norm[g] == (int((grp & 0x7FFF).max()) & 0x7F) << 1
    # n == 1: every (normal) element is its own maximum -> its mantissa moves into the byte
    if n == 1:
        normal = (bits & 0x7F80) != 0
        assert np.all((scaled[normal] & 0x7F) == 0)
        assert np.array_equal(oracle.block_denormalize(scaled, 1, norm)[normal], bits[normal])


def test_power_of_two_maximum_is_the_plain_path(oracle):
    """A group whose largest magnitude is a power of two has base 1.0: byte 0,
    data unchanged, and the lossy reconstruction is the unnormalized one."""
    bits = bf16_bits_normal(4096, 3)
    bits = np.where((bits & 0x7FFF) > 0x3C00, np.uint16(0x3C00) | (bits & 0x8000), bits)  # clamp to 2^-7
    bits[::64] = 0x3C00
    norm, scaled = oracle.block_normalize(bits, 64)
    assert not norm.any() and np.array_equal(scaled, bits)
    for s in (7, 3, 1, 0):
        assert np.array_equal(oracle.reconstruct_normalized(bits, s, 64), closed_form_recon(bits, s))


@pytest.mark.parametrize("s", [3, 1, 0])
def test_normalized_reconstruction_composes(oracle, s):
    bits = bf16_bits_normal(5000, 9)
    for n in (8, 512):
        norm, scaled = oracle.block_normalize(bits, n)
        want = oracle.block_denormalize(closed_form_recon(scaled, s), n, norm)
        assert np.array_equal(oracle.reconstruct_normalized(bits, s, n), want)
        # scaling a whole group by a power of two only moves exponents
        shifted = (bits + np.uint16(3 << 7)).astype(np.uint16)
        assert np.array_equal(oracle.reconstruct_normalized(shifted, s, n),
                              (want + np.uint16(3 << 7)).astype(np.uint16))
