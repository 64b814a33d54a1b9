"""Independent pure-Python reader of the exponent container.

Written from the format description (header | directory | segment records,
64 lanes with two table-ANS states each, 12-bit frequencies, one private bit
stream per lane) without sharing code with the C oracle, so that the two pin
each other on small inputs: the coder tables come from the closed-form rank of
a state among the states of its symbol, where the oracle counts, and the bit
streams are read as one big integer.  Slow: use on a few thousand symbols at
most.
"""
from __future__ import annotations

import struct

import numpy as np

T = 4096
CARRY = 192


def _u32(b, off):
    return struct.unpack_from("<I", b, off)[0]


def parse_table(rec: bytes):
    """-> (freq[256], bytes used) or ('raw', 4)."""
    mode = rec[0]
    if mode == 0xFF:
        return "raw", 4
    live = []
    if 1 <= mode <= 15:
        head = 1 + 2 * mode
        for r in range(mode):
            start, ln = rec[1 + 2 * r], rec[2 + 2 * r] + 1
            live.extend(range(start, start + ln))
    elif mode == 0:
        head = 33
        for s in range(256):
            if (rec[1 + (s >> 3)] >> (s & 7)) & 1:
                live.append(s)
    else:
        raise ValueError("bad table mode")
    freq = [0] * 256
    bits = int.from_bytes(rec[head:head + (12 * len(live) + 7) // 8], "little")
    for i, s in enumerate(live):
        freq[s] = (bits >> (12 * i)) & 0xFFF
    assert sum(freq) == T
    used = (head + (12 * len(live) + 7) // 8 + 3) & ~3
    return freq, used


def state_rank(X: int, c: int, f: int) -> int:
    """Rank of state X among the states of the symbol that owns slots [c, c + f):
    the states Y < X whose slot (Y % 64) * 64 + Y // 64 lies in that range."""
    q, r = X >> 6, X & 63

    def below(m):  # slots i < m with i % 64 < q: states in the rows before X's
        return (m >> 6) * q + min(m & 63, q)

    same_row = r - min(r, (c + 63 - q) >> 6)  # states q * 64 + r', r' < r, on slots >= c
    return below(c + f) - below(c) + same_row


def decode_tables(freq):
    """-> per state X: (symbol, bits to read, next state before the bits)."""
    cum = np.concatenate([[0], np.cumsum(freq)])
    slot2sym = np.repeat(np.arange(256), freq)
    sym, nbits, base = [0] * T, [0] * T, [0] * T
    for X in range(T):
        slot = (X & 63) * 64 + (X >> 6)
        s = int(slot2sym[slot])
        xs = freq[s] + state_rank(X, int(cum[s]), freq[s])
        n = 12 - (xs.bit_length() - 1)
        sym[X], nbits[X], base[X] = s, n, (xs << n) - T
    return sym, nbits, base


def decode_container(comp: bytes, n: int):
    """-> (symbols uint8[n], carried uint8[192 * segments], meaningful for full segments)."""
    comp = bytes(comp)
    magic, version = _u32(comp, 0), _u32(comp, 4)
    assert magic == 0x315A4E41 and version == 5
    assert _u32(comp, 8) | (_u32(comp, 12) << 32) == n
    chunk, lane = _u32(comp, 16), _u32(comp, 20)
    seg = 64 * lane
    spc = -(-chunk // seg)  # the last segment of a chunk holds what remains
    n_segs = (n // chunk) * spc + -(-(n % chunk) // seg)
    assert _u32(comp, 28) == n_segs
    dir_off, rec_off = _u32(comp, 32), _u32(comp, 36)
    out = np.zeros(n, np.uint8)
    carried = np.zeros(CARRY * n_segs, np.uint8)
    table = None
    for k in range(n_segs):
        o0, o1 = _u32(comp, dir_off + 4 * k), _u32(comp, dir_off + 4 * (k + 1))
        rec = comp[rec_off + 4 * o0: rec_off + 4 * o1]
        cpos, kk = divmod(k, spc)
        start = cpos * chunk + kk * seg
        nominal = seg if kk + 1 < spc else chunk - (spc - 1) * seg
        sn = min(nominal, n - start)
        if k % spc == 0:
            table, used = parse_table(rec)
            rec = rec[used:]
            if table != "raw":
                sym, nbits, base = decode_tables(table)
        if table == "raw":
            out[start: start + sn] = np.frombuffer(rec[:sn], np.uint8)
            if sn == nominal:
                pad = (sn + 3) & ~3
                carried[CARRY * k: CARRY * (k + 1)] = np.frombuffer(rec[pad:pad + CARRY], np.uint8)
            continue
        # 64 x (state A | state B << 12), then minlen | w << 24 and 64 w-bit length fields
        states = int.from_bytes(rec[:192], "little")
        xa = [(states >> (24 * l)) & 0xFFF for l in range(64)]
        xb = [(states >> (24 * l + 12)) & 0xFFF for l in range(64)]
        hdr = _u32(rec, 192)
        minlen, w = hdr & 0xFFFFFF, hdr >> 24
        fields = int.from_bytes(rec[196:196 + 8 * w], "little")
        lens = [minlen + ((fields >> (l * w)) & ((1 << w) - 1)) for l in range(64)]
        body = rec[196 + 8 * w:]
        assert len(body) == ((sum(lens) + 7) // 8 + 3) & ~3
        stream = int.from_bytes(body, "little")
        assert stream >> sum(lens) == 0  # zero padding
        ends = np.cumsum(lens).tolist()
        q = list(ends)  # every lane reads its stream from the end downwards
        groups = (sn + 511) // 512
        for g in range(groups):
            for j in range(8):
                x = xb if j & 1 else xa
                for lane_i in range(64):
                    X = x[lane_i]
                    idx = (g * 64 + lane_i) * 8 + j
                    if idx < sn:
                        out[start + idx] = sym[X]
                    q[lane_i] -= nbits[X]
                    x[lane_i] = base[X] + ((stream >> q[lane_i]) & ((1 << nbits[X]) - 1))
        for lane_i in range(64):
            assert q[lane_i] == ends[lane_i] - lens[lane_i]  # every bit of the stream was read
            v = xa[lane_i] | (xb[lane_i] << 12)
            if sn == nominal:
                carried[CARRY * k + 3 * lane_i: CARRY * k + 3 * lane_i + 3] = [v & 0xFF, (v >> 8) & 0xFF, v >> 16]
            else:
                assert v == 0
    return out, carried
