"""Independent pure-Python reader of the exponent container.

Written from the format description (header | directory | segment records,
64 interleaved rANS lanes, 12-bit frequencies, 16-bit renormalisation words)
without sharing code with the C oracle, so that the two pin each other on small
inputs.  Slow: use on a few thousand symbols at most.
"""
from __future__ import annotations

import struct

import numpy as np

M = 4096
L = 1 << 16


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
    assert sum(freq) == M
    used = (head + (12 * len(live) + 7) // 8 + 3) & ~3
    return freq, used


def decode_container(comp: bytes, n: int):
    """-> (symbols uint8[n], carried uint16[64 * full_segments])."""
    comp = bytes(comp)
    magic, version = _u32(comp, 0), _u32(comp, 4)
    assert magic == 0x315A4E41 and version == 4
    assert _u32(comp, 8) | (_u32(comp, 12) << 32) == n
    chunk, lane = _u32(comp, 16), _u32(comp, 20)
    seg = 64 * lane
    spc = -(-chunk // seg)  # the last segment of a chunk holds what remains
    n_segs = (n // chunk) * spc + -(-(n % chunk) // seg)
    assert _u32(comp, 28) == n_segs
    dir_off, rec_off = _u32(comp, 32), _u32(comp, 36)
    out = np.zeros(n, np.uint8)
    carried = np.zeros(64 * n_segs, np.uint16)
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
        if table == "raw":
            out[start: start + sn] = np.frombuffer(rec[:sn], np.uint8)
            if sn == nominal:
                pad = (sn + 3) & ~3
                carried[64 * k: 64 * k + 64] = np.frombuffer(rec[pad:pad + 128], "<u2")
            continue
        freq = table
        cum = np.concatenate([[0], np.cumsum(freq)])
        slot2sym = np.repeat(np.arange(256), freq)
        # 64 two-bit length codes, then the states as little-endian nibbles
        flags = int.from_bytes(rec[:16], "little")
        lens = [5 + ((flags >> (2 * l)) & 3) for l in range(64)]
        total = sum(lens)
        sbytes = ((total + 1) // 2 + 3) & ~3
        stream = int.from_bytes(rec[16:16 + sbytes], "little")
        x, at = [], 0
        for n_l in lens:
            x.append((stream >> (4 * at)) & ((1 << (4 * n_l)) - 1))
            at += n_l
        assert all(v >= L for v in x)
        words = np.frombuffer(rec[16 + sbytes:], "<u2")
        pos = 0
        groups = (sn + 511) // 512
        for g in range(groups):
            for j in range(8):
                for lane_i in range(64):
                    slot = x[lane_i] & (M - 1)
                    s = int(slot2sym[slot])
                    x[lane_i] = freq[s] * (x[lane_i] >> 12) + slot - int(cum[s])
                    idx = (g * 64 + lane_i) * 8 + j
                    if idx < sn:
                        out[start + idx] = s
                    if x[lane_i] < L:
                        x[lane_i] = (x[lane_i] << 16) | int(words[pos])
                        pos += 1
        assert pos <= len(words) and len(words) - pos <= 1
        for lane_i in range(64):
            assert x[lane_i] >> 16 == 1
            if sn == nominal:
                carried[64 * k + lane_i] = x[lane_i] & 0xFFFF
            else:
                assert x[lane_i] == L
    return out, carried
