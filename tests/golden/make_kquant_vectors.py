"""Writes tests/golden/kquant_vectors.json: hand-built k-quant super-blocks whose decoded values
follow from the block layout by a closed-form expression (no decoder is run to make them).

The reference (Llama2.jl) ships no test vectors; these pin the decoders (oracle and GPU) against
the layout described in src/kquants.jl: field order and sizes (:7-35), the 6-bit scale/min
packing (:80-81,102-103), the nibble/bit-plane placement (:92-98, :213-217, :333-343).

    python tests/golden/make_kquant_vectors.py
"""
import json
import os
import struct

import numpy as np


def f16(v):
    return np.float16(v).tobytes()


def pack_scales(sc, m):
    """8 six-bit scales and mins -> 12 bytes (kquants.jl:80-81: bytes 0..3 hold sc[0..3] in the low
    6 bits, bytes 4..7 hold m[0..3]; :102-103: byte 8+k holds the low nibbles of sc[4+k] (low) and
    m[4+k] (high), their top 2 bits sit in bits 6..7 of byte k and of byte 4+k)."""
    b = [0] * 12
    for k in range(4):
        b[k] = sc[k] | ((sc[4 + k] >> 4) << 6)
        b[4 + k] = m[k] | ((m[4 + k] >> 4) << 6)
        b[8 + k] = (sc[4 + k] & 0xF) | ((m[4 + k] & 0xF) << 4)
    return bytes(b)


vectors = []

# --- q4_K A: d=1, dmin=0, sc_s = s+1, m=0; byte k of qs = (k%16) | ((15-k%16)<<4)
qs = bytes(((k % 16) | ((15 - k % 16) << 4)) for k in range(128))
raw = f16(1.0) + f16(0.0) + pack_scales([1, 2, 3, 4, 5, 6, 7, 8], [0] * 8) + qs
exp = np.zeros(256)
for j in range(4):
    for l in range(32):
        exp[64 * j + l] = (2 * j + 1) * (l % 16)            # low nibbles -> sub-block 2j
        exp[64 * j + 32 + l] = (2 * j + 2) * (15 - l % 16)  # high nibbles -> sub-block 2j+1
vectors.append(dict(name="q4_K ramp, scales 1..8", type=12, raw=raw.hex(), expected=exp.tolist()))

# --- q4_K B: top bits of the 6-bit fields: sc = [33]*4 + [63]*4, m = [21]*4 + [42]*4, d=.5, dmin=.25, q=7
sc, m = [33] * 4 + [63] * 4, [21] * 4 + [42] * 4
raw = f16(0.5) + f16(0.25) + pack_scales(sc, m) + bytes([0x77] * 128)
exp = np.repeat([0.5 * sc[s] * 7 - 0.25 * m[s] for s in range(8)], 32)
vectors.append(dict(name="q4_K six-bit fields", type=12, raw=raw.hex(), expected=exp.tolist()))

# --- q4_K C: every sub-block its own scale and min (all 6-bit values distinct)
sc, m = [1, 17, 34, 50, 9, 27, 44, 61], [63, 2, 35, 20, 58, 13, 40, 5]
raw = f16(0.125) + f16(2.0) + pack_scales(sc, m) + bytes([0x3C] * 128)  # low nibble 12, high nibble 3
exp = np.zeros(256)
for s in range(8):
    q = 12 if s % 2 == 0 else 3
    exp[32 * s:32 * s + 32] = 0.125 * sc[s] * q - 2.0 * m[s]
vectors.append(dict(name="q4_K distinct scales/mins", type=12, raw=raw.hex(), expected=exp.tolist()))

# --- q5_K: d=1, dmin=0, sc=1; qs=0; single high bits: bit s of qh[l] adds 16 to element 32*s + l
qh = [0] * 32
marks = [(0, 0), (3, 5), (31, 7), (16, 2), (9, 1)]
for l, s in marks:
    qh[l] |= 1 << s
raw = f16(1.0) + f16(0.0) + pack_scales([1] * 8, [0] * 8) + bytes(qh) + bytes(128)
exp = np.zeros(256)
for l, s in marks:
    exp[32 * s + l] = 16
vectors.append(dict(name="q5_K high-bit placement", type=13, raw=raw.hex(), expected=exp.tolist()))

# --- q5_K: nibbles + high bits + mins
sc, m = [2, 3, 4, 5, 6, 7, 8, 9], [1, 0, 3, 0, 5, 0, 7, 0]
qh = [0xFF if l % 2 == 0 else 0x00 for l in range(32)]     # every even l has all eight high bits set
raw = f16(0.25) + f16(0.5) + pack_scales(sc, m) + bytes(qh) + bytes([0xA5] * 128)  # low nibble 5, high 10
exp = np.zeros(256)
for s in range(8):
    for l in range(32):
        q = (5 if s % 2 == 0 else 10) + (16 if l % 2 == 0 else 0)
        exp[32 * s + l] = 0.25 * sc[s] * q - 0.5 * m[s]
vectors.append(dict(name="q5_K nibbles + bit plane + mins", type=13, raw=raw.hex(), expected=exp.tolist()))

# --- q6_K: ql bytes 0x21, qh bytes 0xE4 (bit pairs 0,1,2,3 from low to high), scales k+1, d=2
ql, qhb = bytes([0x21] * 128), bytes([0xE4] * 64)
scales = bytes(range(1, 17))
raw = ql + qhb + scales + f16(2.0)
exp = np.zeros(256)
qv = [(1 | (0 << 4)) - 32, (1 | (1 << 4)) - 32, (2 | (2 << 4)) - 32, (2 | (3 << 4)) - 32]  # -31, -15, 2, 18
for n in range(2):
    for g in range(4):
        for l in range(32):
            exp[128 * n + 32 * g + l] = 2.0 * (8 * n + l // 16 + 2 * g + 1) * qv[g]
vectors.append(dict(name="q6_K uniform bytes", type=14, raw=raw.hex(), expected=exp.tolist()))

# --- q6_K: negative scales, one distinct ql byte per position class
ql = bytearray(128)
for n in range(2):
    for l in range(64):
        ql[64 * n + l] = ((l % 16) | (((l + n) % 16) << 4))
qhb = bytes([0x1B] * 64)  # bit pairs 3,2,1,0 from low to high
scales = struct.pack("16b", *[(-1) ** k * (k + 3) for k in range(16)])
raw = bytes(ql) + qhb + scales + f16(-0.5)
exp = np.zeros(256)
hi = [3, 2, 1, 0]
for n in range(2):
    for l in range(32):
        lo_a, lo_b = ql[64 * n + l], ql[64 * n + l + 32]
        q = [(lo_a & 0xF) | (hi[0] << 4), (lo_b & 0xF) | (hi[1] << 4), (lo_a >> 4) | (hi[2] << 4), (lo_b >> 4) | (hi[3] << 4)]
        for g in range(4):
            k = 8 * n + l // 16 + 2 * g
            exp[128 * n + 32 * g + l] = -0.5 * ((-1) ** k * (k + 3)) * (q[g] - 32)
vectors.append(dict(name="q6_K negative scales", type=14, raw=raw.hex(), expected=exp.tolist()))

out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kquant_vectors.json")
with open(out, "w") as f:
    json.dump(vectors, f, indent=0)
print("wrote", out, len(vectors), "vectors")
