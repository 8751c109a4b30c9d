"""Writes tests/golden/kquant.json from exact rational arithmetic.

Every fp32 operation of the K-quant -> field map (prover/kquant_cuda.py:42-111:
`(d*sc)*q - dmin*mn` for Q4_K/Q5_K, `(d*sc)*q` for Q6_K, each product and the
difference rounded to binary32, then round-half-even of the value times S) is
evaluated with `fractions.Fraction` and rounded to binary32 by an explicit
round-to-nearest-even routine, so the fixture depends on no floating-point
hardware, on no numpy, on the C oracle or on upstream code.

Blocks: seeded random blocks in the shape of the K-quant benchmark workload (scale/quant
bytes uniform, d and dmin = fp16(|N(0, 0.01)|)), plus hand-made blocks that hit
d = 0, fp16 subnormals, the largest fp16, exact-integer cases and exact .5 ties.

Run:  python tests/golden/make_kquant_fixtures.py
"""
import json
import os
import random
import struct
from fractions import Fraction

P = (1 << 64) - (1 << 32) + 1
HERE = os.path.dirname(os.path.abspath(__file__))
BB = {"Q4_K": 144, "Q5_K": 176, "Q6_K": 210}


def f16_to_frac(h):
    s = -1 if h & 0x8000 else 1
    e, m = (h >> 10) & 31, h & 1023
    assert e != 31
    if e == 0:
        return s * Fraction(m, 1 << 24)
    return s * Fraction(1024 + m, 1024) * Fraction(2) ** (e - 15)


def rne_f32(x):
    """Round a Fraction to the nearest binary32 (ties to even); returns a Fraction."""
    if x == 0:
        return Fraction(0)
    s, a = (-1, -x) if x < 0 else (1, x)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    e = max(e, -126)                    # subnormal range shares the 2^-149 grid
    ulp = Fraction(2) ** (e - 23)
    q, r = divmod(a, ulp)
    q = int(q)
    if r * 2 > ulp or (r * 2 == ulp and (q & 1)):
        q += 1
    res = q * ulp
    assert res < Fraction(2) ** 128
    return s * res


def rne_int(x):
    f = x.numerator // x.denominator
    r = x - f
    if r * 2 > 1 or (r * 2 == 1 and (f & 1)):
        f += 1
    return f


def scale_min(s12, s):
    if s < 4:
        return s12[s] & 0x3F, s12[s + 4] & 0x3F
    j = s - 4
    return ((s12[8 + j] & 0x0F) | ((s12[j] >> 2) & 0x30),
            (s12[8 + j] >> 4) | ((s12[j + 4] >> 2) & 0x30))


def decode_block(qtype, p, S):
    out = []
    for e in range(256):
        if qtype == "Q6_K":
            ql, qh, sc = p[0:128], p[128:192], p[192:208]
            d = f16_to_frac(p[208] | (p[209] << 8))
            lo = (ql[(e >> 7) * 64 + (e & 63)] >> (4 * ((e >> 6) & 1))) & 0xF
            hi = (qh[(e >> 7) * 32 + (e & 31)] >> (2 * ((e >> 5) & 3))) & 3
            q = lo | (hi << 4)
            q = (q - 256 if q > 127 else q) - 32
            s = sc[e >> 4]
            s = s - 256 if s > 127 else s
            v = rne_f32(rne_f32(d * s) * q)
        else:
            d = f16_to_frac(p[0] | (p[1] << 8))
            dmin = f16_to_frac(p[2] | (p[3] << 8))
            sc, mn = scale_min(p[4:16], e >> 5)
            qs = p[16:144] if qtype == "Q4_K" else p[48:176]
            q = (qs[(e >> 6) * 32 + (e & 31)] >> (4 * ((e >> 5) & 1))) & 0xF
            if qtype == "Q5_K":
                q |= ((p[16 + (e & 31)] >> (e >> 5)) & 1) << 4
            v = rne_f32(rne_f32(rne_f32(d * sc) * q) - rne_f32(dmin * mn))
        x = rne_int(v * S)              # S is a power of two here: double(v)*S is exact
        out.append(x % P)
    return out


def f16_bits(x):
    return struct.unpack("<H", struct.pack("<e", x))[0]


def make_block(qtype, rng, d_bits=None, dmin_bits=None):
    b = bytearray(rng.randrange(256) for _ in range(BB[qtype]))
    d = f16_bits(abs(rng.gauss(0, 0.01))) if d_bits is None else d_bits
    dm = f16_bits(abs(rng.gauss(0, 0.01))) if dmin_bits is None else dmin_bits
    if qtype == "Q6_K":
        b[208], b[209] = d & 255, d >> 8
    else:
        b[0], b[1], b[2], b[3] = d & 255, d >> 8, dm & 255, dm >> 8
    return bytes(b)


def main():
    S = 1 << 12
    out = []
    for qtype in ("Q4_K", "Q5_K", "Q6_K"):
        rng = random.Random({"Q4_K": 4, "Q5_K": 5, "Q6_K": 6}[qtype])
        blocks = [make_block(qtype, rng) for _ in range(4)]
        specials = [(0x0000, 0x0000), (0x0001, 0x03FF), (0x7BFF, 0x7BFF), (0x3C00, 0x0000),
                    (0x0A00, 0x0A00),      # 2^-13: with S = 2^12 every odd multiple is a .5 tie
                    (0x0000, 0x0A00), (0x8A00, 0x3800)]
        for d_bits, dm_bits in specials:
            blocks.append(make_block(qtype, rng, d_bits, dm_bits))
        raw = b"".join(blocks)
        vals = []
        for i in range(len(blocks)):
            vals.extend(decode_block(qtype, raw[i * BB[qtype]:(i + 1) * BB[qtype]], S))
        out.append({"qtype": qtype, "S": S, "raw": raw.hex(),
                    "field": [format(v, "016x") for v in vals]})
    json.dump(out, open(os.path.join(HERE, "kquant.json"), "w"))
    print("kquant fixture written")


if __name__ == "__main__":
    main()
