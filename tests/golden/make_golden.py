#!/usr/bin/env python3
"""Writes the known-answer fixtures of this directory.

Nothing here imports the CPU checker, the kernels or the reference: every expected value comes from a
restatement in plain Python integers / fractions of a rule the reference states in its own sources, so
that the checker (tests/test_golden.py) and the kernels (tests/test_gpu_golden.py) are both held
to data that neither of them produced.

  fp16_encode.json      bench/bench.ts:41-51, src/kernel.ts:16-32: truncating binary32 -> binary16
  q8_1_blocks.json      bench/bench.ts:53-72 packQ8_1: d = amax/127, Math.round (ties toward +inf), s = d*sum(q)
  legacy_dequant.json   tests/test_dequant.ts:13-24: byte = lo + 16*hi -> (lo - 8, hi - 8)
  q4k_block.json        144-byte super-block (ggml block_q4_K; the layout BASELINE.json names):
                        scales/mins, nibbles, w = d*sc*nib - dmin*m
  gemv_q4k_q8_1.json    bench/bench.ts:10-38 dot rule on the super-block: exact int32 sub-block dots and the row
                        value as an exact rational, rounded once to binary32
  argmax.json           prototypes/test_argmax.ts:33-44: sin(i)*10 with a spike; ties -> lowest index

Run:  python tests/golden/make_golden.py   (rewrites the .json files next to it)
"""
import json
import math
import os
import struct
from fractions import Fraction

HERE = os.path.dirname(os.path.abspath(__file__))


# ------------------------------------------------------------------ scalar rules, integers only
def f32_bits(x: float) -> int:
    return struct.unpack("<I", struct.pack("<f", x))[0]


def f32_from_bits(b: int) -> float:
    return struct.unpack("<f", struct.pack("<I", b))[0]


def encode_half_trunc(x: float) -> int:
    """bench/bench.ts:41-51: drop 13 mantissa bits, flush below the normal range to signed zero, overflow -> inf."""
    b = f32_bits(x)
    if b & 0x7FFFFFFF == 0:
        return 0
    s, e, m = (b >> 16) & 0x8000, (b >> 23) & 0xFF, b & 0x7FFFFF
    ne = e - 127 + 15
    if ne >= 31:
        return s | 0x7C00
    if ne <= 0:
        return s
    return s | (ne << 10) | (m >> 13)


def half_to_fraction(h: int) -> Fraction:
    s, e, m = h >> 15, (h >> 10) & 31, h & 1023
    v = Fraction(m, 1024) * Fraction(2) ** -14 if e == 0 else (1 + Fraction(m, 1024)) * Fraction(2) ** (e - 15)
    return -v if s else v


def js_round(x: float) -> int:
    """ECMAScript Math.round on a double: nearest integer, ties toward +infinity."""
    f = math.floor(x)
    return f + 1 if x - f >= 0.5 else f


def round_to_f32(fr: Fraction) -> int:
    """Bits of the binary32 nearest (ties to even) to an exact rational (normal range)."""
    if fr == 0:
        return 0
    sign = 0x80000000 if fr < 0 else 0
    a = abs(fr)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    assert Fraction(2) ** e <= a < Fraction(2) ** (e + 1) and -126 <= e <= 127
    scaled = a / Fraction(2) ** (e - 23)           # in [2^23, 2^24)
    n = scaled.numerator // scaled.denominator
    rem = scaled - n
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and n & 1):
        n += 1
    if n == 1 << 24:
        n >>= 1; e += 1
    return sign | ((e + 127) << 23) | (n - (1 << 23))


def pack_q8_1(xs):
    """One block of 32 values (python floats that are exact binary32). Returns (q[32], d_bits16, s_bits16)."""
    amax = max(abs(v) for v in xs)
    d = amax / 127.0                                    # double
    q = [js_round(v / (d if d != 0.0 else 1.0)) for v in xs]
    ssum = sum(q)
    qc = [max(-128, min(127, v)) for v in q]
    to_f32 = lambda v: struct.unpack("<f", struct.pack("<f", v))[0]
    return qc, encode_half_trunc(to_f32(d)), encode_half_trunc(to_f32(ssum * d))


class Lcg:
    """Tiny deterministic generator so that the fixtures do not depend on numpy's bit streams."""
    def __init__(self, seed): self.s = seed & 0xFFFFFFFFFFFFFFFF
    def next(self):
        self.s = (self.s * 6364136223846793005 + 1442695040888963407) & 0xFFFFFFFFFFFFFFFF
        return self.s >> 33
    def below(self, n): return self.next() % n
    def unit(self): return (self.next() % (1 << 24)) / float(1 << 24)
    def normalish(self):                                # sum of uniforms, rounded to binary32
        v = sum(self.unit() for _ in range(6)) - 3.0
        return struct.unpack("<f", struct.pack("<f", v))[0]


def pack_scales(sc, m):
    out = [0] * 12
    for j in range(4):
        out[j] = sc[j] | ((sc[j + 4] >> 4) << 6)
        out[j + 4] = m[j] | ((m[j + 4] >> 4) << 6)
        out[j + 8] = (sc[j + 4] & 15) | ((m[j + 4] & 15) << 4)
    return out


def q4k_block(d_bits, dmin_bits, sc, m, nibbles):
    """nibbles[256] in element order e = 64g + 32h + l -> 144 bytes."""
    qs = [0] * 128
    for e, nib in enumerate(nibbles):
        g, h, l = e // 64, (e // 32) & 1, e % 32
        qs[32 * g + l] |= nib << (4 * h)
    return list(struct.pack("<HH", d_bits, dmin_bits)) + pack_scales(sc, m) + qs


def dump(name, obj):
    with open(os.path.join(HERE, name), "w") as f:
        json.dump(obj, f, indent=1)
        f.write("\n")


def main():
    # ---- fp16 encode
    vals = [0.0, -0.0, 1.0, -1.0, 0.5, 1.0009765625, 1.00146484375, 65504.0, 65520.0, 1e5, -1e5, 6.103515625e-05,
            6.0e-05, 5.960464477539063e-08, 0.1, -0.3333333432674408, 3.14159274101257, 127.0 / 128.0, 2.0 ** -14, 2.0 ** -15]
    dump("fp16_encode.json", {"rule": "bench/bench.ts:41-51", "cases": [{"f32_bits": f32_bits(v), "half_bits": encode_half_trunc(f32_from_bits(f32_bits(v)))} for v in vals]})

    # ---- Q8_1 blocks: ties, a zero block, a random block, a block whose quotients sit on .5 boundaries
    g = Lcg(20260101)
    blocks = []
    ties = [127.0] + [k + 0.5 for k in range(-16, 15)]             # amax = 127 -> d = 1: x/d = k + 0.5 exactly
    blocks.append(ties)
    blocks.append([0.0] * 32)
    blocks.append([g.normalish() for _ in range(32)])
    blocks.append([-254.0] + [(k - 15) * 1.0 + 1.0 for k in range(31)])   # amax 254 -> d = 2: odd x -> .5 ties, negative side too
    blocks.append([g.normalish() * 1e-3 for _ in range(32)])
    out = []
    for xs in blocks:
        q, db, sb = pack_q8_1(xs)
        out.append({"x_f32_bits": [f32_bits(v) for v in xs], "q": q, "d_half_bits": db, "s_half_bits": sb})
    dump("q8_1_blocks.json", {"rule": "bench/bench.ts:53-72 (q[32] @0, fp16 d @32, fp16 s @34)", "blocks": out})

    # ---- legacy 20-byte block: byte j -> elements 2j (low nibble - 8), 2j + 1 (high nibble - 8)
    lb = []
    for _ in range(4):
        raw = [g.below(256) for _ in range(20)]
        exp = []
        for j in range(16):
            exp += [(raw[j] & 15) - 8, (raw[j] >> 4) - 8]
        lb.append({"block_bytes": raw, "int8": exp})
    dump("legacy_dequant.json", {"rule": "tests/test_dequant.ts:13-24 (q[16], fp16 d, fp16 dmin)", "blocks": lb})

    # ---- 144-byte super-block
    sc = [1, 63, 17, 32, 48, 5, 62, 33]
    m = [0, 21, 63, 16, 47, 58, 3, 36]
    nib = [(7 * e + e // 32) % 16 for e in range(256)]
    d_bits, dmin_bits = encode_half_trunc(0.0123), encode_half_trunc(0.0071)
    blk = q4k_block(d_bits, dmin_bits, sc, m, nib)
    d, dmin = half_to_fraction(d_bits), half_to_fraction(dmin_bits)
    w = [round_to_f32(d * sc[e // 32] * nib[e] - dmin * m[e // 32]) for e in range(256)]
    dump("q4k_block.json", {"rule": "ggml block_q4_K: fp16 d @0, fp16 dmin @2, scales[12] @4, qs[128] @16; w = d*sc*nib - dmin*m",
                            "block_bytes": blk, "scales": sc, "mins": m, "nibbles": nib,
                            "w_f32_bits_exact_rounded_once": w})

    # ---- Q4_K x Q8_1 GEMV, N = 6 rows, K = 512
    N, K = 6, 512
    x = [g.normalish() for _ in range(K)]
    xq = [pack_q8_1(x[32 * b: 32 * b + 32]) for b in range(K // 32)]
    xq_bytes = []
    for q, db, sb in xq:
        xq_bytes += [v & 0xFF for v in q] + list(struct.pack("<HH", db, sb))
    W_bytes, subdots, y_bits = [], [], []
    for n in range(N):
        acc = Fraction(0)
        row_dots = []
        for kb in range(K // 256):
            scn = [g.below(64) for _ in range(8)]; mn = [g.below(64) for _ in range(8)]
            nb_ = [g.below(16) for _ in range(256)]
            db_, mb_ = encode_half_trunc(0.002 + 0.02 * g.unit()), encode_half_trunc(0.002 + 0.02 * g.unit())
            W_bytes += q4k_block(db_, mb_, scn, mn, nb_)
            dd, dm = half_to_fraction(db_), half_to_fraction(mb_)
            for j in range(8):
                q8, d8b, s8b = xq[kb * 8 + j]
                I = sum(nb_[32 * j + l] * q8[l] for l in range(32))
                row_dots.append(I)
                acc += dd * half_to_fraction(d8b) * scn[j] * I - dm * half_to_fraction(s8b) * mn[j]
        subdots.append(row_dots)
        y_bits.append(round_to_f32(acc))
    dump("gemv_q4k_q8_1.json", {"rule": "y_n = sum_blk [ d*sum_j sc_j*(d8_j*I_j) - dmin*sum_j m_j*s8_j ], I_j exact int32 (bench/bench.ts:10-38 on the super-block)",
                                "N": N, "K": K, "W_bytes": W_bytes, "x_f32_bits": [f32_bits(v) for v in x], "xq_bytes": xq_bytes,
                                "subdots_int32": subdots, "y_f32_bits_exact_rounded_once": y_bits})

    # ---- argmax
    dump("argmax.json", {"rule": "prototypes/test_argmax.ts:33-44; prototypes/decode.ts:746-791 (strict '>', lowest index wins ties)",
                         "cases": [
                             {"V": 248320, "fill": "float32(sin(i) * 10)", "overrides": {"123456": 999.0}, "idx": 123456, "val_f32_bits": f32_bits(999.0)},
                             {"V": 248320, "fill": "zeros", "overrides": {"70000": 5.0, "4097": 5.0, "200000": 5.0}, "idx": 4097, "val_f32_bits": f32_bits(5.0)},
                             {"V": 5000, "fill": "zeros", "overrides": {}, "idx": 0, "val_f32_bits": 0},
                         ]})


if __name__ == "__main__":
    main()
