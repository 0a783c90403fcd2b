"""Writes tests/golden/q8_0_kat.json: hand-derived known answers for the Q8_0
quantiser of the reference (quantize_row_q8, src/nn/wmat.c:19-44) and for the
F16 rounding of wmat_create_f16 (src/nn/wmat.c:63-75).

Nothing here calls the oracle or the reference.  Every expected byte follows
from exact arithmetic on inputs chosen so that each fp32 operation of the
algorithm is exact (powers of two, small integers), plus the two rounding
rules the algorithm names: roundf = halves away from zero for the int8 codes,
IEEE round-to-nearest-even for the fp16 scale.

Run:  python tests/golden/make_q8_kat.py
"""
import json
import os
import struct
from fractions import Fraction


def f32_bits(x):
    """Bits of a value that must be exactly representable in fp32."""
    b = struct.unpack("<I", struct.pack("<f", float(x)))[0]
    assert Fraction(struct.unpack("<f", struct.pack("<I", b))[0]) == Fraction(x), x
    return b


def round_half_away(fr):
    n = int(abs(fr) + Fraction(1, 2))          # floor(|x| + 1/2)
    return n if fr >= 0 else -n


def i8(v):
    return v & 0xFF


cases = []


def add(name, values, scale_bits, codes):
    assert len(values) == 32 and len(codes) == 32
    cases.append({"name": name, "x_bits": [f32_bits(v) for v in values],
                  "bytes": [scale_bits & 0xFF, scale_bits >> 8] + [i8(c) for c in codes]})


# 1. all-zero block: scale 0, codes 0 (the `scale != 0` branch)
add("zero", [Fraction(0)] * 32, 0x0000, [0] * 32)

# 2. amax = 127 * 2^-10  =>  scale = 2^-10 exactly (fp16 0x1400), inv = 2^10 exactly.
#    x = (k + f) * 2^-10 exercises ties (away from zero) and ordinary rounding.
s = Fraction(1, 1024)
ks = [127, -127, 0, 1, -1, 2, -2, 3, 63, -63, 64, -64, 100, -100, 126, -126]
fr = [Fraction(1, 2), Fraction(-1, 2), Fraction(1, 4), Fraction(-1, 4), Fraction(3, 4), Fraction(-3, 4),
      Fraction(5, 2), Fraction(-5, 2), Fraction(7, 2), Fraction(-7, 2), Fraction(125, 2), Fraction(-125, 2),
      Fraction(1, 8), Fraction(-1, 8), Fraction(253, 2), Fraction(-253, 2)]
vals = [k * s for k in ks] + [f * s for f in fr]
add("pow2_scale_ties", vals, 0x1400, [round_half_away(v / s) for v in vals])

# 3. +-127 saturating block: every element at +-amax, amax = 127  => scale 1.0 (0x3C00)
vals = [Fraction(127 if j % 2 == 0 else -127) for j in range(32)]
add("plus_minus_amax", vals, 0x3C00, [127 if j % 2 == 0 else -127 for j in range(32)])

# 4. fp16 tie for the stored scale, ties-to-even DOWN: amax = 127*(1+2^-11): scale = 1+2^-11
#    is exact in fp32 and lies half-way between fp16 1.0 and 1+2^-10 -> 1.0 (0x3C00).
#    Codes use the UN-rounded scale: x = k*(1+2^-11) -> exactly k (inv is not exact here, so
#    only k whose product stays well inside (k-1/2, k+1/2) are used: all are).
sc = 1 + Fraction(1, 2048)
ks = [127, -127] + list(range(-15, 15))
add("scale_tie_even_down", [k * sc for k in ks], 0x3C00, ks)

# 5. ties-to-even UP: scale = 1+3*2^-11 lies half-way between 0x3C01 and 0x3C02 -> 0x3C02.
sc = 1 + Fraction(3, 2048)
add("scale_tie_even_up", [k * sc for k in ks], 0x3C02, ks)

# 6. negative amax element decides the scale; small magnitudes round to 0
s = Fraction(1, 4)
vals = [Fraction(-127, 4)] + [Fraction(j, 64) for j in range(-15, 16)]      # |x/s| < 1
add("neg_amax_small_values", vals, 0x3400, [-127] + [round_half_away(v / s) for v in vals[1:]])

# --- F16 rounding known answers: (fp32 bits, fp16 bits) ---
f16 = [
    (0x00000000, 0x0000), (0x80000000, 0x8000),
    (0x3F800000, 0x3C00),                      # 1.0
    (0x3F801000, 0x3C00),                      # 1 + 2^-11: tie -> even (down)
    (0x3F803000, 0x3C02),                      # 1 + 3*2^-11: tie -> even (up)
    (0x3F801001, 0x3C01),                      # just above the tie
    (0x477FE000, 0x7BFF),                      # 65504 = max half
    (0x477FEFFF, 0x7BFF),                      # below 65520 stays max
    (0x477FF000, 0x7C00),                      # 65520: tie -> even = inf
    (0x7F800000, 0x7C00), (0xFF800000, 0xFC00),
    (0x38800000, 0x0400),                      # 2^-14 smallest normal
    (0x387FC000, 0x03FF),                      # largest subnormal, exact
    (0x387FE000, 0x0400),                      # tie between 0x3FF and 0x400 -> even 0x400
    (0x33800000, 0x0001),                      # 2^-24 smallest subnormal
    (0x33000000, 0x0000),                      # 2^-25: tie -> even = 0
    (0x33000001, 0x0001),                      # just above 2^-25
    (0x33C00000, 0x0002),                      # 1.5 * 2^-24: tie -> even = 2
    (0x3CA3D70A, 0x251F),                      # 0.02 -> 0.0200043 (nearest)
    (0xBE4CCCCD, 0xB266),                      # -0.2
]

out = {"q8_blocks": cases, "f16": [{"f32_bits": a, "f16_bits": b} for a, b in f16]}
path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "q8_0_kat.json")
with open(path, "w") as fh:
    json.dump(out, fh, indent=1)
print("wrote", path, len(cases), "blocks,", len(f16), "f16 cases")
