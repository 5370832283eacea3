"""Exact models of the hot path's arithmetic, independent of the C oracle and of the kernels.

Everything here is integer / rational arithmetic (fractions.Fraction) with an explicit
round-to-nearest-even, plus a pure-Python Philox4x32-10 transcribed from the published
Random123 description (multipliers 0xD2511F53 / 0xCD9E8D57, Weyl constants 0x9E3779B9 /
0xBB67AE85). It is the source of the committed vectors in this directory and is only fit
for small cases (it runs at a few thousand elements per second).

Formulas modelled:
  dequant  w = bf16(bf16(q - z) * s)                       (utils/quant.py:66-72)
  requant  t = fma(-lr, g, w); r16 = fl(fl(1/s) * 2^16); c16 = fl(z * 2^16 + 1/2); y = fl(t * r16 + c16);
           X = trunc(max(y, 0)) saturated at 2^32 - 1; S = min(X + a, 2^32 - 1); code' = min(S >> 16, 15)
           every fl() one rounding to fp32, NaN- and overflow-free inputs only
  residual codec (utils/cuda_src/multi_random_quant_kernel.cu:46-62, 157-166, host constants :346-351, :385-390):
           level = round(x*c1 + v) etc. with v = S*499 - round(S*499), C round (half away from zero), in two
           readings of the source: a*b + c contracted into one fused multiply-add (what nvcc does by
           default) and not contracted
  draw     a_i = 16-bit half (i & 1) of word (i >> 1) & 3 of Philox(counter = offset + i // 8, key = seed);
           the uniform it stands for is u_i = (a_i + 1/2) * 2^-16
"""
import struct
from fractions import Fraction


def rn(x: Fraction, mant_bits: int, emin: int = -126) -> Fraction:
    """Round an exact rational to a binary float with `mant_bits` significand bits (incl. the
    hidden one), round-to-nearest-even, gradual underflow below 2^emin."""
    if x == 0:
        return Fraction(0)
    sign = -1 if x < 0 else 1
    a = abs(x)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    if Fraction(2) ** (e + 1) <= a:
        e += 1
    e = max(e, emin)
    quantum = Fraction(2) ** (e - (mant_bits - 1))
    n = a / quantum
    fl = n.numerator // n.denominator
    rem = n - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
        fl += 1
    return sign * fl * quantum


def f32(x):
    return rn(x, 24)


def bf16(x):
    return rn(x, 8)


def frac_of_bf16_bits(b: int) -> Fraction:
    return Fraction(struct.unpack("<f", struct.pack("<I", (b & 0xFFFF) << 16))[0])


def frac_of_f32_bits(b: int) -> Fraction:
    return Fraction(struct.unpack("<f", struct.pack("<I", b & 0xFFFFFFFF))[0])


def bf16_bits_of_frac(x: Fraction) -> int:
    """Bits of a rational that is exactly representable in bf16."""
    b = struct.unpack("<I", struct.pack("<f", float(x)))[0]
    assert b & 0xFFFF == 0
    return b >> 16


def dequant_model(q: int, zb: int, sb: int) -> Fraction:
    z, s = frac_of_bf16_bits(zb), frac_of_bf16_bits(sb)
    return bf16(f32(bf16(f32(q - z)) * s))


def requant_model(q: int, zb: int, sb: int, gb: int, lr_bits: int, a: int) -> int:
    """New code of one element for the 16-bit draw a."""
    z, s, g = frac_of_bf16_bits(zb), frac_of_bf16_bits(sb), frac_of_bf16_bits(gb)
    w = dequant_model(q, zb, sb)
    t = f32(w - frac_of_f32_bits(lr_bits) * g)  # one rounding: fused multiply-add
    r16 = f32(f32(1 / s) * 65536)
    c16 = f32(z * 65536 + Fraction(1, 2))
    y = f32(t * r16 + c16)
    x = min(max(y.numerator // y.denominator, 0), 2 ** 32 - 1)  # floor == trunc for y >= 0
    big = min(x + a, 2 ** 32 - 1)
    return min(big >> 16, 15)


def draw_of_uniform(u: Fraction) -> int:
    """16-bit draw taken from an injected uniform in [0, 1): floor(fl(u * 2^16)), at most 65535."""
    v = f32(u * 65536)
    return min(max(v.numerator // v.denominator, 0), 65535)


def philox4x32_10(ctr, key):
    c0, c1, c2, c3 = ctr
    k0, k1 = key
    for _ in range(10):
        p0 = 0xD2511F53 * c0
        p1 = 0xCD9E8D57 * c2
        c0, c1, c2, c3 = ((p1 >> 32) ^ c1 ^ k0) & 0xFFFFFFFF, p1 & 0xFFFFFFFF, ((p0 >> 32) ^ c3 ^ k1) & 0xFFFFFFFF, p0 & 0xFFFFFFFF
        k0 = (k0 + 0x9E3779B9) & 0xFFFFFFFF
        k1 = (k1 + 0xBB67AE85) & 0xFFFFFFFF
    return [c0, c1, c2, c3]


def uniform_draw(i: int, seed: int, offset: int) -> int:
    """16-bit integer a of element i; the uniform it stands for is (a + 1/2) * 2^-16."""
    c = (offset + i // 8) & 0xFFFFFFFFFFFFFFFF
    w = philox4x32_10([c & 0xFFFFFFFF, c >> 32, 0, 0], [seed & 0xFFFFFFFF, seed >> 32])
    return (w[(i >> 1) & 3] >> (16 * (i & 1))) & 0xFFFF


# ------------------------------------------------------------------ 4-bit residual codec -----
def cround(x: Fraction) -> int:
    """C round(): to nearest, halves away from zero."""
    n = (abs(x) + Fraction(1, 2)).__floor__()
    return -n if x < 0 else n


def codec_constants(k1: int, b1: float, k2: int, b2: float, k3: int):
    """Host-side constants of launch_quant / launch_dequant (:346-351, :385-390): b1, b2 arrive as
    C floats; c1, c2, ic1, ic2 are float expressions, c3 and ic3 go through double (the literal 0.5)."""
    fb1, fb2 = f32(Fraction(b1)), f32(Fraction(b2))
    d21 = f32(fb2 - fb1)
    half_b2 = rn(Fraction(1, 2) - fb2, 53, -1022)
    return {"b1": fb1, "b2": fb2, "t1": k1, "t2": k1 + k2,
            "c1": f32(k1 / fb1), "c2": f32(k2 / d21), "c3": f32(rn(k3 / half_b2, 53, -1022)),
            "ic1": f32(fb1 / k1), "ic2": f32(d21 / k2), "ic3": f32(rn(half_b2 / k3, 53, -1022))}


def _mad(a: Fraction, b: Fraction, c: Fraction, fused: bool) -> Fraction:
    return f32(a * b + c) if fused else f32(f32(a * b) + c)


def codec_level(x: Fraction, cst: dict, fused: bool) -> int:
    """The signed level of quant_kernel_bf (:46-60) for a bf16 input x, v0 = 0."""
    S = abs(x)
    v = f32(S * 499)
    v = v - cround(v)  # exact: |v - round(v)| <= 1/2 has no more bits than v
    if S < cst["b1"]:
        return cround(_mad(x, cst["c1"], v, fused))
    if S < cst["b2"]:
        r = cround(_mad(f32(S - cst["b1"]), cst["c2"], v, fused)) + cst["t1"]
    else:
        r = cround(_mad(f32(S - cst["b2"]), cst["c3"], v, fused)) + cst["t2"]
    return -r if x < 0 else r


def codec_nibble(level: int):
    """(:61) a level above 7 wraps to nibble 1 with a carry; a level below -8 converts to unsigned 0."""
    if level > 7:
        return 1, 1
    return max(level + 8, 0) & 0xF, 0


def codec_value(nibble: int, cst: dict, fused: bool) -> Fraction:
    """dequant_kernel_bf (:157-166) for one nibble, rounded to bf16 as its store does."""
    s = nibble - 8
    t1, t2 = cst["t1"], cst["t2"]
    if s < -t2:
        v = _mad(Fraction(s + t2), cst["ic3"], -cst["b2"], fused)
    elif s < -t1:
        v = _mad(Fraction(s + t1), cst["ic2"], -cst["b1"], fused)
    elif s <= t1:
        v = f32(s * cst["ic1"])
    elif s <= t2:
        v = _mad(Fraction(s - t1), cst["ic2"], cst["b1"], fused)
    else:
        v = _mad(Fraction(s - t2), cst["ic3"], cst["b2"], fused)
    return bf16(v)
