#!/usr/bin/env python3
"""Writes tests/golden/hot_path_vectors.json from the exact models in exact_model.py.

    python tests/golden/make_golden.py

The reference ships no vectors for this path, and none of its code is run here: the expected
values come from rational arithmetic and from the published Philox4x32-10 known answers.
Inputs are drawn from Python's `random` with fixed seeds, so the file is reproducible.
"""
import json
import os
import random
import struct
import sys
from fractions import Fraction

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
from tests.golden import exact_model as em  # noqa: E402


def f32_bits(x: float) -> int:
    return struct.unpack("<I", struct.pack("<f", x))[0]


def bf16_bits(x: float) -> int:
    """float -> bf16 bits, round-to-nearest-even, via the exact model."""
    return em.bf16_bits_of_frac(em.bf16(Fraction(x)))


def main():
    rnd = random.Random(20240229)
    out = {"about": "exact-arithmetic vectors for the quantized-linear hot path; see make_golden.py"}

    # Random123 known-answer vectors for Philox4x32-10 (counter, key, output)
    out["philox_kat"] = [
        {"ctr": [0, 0, 0, 0], "key": [0, 0], "out": [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]},
        {"ctr": [0xFFFFFFFF] * 4, "key": [0xFFFFFFFF] * 2, "out": [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]},
        {"ctr": [0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344], "key": [0xA4093822, 0x299F31D0],
         "out": [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]},
    ]
    for k in out["philox_kat"]:
        assert em.philox4x32_10(k["ctr"], k["key"]) == k["out"]

    # uniform stream: 16-bit draws of the first 24 elements for two (seed, offset) pairs,
    # the second one crossing the 32-bit boundary of the counter
    out["uniform"] = []
    for seed, offset in [(7, 0), (0x0123456789ABCDEF, 2 ** 32 - 2)]:
        out["uniform"].append({"seed": seed, "offset": offset, "a16": [em.uniform_draw(i, seed, offset) for i in range(24)]})

    # dequant: (code, zero bits, scale bits) -> weight bits
    cases = []
    for _ in range(96):
        q = rnd.randrange(16)
        z = rnd.choice([6.0, 7.0, 8.0, 9.0, 0.0, 15.0, 7.5, 100.25, 0.30078125])
        s = abs(rnd.gauss(0, 0.02)) / 7 + 1e-6
        zb, sb = bf16_bits(z), bf16_bits(s)
        cases.append([q, zb, sb, em.bf16_bits_of_frac(em.dequant_model(q, zb, sb))])
    out["dequant"] = cases

    # requant: three groups of 128 elements (one row each, K = 128) per setting
    out["requant"] = []
    for lr, gstd, zvals, seed, offset in [(1e-4, 1e-3, [6.0, 7.0, 9.0], 7, 0),
                                          (1.0, 2e-3, [8.0, 7.5, 6.0], 99, 12345),
                                          (3e-2, 1.0, [9.0, 6.0, 0.30078125], 0xDEADBEEFCAFEF00D, 2 ** 32 - 16)]:
        N, K = 3, 128
        codes = [rnd.randrange(16) for _ in range(N * K)]
        sb = [bf16_bits(abs(rnd.gauss(0, 0.02)) / 7 + 1e-6) for _ in range(N)]
        zb = [bf16_bits(z) for z in zvals]
        gb = [bf16_bits(rnd.gauss(0, gstd)) for _ in range(N * K)]
        lrb = f32_bits(lr)
        a16 = [em.uniform_draw(i, seed, offset) for i in range(N * K)]
        new = [em.requant_model(codes[i], zb[i // K], sb[i // K], gb[i], lrb, a16[i]) for i in range(N * K)]
        out["requant"].append({"N": N, "K": K, "lr_bits": lrb, "seed": seed, "offset": offset, "codes": codes,
                               "scale_bits": sb, "zero_bits": zb, "grad_bits": gb, "a16": a16, "new_codes": new})

    # 4-bit residual codec: per companding curve (three_fold_curve_4bit, utils/quant.py:708-716) 96 bf16
    # inputs in [-0.5, 0.5] with nibble and carry from the exact transcription of quant_kernel_bf, and
    # the bf16 value of each of the 16 nibbles from dequant_kernel_bf (fused reading; the unfused one
    # gives the same results on every bf16 input, see tests/test_oracle_pins.py)
    curves = {0: (2, 0.125, 4, 0.25), 1: (2, 0.2666300266320331, 4, 0.375), 2: (2, 0.37272211741724515, 4, 0.4375),
              3: (2, 0.4330623539159437, 4, 0.46875)}
    out["residual_codec"] = []
    for mu, (p1, y1, p2, y2) in curves.items():
        k1, b1, k2, b2, k3 = p1, y1, p2 - p1, y2, 8 - p2
        cst = em.codec_constants(k1, b1, k2, b2, k3)
        xs = [bf16_bits(rnd.uniform(-0.5, 0.5)) for _ in range(88)] + [0x3F00, 0xBF00, 0, 0x8000, bf16_bits(b1), bf16_bits(-b1),
                                                                        bf16_bits(b2), bf16_bits(-b2)]
        nib, carry = [], []
        for b in xs:
            n, c = em.codec_nibble(em.codec_level(em.frac_of_bf16_bits(b), cst, True))
            nib.append(n)
            carry.append(c)
        values = [em.bf16_bits_of_frac(em.codec_value(n, cst, True)) for n in range(16)]
        out["residual_codec"].append({"mu": mu, "k1": k1, "b1": b1, "k2": k2, "b2": b2, "k3": k3, "x_bits": xs,
                                      "nibble": nib, "carry": carry, "value_bits": values})

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hot_path_vectors.json")
    with open(path, "w") as f:
        json.dump(out, f, separators=(",", ":"))
        f.write("\n")
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
