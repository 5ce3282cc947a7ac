"""Writes the golden vectors in this directory.  Run from the repo root:  python tests/golden/make_golden.py

The expected values come from exact rational arithmetic with explicit IEEE roundings (tests/exact.py),
never from the CPU checker or the GPU kernels, so all three can be tested against them.  The reference
ships no vectors of its own (it has no tests), and nothing of the reference is imported or run here: the
formulas are read off triton_functions.py:207-216 (quantize), :483-490 (dequantize), :106-131 (GEMM).

Inputs are seeded (``random.Random``) and stored as bit patterns, so the files are reproducible.
"""
from __future__ import annotations

import json
import os
import random
import struct
import sys
from fractions import Fraction

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import exact  # noqa: E402


def f32_bits(x: float) -> int:
    return struct.unpack("<I", struct.pack("<f", x))[0]


def bits_f32(u: int) -> float:
    return struct.unpack("<f", struct.pack("<I", u))[0]


def fraction_to_f32_bits(fr: Fraction) -> int:
    """fr must be exactly representable in binary32."""
    u = f32_bits(float(fr))
    assert exact.f32_bits_to_fraction(u) == fr, fr
    return u if fr != 0 else 0


def rand_f32_bits(rng, emin=-20, emax=20, dtype="f32"):
    """random finite value with exponent in [emin, emax]; mantissa truncated to the dtype's width"""
    e = rng.randint(emin, emax) + 127
    m = rng.getrandbits(23)
    if dtype == "bf16":
        m &= ~0xFFFF
    elif dtype == "f16":
        m &= ~0x1FFF
    return (rng.getrandbits(1) << 31) | (e << 23) | m


def quant_case(name, bits, dtype, block):
    xs = [exact.f32_bits_to_fraction(u) for u in bits]
    codes, scales = [], []
    for k0 in range(0, len(xs), block):
        s, c = exact.quantize_block_exact(xs[k0:k0 + block])
        scales.append(fraction_to_f32_bits(s))
        codes.extend(c)
    return {"name": name, "dtype": dtype, "block": block, "x_bits": bits, "codes": codes, "scale_bits": scales}


def make_quantize():
    rng = random.Random(20240607)
    cases = []
    # hand-derivable: s = 2; 127*0.5 = 63.5 -> 64 (tie to even); 127*0.25 = 31.75 -> 32
    cases.append(quant_case("hand_half_even", [f32_bits(v) for v in (1.0, -2.0, 0.5, 0.0)], "f32", 4))
    # s = 254: 127*(x/254) is (nearly) x/2 -> a tie for every odd x; the two roundings decide
    cases.append(quant_case("ties_s254", [f32_bits(float(v)) for v in
                                          [254, 1, 3, 5, 7, 9, 11, 13, -1, -3, -5, 125, 127, 129, 251, 253]], "f32", 16))
    cases.append(quant_case("all_zero_block", [0] * 16 + [f32_bits(1.0)] * 16, "f32", 16))
    cases.append(quant_case("negative_zero", [0x80000000, 0, f32_bits(-3.0), f32_bits(1.5)], "f32", 4))
    cases.append(quant_case("ragged_tail", [rand_f32_bits(rng) for _ in range(16 + 5)], "f32", 16))
    # subnormal and near-maximum blocks: the quotient is still an ordinary number in [-1, 1]
    cases.append(quant_case("subnormal_block", [rng.getrandbits(22) | (rng.getrandbits(1) << 31) for _ in range(32)], "f32", 32))
    cases.append(quant_case("tiny_normal_block", [rand_f32_bits(rng, -126, -120) for _ in range(32)], "f32", 32))
    cases.append(quant_case("huge_block", [rand_f32_bits(rng, 120, 127) for _ in range(32)], "f32", 32))
    cases.append(quant_case("wide_range_block", [rand_f32_bits(rng, -126, 127) for _ in range(64)], "f32", 64))
    for dtype in ("f32", "bf16", "f16"):
        lo, hi = (-14, 15) if dtype == "f16" else (-8, 8)
        for block in (16, 32, 64, 128):
            n = 2 * block + (7 if block == 32 else 0)
            cases.append(quant_case(f"random_{dtype}_b{block}", [rand_f32_bits(rng, lo, hi, dtype) for _ in range(n)], dtype, block))
            # same exponent everywhere: codes spread over the whole [-127, 127] range
            cases.append(quant_case(f"flat_{dtype}_b{block}", [rand_f32_bits(rng, 0, 1, dtype) for _ in range(block)], dtype, block))
    return cases


def make_dequantize():
    rng = random.Random(77)
    inv127 = exact.float_to_fraction(bits_f32(f32_bits(1.0 / 127.0)))
    cases = []
    scale_bits = [f32_bits(2.0), f32_bits(1.0), f32_bits(127.0), f32_bits(0.0), 0x00000003, 0x7B000000]
    scale_bits += [rand_f32_bits(rng, -30, 30) for _ in range(26)]
    for sb in scale_bits:
        s = exact.f32_bits_to_fraction(sb)
        codes = [-127, -1, 0, 1, 127] + [rng.randint(-127, 127) for _ in range(11)]
        out32, outbf, outf16 = [], [], []
        for c in codes:
            v = exact.rn32(exact.rn32(s * c) * inv127)
            out32.append(float(v))                      # exact: every binary32 is a binary64
            outbf.append(float(exact.rn_bf16(v)))
            h = exact.rn_f16(v)
            outf16.append(float(h) if abs(h) < 65520 else None)
        # values, not bit patterns: the sign of a zero result is not pinned
        cases.append({"scale_bits": sb, "codes": codes, "out_f32": out32, "out_bf16": outbf, "out_f16": outf16})
    return cases


def make_gemm():
    """Tiny GEMMs evaluated exactly: int partials with Python ints, then the reference's fp32 sequence
    acc += sw * (sx * (float(P) * div)) with a rounding after every operation."""
    rng = random.Random(4242)
    div = exact.float_to_fraction(bits_f32(f32_bits(1.0 / (127.0 * 127.0))))
    cases = []
    for (M, N, K, block) in [(3, 4, 32, 16), (5, 3, 40, 16), (2, 2, 128, 128), (4, 6, 96, 32), (1, 7, 64, 64)]:
        A = [[rng.randint(-127, 127) for _ in range(K)] for _ in range(M)]
        W = [[rng.randint(-127, 127) for _ in range(K)] for _ in range(N)]
        nblk = -(-K // block)
        sa_bits = [[rand_f32_bits(rng, -6, 6) & 0x7FFFFFFF for _ in range(M)] for _ in range(nblk)]
        sw_bits = [[rand_f32_bits(rng, -10, 0) & 0x7FFFFFFF for _ in range(N)] for _ in range(nblk)]
        P = [[[sum(A[m][k] * W[n][k] for k in range(j * block, min(K, (j + 1) * block))) for n in range(N)]
              for m in range(M)] for j in range(nblk)]
        C = []
        for m in range(M):
            row = []
            for n in range(N):
                acc = Fraction(0)
                for j in range(nblk):
                    t0 = exact.rn32(Fraction(P[j][m][n]) * div)
                    t1 = exact.rn32(exact.f32_bits_to_fraction(sa_bits[j][m]) * t0)
                    t2 = exact.rn32(exact.f32_bits_to_fraction(sw_bits[j][n]) * t1)
                    acc = exact.rn32(acc + t2)
                row.append(float(acc))
            C.append(row)
        cases.append({"M": M, "N": N, "K": K, "block": block, "A": A, "W": W, "sa_bits": sa_bits, "sw_bits": sw_bits,
                      "P": P, "C_f32": C})
    return cases


def main():
    for name, fn in (("kat_quantize.json", make_quantize), ("kat_dequantize.json", make_dequantize), ("kat_gemm.json", make_gemm)):
        with open(os.path.join(HERE, name), "w") as f:
            json.dump(fn(), f, separators=(",", ":"))
        print("wrote", name, os.path.getsize(os.path.join(HERE, name)), "bytes")


if __name__ == "__main__":
    main()
