"""Generates the committed fixtures in this directory.  Run from the repository root:

    python tests/golden/make_golden.py

Everything here is computed with exact rational arithmetic (fractions.Fraction) from the closed form
of OCP e4m3fn and a hand-written round-to-nearest-even, independently of oracle/ and of the HIP code,
so the fixtures can pin both.  The reference repository ships no vectors of its own.

  e4m3fn_table.json       value of each of the 256 codes as an exact "numerator/denominator" string
  gemm_16x32x256.json     a 16 x 32 x 256 block-scaled GEMM with small-integer FP8 values and
                          power-of-two scales: every partial sum is exact in fp32, so the expected
                          fp32 result has no rounding freedom; expected bf16 bits are the RNE of it.
                          Arrays are stored in the reference's storage order: a[kk*M+i], b[kk*N+j],
                          a_scale[(kk/128)*M+i], b_scale[(kk/128)*NB+j/128].
"""
import json
import os
import random
import struct
from fractions import Fraction

HERE = os.path.dirname(os.path.abspath(__file__))


def e4m3fn_value(code: int):
    s, e, m = code >> 7, (code >> 3) & 15, code & 7
    if e == 15 and m == 7:
        return None
    v = Fraction(m, 512) if e == 0 else Fraction(2) ** (e - 7) * (1 + Fraction(m, 8))
    return -v if s else v


def bf16_rne_bits(x: Fraction) -> int:
    """bf16 bit pattern of an exactly-fp32-representable rational, round to nearest even."""
    f = float(x)
    assert Fraction(f) == x
    (u,) = struct.unpack("<I", struct.pack("<f", f))
    assert struct.unpack("<f", struct.pack("<I", u))[0] == f, "value must be exact in fp32"
    lsb = (u >> 16) & 1
    return ((u + 0x7FFF + lsb) >> 16) & 0xFFFF


def main():
    table = []
    for code in range(256):
        v = e4m3fn_value(code)
        table.append("nan" if v is None else "%d/%d" % (v.numerator, v.denominator))
    with open(os.path.join(HERE, "e4m3fn_table.json"), "w") as f:
        json.dump({"format": "OCP e4m3fn, exact value per code as numerator/denominator", "values": table}, f, indent=0)

    rnd = random.Random(20250)
    m, n, k = 16, 32, 256
    kb, nb = k // 128, (n + 127) // 128
    # codes whose values are the integers -4..4 and +-0.5 (all exact, products stay tiny)
    val2code = {}
    for code in range(256):
        v = e4m3fn_value(code)
        if v is not None and v in [Fraction(x, 2) for x in range(-8, 9)] and v not in val2code:
            val2code[v] = code
    vals = sorted(val2code)
    a = [val2code[rnd.choice(vals)] for _ in range(k * m)]          # a[kk*m + i]
    b = [val2code[rnd.choice(vals)] for _ in range(k * n)]          # b[kk*n + j]
    a_scale = [2.0 ** rnd.randint(-3, 2) for _ in range(kb * m)]    # as[kbi*m + i]
    b_scale = [2.0 ** rnd.randint(-2, 1) for _ in range(kb * nb)]   # bs[kbi*nb + j/128]
    exp_fp32, exp_bf16 = [], []
    for i in range(m):
        for j in range(n):
            acc = Fraction(0)
            for kk in range(k):
                av = e4m3fn_value(a[kk * m + i]) * Fraction(a_scale[(kk // 128) * m + i])
                bv = e4m3fn_value(b[kk * n + j]) * Fraction(b_scale[(kk // 128) * nb + j // 128])
                acc += av * bv
            exp_fp32.append(float(acc))
            exp_bf16.append(bf16_rne_bits(acc))
    with open(os.path.join(HERE, "gemm_16x32x256.json"), "w") as f:
        json.dump({"m": m, "n": n, "k": k, "a": a, "b": b, "a_scale": a_scale, "b_scale": b_scale,
                   "expected_fp32": exp_fp32, "expected_bf16_bits": exp_bf16}, f)
    print("wrote e4m3fn_table.json and gemm_16x32x256.json")


if __name__ == "__main__":
    main()
