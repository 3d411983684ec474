"""Writes the committed golden fixtures of tests/golden/.

mxfp4_table.npy   bf16 bit pattern of every (e2m1 code, e8m0 scale byte) pair, [16, 256] uint16,
                  computed with exact rational arithmetic (fractions.Fraction) from the definition
                  value = LUT[code] * 2^(scale-127) rounded to bf16 (round-to-nearest-even, overflow
                  to infinity), independent of the C oracle and of any floating-point library.
                  Scale byte 255 stands for 2^128 = +inf in fp32: non-zero codes give +-inf, zero
                  codes NaN (stored as 0x7FC0).
tiny_block.npz    inputs and outputs of the CPU oracle for one tiny MoE block (regression anchor for
                  the oracle itself; the oracle is pinned independently by tests/test_oracle_pins.py).

Run from the repo root:  python tests/golden/make_golden.py
"""
import os
import sys
from fractions import Fraction

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

LUT = [Fraction(0), Fraction(1, 2), Fraction(1), Fraction(3, 2), Fraction(2), Fraction(3), Fraction(4), Fraction(6)]


def bf16_bits_exact(value: Fraction, negative: bool) -> int:
    """Round a non-negative rational to bf16 (RNE, subnormals kept, overflow to inf)."""
    sign = 0x8000 if negative else 0
    if value == 0:
        return sign
    # find e with 2^e <= value < 2^(e+1)
    e = 0
    while Fraction(2) ** e > value:
        e -= 1
    while Fraction(2) ** (e + 1) <= value:
        e += 1
    e_eff = max(e, -126)                 # subnormals share the exponent of the smallest normal
    unit = Fraction(2) ** (e_eff - 7)    # value of one mantissa ulp
    q = value / unit                     # exact
    n = q.numerator // q.denominator
    rem = q - n
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and (n & 1)):
        n += 1
    if e >= -126:
        bits = ((e + 127) << 7) + (n - 128)  # 128 <= n <= 256; n == 256 carries into the exponent
    else:
        bits = n                              # subnormal: n ulps of 2^-133 (n == 128 is the first normal)
    if bits >= 0x7F80:
        bits = 0x7F80
    return sign | bits


def mxfp4_table():
    t = np.zeros((16, 256), dtype=np.uint16)
    for code in range(16):
        neg = bool(code & 8)
        mag = LUT[code & 7]
        for s in range(256):
            if s == 255:
                t[code, s] = 0x7FC0 if mag == 0 else ((0x8000 if neg else 0) | 0x7F80)
                continue
            # fp32 product first: LUT * 2^(s-127) is exact in fp32 unless it overflows (-> inf)
            v = mag * Fraction(2) ** (s - 127)
            if v >= Fraction(2) ** 128:
                t[code, s] = (0x8000 if neg else 0) | 0x7F80
            else:
                t[code, s] = bf16_bits_exact(v, neg)
    return t


def tiny_block():
    import __graft_entry__ as ge
    oracle = ge.import_oracle()
    rng = np.random.default_rng(1234)
    T, H, I, E, K = 5, 64, 64, 4, 2

    def bf(a):  # bf16-representable fp32
        return oracle.bf16_to_f32(oracle.f32_to_bf16(a.astype(np.float32)))

    d = dict(
        t=rng.standard_normal((T, H)).astype(np.float32),
        w_router=bf(rng.standard_normal((E, H)) * 0.1), b_router=bf(rng.standard_normal(E) * 0.1),
        w_mlp1=bf(rng.standard_normal((E, 2 * I, H)) * 0.1), b_mlp1=bf(rng.standard_normal((E, 2 * I)) * 0.1),
        w_mlp2=bf(rng.standard_normal((E, H, I)) * 0.1), b_mlp2=bf(rng.standard_normal((E, H)) * 0.1))
    y, ti, tv, sc = oracle.moe_block(d["t"], d["w_router"], d["b_router"], d["w_mlp1"], d["b_mlp1"], d["w_mlp2"],
                                     d["b_mlp2"], K, want_scores=True)
    d.update(e_agg=y, topk_i=ti, topk_v=tv, router_score=sc, K=np.int32(K))
    return d


if __name__ == "__main__":
    np.save(os.path.join(HERE, "mxfp4_table.npy"), mxfp4_table())
    np.savez(os.path.join(HERE, "tiny_block.npz"), **tiny_block())
    print("wrote", os.listdir(HERE))
