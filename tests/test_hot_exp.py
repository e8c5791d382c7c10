"""The tabulated double-precision exponential of the triplet-reduce kernels (csrc/staf_tri.hpp, HotExp<double>::eval
with a table): its constants are read from the source and checked against what the mathematics fixes -- the table
is 2^(i/128) correctly rounded, the high part of ln2/128 has 32 significant bits (so its product with the integer part
is exact), high + low parts are ln2/128 -- and the function, re-evaluated here with exact fused multiply-adds, stays
within 4e-16 of exp(x) over the range the kernels use.  The kernels themselves are compared with the oracle on the GPU."""
import math
import os
import re
import struct
from decimal import Decimal, getcontext
from fractions import Fraction

import numpy as np

SRC = os.path.join(os.path.dirname(__file__), "..", "alphanesgpu_amd", "csrc", "staf_tri.hpp")
getcontext().prec = 60


def source_constants():
    s = open(SRC).read()
    tab = re.search(r"exp2_frac_128\[128\] = \{(.*?)\};", s, re.S).group(1)
    table = [float(x) for x in tab.replace("\n", " ").split(",") if x.strip()]
    body = s[s.index("__device__ static double eval(double x, const double* tab)"):]
    inv = float(re.search(r"rint\(x \* ([0-9.eE+-]+)\)", body).group(1))
    hi = float(re.search(r"fma\(t, -([0-9.eE+-]+), x\)", body).group(1))
    lo = float(re.search(r"fma\(t, -([0-9.eE+-]+), r\)", body).group(1))
    return table, inv, hi, lo


def fma(a, b, c):
    """Correctly rounded a*b + c."""
    v = Fraction(a) * Fraction(b) + Fraction(c)
    return v.numerator / v.denominator   # int / int division is correctly rounded in Python


def test_table_is_two_to_the_i_over_128_correctly_rounded():
    table, _, _, _ = source_constants()
    assert len(table) == 128
    for i, v in enumerate(table):
        assert v == float(Decimal(2) ** (Decimal(i) / Decimal(128))), i


def test_reduction_constants():
    _, inv, hi, lo = source_constants()
    c = Decimal(2).ln() / 128
    assert inv == float(1 / c)
    bits = struct.unpack("<Q", struct.pack("<d", hi))[0]
    assert bits & ((1 << 21) - 1) == 0          # 32 significant bits: exact products with |t| < 2^21
    assert abs(Decimal(hi) + Decimal(lo) - c) / c < Decimal(10) ** -25   # the low part is itself a rounded double


def test_reevaluated_function_against_exp():
    table, inv, hi, lo = source_constants()
    rng = np.random.Generator(np.random.Philox(5))
    xs = np.concatenate([rng.uniform(-60, 60, 3000), rng.uniform(-2, 2, 1000), [0.0, 1e-300, -1e-300, 700.0, -700.0]])
    worst = 0.0
    for x in xs:
        x = float(x)
        t = float(np.rint(x * inv))
        r = fma(t, -hi, x)
        r = fma(t, -lo, r)
        i = int(t)
        p = fma(r, 8.33333333333333333333e-03, 4.16666666666666666667e-02)
        p = fma(p, r, 1.66666666666666666667e-01)
        p = fma(p, r, 0.5)
        p = fma(p, r, 1.0)
        p = fma(p, r, 1.0)
        got = math.ldexp(table[i & 127] * p, i >> 7)
        want = Decimal(x).exp()
        worst = max(worst, float(abs((Decimal(got) - want) / want)))
    assert worst < 4e-16, worst
