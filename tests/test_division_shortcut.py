"""Host logic of the division shortcut (born_amd/csrc/division.cpp), without a GPU.

The kernels that divide every logit by the temperature replace the correctly rounded division by
q = y * r, e = fma(-q, T, y), q' = fma(e, r, q) with r = RN(1 / T) when the library's host-side check says that this is
exact for the temperature. Checked here: the check's answers, and - in exact rational arithmetic, independent of the
C++ - that the sequence equals RN(y / T) at the edges of the magnitudes the kernels admit to it (2^-100 and 2^100).
"""
import ctypes
import os
import subprocess
from fractions import Fraction

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def shortcut(tmp_path_factory):
    d = tmp_path_factory.mktemp("division")
    wrapper = d / "wrapper.cpp"
    wrapper.write_text('namespace born { float division_shortcut_reciprocal(float T); }\n'
                       'extern "C" float reciprocal(float T) { return born::division_shortcut_reciprocal(T); }\n')
    so = d / "libdivision.so"
    subprocess.check_call(["g++", "-O3", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off",
                           os.path.join(ROOT, "born_amd", "csrc", "division.cpp"), str(wrapper), "-o", str(so)])
    lib = ctypes.CDLL(str(so))
    lib.reciprocal.restype = ctypes.c_float
    lib.reciprocal.argtypes = [ctypes.c_float]
    return lib.reciprocal


def rn32(x):
    """Fraction -> nearest float32 (ties to even), as a Fraction; |x| within the normal range or a denormal."""
    if x == 0:
        return Fraction(0)
    sign = -1 if x < 0 else 1
    x = abs(x)
    e = x.numerator.bit_length() - x.denominator.bit_length()
    if Fraction(2) ** e > x:
        e -= 1
    e = max(e, -126)                                  # denormals share the exponent of the smallest normal
    ulp = Fraction(2) ** (e - 23)
    n, rem = divmod(x, ulp)
    if rem * 2 > ulp or (rem * 2 == ulp and n % 2 == 1):
        n += 1
    return sign * n * ulp


def test_answers(shortcut):
    for T in (0.7, 0.8, 1.2, 1.5, 0.3, 1.3, 0.95):
        r = shortcut(T)
        assert r == np.float32(1.0) / np.float32(T), T          # the shortcut holds for these, and r = RN(1 / T)
        assert shortcut(T) == r                                   # (remembered)
    for T in (1.0, 0.0, -1.0, float("nan"), float("inf"), 1e-9, 3e6):
        assert shortcut(T) == 0.0, T                              # no division needed, or outside the admitted divisors
    assert shortcut(1.9999999) == 0.0                             # a residual that fp32 cannot hold: the kernels divide


@pytest.mark.parametrize("T", [0.7, 1.2, 0.8, 1.05])
def test_sequence_is_the_rounded_quotient_at_the_admitted_magnitudes(shortcut, T):
    r = Fraction(float(shortcut(T)))
    assert r != 0
    Tf = Fraction(float(np.float32(T)))
    rng = np.random.default_rng(int(T * 1000))
    for k in (-100, -99, -50, 0, 1, 60, 99):
        mant = np.concatenate([rng.integers(0, 1 << 23, 300), [0, 1, (1 << 23) - 1, 1 << 22]])
        for m in mant:
            for sign in (1, -1):
                y = sign * (Fraction(1) + Fraction(int(m), 1 << 23)) * Fraction(2) ** k
                q = rn32(y * r)
                e = rn32(y - q * Tf)                              # fma: one rounding of the exact value
                assert e == y - q * Tf                            # .. and the residual is representable (denormal at 2^-100)
                q2 = rn32(q + e * r)
                assert q2 == rn32(y / Tf), (T, k, int(m), sign)
