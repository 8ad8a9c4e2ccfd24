"""An independent statement of `fastapprox::faster::erf` (crate fastapprox 0.3.1, called at
crates/session_interpreter/src/session.rs:929) for the tests: what the crate's bit trick
*means*, written without the trick.

`faster::pow2(p)` stores `2^23 * (max(p, -126) + OFFSET)` in the bits of a float.  Read as a
float, an integer I in the exponent field and a fraction f in the significand are the number
`2^(I-127) * (1 + f)`: the piecewise-linear interpolant of `2^(t-127)` between its values at
integer t, evaluated at `t = max(p, -126) + OFFSET` with f cut to 23 bits.  This module evaluates
that interpolant in exact rational arithmetic; the only floating-point steps are the ones the
crate itself rounds (one fp32 add for t, and for erf one multiply, one add, one divide, one
subtract, all IEEE and done here by numpy float32 scalars).

OFFSET is not an arbitrary fit: the interpolant overestimates 2^t by the factor (1+f)/2^f, whose
base-2 logarithm averages `3/2 - 1/ln 2 = 0.0573049591...` over a unit interval; shifting t down by
that amount makes the mean logarithmic error zero, and `127 - 0.0573049591 = 126.9426950409`, the
constant to every digit the crate prints.  ERF_K (3.3509633149424609) is a fitted constant with no
closed form known to the authors of these tests; it is the one number here that only the crate's
source could confirm.
"""
import math
from fractions import Fraction

import numpy as np

OFFSET = 126.94269504
ERF_K = 3.3509633149424609

F32 = np.float32


def offset_closed_form():
    """127 - (3/2 - 1/ln 2): the shift with zero mean log2 error of the interpolant."""
    return 125.5 + 1.0 / math.log(2.0)


def pow2_interpolant(p):
    """Expected faster::pow2 of each float32 in p, as float32 (NaN where the bits are a NaN)."""
    p = np.asarray(p, dtype=F32).ravel()
    out = np.empty(p.size, dtype=F32)
    for i, v in enumerate(p):
        if np.isnan(v):
            out[i] = 0.0  # Rust's `as u32` maps NaN to 0: all bits clear
            continue
        c = v if v >= F32(-126.0) else F32(-126.0)
        with np.errstate(over="ignore"):
            t = F32(c) + F32(OFFSET)  # the crate's one rounding before the scaling by 2^23 (exact)
        if np.isinf(t) or t >= F32(512.0):
            out[i] = np.nan  # 2^23 t >= 2^32: the cast saturates to all ones, a NaN pattern
            continue
        q = Fraction(float(t))
        whole = q.numerator // q.denominator
        frac = q - whole
        frac = Fraction((frac.numerator << 23) // frac.denominator, 1 << 23)  # the cast truncates
        sign = 1
        if whole >= 256:  # the exponent field overflows into the sign bit
            sign, whole = -1, whole - 256
        if whole == 0:
            val = frac * Fraction(1, 1 << 126)  # subnormal: no hidden one
        elif whole <= 254:
            val = (1 + frac) * (Fraction(2) ** (whole - 127))
        else:
            out[i] = sign * np.inf if frac == 0 else np.nan
            continue
        out[i] = F32(sign * float(val))  # exactly representable by construction
        assert Fraction(float(out[i])) == sign * val
    return out


def erf_expected(x):
    """Expected Op::Erf of each float32 in x: 1 - 2 / (1 + pow2(K x)), every step rounded to fp32."""
    x = np.asarray(x, dtype=F32).ravel()
    with np.errstate(all="ignore"):
        p = F32(ERF_K) * x
        pw = pow2_interpolant(p)
        return F32(1.0) - F32(2.0) / (F32(1.0) + pw)


def erf_vectors(seed=7):
    """Inputs that reach every branch: a dense grid, random normals, the clip at K x = -126, the
    subnormal segment, the exponent-255 segment, the sign-bit wrap, saturation, NaN and infinities."""
    rng = np.random.default_rng(seed)
    dense = np.linspace(-6, 6, 4801, dtype=F32)
    wide = np.linspace(-130, 130, 2081, dtype=F32)
    rand = (rng.standard_normal(4096) * 1.5).astype(F32)
    k = F32(ERF_K)
    edges = np.array([
        0.0, -0.0, 1e-30, -1e-30, 1.0, -1.0,
        -126.0 / k, np.nextafter(F32(-126.0) / k, F32(0)), np.nextafter(F32(-126.0) / k, F32(-np.inf)),
        -37.7, -38.0, -50.0, -1e10,            # clipped: K x < -126
        38.1, 38.2, 38.3, 38.4, 38.45,         # exponent field 255: inf / NaN patterns
        38.6, 39.0, 50.0, 100.0, 114.0,        # sign bit set: negative powers
        115.0, 200.0, 1e10, 3e38,              # saturated cast
        np.inf, -np.inf, np.nan,
    ], dtype=F32)
    return np.concatenate([dense, wide, rand, edges])
