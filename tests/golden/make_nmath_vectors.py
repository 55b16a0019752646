#!/usr/bin/env python3
"""Writes tests/golden/nmath_vectors.npz: correctly rounded results of every NMath
function on the path (the list of ext/cumo/narray/gen/spec.rb:427-457, plus pow), for
SFloat and DFloat arguments, computed with mpmath at 400 bits and rounded ONCE to the
element type (round to nearest even, subnormals and overflow included).

The vectors pin the last bit of these functions independently of any libm: the CPU
oracle (glibc) and the device are both held to them. Run in the build container only
(mpmath is not needed to run the tests):

    python tests/golden/make_nmath_vectors.py

Arrays in the file, per function F and type T in {f32, f64}:
    F_T_x (arguments; F_T_y too for the two-argument functions) and F_T_r (results).
"""
import os
from fractions import Fraction

import mpmath as mp
import numpy as np

mp.mp.prec = 400
HERE = os.path.dirname(os.path.abspath(__file__))

FMT = {"f32": (24, -126, 127, np.float32, np.uint32), "f64": (53, -1022, 1023, np.float64, np.uint64)}


def round_to(v, fmt):
    """mpf (or inf / nan) -> the nearest value of the format, as a Python float (exact for f32 too)."""
    p, emin, emax, _, _ = FMT[fmt]
    if mp.isnan(v):
        return float("nan")
    if mp.isinf(v):
        return float("inf") if v > 0 else float("-inf")
    if v == 0:
        return 0.0
    neg = v < 0
    man, exp = int(v.man), int(v.exp)          # |v| = man * 2^exp exactly
    fr = Fraction(man, 1) * (Fraction(2) ** exp)
    e = man.bit_length() + exp - 1                # floor(log2 |v|)
    e = max(e, emin)
    quantum = Fraction(2) ** (e - (p - 1))        # spacing of the format at this magnitude
    q = fr / quantum
    n = q.numerator // q.denominator
    rem = q - n
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and (n & 1)):
        n += 1
    r = Fraction(n) * quantum
    if r >= Fraction(2) ** (emax + 1):
        out = float("inf")
    else:
        out = float(r)                             # exact: at most 53 significant bits
    return -out if neg else out


def as_type(values, fmt):
    return np.array(values, dtype=np.float64).astype(FMT[fmt][3])


def log_uniform(rng, lo_exp, hi_exp, n, fmt, signed=False):
    e = rng.uniform(lo_exp, hi_exp, n)
    m = rng.uniform(1.0, 2.0, n)
    v = m * np.exp2(np.floor(e))
    if signed:
        v *= rng.choice([-1.0, 1.0], n)
    return as_type(v, fmt)


def uniform(rng, lo, hi, n, fmt):
    return as_type(rng.uniform(lo, hi, n), fmt)


def near(rng, c, n, fmt):
    """values within a few thousand ulps of c"""
    t = FMT[fmt][3]
    u = FMT[fmt][4]
    base = np.array([c], dtype=t).view(u)[0]
    offs = rng.integers(-4000, 4000, n)
    return (base.astype(np.int64) + offs).astype(u).view(t)


def args_for(name, fmt, rng, n):
    big = 126 if fmt == "f32" else 1020
    sub = -149 if fmt == "f32" else -1074
    tiny = np.array([2.0 ** sub, 2.0 ** (sub + 1), 2.0 ** (-126 if fmt == "f32" else -1022)], dtype=np.float64)
    t = FMT[fmt][3]
    parts = []
    if name in ("sqrt",):
        parts = [log_uniform(rng, sub, big, n, fmt), as_type([0.0, 1.0, 2.0, 4.0, 0.25], fmt), as_type(tiny, fmt)]
    elif name == "cbrt":
        parts = [log_uniform(rng, sub, big, n, fmt, signed=True), as_type([0.0, 1.0, -1.0, 8.0, 27.0, -0.125], fmt)]
    elif name in ("log", "log2", "log10"):
        parts = [log_uniform(rng, sub, big, n // 2, fmt), near(rng, 1.0, n // 4, fmt), uniform(rng, 0.5, 2.0, n // 4, fmt),
                 as_type([1.0, 2.0, 10.0, 0.5, 1024.0, 1e-3], fmt), as_type(tiny, fmt)]
    elif name == "exp":
        lo, hi = (-104.0, 88.7) if fmt == "f32" else (-745.0, 709.7)
        parts = [uniform(rng, lo, hi, n // 2, fmt), uniform(rng, -2, 2, n // 4, fmt), log_uniform(rng, -60, -1, n // 4, fmt, signed=True),
                 as_type([0.0, 1.0, -1.0, 0.5], fmt)]
    elif name == "exp2":
        lo, hi = (-150.0, 127.9) if fmt == "f32" else (-1075.0, 1023.9)
        parts = [uniform(rng, lo, hi, n // 2, fmt), uniform(rng, -2, 2, n // 4, fmt), as_type(np.arange(-20, 21), fmt), as_type([0.5, -0.5, 1e-5], fmt)]
    elif name == "exp10":
        lo, hi = (-45.0, 38.5) if fmt == "f32" else (-323.0, 308.2)
        parts = [uniform(rng, lo, hi, n // 2, fmt), uniform(rng, -2, 2, n // 4, fmt), as_type(np.arange(-10, 11), fmt)]
    elif name in ("sin", "cos", "tan"):
        huge = 100 if fmt == "f32" else 70
        parts = [uniform(rng, -8, 8, n // 3, fmt), uniform(rng, -1000, 1000, n // 3, fmt), log_uniform(rng, 10, huge, n // 6, fmt, signed=True),
                 log_uniform(rng, -40, -1, n // 6, fmt, signed=True),
                 as_type([0.0, 1.0, 3.0, 3.14159265358979, 1.5707963267948966, 0.7853981633974483, 1e5, 1e10, 1e22 if fmt == "f64" else 1e20], fmt)]
    elif name in ("asin", "acos"):
        parts = [uniform(rng, -1, 1, n // 2, fmt), near(rng, 1.0, n // 8, fmt), near(rng, -1.0, n // 8, fmt), log_uniform(rng, -60, -1, n // 4, fmt, signed=True),
                 as_type([0.0, 0.5, -0.5, 1.0, -1.0], fmt)]
        parts = [np.clip(p, -1, 1) for p in parts]
    elif name == "atan":
        parts = [log_uniform(rng, -60, 60, n, fmt, signed=True), as_type([0.0, 1.0, -1.0, 1e30], fmt)]
    elif name in ("sinh", "cosh"):
        hi = 88.0 if fmt == "f32" else 709.0
        parts = [uniform(rng, -hi, hi, n // 2, fmt), uniform(rng, -3, 3, n // 4, fmt), log_uniform(rng, -60, -1, n // 4, fmt, signed=True), as_type([0.0, 1.0, -1.0], fmt)]
    elif name == "tanh":
        parts = [uniform(rng, -20, 20, n // 2, fmt), uniform(rng, -1, 1, n // 4, fmt), log_uniform(rng, -60, 6, n // 4, fmt, signed=True), as_type([0.0, 0.5, 19.0, 40.0], fmt)]
    elif name == "asinh":
        parts = [log_uniform(rng, -60, big - 2, n, fmt, signed=True), uniform(rng, -3, 3, n // 4, fmt), as_type([0.0, 1.0, -1.0, 4.19005794e18, 2.74915304e28], fmt)]
    elif name == "acosh":
        parts = [1.0 + log_uniform(rng, -20, 10, n // 2, fmt).astype(np.float64), log_uniform(rng, 0, big - 2, n // 2, fmt), near(rng, 1.0, n // 8, fmt),
                 as_type([1.0, 2.0, 4.19005794e18, 2.74915304e28], fmt)]
        parts = [np.maximum(as_type(p, fmt), t(1.0)) for p in parts]
    elif name == "atanh":
        parts = [uniform(rng, -1, 1, n // 2, fmt), near(rng, 1.0, n // 8, fmt), log_uniform(rng, -60, -1, n // 4, fmt, signed=True), as_type([0.0, 0.5, -0.5], fmt)]
        lim = np.nextafter(t(1.0), t(0.0))
        parts = [np.clip(p, -lim, lim) for p in parts]
    elif name == "sinc":
        parts = [uniform(rng, -30, 30, n // 2, fmt), log_uniform(rng, -40, 20, n // 2, fmt, signed=True), as_type([1.0, 3.0, 0.5], fmt)]
    elif name == "erf":
        parts = [uniform(rng, -6, 6, n // 2, fmt), log_uniform(rng, -60, 3, n // 2, fmt, signed=True), as_type([0.0, 1.0, -1.0, 0.5], fmt)]
    elif name == "erfc":
        hi = 10.0 if fmt == "f32" else 26.5
        parts = [uniform(rng, -6, hi, n // 2, fmt), log_uniform(rng, -60, 2, n // 2, fmt, signed=True), as_type([0.0, 1.0, -1.0, 0.5, 5.0], fmt)]
    elif name == "log1p":
        parts = [log_uniform(rng, -60, big - 2, n // 2, fmt), -log_uniform(rng, -60, -0.001, n // 4, fmt).astype(np.float64), uniform(rng, -0.99, 3, n // 4, fmt),
                 as_type([0.0, 1.0, -0.5, 1e-10, -1e-10], fmt)]
    elif name == "expm1":
        hi = 88.0 if fmt == "f32" else 709.0
        parts = [uniform(rng, -40, hi, n // 2, fmt), uniform(rng, -1, 1, n // 4, fmt), log_uniform(rng, -60, 0, n // 4, fmt, signed=True), as_type([0.0, 1.0, -1.0], fmt)]
    else:
        raise ValueError(name)
    x = np.concatenate([as_type(p, fmt) for p in parts])
    return x[np.isfinite(x)]


def mpf_of(x):
    return mp.mpf(float(x))   # every f32 / f64 value is an exact Python float


def sinc(v):
    return mp.mpf(1) if v == 0 else mp.sin(v) / v


ONE = {
    "sqrt": mp.sqrt, "cbrt": lambda v: mp.cbrt(v) if v >= 0 else -mp.cbrt(-v), "log": mp.log, "log2": lambda v: mp.log(v, 2), "log10": mp.log10,
    "exp": mp.exp, "exp2": lambda v: mp.power(2, v), "exp10": lambda v: mp.power(10, v), "sin": mp.sin, "cos": mp.cos, "tan": mp.tan,
    "asin": mp.asin, "acos": mp.acos, "atan": mp.atan, "sinh": mp.sinh, "cosh": mp.cosh, "tanh": mp.tanh, "asinh": mp.asinh, "acosh": mp.acosh,
    "atanh": mp.atanh, "sinc": sinc, "erf": mp.erf, "erfc": mp.erfc, "log1p": mp.log1p, "expm1": mp.expm1,
}


def main():
    out = {}
    n = 700
    for fi, name in enumerate(sorted(ONE)):
        for fmt in ("f32", "f64"):
            rng = np.random.default_rng(1000 + fi * 2 + (fmt == "f64"))
            x = args_for(name, fmt, rng, n)
            r = np.array([round_to(ONE[name](mpf_of(v)), fmt) for v in x], dtype=np.float64).astype(FMT[fmt][3])
            out["%s_%s_x" % (name, fmt)] = x
            out["%s_%s_r" % (name, fmt)] = r
    # two arguments
    for fmt in ("f32", "f64"):
        t = FMT[fmt][3]
        rng = np.random.default_rng(77 + (fmt == "f64"))
        big = 60 if fmt == "f32" else 500
        y = np.concatenate([log_uniform(rng, -40, 40, n, fmt, signed=True), as_type([0.0, 1.0, -1.0, 0.0, 1.0], fmt)])
        x = np.concatenate([log_uniform(rng, -40, 40, n, fmt, signed=True), as_type([1.0, 0.0, 0.0, -1.0, 1.0], fmt)])
        out["atan2_%s_x" % fmt], out["atan2_%s_y" % fmt] = y, x   # atan2(x = first operand, y = second operand)
        out["atan2_%s_r" % fmt] = np.array([round_to(mp.atan2(mpf_of(a), mpf_of(b)), fmt) for a, b in zip(y, x)], dtype=np.float64).astype(t)
        a = np.concatenate([log_uniform(rng, -big, big, n, fmt, signed=True), as_type([3.0, 0.0, 5.0], fmt)])
        b = np.concatenate([log_uniform(rng, -big, big, n, fmt, signed=True), as_type([4.0, 2.0, 12.0], fmt)])
        # half of the pairs of similar magnitude
        b[: n // 2] = (a[: n // 2].astype(np.float64) * rng.uniform(0.25, 4.0, n // 2)).astype(t)
        out["hypot_%s_x" % fmt], out["hypot_%s_y" % fmt] = a, b
        out["hypot_%s_r" % fmt] = np.array([round_to(mp.hypot(mpf_of(p), mpf_of(q)), fmt) for p, q in zip(a, b)], dtype=np.float64).astype(t)
        # pow: positive bases with real exponents (results in range), and negative bases with integer exponents
        base = np.concatenate([log_uniform(rng, -8, 8, n, fmt), uniform(rng, 0.5, 2.0, n // 2, fmt), -uniform(rng, 0.1, 9.0, 60, fmt)])
        expo = np.concatenate([uniform(rng, -8, 8, n, fmt), uniform(rng, -60, 60, n // 2, fmt), as_type(rng.integers(-9, 10, 60), fmt)])
        out["pow_%s_x" % fmt], out["pow_%s_y" % fmt] = base, expo
        out["pow_%s_r" % fmt] = np.array([round_to(mp.power(mpf_of(p), mpf_of(q)), fmt) for p, q in zip(base, expo)], dtype=np.float64).astype(t)
    path = os.path.join(HERE, "nmath_vectors.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
