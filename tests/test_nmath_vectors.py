"""NMath pinned independently of any libm: tests/golden/nmath_vectors.npz holds correctly
rounded results (mpmath at 400 bits, rounded once; tests/golden/make_nmath_vectors.py) of
every function of ext/cumo/narray/gen/spec.rb:427-457 plus pow, for SFloat and DFloat
arguments. Here, on the CPU:

* the vectors themselves against closed forms a wrong generator would miss;
* the oracle (glibc on this machine) against the vectors: 1 ulp, except the DFloat functions
  whose glibc implementation is itself further from the correctly rounded value (listed
  below with the bound measured on these vectors -- the oracle is no better than that there,
  and tests that compare the device with the oracle use the sum of the two bounds);
* the device's own SFloat / DFloat algorithms (cumo_amd/csrc/ew_ops.h), compiled for the
  host -- every step is an IEEE operation, so the host computes what the device computes --
  against the vectors and, over every 1021st float bit pattern (every pattern with
  CUMO_EXHAUSTIVE=1), against (float)glibc((double)x)."""
import os
import subprocess
import sys

import numpy as np
import pytest

from helpers import ulp_diff

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
import numo_oracle as oracle  # noqa: E402

VECTORS = os.path.join(ROOT, "tests", "golden", "nmath_vectors.npz")
ONE = ("sqrt cbrt log log2 log10 exp exp2 exp10 sin cos tan asin acos atan sinh cosh tanh "
       "asinh acosh atanh sinc erf erfc log1p expm1").split()
TWO = ("atan2", "hypot", "pow")
# glibc's DFloat functions that are measured further than 1 ulp from the correctly rounded
# value on these vectors (ulps). Everything else, and every SFloat function, is within 1.
ORACLE_F64_BOUND = {"cbrt": 3, "exp10": 2, "tanh": 2, "erfc": 2}


@pytest.fixture(scope="module")
def vec():
    return np.load(VECTORS, allow_pickle=False)


def test_vectors_hold_every_function_and_known_values(vec):
    for name in ONE + list(TWO):
        for fmt in ("f32", "f64"):
            assert "%s_%s_x" % (name, fmt) in vec.files and "%s_%s_r" % (name, fmt) in vec.files
            assert vec["%s_%s_x" % (name, fmt)].size >= 500
    # closed forms: exact cases come out exact, and a few published digits
    def at(name, fmt, x):
        xs, rs = vec["%s_%s_x" % (name, fmt)], vec["%s_%s_r" % (name, fmt)]
        i = np.nonzero(xs == x)[0]
        assert i.size, (name, fmt, x)
        return rs[i[0]]
    for fmt, t in (("f32", np.float32), ("f64", np.float64)):
        assert at("sqrt", fmt, t(4.0)) == 2 and at("sqrt", fmt, t(0.25)) == 0.5
        assert at("cbrt", fmt, t(27.0)) == 3 and at("cbrt", fmt, t(-0.125)) == -0.5
        assert at("log", fmt, t(1.0)) == 0 and at("log2", fmt, t(1024.0)) == 10 and at("log10", fmt, t(10.0)) == 1
        assert at("exp", fmt, t(0.0)) == 1 and at("exp2", fmt, t(-3.0)) == 0.125 and at("exp10", fmt, t(3.0)) == 1000
        assert at("sin", fmt, t(0.0)) == 0 and at("cos", fmt, t(0.0)) == 1
        assert at("atan", fmt, t(1.0)) == t(np.pi / 4)
        assert at("expm1", fmt, t(0.0)) == 0 and at("log1p", fmt, t(0.0)) == 0
    assert vec["exp_f64_r"][vec["exp_f64_x"] == 1.0][0] == 2.718281828459045          # e, correctly rounded
    assert vec["sin_f64_r"][vec["sin_f64_x"] == 1e22][0] == -0.8522008497671888        # the classic large-argument case
    assert vec["erf_f64_r"][vec["erf_f64_x"] == 1.0][0] == 0.8427007929497149
    assert vec["exp_f32_r"][vec["exp_f32_x"] == np.float32(1.0)][0] == np.float32(2.7182817)
    # hypot(3, 4) = 5, atan2 quadrant, pow of a negative base with an odd integer exponent keeps the sign
    i = np.nonzero((vec["hypot_f64_x"] == 3.0) & (vec["hypot_f64_y"] == 4.0))[0][0]
    assert vec["hypot_f64_r"][i] == 5.0
    neg = (vec["pow_f64_x"] < 0) & (vec["pow_f64_y"] % 2 == 1)
    assert neg.any() and (vec["pow_f64_r"][neg] < 0).all()
    # monotone functions are monotone in the vectors
    for name in ("exp", "log", "atan", "tanh", "erf", "cbrt"):
        x, r = vec["%s_f64_x" % name], vec["%s_f64_r" % name]
        o = np.argsort(x)
        assert (np.diff(r[o]) >= 0).all(), name


def _oracle_value(name, x, y=None):
    with np.errstate(all="ignore"):
        if name == "pow":
            return oracle.binary("pow", x, y)
        if y is not None:
            return oracle.binary(name, x, y)
        return oracle.unary(name, x)


@pytest.mark.parametrize("name", ONE + list(TWO))
def test_oracle_against_correctly_rounded_vectors(vec, name):
    for fmt in ("f32", "f64"):
        x, r = vec["%s_%s_x" % (name, fmt)], vec["%s_%s_r" % (name, fmt)]
        y = vec["%s_%s_y" % (name, fmt)] if name in TWO else None
        got = _oracle_value(name, x, y)
        bound = ORACLE_F64_BOUND.get(name, 1) if fmt == "f64" else 1
        d = ulp_diff(got, r)
        assert d.max() <= bound, "%s %s: oracle %d ulp from the correctly rounded value at x=%r" % (name, fmt, d.max(), x[np.argmax(d)])


@pytest.fixture(scope="module")
def cores(tmp_path_factory):
    exe = tmp_path_factory.mktemp("cores") / "float_cores_check"
    subprocess.run(["g++", "-O2", "-std=c++17", "-ffp-contract=off", "-o", str(exe), os.path.join(ROOT, "tests", "float_cores_check.cpp")], check=True)
    return str(exe)


SFLOAT_CORES = ("exp", "log", "log2", "log10", "log1p", "tanh", "sinh", "cosh", "expm1", "asinh", "acosh", "atanh", "sin", "cos", "tan",
                "atan", "erf", "asin", "acos", "erfc", "sinc")
DFLOAT_CORES = ("log", "log2", "log10", "tanh", "sinh", "cosh", "erfc", "log1p", "asinh", "acosh", "atanh")


def test_device_algorithms_on_the_host_against_vectors(vec, cores, tmp_path):
    lines = []
    for name in SFLOAT_CORES:
        x = vec["%s_f32_x" % name]
        lines.append("%s f32 %d" % (name, x.size))
        lines += ["%x" % b for b in x.view(np.uint32)]
    for name in DFLOAT_CORES:
        x = vec["%s_f64_x" % name]
        lines.append("%s f64 %d" % (name, x.size))
        lines += ["%x" % b for b in x.view(np.uint64)]
    src = tmp_path / "args.txt"
    src.write_text("\n".join(lines) + "\n")
    out = subprocess.run([cores, "vectors", str(src)], check=True, stdout=subprocess.PIPE, text=True).stdout.split("\n")
    pos = 0
    for name, fmt in [(n, "f32") for n in SFLOAT_CORES] + [(n, "f64") for n in DFLOAT_CORES]:
        head = out[pos].split()
        assert head[:2] == [name, fmt]
        n = int(head[2])
        raw = [int(v, 16) for v in out[pos + 1:pos + 1 + n]]
        pos += 1 + n
        got = np.array(raw, dtype=np.uint32 if fmt == "f32" else np.uint64).view(np.float32 if fmt == "f32" else np.float64)
        d = ulp_diff(got, vec["%s_%s_r" % (name, fmt)])
        assert d.max() <= 1, (name, fmt, int(d.max()))
        if fmt == "f32" and name not in ("asinh", "acosh", "erf", "erfc"):
            # evaluated in double to 2^-40 or better and rounded once: the correctly rounded float
            # itself, bar the rare argument whose exact value lies that close to a rounding boundary
            assert (d > 0).sum() <= 1, (name, int((d > 0).sum()))


def test_device_dfloat_algorithms_on_pairs_against_long_double(cores):
    """tanh, sinh, cosh and erfc of DFloat carry their exponential as a pair of doubles, log1p and the inverse hyperbolic
    functions the argument of their logarithm: the result's one rounding and little else."""
    n = 200000000 if os.environ.get("CUMO_EXHAUSTIVE") else 2000000
    out = subprocess.run([cores, "dsweep", str(n)], check=True, stdout=subprocess.PIPE, text=True).stdout.strip().split("\n")
    assert [line.split()[0] for line in out] == ["tanh", "sinh", "cosh", "erfc", "log1p", "asinh", "acosh", "atanh"]
    for line in out:
        name, tried, worst, where = line.split()
        # (erfc: the series' first-order term is rounded in double, and subnormal results are rounded twice)
        assert int(tried) == n and float(worst) <= (0.8 if name == "erfc" else 0.52), line


def test_device_sfloat_atan2_hypot_and_remainder_against_glibc(cores):
    n = 500000000 if os.environ.get("CUMO_EXHAUSTIVE") else 5000000
    out = subprocess.run([cores, "two", str(n)], check=True, stdout=subprocess.PIPE, text=True).stdout.strip().split("\n")
    assert [line.split()[0] for line in out] == ["atan2", "hypot", "fmod"]
    for line in out:
        name, tried, bad, worst = line.split()
        # evaluated in double to 2^-43 and rounded once: the rare argument next to a rounding boundary may differ by an ulp;
        # the remainder is exact (and its arithmetic covers the quotients below 2^29: a part of the random pairs)
        assert int(tried) >= (n // 10 if name == "fmod" else n * 9 // 10), line
        assert int(bad) <= (0 if name == "fmod" else int(tried) >> 17) and int(worst) <= 1, line


def test_device_sfloat_power_by_whole_numbers_of_halves_against_glibc(cores):
    """x ** y for one exponent that is a whole number of halves goes by squarings, multiplications and one square root
    in double: every float bit pattern of the stride, the rules for zeros, infinities, negative bases and NaN included."""
    stride = 1 if os.environ.get("CUMO_EXHAUSTIVE") else 4099
    out = subprocess.run([cores, "halves", str(stride)], check=True, stdout=subprocess.PIPE, text=True).stdout.strip().split("\n")
    assert len(out) == 22
    for line in out:
        y, tried, bad, worst = line.split()
        assert int(tried) >= (1 << 32) // stride and int(bad) <= int(tried) >> 17 and int(worst) <= 1, line


def test_device_dfloat_power_by_whole_numbers_of_halves_against_long_double(cores):
    n = 20000000 if os.environ.get("CUMO_EXHAUSTIVE") else 200000
    out = subprocess.run([cores, "dhalves", str(n)], check=True, stdout=subprocess.PIPE, text=True).stdout.strip().split("\n")
    assert len(out) == 32
    for line in out:
        y, tried, worst = line.split()
        assert int(tried) == n and float(worst) <= 0.51, line


def test_device_dfloat_power_against_long_double(cores):
    """x ** y of DFloat for a positive normal base and a finite exponent: log2 x and y log2 x as pairs of doubles."""
    n = 300000000 if os.environ.get("CUMO_EXHAUSTIVE") else 3000000
    name, tried, worst, worst_subnormal, wrong_ends, _, _ = subprocess.run(
        [cores, "dpow", str(n)], check=True, stdout=subprocess.PIPE, text=True).stdout.split()
    assert name == "pow" and int(tried) == n
    # (a subnormal result is rounded twice: by the arithmetic and by the scaling)
    assert float(worst) <= 0.54 and float(worst_subnormal) <= 1.0 and int(wrong_ends) == 0


def test_device_sfloat_algorithms_against_glibc_over_float_bit_patterns(cores):
    stride = 1 if os.environ.get("CUMO_EXHAUSTIVE") else 1021
    out = subprocess.run([cores, "sweep", str(stride)], check=True, stdout=subprocess.PIPE, text=True).stdout.strip().split("\n")
    assert len(out) == len(SFLOAT_CORES)
    for line in out:
        name, tried, bad, worst = line.split()
        assert int(tried) >= (1 << 32) // stride
        # one float in about 2^16 lies within 2^-40 of a rounding boundary, where a result that is
        # good to 2^-40 before its one rounding may land on the other side (erf's fits are the
        # loosest: about 4 arguments in a million); never more than one ulp
        allowed = int(tried) >> (14 if name in ("erf", "erfc") else 17)
        assert int(bad) <= allowed and int(worst) <= 1, line
