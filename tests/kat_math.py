"""Literal cases of the reference's test/math_test.rb for the real float types.

Each row: (function, arguments, expected values, cited lines). The reference writes
its expectations with Ruby's Math functions, which are the C library's double
functions; Python's math module calls the same ones. `CLOSE` cases are held to the
reference's own bar (assert_close, math_test.rb:533-536: largest absolute difference
below 1e-6 * max(1, largest expected magnitude)); `EQUAL` cases to assert_equal.
"""
import math

E, PI = math.e, math.pi

CLOSE = [
    ("sqrt", [0, 1, 4, 9, 16], [0, 1, 2, 3, 4], "math_test.rb:19-28"),
    ("cbrt", [-8, -1, 0, 1, 8], [-2, -1, 0, 1, 2], "math_test.rb:64-73"),
    ("log", [1, E, 0.1, 10], [0, 1, math.log(0.1), math.log(10)], "math_test.rb:108-117"),
    ("log2", [1, 0.5, 2, 4], [0, -1, 1, 2], "math_test.rb:126-135"),
    ("log10", [1, 0.1, 5, 10, 100], [0, -1, math.log10(5), 1, 2], "math_test.rb:144-153"),
    ("exp", [-2, -1, 0, 1, 2], [math.exp(-2), math.exp(-1), 1, math.exp(1), math.exp(2)], "math_test.rb:162-171"),
    ("exp2", [-2, -1, 0, 1, 2], [0.25, 0.5, 1, 2, 4], "math_test.rb:180-189"),
    ("exp10", [-2, -1, 0, 1, 2], [0.01, 0.1, 1, 10, 100], "math_test.rb:198-207"),
    ("sin", [-2, -1, 0, 1, 2], [math.sin(-2), math.sin(-1), 0, math.sin(1), math.sin(2)], "math_test.rb:216-225"),
    ("cos", [-2, -1, 0, 1, 2], [math.cos(-2), math.cos(-1), 1, math.cos(1), math.cos(2)], "math_test.rb:234-243"),
    ("tan", [-2, -1, 0, 1, 2], [math.tan(-2), math.tan(-1), 0, math.tan(1), math.tan(2)], "math_test.rb:252-261"),
    ("asin", [-1, -0.5, 0, 0.5, 1], [-PI / 2, math.asin(-0.5), 0, math.asin(0.5), PI / 2], "math_test.rb:270-279"),
    ("acos", [-1, -0.5, 0, 0.5, 1], [PI, math.acos(-0.5), PI / 2, math.acos(0.5), 0], "math_test.rb:288-298"),
    ("atan", [-2, -1, 0, 1, 2], [math.atan(-2), math.atan(-1), 0, math.atan(1), math.atan(2)], "math_test.rb:307-316"),
    ("sinh", [-2, -1, 0, 1, 2], [math.sinh(-2), math.sinh(-1), 0, math.sinh(1), math.sinh(2)], "math_test.rb:325-334"),
    ("cosh", [-2, -1, 0, 1, 2], [math.cosh(-2), math.cosh(-1), 1, math.cosh(1), math.cosh(2)], "math_test.rb:343-352"),
    ("tanh", [-2, -1, 0, 1, 2], [math.tanh(-2), math.tanh(-1), 0, math.tanh(1), math.tanh(2)], "math_test.rb:361-370"),
    ("asinh", [-2, -1, 0, 1, 2], [math.asinh(-2), math.asinh(-1), 0, math.asinh(1), math.asinh(2)], "math_test.rb:379-388"),
    ("acosh", [1, 2, 3, 4], [math.acosh(1), math.acosh(2), math.acosh(3), math.acosh(4)], "math_test.rb:397-406"),
    ("atanh", [-0.2, -0.1, 0, 0.1, 0.2], [math.atanh(-0.2), math.atanh(-0.1), 0, math.atanh(0.1), math.atanh(0.2)],
     "math_test.rb:415-426"),
    ("sinc", [-2, -1, 0, 1, 2], [math.sin(-2) / -2, math.sin(-1) / -1, 1, math.sin(1) / 1, math.sin(2) / 2], "math_test.rb:435-446"),
    ("erf", [-2, -1, 0, 1, 2], [math.erf(-2), math.erf(-1), 0, math.erf(1), math.erf(2)], "math_test.rb:474-477"),
    ("erfc", [-2, -1, 0, 1, 2], [math.erfc(-2), math.erfc(-1), 1, math.erfc(1), math.erfc(2)], "math_test.rb:483-486"),
    ("log1p", [-0.5, 0, 1, 2], [math.log(0.5), math.log(1), math.log(2), math.log(3)], "math_test.rb:492-495"),
    ("expm1", [-1.0, 0.0, 1.0, 2.0], [math.exp(-1) - 1, 0, math.exp(1) - 1, math.exp(2) - 1], "math_test.rb:501-504"),
]

# two arguments, compared with assert_equal after the expectation is stored in the array's own type
EQUAL2 = [
    ("atan2", [0, 1, 0, -1], [1, 0, -1, 0], [0, PI / 2, PI, -PI / 2], "math_test.rb:452-457"),
    ("hypot", [3, 5, 8], [4, 12, 15], [5, 13, 17], "math_test.rb:463-468"),
]
# ldexp takes an Int32 second argument (math_test.rb:510-515); frexp answers [mantissa, Int32 exponent] (521-527)
LDEXP = ([0.0, 0.5, 0.5, 0.75, 0.5, 0.625], [0, 1, 2, 2, 3, 3], [0.0, 1.0, 2.0, 3.0, 4.0, 5.0])
FREXP = ([0.0, 1.0, 2.0, 3.0, 4.0, 5.0], [0.0, 0.5, 0.5, 0.75, 0.5, 0.625], [0, 1, 2, 2, 3, 3])


def close(expected, actual, rtol=1e-6):
    """assert_close of math_test.rb:533-536."""
    scale = max(1.0, max(abs(float(v)) for v in expected))
    worst = max(abs(float(e) - float(a)) for e, a in zip(expected, actual))
    return worst < rtol * scale

# seq and logseq (narray_alt_coverage_test.rb:263-272): (arguments, expected)
SEQ = [((), [0, 1, 2, 3, 4]), ((2,), [2, 3, 4, 5, 6]), ((5, 3), [5, 8, 11, 14, 17])]
LOGSEQ = [(4, (0, 1), [1, 10, 100, 1000]), (5, (4, -1, 2), [16, 8, 4, 2, 1])]
