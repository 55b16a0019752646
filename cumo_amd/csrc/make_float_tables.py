"""Writes float_tables.inc: the tables and polynomial coefficients of the table-driven
log2 / exp2 cores in ew_ops.h (SFloat power, asinh, acosh, atanh).

    python cumo_amd/csrc/make_float_tables.py > cumo_amd/csrc/float_tables.inc

log2: the argument's high word minus 0x3fe6a000 gives the binade k (bits 20 and up), the
interval i (bits 14..19) and, with the binade taken off, a mantissa m in [0.70703125,
1.4140625). Interval i holds the m whose high word lies in [0x3fe6a000 + i 2^14, + 2^14);
its entry is {invc, logc} with invc = 1 / (the interval's midpoint) rounded to double and
logc = -log2(invc) of that rounded value, so that log2 m = logc + log2(1 + z) with
z = m invc - 1, |z| <= 2^-7. 1.0 is the midpoint of interval 37 (0x3ff00000 - 0x3fe6a000 =
37.5 * 2^14): its entry is {1, 0} exactly, so arguments next to 1 lose nothing.
exp2: 2^(j/32), j = 0..31.
Coefficients are the Taylor ones (the intervals are short enough: the remainders are
z^6 / 7 relative for log2(1 + z) and (r ln 2)^5 / 120 for 2^r, |r| <= 1/64)."""
import struct

import mpmath as mp

mp.mp.prec = 200
OFFH = 0x3FE6A000


def dbl(hi, lo=0):
    return struct.unpack("<d", struct.pack("<Q", (hi << 32) | lo))[0]


def to_double(x):
    return float(mp.nstr(x, 40))  # correctly rounded through the decimal string (40 digits >> 17)


def main():
    rows = []
    for i in range(64):
        lo_hi, up_hi = OFFH + (i << 14), OFFH + ((i + 1) << 14)

        def real(h):  # the mantissa value of a high word after the binade is taken off
            t = h - OFFH
            return mp.mpf(dbl(h - (t & 0xFFF00000)))  # (t < 2^20 here: nothing is taken off)
        # interval bounds as reals: a bound in the upper binade is the double with that high word
        a, b = mp.mpf(dbl(lo_hi)), mp.mpf(dbl(up_hi))
        c = (a + b) / 2
        if a < 1 < b:
            assert i == 37
            invc, logc = 1.0, 0.0
        else:
            invc = to_double(1 / c)
            logc = to_double(-mp.log(mp.mpf(invc), 2))
        zmax = max(abs(a * mp.mpf(invc) - 1), abs(b * mp.mpf(invc) - 1))
        assert zmax <= mp.mpf(2) ** -7 * (1 + mp.mpf(2) ** -20), (i, zmax)
        rows.append((invc, logc))
    print("// written by make_float_tables.py; do not edit")
    print("#define CUMO_HIP_LOG2_TABLE \\")
    print(", \\\n".join("    %s, %s" % (float.hex(a), float.hex(b)) for a, b in rows))
    print("#define CUMO_HIP_EXP2_TABLE \\")
    ex = [to_double(mp.mpf(2) ** (mp.mpf(j) / 32)) for j in range(32)]
    print(", \\\n".join("    " + ", ".join(float.hex(v) for v in ex[k:k + 4]) for k in range(0, 32, 4)))
    ln2 = mp.log(2)
    print("// log2(1 + z) = z (L1 + L2 z + ... + L6 z^5)")
    for n in range(1, 7):
        print("#define CUMO_HIP_LOG2_L%d %s" % (n, float.hex(to_double(mp.mpf((-1) ** (n + 1)) / (n * ln2)))))
    print("// 2^r = 1 + r (E1 + E2 r + E3 r^2 + E4 r^3)")
    for n in range(1, 5):
        print("#define CUMO_HIP_EXP2_E%d %s" % (n, float.hex(to_double(ln2 ** n / mp.factorial(n)))))

    # DFloat hyperbolic functions: e^a = 2^(k/32) e^r with a = k (ln 2 / 32) + r; 2^(j/32) as a double and what is
    # left of it, ln 2 / 32 as a 42-bit double (k times it is exact for k < 2^11) and what is left of it
    print("// 2^(j/32) = hi + lo, j = 0..31")
    print("#define CUMO_HIP_EXPDD_TABLE \\")
    dd = []
    for j in range(32):
        v = mp.mpf(2) ** (mp.mpf(j) / 32)
        hi = to_double(v)
        lo = to_double(v - mp.mpf(hi))
        dd.append((hi, lo))
    print(", \\\n".join("    %s, %s" % (float.hex(a), float.hex(b)) for a, b in dd))
    step = ln2 / 32
    hi = mp.ldexp(mp.floor(mp.ldexp(step, 6 + 41)), -(6 + 41))  # step < 2^-5: 42 bits from 2^-6 down
    assert mp.mpf(2) ** -6 <= hi < mp.mpf(2) ** -5
    print("#define CUMO_HIP_LN2_32_HI %s" % float.hex(float(hi)))
    print("#define CUMO_HIP_LN2_32_LO %s" % float.hex(to_double(step - hi)))
    print("#define CUMO_HIP_32_LN2 %s" % float.hex(to_double(32 / ln2)))

    # DFloat power: log2 x as a pair. 128 intervals by the high word minus 0x3fe69000 (1.0 is the midpoint of interval
    # 75, whose entry is {1, 0, 0}); invc has so few bits (7 after the point below 1, 8 above: what the interval's
    # width leaves room for) that z = m invc - 1 is exact in one multiply-add; logc = -log2(invc) as a head on a
    # grid of 2^-42 (so that binade + head is exact) and a tail.
    off = 0x3FE69000
    print("// {invc, logc head, logc tail} for the 128 intervals of the DFloat power's log2")
    print("#define CUMO_HIP_LOG2DD_TABLE \\")
    rows = []
    worst = mp.mpf(0)
    for i in range(128):
        lo_hi, up_hi = off + (i << 13), off + ((i + 1) << 13)
        a, b = mp.mpf(dbl(lo_hi)), mp.mpf(dbl(up_hi))
        if a < 1 < b:
            assert i == 75
            rows.append((1.0, 0.0, 0.0))
            worst = max(worst, 1 - a, b - 1)
            continue
        below = b <= 1
        f = 7 if below else 8
        c = (a + b) / 2
        j = int(mp.nint(mp.ldexp(1 / c, f)))
        invc = mp.ldexp(mp.mpf(j), -f)
        zmax = max(abs(a * invc - 1), abs(b * invc - 1))
        # z is a multiple of 2^(e - 52 - f), e the exponent of m (-1 below 1): it must fit 53 bits
        e = -1 if below else 0
        assert mp.log(zmax, 2) + 52 + f - e <= 53, (i, zmax)
        worst = max(worst, zmax)
        logc = -mp.log(invc, 2)
        head = mp.ldexp(mp.nint(mp.ldexp(logc, 42)), -42)
        tail = to_double(logc - head)
        rows.append((float(invc), float(head), tail))
        assert mp.mpf(float(head)) == head
    print(", \\\n".join("    %s, %s, %s" % tuple(float.hex(v) for v in r) for r in rows))
    print("// largest |z|: %s" % mp.nstr(worst, 8))
    print("// log2(1 + z) = z ((A1 + a1) + (A2 + a2) z + L3 z^2 + ... + L10 z^9)")
    for n in (1, 2):
        v = mp.mpf((-1) ** (n + 1)) / (n * ln2)
        hi = to_double(v)
        print("#define CUMO_HIP_LOG2DD_A%d %s" % (n, float.hex(hi)))
        print("#define CUMO_HIP_LOG2DD_a%d %s" % (n, float.hex(to_double(v - mp.mpf(hi)))))
    for n in range(3, 11):
        print("#define CUMO_HIP_LOG2DD_L%d %s" % (n, float.hex(to_double(mp.mpf((-1) ** (n + 1)) / (n * ln2)))))
    print("// 2^r = 1 + r (F1 + F2 r + ... + F7 r^6), |r| <= 1/64")
    for n in range(1, 8):
        print("#define CUMO_HIP_EXP2DD_F%d %s" % (n, float.hex(to_double(ln2 ** n / mp.factorial(n)))))

    # DFloat erfc: g(x) = e^(x^2) erfc(x) by its Taylor series about the centre of the argument's interval: centres
    # 0, 1/16, ..., 1 for x < 1 + 1/32 (within 1/32 of each), then 32 intervals a binade up to 32 (the centre is the
    # midpoint); per interval {c, g(c) as head and tail, a1 ... a10}. From g' = 2 x g - 2 / sqrt(pi):
    # a1 = 2 c a0 - 2 / sqrt(pi), a(n+1) = (2 c a(n) + 2 a(n-1)) / (n + 1) (run forwards at 1200 bits: the recurrence
    # loses some 150 of them at the far end)
    mp.mp.prec = 1200
    degree = 10
    spans = [(mp.mpf(i) / 16, max(mp.mpf(0), mp.mpf(i) / 16 - mp.mpf(1) / 32), mp.mpf(i) / 16 + mp.mpf(1) / 32) for i in range(17)]
    for e in range(5):
        for j in range(32):
            lo, hi = mp.mpf(2) ** e * (1 + mp.mpf(j) / 32), mp.mpf(2) ** e * (1 + mp.mpf(j + 1) / 32)
            spans.append(((lo + hi) / 2, lo, hi))
    print("// {c, g(c) head, g(c) tail, a1 .. a%d} for the %d intervals of the DFloat erfc" % (degree, len(spans)))
    print("#define CUMO_HIP_ERFC_DEGREE %d" % degree)
    print("#define CUMO_HIP_ERFC_ROWS %d" % len(spans))
    print("#define CUMO_HIP_ERFC_TABLE \\")
    lines = []
    worst = mp.mpf(0)
    for c, lo, hi in spans:
        co = [mp.exp(c * c) * mp.erfc(c)]
        co.append(2 * c * co[0] - 2 / mp.sqrt(mp.pi))
        for n in range(1, degree):
            co.append((2 * c * co[n] + 2 * co[n - 1]) / (n + 1))
        head = to_double(co[0])
        row = [float(c), head, to_double(co[0] - mp.mpf(head))] + [to_double(v) for v in co[1:]]
        assert mp.mpf(float(c)) == c
        for x in (lo, hi, (lo + c) / 2, (hi + c) / 2):
            d = x - c
            got = mp.mpf(row[1]) + mp.mpf(row[2]) + sum(mp.mpf(row[2 + n]) * d ** n for n in range(1, degree + 1))
            worst = max(worst, abs(got / (mp.exp(x * x) * mp.erfc(x)) - 1))
        lines.append("    " + ", ".join(float.hex(v) for v in row))
    assert worst < mp.mpf(2) ** -55, worst   # (the coefficients' own rounding included; the series alone is good to 2^-63)
    print(", \\\n".join(lines))
    print("// largest error of the rounded series at the interval ends: 2^%s" % mp.nstr(mp.log(worst, 2), 5))
    mp.mp.prec = 200


if __name__ == "__main__":
    main()
