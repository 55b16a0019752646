// DFloat functions whose error would show if they were evaluated in double alone: tanh, sinh, cosh and erfc (an
// exponential), x ** y (a logarithm times the exponent, then an exponential), log1p, asinh, acosh and atanh (the
// logarithm of a sum, root or quotient). A double has nothing wider to be evaluated in, so the one quantity that
// matters is carried as a pair of doubles (a value and what is left of it) through exact sums (two-sum), exact
// products (the multiply-add's remainder) and quotients corrected by their exact remainder, and everything else stays
// in double: 60 to 120 double operations an element where the device library's versions, which work on pairs
// throughout, take about 300. The reference calls the CUDA library's functions
// (ext/cumo/include/cumo/types/float_macro_kernel.h:36,101-120).
//
// Every step is an IEEE operation except the reciprocal and reciprocal square root estimates, which only enter
// through correction terms; a CPU build (CUMO_HIP_HOST_CHECK) computes the same up to that, and
// tests/float_cores_check.cpp runs it against the long double functions.
// Included by ew_ops.h, inside namespace cumo_hip, after the tables of float_tables.inc.
#pragma once

constexpr int kExpPairTableDoubles = 64;    // 2^(j/32) as pairs
constexpr int kLog2PairTableDoubles = 384;  // {invc, logc head, logc tail} for 128 intervals
constexpr int kErfcRowDoubles = 3 + CUMO_HIP_ERFC_DEGREE;   // {centre, g head, g tail, a1 ... }
constexpr int kErfcTableDoubles = CUMO_HIP_ERFC_ROWS * kErfcRowDoubles;
#ifdef CUMO_HIP_HOST_CHECK
static const double kPairTablesHost[kExpPairTableDoubles + kLog2PairTableDoubles] = {CUMO_HIP_EXPDD_TABLE, CUMO_HIP_LOG2DD_TABLE};
static const double kErfcTableHost[kErfcTableDoubles] = {CUMO_HIP_ERFC_TABLE};
inline const double* exp_pair_table() { return kPairTablesHost; }
inline const double* log2_pair_table() { return kPairTablesHost + kExpPairTableDoubles; }
inline const double* erfc_table() { return kErfcTableHost; }
#else
__device__ const double kPairTablesDevice[kExpPairTableDoubles + kLog2PairTableDoubles] = {CUMO_HIP_EXPDD_TABLE, CUMO_HIP_LOG2DD_TABLE};
__device__ __forceinline__ double* exp_pair_table_lds() {
    __shared__ double table[kExpPairTableDoubles];
    return table;
}
__device__ __forceinline__ double* log2_pair_table_lds() {
    __shared__ double table[kLog2PairTableDoubles];
    return table;
}
__device__ const double kErfcTableDevice[kErfcTableDoubles] = {CUMO_HIP_ERFC_TABLE};
__device__ __forceinline__ double* erfc_table_lds() {
    __shared__ double table[kErfcTableDoubles];
    return table;
}
__device__ __forceinline__ const double* exp_pair_table() { return exp_pair_table_lds(); }
__device__ __forceinline__ const double* log2_pair_table() { return log2_pair_table_lds(); }
__device__ __forceinline__ const double* erfc_table() { return erfc_table_lds(); }
// with all threads of the block, before the first element
__device__ __forceinline__ void exp_pair_table_prepare() {
    double* t = exp_pair_table_lds();
    for (unsigned i = threadIdx.x; i < (unsigned)kExpPairTableDoubles; i += blockDim.x) t[i] = kPairTablesDevice[i];
    __syncthreads();
}
// (the power reads both tables)
__device__ __forceinline__ void pow_pair_tables_prepare() {
    double* t = exp_pair_table_lds();
    double* l = log2_pair_table_lds();
    for (unsigned i = threadIdx.x; i < (unsigned)kExpPairTableDoubles; i += blockDim.x) t[i] = kPairTablesDevice[i];
    for (unsigned i = threadIdx.x; i < (unsigned)kLog2PairTableDoubles; i += blockDim.x) l[i] = kPairTablesDevice[kExpPairTableDoubles + i];
    __syncthreads();
}
// (erfc reads the exponential's table and its own)
__device__ __forceinline__ void erfc_tables_prepare() {
    double* t = exp_pair_table_lds();
    double* g = erfc_table_lds();
    for (unsigned i = threadIdx.x; i < (unsigned)kExpPairTableDoubles; i += blockDim.x) t[i] = kPairTablesDevice[i];
    for (unsigned i = threadIdx.x; i < (unsigned)kErfcTableDoubles; i += blockDim.x) g[i] = kErfcTableDevice[i];
    __syncthreads();
}
#endif

// (e^a - 1) / 2^down as hi + lo for 0 <= a <= 711 (a NaN travels through), to about 2^-60 of its
// value. `down` (0 or more; 2 where e^a itself would overflow) only shifts exponents: nothing
// is rounded differently for it.
//   a = k (ln 2 / 32) + r, |r| <= ln 2 / 64: k from one multiply-add onto 1.5 * 2^52, k times the
//   42-bit head of ln 2 / 32 taken off exactly, the tail afterwards with its rounding error kept;
//   e^r - 1 = r + r^2 Q(r), the Taylor terms to r^7 (the next is below 2^-61 of r);
//   2^(k/32) = 2^m (T + t) from the table; S = 2^m T, s = 2^m t:
//   e^a - 1 = (S - 1) + S r + [S (e^r - 1 - r) + s e^r], the first sum and the product exact
//   (S - 1 >= 2 |S r| whenever k > 0, which is what the short form of the exact sum needs).
__device__ __forceinline__ void expm1_pair(double a, int down, const double* tab, double& hi, double& lo) {
    const double big = 6755399441055744.0;  // 1.5 * 2^52
    const double t0 = __builtin_fma(a, CUMO_HIP_32_LN2, big);
    const uint32_t ki = (uint32_t)__double2loint(t0);
    const double kd = t0 - big;
    const double rh = __builtin_fma(-kd, CUMO_HIP_LN2_32_HI, a);
    const double tail = kd * CUMO_HIP_LN2_32_LO;
    const double r = rh - tail;
    const double rl = (rh - r) - tail;
    double q = 1.0 / 5040.0;
    q = __builtin_fma(q, r, 1.0 / 720.0);
    q = __builtin_fma(q, r, 1.0 / 120.0);
    q = __builtin_fma(q, r, 1.0 / 24.0);
    q = __builtin_fma(q, r, 1.0 / 6.0);
    q = __builtin_fma(q, r, 0.5);
    const double pl = __builtin_fma(r * r, q, rl);  // e^r - 1 - r
    const uint32_t j = ki & 31u;
    const int m = (int)(ki >> 5) - down;
    const double scale = __hiloint2double((m + 1023) << 20, 0);
    const double one = __hiloint2double((1023 - down) << 20, 0);
    const double sh = tab[2 * j] * scale, sl = tab[2 * j + 1] * scale;
    const double a0 = sh - one;
    const double b0 = (sh - a0) - one;
    const double p = sh * r;
    const double pe = __builtin_fma(sh, r, -p);
    const double rest = __builtin_fma(sh, pl, pe) + __builtin_fma(sl, 1.0 + r, b0);
    const double s1 = a0 + p;
    const double e1 = (p - (s1 - a0)) + rest;
    hi = s1 + e1;
    lo = (s1 - hi) + e1;
}

// (nh + nl) / (dh + dl) rounded once: the quotient of the heads from a reciprocal good to 2^-44, then what that
// quotient leaves of the numerator, exactly, times the reciprocal again
__device__ __forceinline__ double pair_quotient(double nh, double nl, double dh, double dl) {
    const double rc = rcp_refined(dh);
    const double q = nh * rc;
    const double left = __builtin_fma(-q, dl, nl) + __builtin_fma(-q, dh, nh);
    return __builtin_fma(left, rc, q);
}
// the same as a pair (for a sum that follows)
__device__ __forceinline__ void pair_quotient_pair(double nh, double nl, double dh, double dl, double& qh, double& ql) {
    const double rc = rcp_refined(dh);
    qh = nh * rc;
    ql = (__builtin_fma(-qh, dl, nl) + __builtin_fma(-qh, dh, nh)) * rc;
}
// a + b exactly as s + e, whichever is larger
__device__ __forceinline__ void exact_sum(double a, double b, double& s, double& e) {
    s = a + b;
    const double bb = s - a;
    e = (a - (s - bb)) + (b - bb);
}

// tanh|x| = t / (t + 2), t = e^(2|x|) - 1; 2|x| clamped at 44, where the answer is 1 already.
// Measured against the long double function over 4 * 10^8 arguments: within 0.51 ulp.
__device__ __forceinline__ double tanh_double(double x) {
    double a = __builtin_fabs(x);
    a = a + a;
    a = (a > 44.0) ? 44.0 : a;
    double th, tl, dh, dl;
    expm1_pair(a, 0, exp_pair_table(), th, tl);
    exact_sum(th, 2.0, dh, dl);
    return __builtin_copysign(pair_quotient(th, tl, dh, dl + tl), x);
}
// sinh|x| = (t + t / (t + 1)) / 2, t = e^|x| - 1, everything a quarter of its size from |x| = 700 on (the result is
// brought back at the end, and overflows there where it must); |x| clamped at 711, past the last finite answer.
__device__ __forceinline__ double sinh_double(double x) {
    double a = __builtin_fabs(x);
    a = (a > 711.0) ? 711.0 : a;
    const int down = (a > 700.0) ? 2 : 0;
    const double one = down ? 0.25 : 1.0;
    double th, tl, dh, dl, qh, ql, sh, sl;
    expm1_pair(a, down, exp_pair_table(), th, tl);
    exact_sum(th, one, dh, dl);
    pair_quotient_pair(th, tl, dh, dl + tl, qh, ql);
    // t / (t + 1) is a pure number: in the quarter-size world it counts a quarter
    qh *= one;
    ql *= one;
    exact_sum(th, qh, sh, sl);
    const double y = 0.5 * (sh + (sl + (tl + ql)));
    return __builtin_copysign(down ? y * 4.0 : y, x);
}
// cosh x = (e + 1 / e) / 2, e = t + 1, the same way
__device__ __forceinline__ double cosh_double(double x) {
    double a = __builtin_fabs(x);
    a = (a > 711.0) ? 711.0 : a;
    const int down = (a > 700.0) ? 2 : 0;
    const double one = down ? 0.25 : 1.0;
    double th, tl, eh, el, qh, ql, sh, sl;
    expm1_pair(a, down, exp_pair_table(), th, tl);
    exact_sum(th, one, eh, el);
    el += tl;
    // 1 / e in the quarter-size world: (1/4)^2 / (e / 4)
    pair_quotient_pair(one * one, 0.0, eh, el, qh, ql);
    exact_sum(eh, qh, sh, sl);
    const double y = 0.5 * (sh + (sl + (el + ql)));
    return down ? y * 4.0 : y;
}

// ---- DFloat power -------------------------------------------------------------------------
// x^y = 2^(y log2 x) for a positive, finite, normal x and a finite y, with log2 x and the product carried as pairs:
// a result within 2^-53 needs the exponent within 2^-58 or so, and the exponent reaches 1075.
//   log2 x = k + logc + log2(1 + z): the high word minus 0x3fe69000 gives the binade k, the interval (128 of them; 1.0
//   is the midpoint of one, whose entry is {1, 0, 0}) and a mantissa m in [0.7003, 1.4006); z = m invc - 1 is exact
//   because invc has 8 bits or fewer; k + logc's head is exact because the head lies on a grid of 2^-42;
//   log2(1 + z) = z (A1 + a1) + z^2 (A2 + a2) + z^3 (L3 + ... + L10 z^7): the first two products as pairs, the rest
//   (below 2^-15 of the first) in double. |z| < 0.00585: what is left out is below 2^-70 of the first term.
__device__ __forceinline__ void log2_pair(double x, const double* tab, double& lh, double& ll, int more_binades = 0) {
    const uint32_t hx = (uint32_t)__double2hiint(x);
    const uint32_t t = hx - 0x3fe69000u;
    const int k = ((int)t >> 20) + more_binades;   // (log2 of 2^more x)
    const uint32_t i = (t >> 13) & 127u;
    const double m = __hiloint2double((int)(hx - (t & 0xfff00000u)), __double2loint(x));
    const double invc = tab[3 * i], ch = tab[3 * i + 1], cl = tab[3 * i + 2];
    const double z = __builtin_fma(m, invc, -1.0);
    const double p1 = z * CUMO_HIP_LOG2DD_A1;
    const double p1e = __builtin_fma(z, CUMO_HIP_LOG2DD_a1, __builtin_fma(z, CUMO_HIP_LOG2DD_A1, -p1));
    const double z2 = z * z;
    const double z2e = __builtin_fma(z, z, -z2);
    const double p2 = z2 * CUMO_HIP_LOG2DD_A2;
    const double p2e = __builtin_fma(z2e, CUMO_HIP_LOG2DD_A2, __builtin_fma(z2, CUMO_HIP_LOG2DD_a2, __builtin_fma(z2, CUMO_HIP_LOG2DD_A2, -p2)));
    double q = CUMO_HIP_LOG2DD_L10;
    q = __builtin_fma(q, z, CUMO_HIP_LOG2DD_L9);
    q = __builtin_fma(q, z, CUMO_HIP_LOG2DD_L8);
    q = __builtin_fma(q, z, CUMO_HIP_LOG2DD_L7);
    q = __builtin_fma(q, z, CUMO_HIP_LOG2DD_L6);
    q = __builtin_fma(q, z, CUMO_HIP_LOG2DD_L5);
    q = __builtin_fma(q, z, CUMO_HIP_LOG2DD_L4);
    q = __builtin_fma(q, z, CUMO_HIP_LOG2DD_L3);
    const double p3 = (z2 * z) * q;
    // the exact sums in their short form: each left operand is zero or the larger one
    const double base = int_to_double(k) + ch;
    const double s1 = base + p1;
    const double s1e = p1 - (s1 - base);
    const double s2 = s1 + p2;
    const double s2e = p2 - (s2 - s1);
    const double rest = ((s1e + s2e) + (p1e + p2e)) + (p3 + cl);
    lh = s2 + rest;
    ll = (s2 - lh) + rest;
}
// 2^(eh + el) for |eh| <= 1100, |el| tiny: eh = (32 q + j) / 32 + r, 2^(j/32) as a pair from the table, 2^r - 1 from
// seven terms, the exponent q through ldexp (which also rounds a subnormal result and overflows to infinity)
__device__ __forceinline__ double exp2_of_pair(double eh, double el, const double* tab) {
    const double big = 211106232532992.0;  // 1.5 * 2^47: the last mantissa bit is worth 1/32
    const double t0 = eh + big;
    const uint32_t ki = (uint32_t)__double2loint(t0);
    const double r = (eh - (t0 - big)) + el;
    double p = CUMO_HIP_EXP2DD_F7;
    p = __builtin_fma(p, r, CUMO_HIP_EXP2DD_F6);
    p = __builtin_fma(p, r, CUMO_HIP_EXP2DD_F5);
    p = __builtin_fma(p, r, CUMO_HIP_EXP2DD_F4);
    p = __builtin_fma(p, r, CUMO_HIP_EXP2DD_F3);
    p = __builtin_fma(p, r, CUMO_HIP_EXP2DD_F2);
    p = __builtin_fma(p, r, CUMO_HIP_EXP2DD_F1);
    p *= r;
    const uint32_t j = ki & 31u;
    const double th = tab[2 * j], tl = tab[2 * j + 1];
    return ldexp(th + __builtin_fma(th, p, tl), (int)ki >> 5);
}
__device__ __forceinline__ double pow_double_fast(double x, double y) {
    double lh, ll;
    log2_pair(x, log2_pair_table(), lh, ll);
    double eh = y * lh;
    double el = __builtin_fma(y, ll, __builtin_fma(y, lh, -eh));
    // beyond the double range either way (also an infinite product, whose remainder is not a number)
    const bool far = !(__builtin_fabs(eh) <= 1100.0);
    eh = far ? __builtin_copysign(1100.0, eh) : eh;
    el = far ? 0.0 : el;
    return exp2_of_pair(eh, el, exp_pair_table());
}
// every other argument (zero, negative, subnormal, infinite or NaN base; infinite or NaN exponent) goes to the library
__device__ __forceinline__ bool pow_double_is_rare(double x, double y) {
    return !((uint32_t)__double2hiint(x) - 0x00100000u < 0x7fe00000u && __builtin_fabs(y) < (double)INFINITY);
}

// ---- DFloat erfc --------------------------------------------------------------------------
// erfc|x| = e^(-x^2) g(|x|), g(x) = e^(x^2) erfc(x), which varies slowly: 1 at 0, 1 / (x sqrt(pi)) far out.
//   x^2 exactly as a pair (one multiply-add for the product's rounding error), the exponential of its negative as a
//   pair (the reduction and table of expm1_pair; 2^128 times too large, so that 2^m stays a normal number down to the
//   smallest subnormal result: ldexp at the end takes the 128 off and rounds a subnormal result);
//   g from the Taylor series about the centre c of |x|'s interval (centres 0, 1/16 ... 1 below 1 + 1/32, 32 intervals a
//   binade from there: |x| - c is exact and at most 1/32, or 1/64 of c): g(c) as a pair plus d times a polynomial of
//   degree 9 in double, whose rounding shows as 0.02 ulp at most;
//   the product of the two pairs rounded once; erfc(-|x|) = 2 - erfc|x|, the subtraction exact before its rounding.
// The reference calls the CUDA library's erfc (ext/cumo/include/cumo/types/float_macro_kernel.h:120).
__device__ __forceinline__ void exp_pair_scaled_up(double ah, double al, const double* tab, double& hi, double& lo) {
    const double big = 6755399441055744.0;  // 1.5 * 2^52
    const double t0 = __builtin_fma(ah, CUMO_HIP_32_LN2, big);
    const uint32_t ki = (uint32_t)__double2loint(t0);
    const double kd = t0 - big;
    const double rh = __builtin_fma(-kd, CUMO_HIP_LN2_32_HI, ah);
    const double tail = kd * CUMO_HIP_LN2_32_LO;
    // (al is not small beside the reduction's own remainder: it joins r before the polynomial sees it)
    const double r0 = rh - tail;
    const double rl0 = ((rh - r0) - tail) + al;
    const double r = r0 + rl0;
    const double rl = (r0 - r) + rl0;
    double q = 1.0 / 5040.0;
    q = __builtin_fma(q, r, 1.0 / 720.0);
    q = __builtin_fma(q, r, 1.0 / 120.0);
    q = __builtin_fma(q, r, 1.0 / 24.0);
    q = __builtin_fma(q, r, 1.0 / 6.0);
    q = __builtin_fma(q, r, 0.5);
    const double pl = __builtin_fma(r * r, q, rl);  // e^r - 1 - r
    const uint32_t j = ki & 31u;
    const int m = ((int)ki >> 5) + 128;
    const double scale = __hiloint2double((m + 1023) << 20, 0);
    const double sh = tab[2 * j] * scale, sl = tab[2 * j + 1] * scale;
    const double p = sh * r;
    const double pe = __builtin_fma(sh, r, -p);
    const double s1 = sh + p;
    const double rest = (p - (s1 - sh)) + __builtin_fma(sl, 1.0 + r, __builtin_fma(sh, pl, pe));
    hi = s1 + rest;
    lo = (s1 - hi) + rest;
}
__device__ __forceinline__ double erfc_double(double x) {
    const double* tab = erfc_table();
    double a = __builtin_fabs(x);
    a = __builtin_fmin(a, 27.5);   // beyond 27.3 the answer is 0 (a NaN becomes 27.5 here and is put back at the end)
    // the interval: the nearest sixteenth below 1 + 1/32, the binade and five mantissa bits above
    const uint32_t near = (uint32_t)__double2loint(__builtin_fma(a, 16.0, 6755399441055744.0)) & 31u;
    const uint32_t far = 17u + (((uint32_t)__double2hiint(a) - 0x3ff00000u) >> 15);
    const double* row = tab + (a < 1.03125 ? near : far) * (uint32_t)kErfcRowDoubles;
    const double d = a - row[0];
    double p = row[2 + CUMO_HIP_ERFC_DEGREE];
#pragma unroll
    for (int n = CUMO_HIP_ERFC_DEGREE - 1; n >= 1; --n) p = __builtin_fma(p, d, row[2 + n]);
    const double gt = __builtin_fma(d, p, row[2]);
    const double gh = row[1] + gt;
    const double gl = (row[1] - gh) + gt;
    const double xh = a * a;
    const double xl = __builtin_fma(a, a, -xh);
    double eh, el;
    exp_pair_scaled_up(-xh, -xl, exp_pair_table(), eh, el);
    const double ph = eh * gh;
    const double pe = __builtin_fma(eh, gl, __builtin_fma(el, gh, __builtin_fma(eh, gh, -ph)));
    const double rh = ph + pe;
    const double rl = (ph - rh) + pe;
    const double yh = ldexp(rh, -128), yl = ldexp(rl, -128);
    // 2 - (yh + yl) for a negative argument
    const double s = 2.0 - yh;
    const double below = s + (((2.0 - s) - yh) - yl);
    const double y = (x < 0.0) ? below : yh;
    return (x != x) ? x : y;
}

// ---- DFloat log1p, asinh, acosh, atanh ------------------------------------------------------
// Each is the logarithm of a quantity u that is built as a pair (uh + ul, |ul| within a few units in uh's last place):
// ln u = ln 2 * log2 uh + ul / uh, the first term from log2_pair (good to 2^-66 of its value, next to 1 included) times
// ln 2 as a pair, and one rounding at the end. The reference calls the CUDA library's functions
// (ext/cumo/include/cumo/types/float_macro_kernel.h:107-118).
__device__ __forceinline__ double ln_of_pair(double uh, double ul, int more_binades = 0) {
    double lh, ll;
    log2_pair(uh, log2_pair_table(), lh, ll, more_binades);
    const double ln2h = 0x1.62e42fefa39efp-1, ln2l = 0x1.abc9e3b39803fp-56;
    const double ph = lh * ln2h;
    const double pe = __builtin_fma(ll, ln2h, __builtin_fma(lh, ln2l, __builtin_fma(lh, ln2h, -ph)));
    return ph + __builtin_fma(ul, rcp_refined(uh), pe);
}
// a + b exactly as s + e for |a| >= |b| (or a == 0)
__device__ __forceinline__ void exact_sum_ordered(double a, double b, double& s, double& e) {
    s = a + b;
    e = b - (s - a);
}
// sqrt(wh + wl) as a pair for a positive normal wh: the refined estimate, then what its square leaves of w, exactly
__device__ __forceinline__ void sqrt_pair(double wh, double wl, double& sh, double& sl) {
#ifdef CUMO_HIP_HOST_CHECK
    sh = sqrt(wh);
    const double half_over = 0.5 / sh;
#else
    const double y = __builtin_amdgcn_rsq(wh);
    const double g = wh * y;
    sh = __builtin_fma(__builtin_fma(-g, g, wh) * 0.5, y, g);
    const double half_over = 0.5 * y;
#endif
    sl = (__builtin_fma(-sh, sh, wh) + wl) * half_over;
}
// log1p: u = 1 + x exactly as a pair; below 2^-54 the answer is x itself (the sign of a zero included)
__device__ __forceinline__ double log1p_double(double x) {
    double uh, ul;
    exact_sum(1.0, x, uh, ul);
    const bool fine = uh >= 2.2250738585072014e-308 && uh < (double)INFINITY;   // (x > -1, finite)
    double y = ln_of_pair(fine ? uh : 1.0, fine ? ul : 0.0);
    y = (__builtin_fabs(x) < 0x1p-54) ? x : y;
    y = (x == -1.0) ? (double)-INFINITY : y;
    y = (x < -1.0) ? (double)NAN : y;
    y = (x == (double)INFINITY) ? x : y;
    return (x != x) ? x : y;
}
// asinh|x| = ln(1 + v), v = |x| + x^2 / (1 + sqrt(1 + x^2)), every step a pair; beyond 2^500 (where x^2 would leave the
// range) ln(2|x|); below 2^-28 x itself
__device__ __forceinline__ double asinh_double(double x) {
    const double a = __builtin_fabs(x);
    const bool huge = !(a <= 0x1p500);   // (a NaN too: it is put back at the end)
    const double am = huge ? 1.0 : a;
    const double x2h = am * am;
    const double x2l = __builtin_fma(am, am, -x2h);
    double wh, wl, sh, sl, dh, dl, qh, ql, vh, vl, uh, ul;
    exact_sum(1.0, x2h, wh, wl);
    sqrt_pair(wh, wl + x2l, sh, sl);
    exact_sum_ordered(sh, 1.0, dh, dl);
    pair_quotient_pair(x2h, x2l, dh, dl + sl, qh, ql);
    exact_sum_ordered(am, qh, vh, vl);
    exact_sum(1.0, vh, uh, ul);
    ul += vl + ql;
    const bool far = huge && a < (double)INFINITY;
    double y = ln_of_pair(far ? a : uh, far ? 0.0 : ul, far ? 1 : 0);
    y = (a < 0x1p-28) ? a : y;
    y = (a == (double)INFINITY) ? a : y;
    y = __builtin_copysign(y, x);
    return (x != x) ? x : y;
}
// acosh x = ln(x + sqrt(x^2 - 1)), x^2 - 1 exactly as a pair; beyond 2^500 ln(2x)
__device__ __forceinline__ double acosh_double(double x) {
    const bool huge = !(x <= 0x1p500);
    const bool inside = x >= 1.0;
    const double am = (huge || !inside) ? 1.0 : x;
    const double x2h = am * am;
    const double x2l = __builtin_fma(am, am, -x2h);
    double wh, wl, sh, sl, uh, ul;
    exact_sum_ordered(x2h, -1.0, wh, wl);
    wl += x2l;
    // (x next to 1: the head may cancel to nothing while the tail does not)
    const double w0 = wh + wl;
    const double w1 = (wh - w0) + wl;
    const bool none = !(w0 > 0.0);
    sqrt_pair(none ? 1.0 : w0, none ? 0.0 : w1, sh, sl);
    sh = none ? 0.0 : sh;
    sl = none ? 0.0 : sl;
    exact_sum_ordered(am, sh, uh, ul);
    ul += sl;
    const bool far = huge && x < (double)INFINITY;
    double y = ln_of_pair(far ? x : uh, far ? 0.0 : ul, far ? 1 : 0);
    y = (x == (double)INFINITY) ? x : y;
    y = (x < 1.0) ? (double)NAN : y;
    return (x != x) ? x : y;
}
// atanh|x| = ln((1 + |x|) / (1 - |x|)) / 2, numerator, denominator and quotient as pairs; below 2^-28 x itself
__device__ __forceinline__ double atanh_double(double x) {
    const double a = __builtin_fabs(x);
    const bool inside = a < 1.0;
    const double am = inside ? a : 0.5;
    double nh, nl, dh, dl, qh, ql;
    exact_sum_ordered(1.0, am, nh, nl);
    exact_sum_ordered(1.0, -am, dh, dl);
    pair_quotient_pair(nh, nl, dh, dl, qh, ql);
    // (the quotient's head and tail overlap by a few bits: ln_of_pair's u wants them apart)
    const double uh = qh + ql;
    const double ul = (qh - uh) + ql;
    double y = 0.5 * ln_of_pair(uh, ul);
    y = (a < 0x1p-28) ? a : y;
    y = (a == 1.0) ? (double)INFINITY : y;
    y = (a > 1.0) ? (double)NAN : y;
    y = __builtin_copysign(y, x);
    return (x != x) ? x : y;
}

// ---- DFloat ** y for one exponent that is a whole number of halves, up to 8 either way ---------------------
// (x ** 0.5, x ** -1.5, x ** 2.5): the whole part by squarings and multiplications of pairs (the first square is exact),
// the half by sqrt_pair, a negative exponent by a reciprocal corrected with its exact remainder, one rounding at the
// end. For bases between 2^-100 and 2^100 (no intermediate leaves the normal range there); every other base is the
// device library's pow, out of line.
__device__ __forceinline__ void pair_product(double ah, double al, double bh, double bl, double& ph, double& pl) {
    const double p = ah * bh;
    const double e = __builtin_fma(ah, bl, __builtin_fma(al, bh, __builtin_fma(ah, bh, -p)));
    ph = p + e;
    pl = (p - ph) + e;
}
template <bool NEG>
__device__ __forceinline__ double pow_halves_double_fast(double x, int twice) {
    const unsigned m = (unsigned)(twice < 0 ? -twice : twice);
    double rh = 1.0, rl = 0.0, bh = x, bl = 0.0;
    for (unsigned q = m >> 1; q != 0; q >>= 1) {   // (the same turns for every lane)
        if (q & 1u) pair_product(rh, rl, bh, bl, rh, rl);
        if (q > 1u) pair_product(bh, bl, bh, bl, bh, bl);
    }
    if (m & 1u) {
        double sh, sl;
        sqrt_pair(x, 0.0, sh, sl);
        pair_product(rh, rl, sh, sl, rh, rl);
    }
    if (NEG) {
        // 1 / (rh + rl): the estimate's remainder, exactly, times the estimate again
        const double q = rcp_refined(rh);
        const double left = __builtin_fma(-q, rl, __builtin_fma(-q, rh, 1.0));
        return __builtin_fma(left, q, q);
    }
    return rh + rl;
}
__device__ __forceinline__ bool pow_halves_double_is_rare(double x) {
    // positive, between 2^-100 and 2^100 (a NaN fails)
    return !(x >= 0x1p-100 && x <= 0x1p100);
}
