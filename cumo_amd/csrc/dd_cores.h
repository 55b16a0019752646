// DFloat tanh, sinh and cosh from an exponential carried as a pair of doubles (a value and what
// is left of it), so that the one rounding of the result is the only one that shows: about 60
// double operations an element where the device library's versions, which work on such pairs
// throughout, take some 300. The reference calls the CUDA library's tanh / sinh / cosh
// (ext/cumo/include/cumo/types/float_macro_kernel.h:101-106).
//
// Every step is an IEEE operation except the reciprocal estimate, which only enters through a
// correction term; a CPU build (CUMO_HIP_HOST_CHECK) computes the same up to that.
// Included by ew_ops.h, inside namespace cumo_hip, after the tables of float_tables.inc.
#pragma once

constexpr int kExpPairTableDoubles = 64;
#ifdef CUMO_HIP_HOST_CHECK
static const double kExpPairTableHost[kExpPairTableDoubles] = {CUMO_HIP_EXPDD_TABLE};
inline const double* exp_pair_table() { return kExpPairTableHost; }
#else
__device__ const double kExpPairTableDevice[kExpPairTableDoubles] = {CUMO_HIP_EXPDD_TABLE};
__device__ __forceinline__ double* exp_pair_table_lds() {
    __shared__ double table[kExpPairTableDoubles];
    return table;
}
__device__ __forceinline__ const double* exp_pair_table() { return exp_pair_table_lds(); }
// with all threads of the block, before the first element
__device__ __forceinline__ void exp_pair_table_prepare() {
    double* t = exp_pair_table_lds();
    for (unsigned i = threadIdx.x; i < (unsigned)kExpPairTableDoubles; i += blockDim.x) t[i] = kExpPairTableDevice[i];
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
