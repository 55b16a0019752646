// Element functors for the elementwise kernels.
//
// Semantics follow the reference's device macros
// (ext/cumo/include/cumo/types/float_macro_kernel.h:28-123,
// xint_macro_kernel.h:15-42, int_macro_kernel.h:8-27) with one deliberate
// difference: for SFloat, every libm function is evaluated in double and
// rounded once, which is what the host macros (types/float_macro.h:84-118)
// compile to on the CPU that Numo runs on, instead of the device's float
// overload. The kernels are bandwidth bound, so the wider evaluation is free.
#ifndef CUMO_HIP_EW_OPS_H
#define CUMO_HIP_EW_OPS_H

// CUMO_HIP_HOST_CHECK: a CPU build of the element functions, for tests that run the
// float algorithms below on the host against reference values. The including file then
// supplies __device__, __forceinline__ and the bit-cast intrinsics.
#ifndef CUMO_HIP_HOST_CHECK
#include <hip/hip_runtime.h>
#endif
#include <stdint.h>
#include <float.h>

#include "div31.h"

namespace cumo_hip {

// 1 / x to about one ulp (v_rcp_f32); only used where that is more than enough
__device__ __forceinline__ float rcp_approx(float x) {
#ifdef CUMO_HIP_HOST_CHECK
    return 1.0f / x;
#else
    return __builtin_amdgcn_rcpf(x);
#endif
}
// 1 / b for a finite, normal, non-zero double to about 2^-44: the hardware's estimate (good to
// some 2^-23) and one Newton step, 6 instructions where the IEEE division takes about 25. For
// results that are rounded to float afterwards.
__device__ __forceinline__ double rcp_refined(double b) {
#ifdef CUMO_HIP_HOST_CHECK
    return 1.0 / b;
#else
    const double r = __builtin_amdgcn_rcp(b);
    return __builtin_fma(__builtin_fma(-b, r, 1.0), r, r);
#endif
}
// sqrt(a) for a positive, finite, normal double to about 2^-44, the same way
__device__ __forceinline__ double sqrt_refined(double a) {
#ifdef CUMO_HIP_HOST_CHECK
    return sqrt(a);
#else
    const double y = __builtin_amdgcn_rsq(a);
    const double s = a * y;
    return __builtin_fma(__builtin_fma(-s, s, a) * 0.5, y, s);
#endif
}
// (double)k without the quarter-rate conversion: 2^52 + 2^31 + k sits in the mantissa
__device__ __forceinline__ double int_to_double(int k) {
    return __hiloint2double(0x43300000, (int)((uint32_t)k ^ 0x80000000u)) - 4503601774854144.0;
}

// ---- table-driven log2 and exp2 (for results that are rounded to float) ------------------
// 64 entries {1 / c, log2 c} for the logarithm and 32 values 2^(j/32) for the exponential take
// the place of a division and of half a polynomial each (float_tables.inc, written by
// make_float_tables.py, says how they are laid out). On the device the tables live in LDS: an
// operator that reads them declares USES_TABLES, and a kernel that runs such an operator
// calls float_tables_prepare() with all its threads before the first element.
#include "float_tables.inc"
constexpr int kFloatTableDoubles = 128 + 32;
#ifdef CUMO_HIP_HOST_CHECK
static const double kFloatTablesHost[kFloatTableDoubles] = {CUMO_HIP_LOG2_TABLE, CUMO_HIP_EXP2_TABLE};
inline const double* float_tables() { return kFloatTablesHost; }
#else
__device__ const double kFloatTablesDevice[kFloatTableDoubles] = {CUMO_HIP_LOG2_TABLE, CUMO_HIP_EXP2_TABLE};
__device__ __forceinline__ double* float_tables_lds() {
    __shared__ double tables[kFloatTableDoubles];
    return tables;
}
__device__ __forceinline__ const double* float_tables() { return float_tables_lds(); }
__device__ __forceinline__ void float_tables_prepare() {
    double* t = float_tables_lds();
    for (unsigned i = threadIdx.x; i < (unsigned)kFloatTableDoubles; i += blockDim.x) t[i] = kFloatTablesDevice[i];
    __syncthreads();
}
#endif
// log2(x) for a positive, finite, normal double to 2^-44 relative (also next to 1, where the
// entry {1, 0} leaves the polynomial alone): 8 multiply-adds and one 16-byte table read.
__device__ __forceinline__ double log2_by_table(double x, const double* tab) {
    const uint32_t hx = (uint32_t)__double2hiint(x);
    const uint32_t t = hx - 0x3fe6a000u;
    const int k = (int)t >> 20;
    const uint32_t i = (t >> 14) & 63u;
    const double m = __hiloint2double((int)(hx - (t & 0xfff00000u)), __double2loint(x));
    const double invc = tab[2 * i], logc = tab[2 * i + 1];
    const double z = __builtin_fma(m, invc, -1.0);
    double p = CUMO_HIP_LOG2_L6;
    p = __builtin_fma(p, z, CUMO_HIP_LOG2_L5);
    p = __builtin_fma(p, z, CUMO_HIP_LOG2_L4);
    p = __builtin_fma(p, z, CUMO_HIP_LOG2_L3);
    p = __builtin_fma(p, z, CUMO_HIP_LOG2_L2);
    p = __builtin_fma(p, z, CUMO_HIP_LOG2_L1);
    return __builtin_fma(z, p, logc + int_to_double(k));
}
// 2^e for -1000 < e < 1000 to 2^-39 relative: e = (32 q + j) / 32 + r with |r| <= 1/64 from one
// addition of 1.5 * 2^47 (whose last mantissa bit is worth 1/32), 2^(j/32) from the table with
// q added to its exponent field, 2^r from four multiply-adds.
__device__ __forceinline__ double exp2_by_table(double e, const double* tab) {
    const double big = 211106232532992.0;  // 1.5 * 2^47
    const double t0 = e + big;
    const uint32_t ki = (uint32_t)__double2loint(t0);
    const double r = e - (t0 - big);
    const double sj = tab[128 + (ki & 31u)];
    const double s = __hiloint2double((int)((uint32_t)__double2hiint(sj) + (uint32_t)(((int)ki >> 5) << 20)), __double2loint(sj));
    double p = CUMO_HIP_EXP2_E4;
    p = __builtin_fma(p, r, CUMO_HIP_EXP2_E3);
    p = __builtin_fma(p, r, CUMO_HIP_EXP2_E2);
    p = __builtin_fma(p, r, CUMO_HIP_EXP2_E1);
    return __builtin_fma(s * r, p, s);
}

#include "dd_cores.h"

#define CUMO_HIP_OP_COMMON(TA, TB, TR, NIN_, BIT_, CHK_) \
    typedef TA A; typedef TB B; typedef TR R; typedef TA S; \
    static constexpr int NIN = NIN_; static constexpr bool BIT_OUT = BIT_; static constexpr bool CHECKED = CHK_;

// ---- binary, float ---------------------------------------------------------
#define CUMO_HIP_FBIN(NAME, EXPR) \
    template <class T> struct NAME { CUMO_HIP_OP_COMMON(T, T, T, 2, false, false) \
        __device__ __forceinline__ bool operator()(T x, T y, T& z) const { z = (T)(EXPR); return true; } };
CUMO_HIP_FBIN(OpAdd, x + y)
CUMO_HIP_FBIN(OpSub, x - y)
CUMO_HIP_FBIN(OpMul, x * y)
CUMO_HIP_FBIN(OpDiv, x / y)
// (OpFMod: further down, with its SFloat core)
CUMO_HIP_FBIN(OpCopysign, copysign((double)x, (double)y))
// (OpAtan2 and OpHypot: further down, beside the cores they share with atan)
// the second operand arrives in the float type and converts to int (types/float_macro_kernel.h:122)
CUMO_HIP_FBIN(OpLdexp, ldexp((double)x, (int)y))

// ---- binary, int32 (wrapping arithmetic done in unsigned) -------------------
#define CUMO_HIP_IBIN(NAME, EXPR) \
    struct NAME { CUMO_HIP_OP_COMMON(int32_t, int32_t, int32_t, 2, false, false) \
        __device__ __forceinline__ bool operator()(int32_t x, int32_t y, int32_t& z) const { z = (int32_t)(EXPR); return true; } };
CUMO_HIP_IBIN(OpIAdd, (uint32_t)x + (uint32_t)y)
CUMO_HIP_IBIN(OpISub, (uint32_t)x - (uint32_t)y)
CUMO_HIP_IBIN(OpIMul, (uint32_t)x * (uint32_t)y)
CUMO_HIP_IBIN(OpIAnd, x & y)
CUMO_HIP_IBIN(OpIOr, x | y)
CUMO_HIP_IBIN(OpIXor, x ^ y)
CUMO_HIP_IBIN(OpIShl, (uint32_t)x << (y & 31))
CUMO_HIP_IBIN(OpIShr, x >> (y & 31))

// division by zero rejects the element and raises the flag
// (reference: narray/gen/tmpl/binary_kernel.cu:3-8)
struct OpIDiv { CUMO_HIP_OP_COMMON(int32_t, int32_t, int32_t, 2, false, true)
    __device__ __forceinline__ bool operator()(int32_t x, int32_t y, int32_t& z) const {
        if (y == 0) return false;
        z = (x == INT32_MIN && y == -1) ? INT32_MIN : x / y;
        return true; } };
struct OpIMod { CUMO_HIP_OP_COMMON(int32_t, int32_t, int32_t, 2, false, true)
    __device__ __forceinline__ bool operator()(int32_t x, int32_t y, int32_t& z) const {
        if (y == 0) return false;
        z = (y == -1) ? 0 : x % y;
        return true; } };

// Division and remainder by one divisor for the whole launch (array / 7, array % 7), the divisor neither 0 nor the
// element being rejected: the quotient of the magnitudes by a multiplication and a shift (div31.h: exact up to 2^31,
// which is the magnitude of the smallest Int32), the sign put back; the remainder from the quotient. Truncating, as
// the C operators the reference's macros use (types/int_macro_kernel.h m_div, m_mod); every result wraps like theirs.
struct OpIDivBy { CUMO_HIP_OP_COMMON(int32_t, int32_t, int32_t, 1, false, false)
    Div31 magic;
    int32_t d;
    __device__ __forceinline__ uint32_t quotient(int32_t x) const {
        const uint32_t ax = x < 0 ? 0u - (uint32_t)x : (uint32_t)x;
        const uint32_t q = div31(ax, magic);
        return ((x ^ d) < 0) ? 0u - q : q;
    }
    __device__ __forceinline__ bool operator()(int32_t x, int32_t, int32_t& z) const { z = (int32_t)quotient(x); return true; } };
struct OpIModBy : OpIDivBy {
    __device__ __forceinline__ bool operator()(int32_t x, int32_t, int32_t& z) const {
        z = (int32_t)((uint32_t)x - quotient(x) * (uint32_t)d);
        return true; } };

// ---- unary -----------------------------------------------------------------
#define CUMO_HIP_FUN(NAME, EXPR) \
    template <class T> struct NAME { CUMO_HIP_OP_COMMON(T, T, T, 1, false, false) \
        __device__ __forceinline__ bool operator()(T x, T, T& z) const { z = (T)(EXPR); return true; } };
CUMO_HIP_FUN(OpMinus, -x)
CUMO_HIP_FUN(OpReciprocal, 1 / x)
CUMO_HIP_FUN(OpSquare, x * x)
CUMO_HIP_FUN(OpSign, (x == 0) ? 0.0 : ((x > 0) ? 1.0 : ((x < 0) ? -1.0 : (double)x)))
CUMO_HIP_FUN(OpFAbs, fabs((double)x))
CUMO_HIP_FUN(OpFloor, floor((double)x))
CUMO_HIP_FUN(OpRound, round((double)x))
CUMO_HIP_FUN(OpCeil, ceil((double)x))
CUMO_HIP_FUN(OpTrunc, trunc((double)x))
CUMO_HIP_FUN(OpRint, rint((double)x))
// NMath (reference list: narray/gen/spec.rb:427-457). HEAVY: many instructions per element.
#define CUMO_HIP_FUN_H(NAME, EXPR) \
    template <class T> struct NAME { CUMO_HIP_OP_COMMON(T, T, T, 1, false, false) static constexpr bool HEAVY = true; \
        __device__ __forceinline__ bool operator()(T x, T, T& z) const { z = (T)(EXPR); return true; } };
CUMO_HIP_FUN(OpSqrt, sqrt((double)x))
CUMO_HIP_FUN_H(OpCbrt, cbrt((double)x))
// SFloat exp: the double-precision exp of the argument, rounded to float once.
// The argument has 24 significant bits, so k = rint(x / ln 2) times the upper part
// of ln 2 is exact; exp(r) on |r| <= ln(2)/2 is a degree-10 polynomial (2^-50; four
// multiply-adds fewer than the Taylor polynomial of the same accuracy), scaled by 2^k. Only full-rate instructions besides the
// two conversions: k is rounded by adding 1.5 * 2^52 (its integer value is then
// the low word of the sum), and 2^k is applied by adding k to the exponent field,
// which is safe because the clamp keeps the result a normal double. Outside
// [-105, 89] the float answer is already 0 or inf. No branch anywhere, so the
// elements of a vector are evaluated side by side: NaN goes through the clamp
// (the comparisons are false) and comes back in through xc - xc at the end,
// which is +0 for every other argument.
__device__ __forceinline__ float exp_float_rounded_once(float xf) {
    float xc = (xf < -105.0f) ? -105.0f : xf;
    xc = (xc > 89.0f) ? 89.0f : xc;
    const double x = (double)xc;
    const double big = 6755399441055744.0;  // 1.5 * 2^52
    const double t = __builtin_fma(x, 1.44269504088896338700e+00, big);
    const double k = t - big;
    const int ki = (int)(uint32_t)__double_as_longlong(t);
    double r = __builtin_fma(k, -6.93147180369123816490e-01, x);  // ln 2, upper 32 bits
    r = __builtin_fma(k, -1.90821492927058770002e-10, r);         // ln 2, the rest
    // exp(r) = 1 + r (1 + r E(r)) with a degree-8 fit of E = (exp(r) - 1 - r) / r^2 (2^-50 relative on |r| <= ln(2)/2)
    double p = 2.762343374154865e-07;
    p = __builtin_fma(p, r, 2.7625077174598027e-06);
    p = __builtin_fma(p, r, 2.480151290638607e-05);
    p = __builtin_fma(p, r, 0.00019841208813878425);
    p = __builtin_fma(p, r, 0.00138888889238219);
    p = __builtin_fma(p, r, 0.008333333353676958);
    p = __builtin_fma(p, r, 0.04166666666660734);
    p = __builtin_fma(p, r, 0.16666666666648428);
    p = __builtin_fma(p, r, 0.5000000000000002);
    p = __builtin_fma(p, r, 1.0);
    p = __builtin_fma(p, r, 1.0);
    const int hi = __double2hiint(p) + (ki << 20);
    const float y = (float)__hiloint2double(hi, __double2loint(p));
    return y + (xc - xc);
}
// SFloat log, log2, log10: the double-precision logarithm of the argument, rounded to
// float once, by the classic reduction x = 2^k (1 + f), sqrt(2)/2 < 1 + f < sqrt(2),
// s = f / (2 + f), log(1 + f) = f - f^2/2 + s (f^2/2 + R(s^2)) with a degree-7 polynomial R
// (the public fdlibm scheme and coefficients), every step an IEEE double operation, no
// branch on the data. BASE 0: k ln2 + log(1 + f) with ln2 in two parts; BASE 2:
// k + log(1 + f) / ln2 in one fused multiply-add; BASE 10: k log10(2) in two parts plus
// log(1 + f) / ln10. Run on the CPU against glibc's log, log2 and log10 over every
// non-negative float bit pattern, the float results differ nowhere. A subnormal float is
// a normal double, so only 0, negative arguments, infinity and NaN are special.
template <int BASE>
__device__ __forceinline__ double log_core(double x, int kadj = 0) {  // x positive, finite, normal; answers log(x) + kadj log(2)
    uint32_t hx = (uint32_t)__double2hiint(x);
    int k = (int)(hx >> 20) - 1023 + kadj;
    hx &= 0x000fffffu;
    const uint32_t i = (hx + 0x95f64u) & 0x100000u;  // mantissa >= sqrt(2): halve it
    k += (int)(i >> 20);
    const double m = __hiloint2double((int)(hx | (i ^ 0x3ff00000u)), __double2loint(x));
    const double f = m - 1.0;
    const double s = f / (2.0 + f);
    const double dk = (double)k;
    const double z = s * s, w = z * z;
    const double t1 = w * __builtin_fma(w, __builtin_fma(w, 1.531383769920937332e-01, 2.222219843214978396e-01), 3.999999999940941908e-01);
    const double t2 = z * __builtin_fma(w, __builtin_fma(w, __builtin_fma(w, 1.479819860511658591e-01, 1.818357216161805012e-01),
                                                         2.857142874366239149e-01), 6.666666666666735130e-01);
    const double R = t2 + t1;
    const double hfsq = 0.5 * f * f;
    if (BASE == 2) {
        const double lm = f - (hfsq - s * (hfsq + R));
        return __builtin_fma(lm, 1.44269504088896338700e+00, dk);
    }
    if (BASE == 10) {
        const double lm = f - (hfsq - s * (hfsq + R));
        return __builtin_fma(dk, 3.69423907715893078616e-13, 4.34294481903251816668e-01 * lm) + dk * 3.01029995663611771306e-01;
    }
    return dk * 6.93147180369123816490e-01 - ((hfsq - (s * (hfsq + R) + dk * 1.90821492927058770002e-10)) - f);
}
// The same logarithm for a result that is rounded to float: log(1 + f) = 2 s + s z R(z), z = s^2,
// with a degree-4 fit of R (2^-43 relative on 0 <= z <= 0.0295), the division by the refined
// reciprocal and k converted through the mantissa trick: about half the instructions of the
// form above. x positive, finite and normal.
template <int BASE, bool EXTRA = false>
__device__ __forceinline__ double log_core_for_float(double x) {
    uint32_t hx = (uint32_t)__double2hiint(x);
    int k = (int)(hx >> 20) - 1023;
    hx &= 0x000fffffu;
    const uint32_t i = (hx + 0x95f64u) & 0x100000u;
    k += (int)(i >> 20);
    const double m = __hiloint2double((int)(hx | (i ^ 0x3ff00000u)), __double2loint(x));
    const double f = m - 1.0;
    const double d = 2.0 + f;
    double rd = rcp_refined(d);
    double R;
    if (EXTRA) {  // 2^-50: a second Newton step and one more term (for pow, whose exponent multiplies the error)
        rd = __builtin_fma(__builtin_fma(-d, rd, 1.0), rd, rd);
        R = 0.16625981808365656;
    }
    const double s = f * rd;
    const double z = s * s;
    if (EXTRA) {
        R = __builtin_fma(R, z, 0.181399072797897);
        R = __builtin_fma(R, z, 0.22222869146289312);
        R = __builtin_fma(R, z, 0.28571424071527063);
        R = __builtin_fma(R, z, 0.4000000001143263);
        R = __builtin_fma(R, z, 0.6666666666666199);
    } else {
        R = 0.19366868181730357;
        R = __builtin_fma(R, z, 0.22191171841584165);
        R = __builtin_fma(R, z, 0.2857175839580272);
        R = __builtin_fma(R, z, 0.3999999877669915);
        R = __builtin_fma(R, z, 0.6666666666739216);
    }
    const double lm = __builtin_fma(s * z, R, s + s);
    const double dk = int_to_double(k);
    if (BASE == 2) return __builtin_fma(lm, 1.44269504088896338700e+00, dk);
    if (BASE == 10) return __builtin_fma(dk, 3.01029995663981198017e-01, 4.34294481903251816668e-01 * lm);
    if (EXTRA) return __builtin_fma(dk, 6.93147180369123816490e-01, __builtin_fma(dk, 1.90821492927058770002e-10, lm));
    return __builtin_fma(dk, 6.93147180559945286227e-01, lm);
}
template <int BASE>
__device__ __forceinline__ float log_float_rounded_once(float xf) {
    // No branch on the data, so that the elements of a vector are evaluated side by side. A
    // subnormal float is a normal double. NaN comes back in through xf - xf (which is NaN for an
    // infinity too); then, on the float: 0 -> -inf, negative -> NaN, +inf -> +inf
    float y = (float)log_core_for_float<BASE>((double)xf) + (xf - xf);
    y = (xf == 0.0f) ? -INFINITY : y;
    y = (xf < 0.0f) ? NAN : y;
    y = (xf == INFINITY) ? INFINITY : y;
    return y;
}
// DFloat log, log2, log10: the same algorithm on a double argument (a subnormal one is
// scaled by 2^54 first). Against glibc on 2 * 10^8 random doubles per function (all
// binades, near 1, subnormals): log differs by at most 1 ulp, log2 and log10 by at most 2.
template <int BASE>
__device__ __forceinline__ double log_double(double x) {
    const bool sub = x < 2.2250738585072014e-308;  // subnormal (or zero or negative, settled below)
    const double xs = sub ? x * 18014398509481984.0 : x;
    double r = log_core<BASE>(xs, sub ? -54 : 0) + (x - x);
    r = (x == 0.0) ? (double)-INFINITY : r;
    r = (x < 0.0) ? (double)NAN : r;
    r = (x == (double)INFINITY) ? (double)INFINITY : r;
    return r;
}
// SFloat log1p: 1 + x is exact in double for |x| >= 2^-29 (a float has 24 bits), so the
// logarithm above applies to it unchanged; below that the answer rounds to x itself.
// Checked like the others, over every float bit pattern.
__device__ __forceinline__ float log1p_float_rounded_once(float xf) {
    float y = (float)log_core_for_float<0>(1.0 + (double)xf) + (xf - xf);
    y = (__builtin_fabsf(xf) < 1.862645149230957e-09f) ? xf : y;
    y = (xf == -1.0f) ? -INFINITY : y;
    y = (xf < -1.0f) ? NAN : y;
    y = (xf == INFINITY) ? INFINITY : y;
    return y;
}
#define CUMO_HIP_LOG_OP(NAME, BASE)                                                                                         \
    template <class T> struct NAME { CUMO_HIP_OP_COMMON(T, T, T, 1, false, false) static constexpr bool HEAVY = true;       \
        __device__ __forceinline__ bool operator()(T x, T, T& z) const {                                                    \
            if constexpr (sizeof(T) == 4) z = (T)log_float_rounded_once<BASE>((float)x);                                    \
            else z = (T)log_double<BASE>((double)x);                                                                        \
            return true; } };
CUMO_HIP_LOG_OP(OpLog, 0)
CUMO_HIP_LOG_OP(OpLog2, 2)
CUMO_HIP_LOG_OP(OpLog10, 10)
// (DFloat: log1p_double of dd_cores.h, which reads the table of the power's logarithm)
template <class T> struct OpLog1p { CUMO_HIP_OP_COMMON(T, T, T, 1, false, false) static constexpr bool HEAVY = true;
    static constexpr bool USES_POW_PAIR_TABLES = sizeof(T) == 8;
    __device__ __forceinline__ bool operator()(T x, T, T& z) const {
        if constexpr (sizeof(T) == 4) z = (T)log1p_float_rounded_once((float)x);
        else z = (T)log1p_double((double)x);
        return true; } };

// exp(x) - 1 for x inside [-745, 709] and a result that is rounded to float, from the reduction
// of exp above: with q = (exp(r) - 1) / r (a degree-8 fit, 2^-44 relative on |r| <= ln(2)/2),
// exp(x) - 1 = 2^k (1 + q r) - 1 = (2^k - 1) + (2^k q) r comes out of one fused multiply-add,
// without the cancellation of exp(x) - 1 near 0.
// EXPM1 false: exp(x) itself, 2^k (1 + q r), for x inside [-700, 700].
template <bool EXPM1>
__device__ __forceinline__ double exp_core_for_float(double x) {
    const double big = 6755399441055744.0;  // 1.5 * 2^52
    const double t0 = __builtin_fma(x, 1.44269504088896338700e+00, big);
    const double k = t0 - big;
    const uint32_t ki = (uint32_t)__double2loint(t0);  // k as a two's-complement integer (anything for a NaN, which r carries on)
    double r = __builtin_fma(k, -6.93147180369123816490e-01, x);
    r = __builtin_fma(k, -1.90821492927058770002e-10, r);
    double q = 2.7632704798457074e-06;
    q = __builtin_fma(q, r, 2.486788542787532e-05);
    q = __builtin_fma(q, r, 0.0001984119277622577);
    q = __builtin_fma(q, r, 0.0013888839087169604);
    q = __builtin_fma(q, r, 0.008333333363318172);
    q = __builtin_fma(q, r, 0.04166666678635317);
    q = __builtin_fma(q, r, 0.16666666666633861);
    q = __builtin_fma(q, r, 0.4999999999995511);
    q = __builtin_fma(q, r, 1.0);
    if (!EXPM1) {
        const double e = __builtin_fma(q, r, 1.0);
        return __hiloint2double((int)((uint32_t)__double2hiint(e) + (ki << 20)), __double2loint(e));
    }
    const double qs = __hiloint2double((int)((uint32_t)__double2hiint(q) + (ki << 20)), __double2loint(q));
    const double p2k = __hiloint2double((int)((1023u + ki) << 20), 0);
    return __builtin_fma(qs, r, p2k - 1.0);
}
__device__ __forceinline__ double expm1_core(double x) { return exp_core_for_float<true>(x); }

// SFloat tanh, sinh, cosh, expm1: the function evaluated in double (to 2^-43 or better) and
// rounded to float once, each from t = exp(a) - 1 above and one refined reciprocal:
// tanh|x| = t / (t + 2) with a = 2|x| (clamped at 40, where the answer is 1 in double already);
// sinh|x| = (t + t / (t + 1)) / 2 and cosh x = (e + 1 / e) / 2, e = t + 1, with a = |x| clamped
// at 90 (beyond float range either way); expm1 with a = x clamped to [-40, 89]. A NaN argument
// fails the clamps' comparisons and travels through the arithmetic.
__device__ __forceinline__ float tanh_float_rounded_once(float xf) {
    float ax = __builtin_fabsf(xf);
    ax = (ax > 20.0f) ? 20.0f : ax;
    const double t = expm1_core(2.0 * (double)ax);
    return __builtin_copysignf((float)(t * rcp_refined(t + 2.0)), xf);
}
__device__ __forceinline__ float sinh_float_rounded_once(float xf) {
    float ax = __builtin_fabsf(xf);
    ax = (ax > 90.0f) ? 90.0f : ax;
    const double t = expm1_core((double)ax);
    return __builtin_copysignf((float)(0.5 * __builtin_fma(t, rcp_refined(t + 1.0), t)), xf);
}
__device__ __forceinline__ float cosh_float_rounded_once(float xf) {
    float ax = __builtin_fabsf(xf);
    ax = (ax > 90.0f) ? 90.0f : ax;
    const double e = expm1_core((double)ax) + 1.0;
    return (float)(0.5 * (e + rcp_refined(e)));
}
__device__ __forceinline__ float expm1_float_rounded_once(float xf) {
    float xc = (xf < -40.0f) ? -40.0f : xf;
    xc = (xc > 89.0f) ? 89.0f : xc;
    const float y = (float)expm1_core((double)xc);
    return (xf == 0.0f) ? xf : y;  // keeps the sign of a zero argument
}
// SFloat asinh, acosh, atanh: the function evaluated in double and rounded to float once, on the
// logarithm above (the form for float results, refined reciprocal and square root). log(1 + u)
// for a double u >= 0 whose sum 1 + u is not exact: the part c of u that the sum w loses comes
// back as c / w. asinh|x| = log1p(a + a^2 / (1 + sqrt(1 + a^2))) and acosh x =
// log1p(t + sqrt(t^2 + 2 t)), t = x - 1 (exact), hold over the whole float range (a^2 and t^2
// are exact in double and stay far below its overflow); atanh|x| = log1p(2a / (1 - a)) / 2 with
// 1 - a exact. Below 2^-29 asinh and atanh round to the argument.
__device__ __forceinline__ double log1p_core(double u) {
    const double w = 1.0 + u;
    const double c = u - (w - 1.0);
    // c / w: c is below 2^-53 w, so the term only counts where u is small, and there 1 / w = 1 - u
    // will do (past u = 2^-10 it is below 2^-43 of the answer, past 1 it is left out)
    const double um = (u < 1.0) ? u : 1.0;
    // the logarithm from the table-driven core (2^-44 relative, next to 1 as well), times ln 2
    return __builtin_fma(c, 1.0 - um, 6.93147180559945286227e-01 * log2_by_table(w, float_tables()));
}
// asinh|x| = log(a + sqrt(1 + a^2)) directly from 2^-11 on: with the square root good to 2^-52 (a second refining
// step) the sum is off by 2^-52 next to 1, where the answer is about a, so by 2^-41 of the answer at most; the
// logarithm's table has 1.0 as the midpoint of an interval, so a sum next to 1 loses nothing. Below 2^-11
// a - a^3 / 6 (the next term is below 2^-44 of a). This saves the reciprocal and the lost-bits bookkeeping of
// the log1p form: 47 -> 39 vector instructions an element.
__device__ __forceinline__ float asinh_float_rounded_once(float xf) {
    const float af = __builtin_fabsf(xf);
    const double a = (double)af;
    const double a2 = a * a;
    const double w = 1.0 + a2;
#ifdef CUMO_HIP_HOST_CHECK
    const double s = sqrt(w);
#else
    const double r = __builtin_amdgcn_rsq(w);
    double s = w * r;
    s = __builtin_fma(__builtin_fma(-s, s, w) * 0.5, r, s);
    s = __builtin_fma(__builtin_fma(-s, s, w) * 0.5, r, s);
#endif
    // (the table-driven logarithm works on the argument's bits: a NaN comes back in through a - a, which is NaN for an infinity too)
    const double big = __builtin_fma(6.93147180559945286227e-01, log2_by_table(a + s, float_tables()), a - a);
    const double small = __builtin_fma(a2 * a, -1.0 / 6.0, a);
    float y = (float)((af < 4.8828125e-04f) ? small : big);   // NaN travels through; an infinity gives NaN here and is put right below
    y = (af == INFINITY) ? INFINITY : y;
    return __builtin_copysignf(y, xf);
}
// acosh x = log(x + sqrt((x - 1)(x + 1))): both factors and their product are exact in double, so the square root
// is good to 2^-44 of itself next to 1 as well, where it is the answer's leading term.
__device__ __forceinline__ float acosh_float_rounded_once(float xf) {
    const float xc = (xf < 1.0f) ? 1.0f : xf;  // keeps the square root's argument in range; a NaN stays
    const double x = (double)xc;
    const double q = (x - 1.0) * (x + 1.0);
    const double u = x + ((q > 0.0) ? sqrt_refined(q) : 0.0);   // a NaN gives 0 here and comes back through x
    float y = (float)__builtin_fma(6.93147180559945286227e-01, log2_by_table(u, float_tables()), x - x);   // (a NaN comes back in through x - x)
    y = (xf < 1.0f) ? NAN : y;
    y = (xf == INFINITY) ? INFINITY : y;
    return y;
}
__device__ __forceinline__ float atanh_float_rounded_once(float xf) {
    const float af = __builtin_fabsf(xf);
    const float ac = (af < 1.0f) ? af : 0.5f;   // a stand-in for |x| >= 1, settled below
    const double a = (double)ac;
    float y = (float)(0.5 * log1p_core((a + a) * rcp_refined(1.0 - a)));
    y = (af < 1.862645149230957e-09f) ? af : y;
    y = (af == 1.0f) ? INFINITY : y;
    y = (af > 1.0f) ? NAN : y;
    y = (xf != xf) ? xf : y;
    return __builtin_copysignf(y, xf);
}
// SFloat sin, cos, tan: evaluated in double and rounded to float once. Below 10^6 in magnitude:
// k = rint(x 2/pi) by the 1.5 * 2^52 trick, r = x - k pi/2 with pi/2 in two parts (the upper 33
// bits, so that k times it is exact), then sin r = r + r z S(z) and cos r = 1 - z/2 + z^2 C(z),
// z = r^2, from degree-4 and degree-3 fits (2^-35 and 2^-40 relative on |r| <= pi/4), both
// evaluated, the quadrant choosing between them and the sign. Beyond that the device library's
// double function (its argument reduction is a branch of its own). WHICH: 0 sin, 1 cos, 2 tan.
// (out of line for the same reason as the library's pow further down)
template <int WHICH>
__device__ __attribute__((noinline)) float trig_by_the_library(float xf) {
    if (WHICH == 0) return (float)sin((double)xf);
    if (WHICH == 1) return (float)cos((double)xf);
    return (float)tan((double)xf);
}
// the arithmetic alone, before the rounding to float: right below 10^6 in magnitude, some
// finite number or NaN beyond
template <int WHICH>
__device__ __forceinline__ double trig_core(float xf) {
    const double x = (double)xf;
    const double big = 6755399441055744.0;  // 1.5 * 2^52
    const double t = __builtin_fma(x, 6.36619772367581382433e-01, big);
    const double k = t - big;
    const uint32_t ki = (uint32_t)__double2loint(t);
    double r = __builtin_fma(k, -1.57079632673412561417e+00, x);  // pi/2, upper 33 bits
    r = __builtin_fma(k, -6.07710050650619224932e-11, r);         // pi/2, the rest
    const double z = r * r;
    double ps = -2.4805649861027395e-08;
    ps = __builtin_fma(ps, z, 2.7555991132757367e-06);
    ps = __builtin_fma(ps, z, -0.0001984126691790408);
    ps = __builtin_fma(ps, z, 0.008333333331080512);
    ps = __builtin_fma(ps, z, -0.16666666666663896);
    const double sn = __builtin_fma(r * z, ps, r);
    double pc = -2.7300987836458486e-07;
    pc = __builtin_fma(pc, z, 2.480060068144107e-05);
    pc = __builtin_fma(pc, z, -0.0013888887672811724);
    pc = __builtin_fma(pc, z, 0.04166666666432424);
    const double cs = __builtin_fma(z * z, pc, __builtin_fma(z, -0.5, 1.0));
    if (WHICH == 2) {
        const bool odd = (ki & 1u) != 0;
        return (odd ? -cs : sn) * rcp_refined(odd ? sn : cs);
    }
    // sin: quadrant 0 s, 1 c, 2 -s, 3 -c; cos is sin a quadrant further on
    const uint32_t q = WHICH == 0 ? ki : ki + 1u;
    const double v = (q & 1u) ? cs : sn;
    return __hiloint2double(__double2hiint(v) ^ (int)((q & 2u) << 30), __double2loint(v));
}
template <int WHICH>
__device__ __forceinline__ float trig_fast(float xf) {
    const float y = (float)trig_core<WHICH>(xf);
    return (WHICH != 1 && xf == 0.0f) ? xf : y;  // keeps the sign of a zero argument
}
__device__ __forceinline__ bool trig_is_rare(float xf) { return !(__builtin_fabsf(xf) < 1.0e6f); }  // large, infinite or NaN
template <int WHICH>
__device__ __forceinline__ float trig_float_rounded_once(float xf) {
    // the rare argument after the arithmetic, so that the elements of a vector are evaluated side by side
    float y = trig_fast<WHICH>(xf);
    if (trig_is_rare(xf)) y = trig_by_the_library<WHICH>(xf);
    return y;
}
// SFloat atan, the same way: one refined reciprocal brings the argument below tan(pi/8)
// (t = a there, (a - 1)/(a + 1) plus pi/4 up to tan(3 pi/8), -1/a plus pi/2 above), then
// atan t = t + t z A(z), z = t^2, with a degree-7 fit of A (2^-43 relative).
__device__ __forceinline__ float atan_float_rounded_once(float xf) {
    const float af = __builtin_fabsf(xf);
    const double a = (double)((af > 1.0e30f) ? 1.0e30f : af);  // the answer is pi/2 in float from 2^25 on; a NaN passes
    const bool mid = af > 0.41421356f, top = af > 2.41421356f;
    const double num = top ? -1.0 : (mid ? a - 1.0 : a);
    const double den = top ? a : (mid ? a + 1.0 : 1.0);
    const double off = top ? 1.57079632679489655800e+00 : (mid ? 7.85398163397448278999e-01 : 0.0);
    const double t = num * rcp_refined(den);
    const double z = t * t;
    double p = 0.033038827515269494;
    p = __builtin_fma(p, z, -0.06032248119994454);
    p = __builtin_fma(p, z, 0.07605969344616582);
    p = __builtin_fma(p, z, -0.09084239163280672);
    p = __builtin_fma(p, z, 0.11110827992295265);
    p = __builtin_fma(p, z, -0.1428570834807845);
    p = __builtin_fma(p, z, 0.19999999952417688);
    p = __builtin_fma(p, z, -0.33333333333270726);
    return __builtin_copysignf((float)(off + __builtin_fma(t * z, p, t)), xf);
}
// SFloat asin, acos, the same way: up to 1/2, asin a = a + a z P(z), z = a^2, with a degree-8 fit
// of P (2^-42 relative on z <= 1/4); beyond, the same series at s = sqrt((1 - a) / 2) (1 - a is
// exact, the square root refined) gives asin a = pi/2 - 2 asin s. acos x is 2 asin s above 1/2,
// pi - 2 asin s below -1/2 and pi/2 - asin x between.
template <bool ACOS>
__device__ __forceinline__ float asin_acos_float_rounded_once(float xf) {
    const float af = __builtin_fabsf(xf);
    const double a = (double)af;
    const bool outer = af > 0.5f;
    const double z = outer ? 0.5 * (1.0 - a) : a * a;
    const bool z_pos = z > 0.0;
    double s = sqrt_refined((outer && z_pos) ? z : 1.0);
    s = outer ? (z_pos ? s : 0.0) : a;     // (|x| = 1: s = 0; |x| > 1 is settled below; a NaN passes through a)
    double p = 0.02857943531987056;
    p = __builtin_fma(p, z, 0.0008360525284043926);
    p = __builtin_fma(p, z, 0.01695759046734276);
    p = __builtin_fma(p, z, 0.016883023346408812);
    p = __builtin_fma(p, z, 0.022414706851110307);
    p = __builtin_fma(p, z, 0.030379800562048823);
    p = __builtin_fma(p, z, 0.04464291095965551);
    p = __builtin_fma(p, z, 0.0749999994813725);
    p = __builtin_fma(p, z, 0.16666666666748844);
    const double as = __builtin_fma(s * z, p, s);   // asin s
    const double pio2 = 1.57079632679489655800e+00, pi = 3.14159265358979311600e+00;
    float y;
    if (ACOS) {
        const double neg = (xf < 0.0f) ? -as : as;
        const double r = outer ? ((xf < 0.0f) ? pi - 2.0 * as : 2.0 * as) : pio2 - neg;
        y = (float)r;
    } else {
        y = __builtin_copysignf((float)(outer ? pio2 - 2.0 * as : as), xf);
    }
    return (af > 1.0f) ? NAN : y;
}
// SFloat erf, the same way, in one form over the whole range: erf a = 1 - exp(-a S(a)) with a
// degree-14 fit of S = -log(erfc a) / a on [0, 4] (2^-41 relative in erf, near 0 included:
// S(0) = 2/sqrt(pi)) and exp(.) - 1 from the core above, which keeps the small results whole.
// In float, erf is 1 from 3.92 on.
__device__ __forceinline__ float erf_float_rounded_once(float xf) {
    const float af = __builtin_fabsf(xf);
    const double a = (double)((af > 4.0f) ? 4.0f : af);  // a NaN passes
    double sp = 1.2454485957275264e-09;
    sp = __builtin_fma(sp, a, -3.292031665613006e-08);
    sp = __builtin_fma(sp, a, 3.959960484006724e-07);
    sp = __builtin_fma(sp, a, -2.8566560041378794e-06);
    sp = __builtin_fma(sp, a, 1.3576807482500019e-05);
    sp = __builtin_fma(sp, a, -4.281130444734605e-05);
    sp = __builtin_fma(sp, a, 7.680414177713242e-05);
    sp = __builtin_fma(sp, a, 1.7468095488586178e-05);
    sp = __builtin_fma(sp, a, -0.0005860400176985031);
    sp = __builtin_fma(sp, a, 0.0016948435469004315);
    sp = __builtin_fma(sp, a, -0.00020889888424513057);
    sp = __builtin_fma(sp, a, -0.019128485397176796);
    sp = __builtin_fma(sp, a, 0.10277260588324502);
    sp = __builtin_fma(sp, a, 0.6366197723000346);
    sp = __builtin_fma(sp, a, 1.1283791670957979);
    return __builtin_copysignf((float)(-expm1_core(-a * sp)), xf);
}
// SFloat erfc, the same way: erfc a = t exp(-a^2 + P(t)), t = 2 / (2 + a), with a degree-16 fit
// of P on 0 <= a <= 10.2 (2^-39 relative in erfc; a^2 is exact in double, and beyond 10.06 the
// float answer is 0); erfc(-a) = 2 - erfc a.
__device__ __forceinline__ float erfc_float_rounded_once(float xf) {
    const float af = __builtin_fabsf(xf);
    const double a = (double)((af > 10.2f) ? 10.2f : af);  // a NaN passes
    const double t = 2.0 * rcp_refined(2.0 + a);
    double p = 0.08559139243524283;
    p = __builtin_fma(p, t, -0.6542044248194727);
    p = __builtin_fma(p, t, 1.9990352510531308);
    p = __builtin_fma(p, t, -2.5941568730621682);
    p = __builtin_fma(p, t, -0.8737363806023866);
    p = __builtin_fma(p, t, 8.652953555628644);
    p = __builtin_fma(p, t, -14.909187280785874);
    p = __builtin_fma(p, t, 14.312468419074285);
    p = __builtin_fma(p, t, -9.029793572490398);
    p = __builtin_fma(p, t, 4.291175130459545);
    p = __builtin_fma(p, t, -1.5542215474097043);
    p = __builtin_fma(p, t, 0.22800239714528087);
    p = __builtin_fma(p, t, -0.1551378787683726);
    p = __builtin_fma(p, t, 0.09249811135208773);
    p = __builtin_fma(p, t, 0.3741830048987767);
    p = __builtin_fma(p, t, 1.000043891501855);
    p = __builtin_fma(p, t, -1.2655131956093486);
    // exp(q) = 2^(q log2 e), q in [-106, 0]: the product is off by 2^-46 at most, the table-driven 2^x by 2^-39 relative
    const double e = t * exp2_by_table(1.44269504088896338700e+00 * __builtin_fma(-a, a, p), float_tables());
    const float y = (float)((xf < 0.0f) ? 2.0 - e : e);
    return (xf != xf) ? xf : y;
}
#define CUMO_HIP_OWN_OP(NAME, FEXPR, DEXPR)                                                                                 \
    template <class T> struct NAME { CUMO_HIP_OP_COMMON(T, T, T, 1, false, false) static constexpr bool HEAVY = true;       \
        __device__ __forceinline__ bool operator()(T x, T, T& z) const {                                                    \
            if constexpr (sizeof(T) == 4) z = (T)FEXPR((float)x);                                                           \
            else z = (T)(DEXPR);                                                                                            \
            return true; } };
// (DFloat: the cores of dd_cores.h, which read the table of 2^(j/32) as pairs)
#define CUMO_HIP_OWN_OP_WITH_PAIR_TABLE(NAME, FEXPR, DEXPR)                                                                 \
    template <class T> struct NAME { CUMO_HIP_OP_COMMON(T, T, T, 1, false, false) static constexpr bool HEAVY = true;       \
        static constexpr bool USES_PAIR_TABLE = sizeof(T) == 8;                                                             \
        __device__ __forceinline__ bool operator()(T x, T, T& z) const {                                                    \
            if constexpr (sizeof(T) == 4) z = (T)FEXPR((float)x);                                                           \
            else z = (T)(DEXPR);                                                                                            \
            return true; } };
CUMO_HIP_OWN_OP_WITH_PAIR_TABLE(OpTanh, tanh_float_rounded_once, tanh_double((double)x))
CUMO_HIP_OWN_OP_WITH_PAIR_TABLE(OpSinh, sinh_float_rounded_once, sinh_double((double)x))
CUMO_HIP_OWN_OP_WITH_PAIR_TABLE(OpCosh, cosh_float_rounded_once, cosh_double((double)x))
CUMO_HIP_OWN_OP(OpExpm1, expm1_float_rounded_once, (x == 0) ? (double)x : expm1((double)x))  // the library answers +0 for -0

// (not HEAVY: with the short polynomial a lane's single vector keeps up with memory, and the transposed
// kernel's one-tile form is as fast as the prefetching one; DFloat exp of 2^26: 80 -> 83 % of peak)
template <class T> struct OpExp { CUMO_HIP_OP_COMMON(T, T, T, 1, false, false)
    __device__ __forceinline__ bool operator()(T x, T, T& z) const {
        if constexpr (sizeof(T) == 4) z = (T)exp_float_rounded_once((float)x);
        else z = (T)exp((double)x);
        return true; } };
CUMO_HIP_FUN_H(OpExp2, exp2((double)x))
CUMO_HIP_FUN_H(OpExp10, exp10((double)x))
// SFloat ops whose arithmetic covers all but a rare kind of argument also offer the three parts
// apart (fast: the arithmetic; rare: whether the argument is of that kind; slow: the out-of-line
// answer for it), for kernels that evaluate a lane's elements first and mend the rare ones after.
#define CUMO_HIP_TRIG_OP(NAME, WHICH, DEXPR)                                                                                \
    template <class T> struct NAME { CUMO_HIP_OP_COMMON(T, T, T, 1, false, false) static constexpr bool HEAVY = true;       \
        static constexpr bool HAS_RARE = sizeof(T) == 4;                                                                    \
        __device__ __forceinline__ bool operator()(T x, T, T& z) const {                                                    \
            if constexpr (sizeof(T) == 4) z = (T)trig_float_rounded_once<WHICH>((float)x);                                  \
            else z = (T)(DEXPR);                                                                                            \
            return true; }                                                                                                  \
        __device__ __forceinline__ void fast(T x, T, T& z) const { z = (T)trig_fast<WHICH>((float)x); }                    \
        __device__ __forceinline__ bool rare(T x, T) const { return trig_is_rare((float)x); }                              \
        __device__ __forceinline__ T slow(T x, T) const { return (T)trig_by_the_library<WHICH>((float)x); } };
CUMO_HIP_TRIG_OP(OpSin, 0, sin((double)x))
CUMO_HIP_TRIG_OP(OpCos, 1, cos((double)x))
CUMO_HIP_TRIG_OP(OpTan, 2, tan((double)x))
CUMO_HIP_OWN_OP(OpAsin, asin_acos_float_rounded_once<false>, asin((double)x))
CUMO_HIP_OWN_OP(OpAcos, asin_acos_float_rounded_once<true>, acos((double)x))
CUMO_HIP_OWN_OP(OpAtan, atan_float_rounded_once, atan((double)x))
// SFloat atan2(y, x) for finite arguments that are not zero, with atan's polynomial: the quotient's reduction is done on
// numerator and denominator (t = |y| / |x| up to tan(pi/8), (|y| - |x|) / (|y| + |x|) plus pi/4 up to tan(3 pi/8),
// -|x| / |y| plus pi/2 above; the sums are exact or good to 2^-53 in double), pi minus that for a negative x, y's sign.
// Every other argument (a zero, an infinity, a NaN: the rules about signs and quadrants) is the device library's atan2.
// (reference: types/float_macro_kernel.h m_atan2 -> atan2)
__device__ __attribute__((noinline)) float atan2_by_the_library(float yf, float xf) { return (float)atan2((double)yf, (double)xf); }
__device__ __forceinline__ float atan2_fast(float yf, float xf) {
    const double ay = (double)__builtin_fabsf(yf), ax = (double)__builtin_fabsf(xf);
    const bool mid = ay > 0.41421356237309503 * ax, top = ay > 2.4142135623730951 * ax;
    const double num = top ? -ax : (mid ? ay - ax : ay);
    const double den = top ? ay : (mid ? ay + ax : ax);
    const double off = top ? 1.57079632679489655800e+00 : (mid ? 7.85398163397448278999e-01 : 0.0);
    const double t = num * rcp_refined(den);
    const double z = t * t;
    double p = 0.033038827515269494;
    p = __builtin_fma(p, z, -0.06032248119994454);
    p = __builtin_fma(p, z, 0.07605969344616582);
    p = __builtin_fma(p, z, -0.09084239163280672);
    p = __builtin_fma(p, z, 0.11110827992295265);
    p = __builtin_fma(p, z, -0.1428570834807845);
    p = __builtin_fma(p, z, 0.19999999952417688);
    p = __builtin_fma(p, z, -0.33333333333270726);
    double r = off + __builtin_fma(t * z, p, t);
    r = (xf < 0.0f) ? 3.14159265358979311600e+00 - r : r;
    return __builtin_copysignf((float)r, yf);
}
// (finite and not zero, both)
__device__ __forceinline__ bool atan2_is_rare(float yf, float xf) {
    return !(__float_as_uint(__builtin_fabsf(yf)) - 1u < 0x7f7fffffu && __float_as_uint(__builtin_fabsf(xf)) - 1u < 0x7f7fffffu);
}
__device__ __forceinline__ float atan2_float_rounded_once(float yf, float xf) {
    float z = atan2_fast(yf, xf);
    if (atan2_is_rare(yf, xf)) z = atan2_by_the_library(yf, xf);
    return z;
}
template <class T> struct OpAtan2 { CUMO_HIP_OP_COMMON(T, T, T, 2, false, false) static constexpr bool HEAVY = true;
    static constexpr bool HAS_RARE = sizeof(T) == 4;
    __device__ __forceinline__ bool operator()(T x, T y, T& z) const {
        if constexpr (sizeof(T) == 4) z = (T)atan2_float_rounded_once((float)x, (float)y);
        else z = (T)atan2((double)x, (double)y);
        return true; }
    __device__ __forceinline__ void fast(T x, T y, T& z) const { z = (T)atan2_fast((float)x, (float)y); }
    __device__ __forceinline__ bool rare(T x, T y) const { return atan2_is_rare((float)x, (float)y); }
    __device__ __forceinline__ T slow(T x, T y) const { return (T)atan2_by_the_library((float)x, (float)y); } };
// SFloat remainder x % y (the C fmod: the sign of x, exact) where the quotient stays below 2^29: its integer part from
// a refined reciprocal (off by one at most, next to a whole number), taken off in one multiply-add, which is exact there
// (29 + 24 bits), and put right by one addition or subtraction of |y|. Larger quotients, a zero divisor, infinities and
// NaN are the device library's fmod (reference: types/float_macro_kernel.h m_mod -> fmod).
__device__ __attribute__((noinline)) float fmod_by_the_library(float xf, float yf) { return (float)fmod((double)xf, (double)yf); }
__device__ __forceinline__ float fmod_fast(float xf, float yf) {
    const double ax = (double)__builtin_fabsf(xf), ay = (double)__builtin_fabsf(yf);
    const double q = __builtin_trunc(ax * rcp_refined(ay));
    double r = __builtin_fma(-q, ay, ax);
    r = (r < 0.0) ? r + ay : r;
    r = (r >= ay) ? r - ay : r;
    return __builtin_copysignf((float)r, xf);
}
__device__ __forceinline__ bool fmod_is_rare(float xf, float yf) {
    const float ax = __builtin_fabsf(xf), ay = __builtin_fabsf(yf);
    // (false for a NaN on either side, a zero or infinite divisor, an infinite dividend)
    return !(ax < 536870912.0f * ay && ay < INFINITY && ax < INFINITY);
}
__device__ __forceinline__ float fmod_float(float xf, float yf) {
    float z = fmod_fast(xf, yf);
    if (fmod_is_rare(xf, yf)) z = fmod_by_the_library(xf, yf);
    return z;
}
template <class T> struct OpFMod { CUMO_HIP_OP_COMMON(T, T, T, 2, false, false)
    static constexpr bool HAS_RARE = sizeof(T) == 4;
    __device__ __forceinline__ bool operator()(T x, T y, T& z) const {
        if constexpr (sizeof(T) == 4) z = (T)fmod_float((float)x, (float)y);
        else z = (T)fmod((double)x, (double)y);
        return true; }
    __device__ __forceinline__ void fast(T x, T y, T& z) const { z = (T)fmod_fast((float)x, (float)y); }
    __device__ __forceinline__ bool rare(T x, T y) const { return fmod_is_rare((float)x, (float)y); }
    __device__ __forceinline__ T slow(T x, T y) const { return (T)fmod_by_the_library((float)x, (float)y); } };
// SFloat hypot: x^2 + y^2 cannot leave the double range and is good to 2^-53 there; one refined square root. An
// infinity on either side answers infinity, whatever the other is (types/float_macro_kernel.h m_hypot -> hypot).
__device__ __forceinline__ float hypot_float_rounded_once(float xf, float yf) {
    const double x = (double)xf, y = (double)yf;
    const double s = __builtin_fma(x, x, y * y);
    float r = (float)sqrt_refined((s > 0.0) ? s : 1.0);
    r = (s == 0.0) ? 0.0f : r;
    r = (s != s) ? (float)s : r;
    return (__builtin_fabsf(xf) == INFINITY || __builtin_fabsf(yf) == INFINITY) ? INFINITY : r;
}
template <class T> struct OpHypot { CUMO_HIP_OP_COMMON(T, T, T, 2, false, false)
    __device__ __forceinline__ bool operator()(T x, T y, T& z) const {
        if constexpr (sizeof(T) == 4) z = (T)hypot_float_rounded_once((float)x, (float)y);
        else z = (T)hypot((double)x, (double)y);
        return true; } };
// (DFloat: the cores of dd_cores.h, which read the table of the power's logarithm)
#define CUMO_HIP_OWN_OP_WITH_TABLES(NAME, FEXPR, DEXPR)                                                                     \
    template <class T> struct NAME { CUMO_HIP_OP_COMMON(T, T, T, 1, false, false) static constexpr bool HEAVY = true;       \
        static constexpr bool USES_TABLES = sizeof(T) == 4;                                                                 \
        static constexpr bool USES_POW_PAIR_TABLES = sizeof(T) == 8;                                                        \
        __device__ __forceinline__ bool operator()(T x, T, T& z) const {                                                    \
            if constexpr (sizeof(T) == 4) z = (T)FEXPR((float)x);                                                           \
            else z = (T)(DEXPR);                                                                                            \
            return true; } };
CUMO_HIP_OWN_OP_WITH_TABLES(OpAsinh, asinh_float_rounded_once, asinh_double((double)x))
CUMO_HIP_OWN_OP_WITH_TABLES(OpAcosh, acosh_float_rounded_once, acosh_double((double)x))
CUMO_HIP_OWN_OP_WITH_TABLES(OpAtanh, atanh_float_rounded_once, atanh_double((double)x))
// the host macro guards x == 0 (types/float_macro.h:113); the reference's device
// macro does not and answers NaN there, which Numo does not
__device__ __attribute__((noinline)) float sinc_by_the_library(float xf) { return (float)(sin((double)xf) / (double)xf); }
__device__ __forceinline__ float sinc_float_rounded_once(float xf) {
    float y = (float)(trig_core<0>(xf) * rcp_refined((double)xf));
    if (trig_is_rare(xf)) y = sinc_by_the_library(xf);
    return (xf == 0.0f) ? 1.0f : y;
}
CUMO_HIP_OWN_OP(OpSinc, sinc_float_rounded_once, (x == 0) ? 1.0 : (sin((double)x) / (double)x))
CUMO_HIP_OWN_OP(OpErf, erf_float_rounded_once, erf((double)x))
// (DFloat: erfc_double of dd_cores.h, which reads its interval table and the exponential's)
template <class T> struct OpErfc { CUMO_HIP_OP_COMMON(T, T, T, 1, false, false) static constexpr bool HEAVY = true;
    static constexpr bool USES_TABLES = sizeof(T) == 4;
    static constexpr bool USES_ERFC_TABLES = sizeof(T) == 8;
    __device__ __forceinline__ bool operator()(T x, T, T& z) const {
        if constexpr (sizeof(T) == 4) z = (T)erfc_float_rounded_once((float)x);
        else z = (T)erfc_double((double)x);
        return true; } };

#define CUMO_HIP_IUN(NAME, EXPR) \
    struct NAME { CUMO_HIP_OP_COMMON(int32_t, int32_t, int32_t, 1, false, false) \
        __device__ __forceinline__ bool operator()(int32_t x, int32_t, int32_t& z) const { z = (int32_t)(EXPR); return true; } };
CUMO_HIP_IUN(OpIMinus, 0u - (uint32_t)x)
CUMO_HIP_IUN(OpISquare, (uint32_t)x * (uint32_t)x)
CUMO_HIP_IUN(OpISign, (x == 0) ? 0 : ((x > 0) ? 1 : -1))
CUMO_HIP_IUN(OpINot, ~x)
// reference: types/int_macro_kernel.h:12-24 and narray/gen/tmpl/unary_kernel.cu:4-9
struct OpIReciprocal { CUMO_HIP_OP_COMMON(int32_t, int32_t, int32_t, 1, false, true)
    __device__ __forceinline__ bool operator()(int32_t x, int32_t, int32_t& z) const {
        if (x == 0) return false;
        z = (x == 1) ? 1 : ((x == -1) ? -1 : 0);
        return true; } };
// reference: narray/gen/tmpl/unary2_kernel.cu:4-9
struct OpIAbs { CUMO_HIP_OP_COMMON(int32_t, int32_t, int32_t, 1, false, true)
    __device__ __forceinline__ bool operator()(int32_t x, int32_t, int32_t& z) const {
        if (x == INT32_MIN) return false;
        z = (x < 0) ? -x : x;
        return true; } };

// ---- pow, maximum/minimum, clip ----------------------------------------------
// Float ** float: the host macro's pow in double, rounded once
// (reference: types/float_macro.h m_pow; device types/float_macro_kernel.h:36).
// SFloat: for a positive finite base and a finite exponent, 2^(y log2 x) in double from the two
// table-driven cores above: the logarithm is good to 2^-44 relative and |y log2 x| stays below 160
// wherever the float answer is neither 0 nor infinite, so the exponent is off by less than 2^-36
// and the result by less than 2^-12 of a float's last place before the one rounding; everything
// else (zero, negative, infinite or NaN base, infinite or NaN exponent: the sign, domain and
// limit rules) is the device library's pow.
// kept out of line: inlined next to every element it would spread the few instructions
// that run over many times their size of instructions that almost never do
__device__ __attribute__((noinline)) float pow_by_the_library(float xf, float yf) { return (float)pow((double)xf, (double)yf); }
__device__ __forceinline__ float pow_fast(float xf, float yf) {
    const double* tab = float_tables();
    double e = (double)yf * log2_by_table((double)xf, tab);
    e = __builtin_fmin(__builtin_fmax(e, -160.0), 130.0);  // (a NaN only comes from a rare argument)
    return (float)exp2_by_table(e, tab);
}
__device__ __forceinline__ bool pow_is_rare(float xf, float yf) { return !(__float_as_uint(xf) - 1u < 0x7f7fffffu && __builtin_fabsf(yf) < INFINITY); }
__device__ __forceinline__ float pow_float_rounded_once(float xf, float yf) {
    // the rare other case after the arithmetic, so that the elements of a vector are evaluated side by side
    float z = pow_fast(xf, yf);
    if (pow_is_rare(xf, yf)) z = pow_by_the_library(xf, yf);
    return z;
}
// DFloat: the same split with log2 x and y log2 x carried as pairs of doubles (dd_cores.h); a subnormal base goes to the
// library too.
__device__ __attribute__((noinline)) double pow_double_by_the_library(double x, double y) { return pow(x, y); }
template <class T> struct OpPow { CUMO_HIP_OP_COMMON(T, T, T, 2, false, false) static constexpr bool HEAVY = true;
    static constexpr bool HAS_RARE = true;
    static constexpr bool USES_TABLES = sizeof(T) == 4;
    static constexpr bool USES_POW_PAIR_TABLES = sizeof(T) == 8;
    __device__ __forceinline__ bool operator()(T x, T y, T& z) const {
        fast(x, y, z);
        if (rare(x, y)) z = slow(x, y);
        return true; }
    __device__ __forceinline__ void fast(T x, T y, T& z) const {
        if constexpr (sizeof(T) == 4) z = (T)pow_fast((float)x, (float)y);
        else z = (T)pow_double_fast((double)x, (double)y); }
    __device__ __forceinline__ bool rare(T x, T y) const {
        if constexpr (sizeof(T) == 4) return pow_is_rare((float)x, (float)y);
        else return pow_double_is_rare((double)x, (double)y); }
    __device__ __forceinline__ T slow(T x, T y) const {
        if constexpr (sizeof(T) == 4) return (T)pow_by_the_library((float)x, (float)y);
        else return (T)pow_double_by_the_library((double)x, (double)y); } };

// SFloat ** y for one exponent that is a whole number of halves, up to 32 either way (x ** 0.5, x ** -1.5, x ** 2.5,
// x ** 3.0): the whole part by squaring and multiplying, the half by one refined square root, a negative exponent by one
// division, all in double (whose range holds every intermediate whose result a float can hold; beyond it the float
// answer is 0 or infinite either way) and rounded to float once. The rules of pow for the arguments that arithmetic
// would get wrong are spelt out: with an exponent that is not whole a zero base counts as +0 and -inf as +inf
// (a negative base answers NaN through the square root); x ** 0 is 1 whatever x is.
// (NEG, a negative exponent, at compile time: left to run time the compiler evaluates the division for every element
// and then picks, 25 issue slots an element)
template <bool NEG>
struct OpPowHalves { CUMO_HIP_OP_COMMON(float, float, float, 1, false, false)
    int twice;   // 2 y (negative exactly when NEG)
    __device__ __forceinline__ bool operator()(float xf, float, float& z) const {
        const unsigned m = (unsigned)(twice < 0 ? -twice : twice);
        const bool half = (m & 1u) != 0;
        double x = (double)xf;
        if (half) {
            x = (xf == 0.0f) ? 0.0 : x;
            x = (xf == -INFINITY) ? (double)INFINITY : x;
        }
        double r = 1.0, b = x;
        for (unsigned q = m >> 1; q != 0; q >>= 1) {   // (the same turns for every lane)
            if (q & 1u) r *= b;
            b *= b;
        }
        if (half) {
            const bool inside = x > 0.0 && x < (double)INFINITY;
            double s = sqrt_refined(inside ? x : 1.0);
            s = inside ? s : ((x == 0.0 || x == (double)INFINITY) ? x : (double)NAN);   // (a NaN base fails every comparison)
            r *= s;
        }
        if (NEG) r = 1.0 / r;
        z = (float)r;
        return true; } };

// DFloat ** y for one exponent that is a whole number of halves up to 8 either way (dd_cores.h)
template <bool NEG>
struct OpPowHalvesD { CUMO_HIP_OP_COMMON(double, double, double, 1, false, false) static constexpr bool HEAVY = true;
    static constexpr bool HAS_RARE = true;
    int twice;   // 2 y (negative exactly when NEG)
    __device__ __forceinline__ bool operator()(double x, double, double& z) const {
        fast(x, 0.0, z);
        if (rare(x, 0.0)) z = slow(x, 0.0);
        return true; }
    __device__ __forceinline__ void fast(double x, double, double& z) const { z = pow_halves_double_fast<NEG>(x, twice); }
    __device__ __forceinline__ bool rare(double x, double) const { return pow_halves_double_is_rare(x); }
    __device__ __forceinline__ double slow(double x, double) const { return pow_double_by_the_library(x, 0.5 * (double)twice); } };

// Float ** Int32 (reference: types/float_macro_kernel.h:125-149): products in the
// element type for small exponents, pow() beyond 64, the reciprocal for negative ones.
// (out of line: inlined at every element, the library's pow took 66 registers of a kernel that needs 10)
template <class T>
__device__ __attribute__((noinline)) T pow_float_int_by_the_library(T x, uint32_t q) { return (T)pow((double)x, (double)q); }

template <class T>
__device__ __forceinline__ T pow_float_int(T x, int32_t p) {
    const bool neg = p < 0;
    uint32_t q = neg ? (0u - (uint32_t)p) : (uint32_t)p;
    T r = 1;
    switch (q) {
        case 0: r = 1; break;
        case 1: r = x; break;
        case 2: r = x * x; break;
        case 3: r = x * x * x; break;
        case 4: x = x * x; r = x * x; break;
        default:
            if (q > 64) {
                r = pow_float_int_by_the_library<T>(x, q);
            } else {
                while (q) {
                    if (q & 1u) r *= x;
                    x *= x;
                    q >>= 1;
                }
            }
    }
    return neg ? (T)1 / r : r;
}
template <class T> struct OpPowInt { typedef T A; typedef int32_t B; typedef T R; typedef T S;
    static constexpr int NIN = 2; static constexpr bool BIT_OUT = false; static constexpr bool CHECKED = false;
    __device__ __forceinline__ bool operator()(T x, int32_t y, T& z) const { z = pow_float_int<T>(x, y); return true; } };
// the exponent is one Int32 for the whole launch
template <class T> struct OpPowIntS { CUMO_HIP_OP_COMMON(T, T, T, 1, false, false)
    int32_t p;
    __device__ __forceinline__ bool operator()(T x, T, T& z) const { z = pow_float_int<T>(x, p); return true; } };
// the base is one number for the whole launch, the exponents are an Int32 array
template <class T> struct OpPowIntLeft { typedef int32_t A; typedef int32_t B; typedef T R; typedef int32_t S;
    static constexpr int NIN = 1; static constexpr bool BIT_OUT = false; static constexpr bool CHECKED = false;
    T base;
    __device__ __forceinline__ bool operator()(int32_t y, int32_t, T& z) const { z = pow_float_int<T>(base, y); return true; } };

// Int32 ** Int32 (reference: types/int_macro_kernel.h:26-42): wrapping products, 0 for a negative exponent
__device__ __forceinline__ int32_t pow_int32(int32_t x, int32_t p) {
    uint32_t ux = (uint32_t)x, r = 1u;
    switch (p) {
        case 0: return 1;
        case 1: return x;
        case 2: return (int32_t)(ux * ux);
        case 3: return (int32_t)(ux * ux * ux);
    }
    if (p < 0) return 0;
    uint32_t q = (uint32_t)p;
    while (q) {
        if (q & 1u) r *= ux;
        ux *= ux;
        q >>= 1;
    }
    return (int32_t)r;
}
struct OpIPow { CUMO_HIP_OP_COMMON(int32_t, int32_t, int32_t, 2, false, false)
    __device__ __forceinline__ bool operator()(int32_t x, int32_t y, int32_t& z) const { z = pow_int32(x, y); return true; } };
struct OpIPowS { CUMO_HIP_OP_COMMON(int32_t, int32_t, int32_t, 1, false, false)
    int32_t p;
    __device__ __forceinline__ bool operator()(int32_t x, int32_t, int32_t& z) const { z = pow_int32(x, p); return true; } };
struct OpIPowLeft { CUMO_HIP_OP_COMMON(int32_t, int32_t, int32_t, 1, false, false)
    int32_t base;
    __device__ __forceinline__ bool operator()(int32_t y, int32_t, int32_t& z) const { z = pow_int32(base, y); return true; } };

// maximum / minimum of two arrays (reference: types/real_accum_kernel.h:28-70,
// xint_macro_kernel.h:54-68). The plain form answers the other operand when one
// is NaN; the _nan form answers the NaN.
template <class T> struct OpMaximum { CUMO_HIP_OP_COMMON(T, T, T, 2, false, false)
    __device__ __forceinline__ bool operator()(T x, T y, T& z) const { z = (x >= y) ? x : ((y == y) ? y : x); return true; } };
template <class T> struct OpMaximumNan { CUMO_HIP_OP_COMMON(T, T, T, 2, false, false)
    __device__ __forceinline__ bool operator()(T x, T y, T& z) const { z = (x >= y) ? x : ((x != x) ? x : y); return true; } };
template <class T> struct OpMinimum { CUMO_HIP_OP_COMMON(T, T, T, 2, false, false)
    __device__ __forceinline__ bool operator()(T x, T y, T& z) const { z = (x <= y) ? x : ((y == y) ? y : x); return true; } };
template <class T> struct OpMinimumNan { CUMO_HIP_OP_COMMON(T, T, T, 2, false, false)
    __device__ __forceinline__ bool operator()(T x, T y, T& z) const { z = (x <= y) ? x : ((x != x) ? x : y); return true; } };

// clip against one bound that is an array or the scalar, and against two scalar
// bounds (reference: narray/gen/tmpl/clip_kernel.cu:7-44)
template <class T> struct OpClipMin { CUMO_HIP_OP_COMMON(T, T, T, 2, false, false)
    __device__ __forceinline__ bool operator()(T x, T lo, T& z) const { z = (x < lo) ? lo : x; return true; } };
template <class T> struct OpClipMax { CUMO_HIP_OP_COMMON(T, T, T, 2, false, false)
    __device__ __forceinline__ bool operator()(T x, T hi, T& z) const { z = (x > hi) ? hi : x; return true; } };
template <class T> struct OpClipS { CUMO_HIP_OP_COMMON(T, T, T, 1, false, false)
    T lo, hi;
    __device__ __forceinline__ bool operator()(T x, T, T& z) const {
        if (x < lo) x = lo;
        if (x > hi) x = hi;
        z = x;
        return true; } };

// ---- comparisons into Bit ---------------------------------------------------
#define CUMO_HIP_CMP(NAME, EXPR) \
    template <class T> struct NAME { CUMO_HIP_OP_COMMON(T, T, uint32_t, 2, true, false) \
        __device__ __forceinline__ bool operator()(T x, T y, uint32_t& z) const { z = (EXPR) ? 1u : 0u; return true; } };
CUMO_HIP_CMP(OpEq, x == y)
CUMO_HIP_CMP(OpNe, x != y)
CUMO_HIP_CMP(OpGt, x > y)
CUMO_HIP_CMP(OpGe, x >= y)
CUMO_HIP_CMP(OpLt, x < y)
CUMO_HIP_CMP(OpLe, x <= y)
// reference: types/sfloat_kernel.h:9, dfloat_kernel.h (the float form does the
// subtraction in float and everything else in double)
template <class T> struct OpNearlyEq { CUMO_HIP_OP_COMMON(T, T, uint32_t, 2, true, false)
    __device__ __forceinline__ bool operator()(T x, T y, uint32_t& z) const {
        const double eps = (sizeof(T) == 4) ? (double)FLT_EPSILON : DBL_EPSILON;
        z = (fabs((double)(T)(x - y)) <= (fabs((double)x) + fabs((double)y)) * eps * 2) ? 1u : 0u;
        return true; } };

#define CUMO_HIP_CND(NAME, EXPR) \
    template <class T> struct NAME { CUMO_HIP_OP_COMMON(T, T, uint32_t, 1, true, false) \
        __device__ __forceinline__ bool operator()(T x, T, uint32_t& z) const { z = (EXPR) ? 1u : 0u; return true; } };
CUMO_HIP_CND(OpIsNan, x != x)
CUMO_HIP_CND(OpIsInf, isinf(x))
CUMO_HIP_CND(OpIsPosInf, isinf(x) && !signbit(x))
CUMO_HIP_CND(OpIsNegInf, isinf(x) && signbit(x))
CUMO_HIP_CND(OpIsFinite, isfinite(x))
CUMO_HIP_CND(OpSignbit, signbit(x))

// ---- store/cast, fill --------------------------------------------------------
// dst = (dst type)src, the plain C conversion of the reference's device macros
// (types/float_macro_kernel.h:21-27, xint_macro_kernel.h:7-13)
template <class TD, class TS> struct OpCast { CUMO_HIP_OP_COMMON(TS, TS, TD, 1, false, false)
    __device__ __forceinline__ bool operator()(TS x, TS, TD& z) const { z = (TD)x; return true; } };

template <class T> struct OpFill { CUMO_HIP_OP_COMMON(T, T, T, 0, false, false)
    T value;
    __device__ __forceinline__ bool operator()(T, T, T& z) const { z = value; return true; } };

}  // namespace cumo_hip

#endif
