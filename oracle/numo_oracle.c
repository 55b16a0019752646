/*
 * numo_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A single-threaded CPU restatement of the Numo/Cumo semantics of the array
 * hot path: elementwise unary/binary/compare/cast ops with broadcasting over
 * strided views, Bit packing, count_true and the axis reductions.  Only the
 * tests, the smoke check and the cpu_baseline leg of the benchmark may load
 * it; nothing the library ships links or calls it.
 *
 * Every function cites the reference file (relative to the reference tree)
 * whose behaviour it restates.  The loops are deliberately the plain
 * sequential shapes of the host macros, because the host f_* loops are what
 * Numo compiles to, and their order of evaluation is part of the answer.
 *
 * Pinning status (what fixes each function independently of this file):
 *   - add/sub/mul/div/minus/square/abs/compare : IEEE-754 single operation,
 *     checked bit-for-bit against numpy.
 *   - Int32 ops                                : C integer semantics, checked
 *     against numpy int32 / Python ints.
 *   - addressing / broadcast                   : brute force vs numpy
 *     as_strided.
 *   - sum/mean/var/stddev/rms                  : closed forms, exact rational
 *     arithmetic and literals held by the reference tests.
 *   - min/max/argmin/argmax (NaN, ties, +-0)   : enumerated cases from the
 *     reference tests, brute force on small inputs.
 *   - Bit packing / count_true                 : popcount closed form, brute
 *     force.
 *   - SFloat/DFloat NMath functions and pow    : restated as (float)f((double)x)
 *     / f(x) per types/float_macro.h:84-118, which is what the host macros
 *     compile to, with this machine's glibc for f. Pinned against correctly
 *     rounded vectors (tests/golden/nmath_vectors.npz, mpmath at 400 bits):
 *     every SFloat function and most DFloat ones are within 1 ulp of them;
 *     glibc's DFloat cbrt (3 ulp), exp10, tanh and erfc (2 ulp) are not, and
 *     the tests say so where they use them. Which libm Numo links on another
 *     machine is not observable; the vectors are the fixed point instead.
 */
#define _GNU_SOURCE
#include <math.h>
#include <stdint.h>
#include <stddef.h>
#include <string.h>
#include <sys/types.h>
#include <float.h>

#define MAXD 12  /* include/cumo/narray.h:489 CUMO_NA_MAX_DIMENSION */
#define NB 32    /* include/cumo/narray.h:492-494: Bit word is unsigned int */

enum { T_SFLOAT = 0, T_DFLOAT = 1, T_INT32 = 2, T_INT64 = 3, T_UINT64 = 4 };

/* ------------------------------------------------------------------ */
/* N-d iteration in row-major order (narray/ndloop.c:1459-1616: the    */
/* innermost loop runs over the last dimension).                       */
/* ------------------------------------------------------------------ */
typedef struct {
    int ndim;
    size_t shape[MAXD];
    size_t idx[MAXD];
} iter_t;

static void iter_init(iter_t *it, int ndim, const size_t *shape)
{
    it->ndim = ndim;
    for (int d = 0; d < ndim; ++d) { it->shape[d] = shape[d]; it->idx[d] = 0; }
}

static int iter_next(iter_t *it)
{
    for (int d = it->ndim; --d >= 0;) {
        if (++it->idx[d] < it->shape[d]) return 1;
        it->idx[d] = 0;
    }
    return 0;
}

static ssize_t iter_off(const iter_t *it, const ssize_t *step)
{
    ssize_t o = 0;
    for (int d = 0; d < it->ndim; ++d) o += (ssize_t)it->idx[d] * step[d];
    return o;
}

static size_t total_of(int ndim, const size_t *shape)
{
    size_t t = 1;
    for (int d = 0; d < ndim; ++d) t *= shape[d];
    return t;
}

/* ------------------------------------------------------------------ */
/* Bit load/store: include/cumo/template.h:110-138 (LSB-first inside a */
/* 32-bit word, position counted in bits from the word pointer).       */
/* ------------------------------------------------------------------ */
static unsigned load_bit(const uint32_t *a, size_t pos)
{
    return (a[pos / NB] >> (pos % NB)) & 1u;
}

static void store_bit(uint32_t *a, size_t pos, unsigned v)
{
    size_t dig = pos / NB; int bit = (int)(pos % NB);
    a[dig] = (a[dig] & ~(1u << bit)) | ((v & 1u) << bit);
}

/* ------------------------------------------------------------------ */
/* Element operations.                                                 */
/* Float: include/cumo/types/float_macro.h:26-118. With dtype float the*/
/* arithmetic macros are float operations, and every libm call is the  */
/* double function on the promoted argument, rounded once on store.    */
/* ------------------------------------------------------------------ */
#define FLOAT_BINARY(T)                                                        \
static int T##_binary(const char *op, T x, T y, T *z)                          \
{                                                                              \
    if (!strcmp(op, "add")) { *z = x + y; return 1; }                          \
    if (!strcmp(op, "sub")) { *z = x - y; return 1; }                          \
    if (!strcmp(op, "mul")) { *z = x * y; return 1; }                          \
    if (!strcmp(op, "div")) { *z = x / y; return 1; }                          \
    if (!strcmp(op, "mod")) { *z = (T)fmod(x, y); return 1; }                  \
    if (!strcmp(op, "copysign")) { *z = (T)copysign(x, y); return 1; }         \
    if (!strcmp(op, "atan2")) { *z = (T)atan2(x, y); return 1; }               \
    if (!strcmp(op, "hypot")) { *z = (T)hypot(x, y); return 1; }               \
    if (!strcmp(op, "ldexp")) { /* types/float_macro.h:117; the second    */   \
        *z = (T)ldexp(x, (int)y); return 1; } /* operand converts to int  */   \
    if (!strcmp(op, "maximum")) { /* types/real_accum.h:444-453 */             \
        *z = (x >= y) ? x : ((y == y) ? y : x); return 1; }                    \
    if (!strcmp(op, "minimum")) { /* types/real_accum.h:466-475 */             \
        *z = (x <= y) ? x : ((y == y) ? y : x); return 1; }                    \
    if (!strcmp(op, "maximum_nan")) { /* types/real_accum.h:455-464 */         \
        *z = (x >= y) ? x : ((x != x) ? x : y); return 1; }                    \
    if (!strcmp(op, "minimum_nan")) { /* types/real_accum.h:477-486 */         \
        *z = (x <= y) ? x : ((x != x) ? x : y); return 1; }                    \
    if (!strcmp(op, "pow")) { *z = (T)pow(x, y); return 1; } /* float_macro.h:33 */ \
    /* narray/gen/tmpl/clip.c:74-75,106-107: one-sided clip */                 \
    if (!strcmp(op, "clip_min")) { *z = (x < y) ? y : x; return 1; }           \
    if (!strcmp(op, "clip_max")) { *z = (x > y) ? y : x; return 1; }           \
    return 0;                                                                  \
}
FLOAT_BINARY(float)
FLOAT_BINARY(double)

/* types/float_macro.h:36-47,84-118; sinc on the host guards x==0
 * (float_macro.h:113). */
#define FLOAT_UNARY(T)                                                         \
static int T##_unary(const char *op, T x, T *z)                                \
{                                                                              \
    if (!strcmp(op, "minus")) { *z = -x; return 1; }                           \
    if (!strcmp(op, "abs")) { *z = (T)fabs(x); return 1; }                     \
    if (!strcmp(op, "reciprocal")) { *z = 1 / x; return 1; }                   \
    if (!strcmp(op, "square")) { *z = x * x; return 1; }                       \
    if (!strcmp(op, "sign")) {                                                 \
        *z = (T)((x == 0) ? 0.0 : ((x > 0) ? 1.0 : ((x < 0) ? -1.0 : x)));     \
        return 1; }                                                            \
    if (!strcmp(op, "floor")) { *z = (T)floor(x); return 1; }                  \
    if (!strcmp(op, "round")) { *z = (T)round(x); return 1; }                  \
    if (!strcmp(op, "ceil")) { *z = (T)ceil(x); return 1; }                    \
    if (!strcmp(op, "trunc")) { *z = (T)trunc(x); return 1; }                  \
    if (!strcmp(op, "rint")) { *z = (T)rint(x); return 1; }                    \
    if (!strcmp(op, "sqrt")) { *z = (T)sqrt(x); return 1; }                    \
    if (!strcmp(op, "cbrt")) { *z = (T)cbrt(x); return 1; }                    \
    if (!strcmp(op, "log")) { *z = (T)log(x); return 1; }                      \
    if (!strcmp(op, "log2")) { *z = (T)log2(x); return 1; }                    \
    if (!strcmp(op, "log10")) { *z = (T)log10(x); return 1; }                  \
    if (!strcmp(op, "exp")) { *z = (T)exp(x); return 1; }                      \
    if (!strcmp(op, "exp2")) { *z = (T)exp2(x); return 1; }                    \
    if (!strcmp(op, "exp10")) { *z = (T)exp10(x); return 1; }                  \
    if (!strcmp(op, "expm1")) { *z = (T)expm1(x); return 1; }                  \
    if (!strcmp(op, "log1p")) { *z = (T)log1p(x); return 1; }                  \
    if (!strcmp(op, "sin")) { *z = (T)sin(x); return 1; }                      \
    if (!strcmp(op, "cos")) { *z = (T)cos(x); return 1; }                      \
    if (!strcmp(op, "tan")) { *z = (T)tan(x); return 1; }                      \
    if (!strcmp(op, "asin")) { *z = (T)asin(x); return 1; }                    \
    if (!strcmp(op, "acos")) { *z = (T)acos(x); return 1; }                    \
    if (!strcmp(op, "atan")) { *z = (T)atan(x); return 1; }                    \
    if (!strcmp(op, "sinh")) { *z = (T)sinh(x); return 1; }                    \
    if (!strcmp(op, "cosh")) { *z = (T)cosh(x); return 1; }                    \
    if (!strcmp(op, "tanh")) { *z = (T)tanh(x); return 1; }                    \
    if (!strcmp(op, "asinh")) { *z = (T)asinh(x); return 1; }                  \
    if (!strcmp(op, "acosh")) { *z = (T)acosh(x); return 1; }                  \
    if (!strcmp(op, "atanh")) { *z = (T)atanh(x); return 1; }                  \
    if (!strcmp(op, "sinc")) { *z = (T)((x == 0) ? 1.0 : (sin(x) / x)); return 1; } \
    if (!strcmp(op, "erf")) { *z = (T)erf(x); return 1; }                      \
    if (!strcmp(op, "erfc")) { *z = (T)erfc(x); return 1; }                    \
    return 0;                                                                  \
}
FLOAT_UNARY(float)
FLOAT_UNARY(double)

/* types/float_macro.h:50-61; nearly_eq: types/sfloat.h:42, dfloat.h. */
#define FLOAT_COND(T, EPS)                                                     \
static int T##_cmp(const char *op, T x, T y, unsigned *b)                      \
{                                                                              \
    if (!strcmp(op, "eq")) { *b = (x == y); return 1; }                        \
    if (!strcmp(op, "ne")) { *b = (x != y); return 1; }                        \
    if (!strcmp(op, "gt")) { *b = (x > y); return 1; }                         \
    if (!strcmp(op, "ge")) { *b = (x >= y); return 1; }                        \
    if (!strcmp(op, "lt")) { *b = (x < y); return 1; }                         \
    if (!strcmp(op, "le")) { *b = (x <= y); return 1; }                        \
    if (!strcmp(op, "nearly_eq")) {                                            \
        *b = (fabs(x - y) <= (fabs(x) + fabs(y)) * EPS * 2); return 1; }       \
    return 0;                                                                  \
}                                                                              \
static int T##_cond1(const char *op, T x, unsigned *b)                         \
{                                                                              \
    if (!strcmp(op, "isnan")) { *b = isnan(x) ? 1 : 0; return 1; }             \
    if (!strcmp(op, "isinf")) { *b = isinf(x) ? 1 : 0; return 1; }             \
    if (!strcmp(op, "isposinf")) { *b = (isinf(x) && !signbit(x)) ? 1 : 0; return 1; } \
    if (!strcmp(op, "isneginf")) { *b = (isinf(x) && signbit(x)) ? 1 : 0; return 1; }  \
    if (!strcmp(op, "isfinite")) { *b = isfinite(x) ? 1 : 0; return 1; }       \
    if (!strcmp(op, "signbit")) { *b = signbit(x) ? 1 : 0; return 1; }         \
    return 0;                                                                  \
}
FLOAT_COND(float, FLT_EPSILON)
FLOAT_COND(double, DBL_EPSILON)

/* Int32: include/cumo/types/xint_macro.h:16-42, int_macro.h:3-24.
 * Division by zero does not store and raises a flag
 * (narray/gen/tmpl/binary_kernel.cu:3-8); int_reciprocal of 0 likewise
 * (tmpl/unary_kernel.cu:4-9); abs(INT_MIN) likewise
 * (tmpl/unary2_kernel.cu:4-9). Wrapping arithmetic is done in unsigned so
 * this file has no undefined behaviour of its own. */
static int i32_binary(const char *op, int32_t x, int32_t y, int32_t *z, int *flag)
{
    if (!strcmp(op, "add")) { *z = (int32_t)((uint32_t)x + (uint32_t)y); return 1; }
    if (!strcmp(op, "sub")) { *z = (int32_t)((uint32_t)x - (uint32_t)y); return 1; }
    if (!strcmp(op, "mul")) { *z = (int32_t)((uint32_t)x * (uint32_t)y); return 1; }
    if (!strcmp(op, "div")) {
        if (y == 0) { *flag = 1; return 2; }
        *z = (x == INT32_MIN && y == -1) ? INT32_MIN : x / y; return 1; }
    if (!strcmp(op, "mod")) {
        if (y == 0) { *flag = 1; return 2; }
        *z = (y == -1) ? 0 : x % y; return 1; }
    if (!strcmp(op, "bit_and")) { *z = x & y; return 1; }
    if (!strcmp(op, "bit_or")) { *z = x | y; return 1; }
    if (!strcmp(op, "bit_xor")) { *z = x ^ y; return 1; }
    if (!strcmp(op, "left_shift")) { *z = (int32_t)((uint32_t)x << (y & 31)); return 1; }
    if (!strcmp(op, "right_shift")) { *z = x >> (y & 31); return 1; }
    if (!strcmp(op, "maximum")) { *z = (x >= y) ? x : y; return 1; }
    if (!strcmp(op, "minimum")) { *z = (x <= y) ? x : y; return 1; }
    if (!strcmp(op, "clip_min")) { *z = (x < y) ? y : x; return 1; }
    if (!strcmp(op, "clip_max")) { *z = (x > y) ? y : x; return 1; }
    if (!strcmp(op, "pow")) { /* types/int_macro_kernel.h:26-42 (the host copy in int_macro.h:26-42 is commented out) */
        uint32_t ux = (uint32_t)x, r = 1u; int32_t p = y;
        switch (p) {
        case 0: *z = 1; return 1;
        case 1: *z = x; return 1;
        case 2: *z = (int32_t)(ux * ux); return 1;
        case 3: *z = (int32_t)(ux * ux * ux); return 1;
        }
        if (p < 0) { *z = 0; return 1; }
        while (p) { if (p & 1) r *= ux; ux *= ux; p >>= 1; }
        *z = (int32_t)r; return 1; }
    return 0;
}

static int i32_unary(const char *op, int32_t x, int32_t *z, int *flag)
{
    if (!strcmp(op, "minus")) { *z = (int32_t)(0u - (uint32_t)x); return 1; }
    if (!strcmp(op, "abs")) {
        if (x == INT32_MIN) { *flag = 1; return 2; }
        *z = (x < 0) ? -x : x; return 1; }
    if (!strcmp(op, "reciprocal")) {
        if (x == 0) { *flag = 1; return 2; }
        *z = (x == 1) ? 1 : ((x == -1) ? -1 : 0); return 1; }
    if (!strcmp(op, "square")) { *z = (int32_t)((uint32_t)x * (uint32_t)x); return 1; }
    if (!strcmp(op, "sign")) { *z = (x == 0) ? 0 : ((x > 0) ? 1 : -1); return 1; }
    if (!strcmp(op, "bit_not")) { *z = ~x; return 1; }
    return 0;
}

static int i32_cmp(const char *op, int32_t x, int32_t y, unsigned *b)
{
    if (!strcmp(op, "eq") || !strcmp(op, "nearly_eq")) { *b = (x == y); return 1; }
    if (!strcmp(op, "ne")) { *b = (x != y); return 1; }
    if (!strcmp(op, "gt")) { *b = (x > y); return 1; }
    if (!strcmp(op, "ge")) { *b = (x >= y); return 1; }
    if (!strcmp(op, "lt")) { *b = (x < y); return 1; }
    if (!strcmp(op, "le")) { *b = (x <= y); return 1; }
    return 0;
}

/* ------------------------------------------------------------------ */
/* Elementwise drivers. Steps are signed byte strides, 0 = broadcast   */
/* (narray/ndloop.c:493-595). A NULL operand pointer for p2 means the  */
/* scalar form: sv carries the Ruby number and scalar_is_left says on  */
/* which side it sits (narray/gen/tmpl/binary_kernel.cu:13-35).        */
/* Returns -1 for an unknown op; otherwise the error flag (0/1).       */
/* ------------------------------------------------------------------ */
int numo_binary(const char *op, int dtype, int ndim, const size_t *shape,
                const char *p1, const ssize_t *s1,
                const char *p2, const ssize_t *s2,
                char *p3, const ssize_t *s3,
                double sv, int scalar_is_left)
{
    iter_t it; int flag = 0;
    if (total_of(ndim, shape) == 0) return 0;
    iter_init(&it, ndim, shape);
    do {
        const char *a = p1 + iter_off(&it, s1);
        char *c = p3 + iter_off(&it, s3);
        if (dtype == T_SFLOAT) {
            float x = *(const float *)a, y, z;
            if (p2) y = *(const float *)(p2 + iter_off(&it, s2));
            else if (scalar_is_left) { y = x; x = (float)sv; }
            else y = (float)sv;
            if (!float_binary(op, x, y, &z)) return -1;
            *(float *)c = z;
        } else if (dtype == T_DFLOAT) {
            double x = *(const double *)a, y, z;
            if (p2) y = *(const double *)(p2 + iter_off(&it, s2));
            else if (scalar_is_left) { y = x; x = sv; }
            else y = sv;
            if (!double_binary(op, x, y, &z)) return -1;
            *(double *)c = z;
        } else {
            int32_t x = *(const int32_t *)a, y, z; int r;
            if (p2) y = *(const int32_t *)(p2 + iter_off(&it, s2));
            else if (scalar_is_left) { y = x; x = (int32_t)sv; }
            else y = (int32_t)sv;
            r = i32_binary(op, x, y, &z, &flag);
            if (!r) return -1;
            if (r == 1) *(int32_t *)c = z;
        }
    } while (iter_next(&it));
    return flag;
}

int numo_unary(const char *op, int dtype, int ndim, const size_t *shape,
               const char *p1, const ssize_t *s1, char *p2, const ssize_t *s2)
{
    iter_t it; int flag = 0;
    if (total_of(ndim, shape) == 0) return 0;
    iter_init(&it, ndim, shape);
    do {
        const char *a = p1 + iter_off(&it, s1);
        char *c = p2 + iter_off(&it, s2);
        if (dtype == T_SFLOAT) {
            float z; if (!float_unary(op, *(const float *)a, &z)) return -1;
            *(float *)c = z;
        } else if (dtype == T_DFLOAT) {
            double z; if (!double_unary(op, *(const double *)a, &z)) return -1;
            *(double *)c = z;
        } else {
            int32_t z; int r = i32_unary(op, *(const int32_t *)a, &z, &flag);
            if (!r) return -1;
            if (r == 1) *(int32_t *)c = z;
        }
    } while (iter_next(&it));
    return flag;
}

/* Compare into a Bit array: narray/gen/tmpl/cond_binary_kernel.cu:7-24.
 * pos3 and bs3 are in bits. */
int numo_compare(const char *op, int dtype, int ndim, const size_t *shape,
                 const char *p1, const ssize_t *s1,
                 const char *p2, const ssize_t *s2,
                 uint32_t *bits, size_t pos3, const ssize_t *bs3,
                 double sv, int scalar_is_left)
{
    iter_t it;
    if (total_of(ndim, shape) == 0) return 0;
    iter_init(&it, ndim, shape);
    do {
        const char *a = p1 + iter_off(&it, s1);
        size_t bp = pos3 + (size_t)iter_off(&it, bs3);
        unsigned b = 0; int ok;
        if (dtype == T_SFLOAT) {
            float x = *(const float *)a, y;
            if (p2) y = *(const float *)(p2 + iter_off(&it, s2));
            else if (scalar_is_left) { y = x; x = (float)sv; }
            else y = (float)sv;
            ok = float_cmp(op, x, y, &b);
        } else if (dtype == T_DFLOAT) {
            double x = *(const double *)a, y;
            if (p2) y = *(const double *)(p2 + iter_off(&it, s2));
            else if (scalar_is_left) { y = x; x = sv; }
            else y = sv;
            ok = double_cmp(op, x, y, &b);
        } else {
            int32_t x = *(const int32_t *)a, y;
            if (p2) y = *(const int32_t *)(p2 + iter_off(&it, s2));
            else if (scalar_is_left) { y = x; x = (int32_t)sv; }
            else y = (int32_t)sv;
            ok = i32_cmp(op, x, y, &b);
        }
        if (!ok) return -1;
        store_bit(bits, bp, b);
    } while (iter_next(&it));
    return 0;
}

/* narray/gen/tmpl/cond_unary_kernel.cu:3-12 */
int numo_cond_unary(const char *op, int dtype, int ndim, const size_t *shape,
                    const char *p1, const ssize_t *s1,
                    uint32_t *bits, size_t pos2, const ssize_t *bs2)
{
    iter_t it;
    if (total_of(ndim, shape) == 0) return 0;
    iter_init(&it, ndim, shape);
    do {
        const char *a = p1 + iter_off(&it, s1);
        unsigned b = 0; int ok;
        if (dtype == T_SFLOAT) ok = float_cond1(op, *(const float *)a, &b);
        else if (dtype == T_DFLOAT) ok = double_cond1(op, *(const double *)a, &b);
        else return -1;
        if (!ok) return -1;
        store_bit(bits, pos2 + (size_t)iter_off(&it, bs2), b);
    } while (iter_next(&it));
    return 0;
}

/* Typed store/cast dst = m_from_X(src): narray/gen/tmpl/store_from_kernel.cu:3-13
 * with the conversion macros of types/float_macro.h:18-24 (plain C conversion)
 * and types/xint_macro.h (device: plain conversion). */
static double load_as_double(int t, const char *p, int64_t *iv, int *is_int)
{
    *is_int = 0;
    switch (t) {
    case T_SFLOAT: return *(const float *)p;
    case T_DFLOAT: return *(const double *)p;
    case T_INT32: *is_int = 1; *iv = *(const int32_t *)p; return (double)*iv;
    case T_INT64: *is_int = 1; *iv = *(const int64_t *)p; return (double)*iv;
    default: *is_int = 1; *iv = (int64_t)*(const uint64_t *)p; return (double)*(const uint64_t *)p;
    }
}

int numo_store(int dst_t, int src_t, int ndim, const size_t *shape,
               char *pd, const ssize_t *sd, const char *ps, const ssize_t *ss)
{
    iter_t it;
    if (total_of(ndim, shape) == 0) return 0;
    iter_init(&it, ndim, shape);
    do {
        char *d = pd + iter_off(&it, sd);
        const char *s = ps + iter_off(&it, ss);
        int64_t iv = 0; int is_int;
        double v = load_as_double(src_t, s, &iv, &is_int);
        switch (dst_t) {
        case T_SFLOAT:
            if (src_t == T_SFLOAT) *(float *)d = *(const float *)s;
            else if (is_int) *(float *)d = (float)iv;
            else *(float *)d = (float)v;
            break;
        case T_DFLOAT: *(double *)d = is_int ? (double)iv : v; break;
        case T_INT32: *(int32_t *)d = is_int ? (int32_t)iv : (int32_t)v; break;
        case T_INT64: *(int64_t *)d = is_int ? iv : (int64_t)v; break;
        default: return -1;
        }
    } while (iter_next(&it));
    return 0;
}

/* Bit -> number (0/1): narray/gen/tmpl/store_bit_kernel.cu:3-12 */
int numo_store_bit(int dst_t, int ndim, const size_t *shape,
                   char *pd, const ssize_t *sd,
                   const uint32_t *bits, size_t pos, const ssize_t *bs)
{
    iter_t it;
    if (total_of(ndim, shape) == 0) return 0;
    iter_init(&it, ndim, shape);
    do {
        char *d = pd + iter_off(&it, sd);
        unsigned b = load_bit(bits, pos + (size_t)iter_off(&it, bs));
        switch (dst_t) {
        case T_SFLOAT: *(float *)d = (float)b; break;
        case T_DFLOAT: *(double *)d = (double)b; break;
        case T_INT32: *(int32_t *)d = (int32_t)b; break;
        default: return -1;
        }
    } while (iter_next(&it));
    return 0;
}

/* copy of any view, byte-wise: narray/data_kernel.cu:47-55 */
int numo_copy_bytes(size_t elmsz, int ndim, const size_t *shape,
                    const char *ps, const ssize_t *ss, char *pd, const ssize_t *sd)
{
    iter_t it;
    if (total_of(ndim, shape) == 0) return 0;
    iter_init(&it, ndim, shape);
    do {
        memcpy(pd + iter_off(&it, sd), ps + iter_off(&it, ss), elmsz);
    } while (iter_next(&it));
    return 0;
}

/* fill: narray/gen/tmpl/fill_kernel.cu:3-10 */
int numo_fill(int dtype, int ndim, const size_t *shape, char *p, const ssize_t *s, double v)
{
    iter_t it;
    if (total_of(ndim, shape) == 0) return 0;
    iter_init(&it, ndim, shape);
    do {
        char *d = p + iter_off(&it, s);
        if (dtype == T_SFLOAT) *(float *)d = (float)v;
        else if (dtype == T_DFLOAT) *(double *)d = v;
        else *(int32_t *)d = (int32_t)v;
    } while (iter_next(&it));
    return 0;
}

/* ------------------------------------------------------------------ */
/* Bit ops. narray/gen/tmpl_bit/binary_kernel.cu:1-12 (per-bit form),  */
/* types/bit.h:23-31.                                                  */
/* ------------------------------------------------------------------ */
int numo_bit_binary(const char *op, int ndim, const size_t *shape,
                    const uint32_t *a1, size_t p1, const ssize_t *s1,
                    const uint32_t *a2, size_t p2, const ssize_t *s2,
                    uint32_t *a3, size_t p3, const ssize_t *s3)
{
    iter_t it;
    if (total_of(ndim, shape) == 0) return 0;
    iter_init(&it, ndim, shape);
    do {
        unsigned x = load_bit(a1, p1 + (size_t)iter_off(&it, s1));
        unsigned y = a2 ? load_bit(a2, p2 + (size_t)iter_off(&it, s2)) : 0;
        unsigned z;
        if (!strcmp(op, "and")) z = x & y;
        else if (!strcmp(op, "or")) z = x | y;
        else if (!strcmp(op, "xor")) z = x ^ y;
        else if (!strcmp(op, "eq")) z = ~(x ^ y);
        else if (!strcmp(op, "not")) z = ~x;
        else if (!strcmp(op, "copy")) z = x;
        else return -1;
        store_bit(a3, p3 + (size_t)iter_off(&it, s3), z & 1u);
    } while (iter_next(&it));
    return 0;
}

/* count_true / count_false along a 1-d run of n bits, added onto *out the
 * way the device kernel adds (narray/gen/tmpl_bit/bit_count_kernel.cu:15-24). */
uint64_t numo_bit_count(const uint32_t *a, size_t pos, ssize_t step, uint64_t n, int count_false)
{
    uint64_t c = 0;
    for (uint64_t i = 0; i < n; ++i) {
        unsigned x = load_bit(a, (size_t)((ssize_t)pos + (ssize_t)i * step));
        c += count_false ? (x == 0) : (x != 0);
    }
    return c;
}

/* ------------------------------------------------------------------ */
/* Reductions. One output element at a time; the reduce axes are the   */
/* trailing dims of the (already transposed) input and are walked flat */
/* in row-major order (narray/ndloop.c:421-451 and the FLAT_REDUCE     */
/* contraction), each with the sequential loop of                      */
/* include/cumo/types/real_accum.h:25-441 (float) or                   */
/* include/cumo/types/xint_macro.h f_sum/f_min/... (int).              */
/* ------------------------------------------------------------------ */
#define not_nan(x) ((x) == (x))

/* gather one output's reduce slice into a contiguous scratch so the f_* loops
 * below read exactly the sequence Numo's flat loop reads */
static void gather(char *dst, size_t elmsz, const char *base, int rnd,
                   const size_t *rshape, const ssize_t *rstep)
{
    iter_t it;
    size_t k = 0;
    if (rnd == 0) { memcpy(dst, base, elmsz); return; }
    iter_init(&it, rnd, rshape);
    do {
        memcpy(dst + k * elmsz, base + iter_off(&it, rstep), elmsz);
        ++k;
    } while (iter_next(&it));
}

#define FLOAT_REDUCE(T, SQRT_FN)                                                \
/* real_accum.h:25-36 */                                                       \
static T T##_f_sum(size_t n, const T *p) { T y = 0; for (size_t i = 0; i < n; ++i) y = p[i] + y; return y; } \
/* real_accum.h:38-51 */                                                       \
static T T##_f_sum_nan(size_t n, const T *p) { T y = 0; for (size_t i = 0; i < n; ++i) if (not_nan(p[i])) y = p[i] + y; return y; } \
/* real_accum.h:54-65 */                                                       \
static T T##_f_prod(size_t n, const T *p) { T y = 1; for (size_t i = 0; i < n; ++i) y = p[i] * y; return y; } \
static T T##_f_prod_nan(size_t n, const T *p) { T y = 1; for (size_t i = 0; i < n; ++i) if (not_nan(p[i])) y = p[i] * y; return y; } \
/* real_accum.h:82-95: the divisor is the size_t count converted to dtype */  \
static T T##_f_mean(size_t n, const T *p) { T y = 0; size_t c = 0; for (size_t i = 0; i < n; ++i) { y = p[i] + y; c++; } return y / (T)c; } \
static T T##_f_mean_nan(size_t n, const T *p) { T y = 0; size_t c = 0; for (size_t i = 0; i < n; ++i) if (not_nan(p[i])) { y = p[i] + y; c++; } return y / (T)c; } \
/* real_accum.h:114-131: two passes, fabs goes through double */              \
static T T##_f_var(size_t n, const T *p) {                                     \
    T m = T##_f_mean(n, p), y = 0; size_t c = 0;                               \
    for (size_t i = 0; i < n; ++i) { T a = (T)fabs(p[i] - m); y = y + a * a; c++; } \
    return y / (T)(c - 1); }                                                   \
static T T##_f_var_nan(size_t n, const T *p) {                                 \
    T m = T##_f_mean_nan(n, p), y = 0; size_t c = 0;                           \
    for (size_t i = 0; i < n; ++i) if (not_nan(p[i])) { T a = (T)fabs(p[i] - m); y = y + a * a; c++; } \
    return y / (T)(c - 1); }                                                   \
/* real_accum.h:154-162 */                                                     \
static T T##_f_stddev(size_t n, const T *p) { return (T)SQRT_FN(T##_f_var(n, p)); } \
static T T##_f_stddev_nan(size_t n, const T *p) { return (T)SQRT_FN(T##_f_var_nan(n, p)); } \
/* real_accum.h:164-194 */                                                     \
static T T##_f_rms(size_t n, const T *p) { T y = 0; size_t c = 0;              \
    for (size_t i = 0; i < n; ++i) { T a = (T)fabs(p[i]); y = y + a * a; c++; } \
    return (T)SQRT_FN(y / (T)c); }                                             \
static T T##_f_rms_nan(size_t n, const T *p) { T y = 0; size_t c = 0;          \
    for (size_t i = 0; i < n; ++i) if (not_nan(p[i])) { T a = (T)fabs(p[i]); y = y + a * a; c++; } \
    return (T)SQRT_FN(y / (T)c); }                                             \
/* real_accum.h:217-237: skip leading NaN, later NaN lose the comparison */   \
static T T##_f_min(size_t n, const T *p) { T y = 0; size_t i = 0;              \
    for (; i < n;) { y = p[i++]; if (not_nan(y)) { for (; i < n; ++i) if (p[i] < y) y = p[i]; break; } } \
    return y; }                                                                \
static T T##_f_max(size_t n, const T *p) { T y = 0; size_t i = 0;              \
    for (; i < n;) { y = p[i++]; if (not_nan(y)) { for (; i < n; ++i) if (p[i] > y) y = p[i]; break; } } \
    return y; }                                                                \
/* real_accum.h:198-215,239-256: first NaN wins */                             \
static T T##_f_min_nan(size_t n, const T *p) { T y = p[0]; if (!not_nan(y)) return y; \
    for (size_t i = 1; i < n; ++i) { if (!not_nan(p[i])) return p[i]; if (p[i] < y) y = p[i]; } return y; } \
static T T##_f_max_nan(size_t n, const T *p) { T y = p[0]; if (!not_nan(y)) return y; \
    for (size_t i = 1; i < n; ++i) { if (!not_nan(p[i])) return p[i]; if (p[i] > y) y = p[i]; } return y; } \
/* real_accum.h:300-322,344-366 */                                             \
static size_t T##_f_min_index(size_t n, const T *p) {                          \
    size_t j = 0, i = 0;                                                       \
    while (i < n && !not_nan(p[i])) ++i;                                       \
    if (i < n) {                                                               \
        T y = p[i]; j = i;                                                     \
        for (++i; i < n; ++i) { if (p[i] < y) { y = p[i]; j = i; } }           \
    }                                                                          \
    return j; }                                                                \
static size_t T##_f_max_index(size_t n, const T *p) {                          \
    size_t j = 0, i = 0;                                                       \
    while (i < n && !not_nan(p[i])) ++i;                                       \
    if (i < n) {                                                               \
        T y = p[i]; j = i;                                                     \
        for (++i; i < n; ++i) { if (p[i] > y) { y = p[i]; j = i; } }           \
    }                                                                          \
    return j; }                                                                \
/* real_accum.h:280-298,324-342 */                                             \
static size_t T##_f_min_index_nan(size_t n, const T *p) { size_t j = 0; T y = p[0]; \
    if (!not_nan(y)) return 0;                                                 \
    for (size_t i = 1; i < n; ++i) { if (!not_nan(p[i])) return i; if (p[i] < y) { y = p[i]; j = i; } } return j; } \
static size_t T##_f_max_index_nan(size_t n, const T *p) { size_t j = 0; T y = p[0]; \
    if (!not_nan(y)) return 0;                                                 \
    for (size_t i = 1; i < n; ++i) { if (!not_nan(p[i])) return i; if (p[i] > y) { y = p[i]; j = i; } } return j; }

FLOAT_REDUCE(float, sqrt)
FLOAT_REDUCE(double, sqrt)

/* xint_macro.h: f_sum/f_prod widen to int64; f_min/f_max/f_*_index are the
 * plain first-wins scans. */
static int64_t i32_f_sum(size_t n, const int32_t *p) { int64_t y = 0; for (size_t i = 0; i < n; ++i) y += p[i]; return y; }
static int64_t i32_f_prod(size_t n, const int32_t *p) { uint64_t y = 1; for (size_t i = 0; i < n; ++i) y *= (uint64_t)(int64_t)p[i]; return (int64_t)y; }
static int32_t i32_f_min(size_t n, const int32_t *p) { int32_t y = p[0]; for (size_t i = 1; i < n; ++i) if (p[i] < y) y = p[i]; return y; }
static int32_t i32_f_max(size_t n, const int32_t *p) { int32_t y = p[0]; for (size_t i = 1; i < n; ++i) if (p[i] > y) y = p[i]; return y; }
static size_t i32_f_min_index(size_t n, const int32_t *p) { size_t j = 0; int32_t y = p[0]; for (size_t i = 1; i < n; ++i) if (p[i] < y) { y = p[i]; j = i; } return j; }
static size_t i32_f_max_index(size_t n, const int32_t *p) { size_t j = 0; int32_t y = p[0]; for (size_t i = 1; i < n; ++i) if (p[i] > y) { y = p[i]; j = i; } return j; }

/* 1-d entry points of the f_* loops (tests, and the benchmark's CPU leg). */
float numo_sfloat_f(const char *op, size_t n, const float *p);
double numo_dfloat_f(const char *op, size_t n, const double *p);

#define FLOAT_F_DISPATCH(T, NAME)                                              \
T NAME(const char *op, size_t n, const T *p)                                   \
{                                                                              \
    if (!strcmp(op, "sum")) return T##_f_sum(n, p);                            \
    if (!strcmp(op, "sum_nan")) return T##_f_sum_nan(n, p);                    \
    if (!strcmp(op, "prod")) return T##_f_prod(n, p);                          \
    if (!strcmp(op, "prod_nan")) return T##_f_prod_nan(n, p);                  \
    if (!strcmp(op, "mean")) return T##_f_mean(n, p);                          \
    if (!strcmp(op, "mean_nan")) return T##_f_mean_nan(n, p);                  \
    if (!strcmp(op, "var")) return T##_f_var(n, p);                            \
    if (!strcmp(op, "var_nan")) return T##_f_var_nan(n, p);                    \
    if (!strcmp(op, "stddev")) return T##_f_stddev(n, p);                      \
    if (!strcmp(op, "stddev_nan")) return T##_f_stddev_nan(n, p);              \
    if (!strcmp(op, "rms")) return T##_f_rms(n, p);                            \
    if (!strcmp(op, "rms_nan")) return T##_f_rms_nan(n, p);                    \
    if (!strcmp(op, "min")) return T##_f_min(n, p);                            \
    if (!strcmp(op, "min_nan")) return T##_f_min_nan(n, p);                    \
    if (!strcmp(op, "max")) return T##_f_max(n, p);                            \
    if (!strcmp(op, "max_nan")) return T##_f_max_nan(n, p);                    \
    if (!strcmp(op, "ptp")) return T##_f_max(n, p) - T##_f_min(n, p);          \
    if (!strcmp(op, "ptp_nan")) { /* real_accum.h:368-404 */                   \
        T mn = T##_f_min_nan(n, p), mx = T##_f_max_nan(n, p);                  \
        return not_nan(mn) ? (mx - mn) : (mn - mn); }                          \
    return (T)NAN;                                                             \
}
FLOAT_F_DISPATCH(float, numo_sfloat_f)
FLOAT_F_DISPATCH(double, numo_dfloat_f)

int64_t numo_sfloat_index_f(const char *op, size_t n, const float *p)
{
    if (!strcmp(op, "min_index") || !strcmp(op, "argmin")) return (int64_t)float_f_min_index(n, p);
    if (!strcmp(op, "max_index") || !strcmp(op, "argmax")) return (int64_t)float_f_max_index(n, p);
    if (!strcmp(op, "min_index_nan") || !strcmp(op, "argmin_nan")) return (int64_t)float_f_min_index_nan(n, p);
    if (!strcmp(op, "max_index_nan") || !strcmp(op, "argmax_nan")) return (int64_t)float_f_max_index_nan(n, p);
    return -1;
}

int64_t numo_dfloat_index_f(const char *op, size_t n, const double *p)
{
    if (!strcmp(op, "min_index") || !strcmp(op, "argmin")) return (int64_t)double_f_min_index(n, p);
    if (!strcmp(op, "max_index") || !strcmp(op, "argmax")) return (int64_t)double_f_max_index(n, p);
    if (!strcmp(op, "min_index_nan") || !strcmp(op, "argmin_nan")) return (int64_t)double_f_min_index_nan(n, p);
    if (!strcmp(op, "max_index_nan") || !strcmp(op, "argmax_nan")) return (int64_t)double_f_max_index_nan(n, p);
    return -1;
}

/* The N-d reduction driver.
 *   in_ndim dims of the input, the first out_ndim are output dims and the rest
 *   are reduced (include/cumo/indexer.h:189-220).
 *   out element type: dtype for float ops; int64 for Int32 sum/prod
 *   (narray/gen/spec.rb:308-319); idx_bytes (4 or 8) wide signed integers for
 *   argmin/argmax and min_index/max_index (narray/gen/tmpl/accum_arg.c:92-110).
 * For arg ops the answer is the position along the flattened reduce axes; for
 * the _index ops it is the element offset from in (in elements) which requires a
 * contiguous input, as the reference requires (tmpl/accum_index.c).
 * scratch must hold reduce_total elements.
 * Returns -1 for an unknown op. */
int numo_reduce(const char *op, int dtype, int in_ndim, int out_ndim,
                const size_t *shape, const char *pin, const ssize_t *sin,
                char *pout, const ssize_t *sout, int idx_bytes, char *scratch)
{
    iter_t it;
    int rnd = in_ndim - out_ndim;
    size_t n = total_of(rnd, shape + out_ndim);
    size_t elmsz = (dtype == T_DFLOAT) ? 8 : 4;
    int is_arg = !strncmp(op, "arg", 3);
    int is_index = (strstr(op, "_index") != NULL);
    if (total_of(out_ndim, shape) == 0) return 0;
    iter_init(&it, out_ndim, shape);
    do {
        ssize_t in_off = iter_off(&it, sin);
        char *o = pout + iter_off(&it, sout);
        gather(scratch, elmsz, pin + in_off, rnd, shape + out_ndim, sin + out_ndim);
        if (is_arg || is_index) {
            int64_t j;
            if (dtype == T_SFLOAT) j = numo_sfloat_index_f(op, n, (const float *)scratch);
            else if (dtype == T_DFLOAT) j = numo_dfloat_index_f(op, n, (const double *)scratch);
            else {
                const int32_t *p = (const int32_t *)scratch;
                if (strstr(op, "min")) j = (int64_t)i32_f_min_index(n, p);
                else j = (int64_t)i32_f_max_index(n, p);
            }
            if (j < 0) return -1;
            if (is_index) {
                /* position in the slice -> offset of that element from the start of
                 * the array, in elements (tmpl/accum_index.c: the answer indexes the
                 * flattened array) */
                ssize_t off = in_off;
                int64_t r = j;
                for (int d = rnd; --d >= 0;) {
                    int64_t nd_ = (int64_t)shape[out_ndim + d];
                    off += (ssize_t)(r % nd_) * sin[out_ndim + d];
                    r /= nd_;
                }
                j = (int64_t)(off / (ssize_t)elmsz);
            }
            if (idx_bytes == 4) *(int32_t *)o = (int32_t)j; else *(int64_t *)o = j;
        } else if (dtype == T_SFLOAT) {
            float r = numo_sfloat_f(op, n, (const float *)scratch);
            *(float *)o = r;
        } else if (dtype == T_DFLOAT) {
            double r = numo_dfloat_f(op, n, (const double *)scratch);
            *(double *)o = r;
        } else {
            const int32_t *p = (const int32_t *)scratch;
            if (!strcmp(op, "sum")) *(int64_t *)o = i32_f_sum(n, p);
            else if (!strcmp(op, "prod")) *(int64_t *)o = i32_f_prod(n, p);
            else if (!strcmp(op, "min")) *(int32_t *)o = i32_f_min(n, p);
            else if (!strcmp(op, "max")) *(int32_t *)o = i32_f_max(n, p);
            else if (!strcmp(op, "ptp")) *(int32_t *)o = (int32_t)((uint32_t)i32_f_max(n, p) - (uint32_t)i32_f_min(n, p));
            else return -1;
        }
    } while (iter_next(&it));
    return 0;
}

/* ------------------------------------------------------------------ */
/* Row loops for the CPU baseline timing. Numo's ndloop walks the outer */
/* dimensions on the host and hands each innermost run to the iterator, */
/* whose loop shapes are those of narray/gen/tmpl/binary.c:38-97: an    */
/* indexed loop when every step is the element size, a pointer-bumping  */
/* loop otherwise, the right operand read once when its step is 0.      */
/* The benchmark times these, not the generic N-d driver above.         */
/* ------------------------------------------------------------------ */
#define ROW_LOOP(T, EXPR)                                                        \
    for (size_t r = 0; r < nrows; ++r) {                                         \
        const char *a = p1 + (ssize_t)r * r1, *b = p2 + (ssize_t)r * r2;         \
        char *c = p3 + (ssize_t)r * r3;                                          \
        if (s1 == (ssize_t)sizeof(T) && s2 == (ssize_t)sizeof(T) && s3 == (ssize_t)sizeof(T)) { \
            const T *x_ = (const T *)a, *y_ = (const T *)b; T *z_ = (T *)c;      \
            for (size_t i = 0; i < n; ++i) { T x = x_[i], y = y_[i]; z_[i] = (EXPR); } \
        } else if (s2 == 0 && s1 == (ssize_t)sizeof(T) && s3 == (ssize_t)sizeof(T)) { \
            const T *x_ = (const T *)a; T y = *(const T *)b; T *z_ = (T *)c;     \
            for (size_t i = 0; i < n; ++i) { T x = x_[i]; z_[i] = (EXPR); }      \
        } else {                                                                 \
            for (size_t i = 0; i < n; ++i) {                                     \
                T x = *(const T *)a, y = *(const T *)b;                          \
                *(T *)c = (EXPR);                                                \
                a += s1; b += s2; c += s3;                                       \
            }                                                                    \
        }                                                                        \
    }

#define ROWS_BY_OP(T)                                                            \
    if (!strcmp(op, "add")) { ROW_LOOP(T, x + y) return 0; }                     \
    if (!strcmp(op, "sub")) { ROW_LOOP(T, x - y) return 0; }                     \
    if (!strcmp(op, "mul")) { ROW_LOOP(T, x * y) return 0; }                     \
    if (!strcmp(op, "div")) { ROW_LOOP(T, x / y) return 0; }

int numo_rows_binary(const char *op, int dtype, size_t nrows, size_t n,
                     const char *p1, ssize_t r1, ssize_t s1,
                     const char *p2, ssize_t r2, ssize_t s2,
                     char *p3, ssize_t r3, ssize_t s3)
{
    if (dtype == T_SFLOAT) { ROWS_BY_OP(float) }
    else if (dtype == T_DFLOAT) { ROWS_BY_OP(double) }
    return -1;
}

/* one f_<op> per contiguous row (types/real_accum.h), result per row */
int numo_rows_reduce(const char *op, int dtype, size_t nrows, size_t n,
                     const char *p, ssize_t row_step, char *out)
{
    for (size_t r = 0; r < nrows; ++r) {
        if (dtype == T_SFLOAT) ((float *)out)[r] = numo_sfloat_f(op, n, (const float *)(p + (ssize_t)r * row_step));
        else if (dtype == T_DFLOAT) ((double *)out)[r] = numo_dfloat_f(op, n, (const double *)(p + (ssize_t)r * row_step));
        else return -1;
    }
    return 0;
}

/* ------------------------------------------------------------------ */
/* Float ** Int32: types/float_macro.h:125-144 (pow_int). Products in  */
/* the element type up to an exponent of 64, pow() beyond, 1/.. for a  */
/* negative exponent. Flat arrays of n elements; p_step 0 repeats one  */
/* exponent, x_step 0 one base.                                        */
/* ------------------------------------------------------------------ */
#define POW_INT(T)                                                             \
static T T##_pow_int(T x, int p)                                               \
{                                                                              \
    T r = 1;                                                                   \
    switch (p) {                                                               \
    case 0: return 1;                                                          \
    case 1: return x;                                                          \
    case 2: return x * x;                                                      \
    case 3: return x * x * x;                                                  \
    case 4: x = x * x; return x * x;                                           \
    }                                                                          \
    if (p < 0) return 1 / T##_pow_int(x, (int)(0u - (unsigned)p));             \
    if (p > 64) return (T)pow(x, p);                                           \
    while (p) { if (p & 1) r *= x; x *= x; p >>= 1; }                          \
    return r;                                                                  \
}
POW_INT(float)
POW_INT(double)

int numo_pow_int(int dtype, size_t n, const void *x, ssize_t x_step, const int32_t *p, ssize_t p_step, void *out)
{
    for (size_t i = 0; i < n; ++i) {
        const int32_t e = p[(ssize_t)i * p_step];
        if (dtype == T_SFLOAT) ((float *)out)[i] = float_pow_int(((const float *)x)[(ssize_t)i * x_step], e);
        else if (dtype == T_DFLOAT) ((double *)out)[i] = double_pow_int(((const double *)x)[(ssize_t)i * x_step], e);
        else return -1;
    }
    return 0;
}

/* ------------------------------------------------------------------ */
/* cumsum / cumprod along one run: the host loop of                    */
/* narray/gen/tmpl/cum.c:32-45 with the operators of                   */
/* types/real_accum.h:9-23 and xint_macro.h:46-47. The first element   */
/* is copied through; each later one updates the running value.        */
/* ------------------------------------------------------------------ */
#define CUM_RUN(T, ISNAN)                                                      \
static void T##_cum_run(int prod, int nan, size_t n, const char *p1, ssize_t s1, char *p2, ssize_t s2) \
{                                                                              \
    if (n == 0) return;                                                        \
    T x = *(const T *)p1;                                                      \
    *(T *)p2 = x;                                                              \
    for (size_t i = 1; i < n; ++i) {                                           \
        const T y = *(const T *)(p1 + (ssize_t)i * s1);                        \
        if (nan) {                                                             \
            if (ISNAN(x)) x = y;                                               \
            else if (!ISNAN(y)) x = prod ? x * y : x + y;                      \
        } else {                                                               \
            x = prod ? x * y : x + y;                                          \
        }                                                                      \
        *(T *)(p2 + (ssize_t)i * s2) = x;                                      \
    }                                                                          \
}
#define FISNAN(v) ((v) != (v))
CUM_RUN(float, FISNAN)
CUM_RUN(double, FISNAN)

int numo_cum_run(int prod, int dtype, int nan, size_t n, const char *p1, ssize_t s1, char *p2, ssize_t s2)
{
    if (dtype == T_SFLOAT) float_cum_run(prod, nan, n, p1, s1, p2, s2);
    else if (dtype == T_DFLOAT) double_cum_run(prod, nan, n, p1, s1, p2, s2);
    else if (dtype == T_INT32) {
        if (n == 0) return 0;
        uint32_t x = *(const uint32_t *)p1;
        *(uint32_t *)p2 = x;
        for (size_t i = 1; i < n; ++i) {
            const uint32_t y = *(const uint32_t *)(p1 + (ssize_t)i * s1);
            x = prod ? x * y : x + y;   /* wrapping, done in unsigned */
            *(uint32_t *)(p2 + (ssize_t)i * s2) = x;
        }
    } else return -1;
    return 0;
}

/* mulsum over one run, added onto *acc: narray/gen/tmpl/accum_binary.c:27-38   */
/* with types/real_accum.h:3-7 and xint_macro.h:44. Product and sum are two     */
/* roundings in the element type (this file is built with -ffp-contract=off).   */
int numo_mulsum_run(int dtype, int nan, size_t n, const char *p1, ssize_t s1, const char *p2, ssize_t s2, void *acc)
{
    if (dtype == T_SFLOAT) {
        float z = *(float *)acc;
        for (size_t i = 0; i < n; ++i) {
            const float x = *(const float *)(p1 + (ssize_t)i * s1), y = *(const float *)(p2 + (ssize_t)i * s2);
            if (nan && (x != x || y != y)) continue;
            z = x * y + z;
        }
        *(float *)acc = z;
    } else if (dtype == T_DFLOAT) {
        double z = *(double *)acc;
        for (size_t i = 0; i < n; ++i) {
            const double x = *(const double *)(p1 + (ssize_t)i * s1), y = *(const double *)(p2 + (ssize_t)i * s2);
            if (nan && (x != x || y != y)) continue;
            z = x * y + z;
        }
        *(double *)acc = z;
    } else if (dtype == T_INT32) {
        uint32_t z = *(uint32_t *)acc;
        for (size_t i = 0; i < n; ++i)
            z += *(const uint32_t *)(p1 + (ssize_t)i * s1) * *(const uint32_t *)(p2 + (ssize_t)i * s2);
        *(uint32_t *)acc = z;
    } else return -1;
    return 0;
}
