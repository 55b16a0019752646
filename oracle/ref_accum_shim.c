/*
 * ref_accum_shim.c -- TEST INFRASTRUCTURE. Compiles the reference's own
 * sequential reduction loops (ext/cumo/include/cumo/types/real_accum.h, the
 * f_sum ... f_max_index functions that Numo's C is made of) for one element
 * type, so that the restatement in numo_oracle.c can be checked against the
 * real thing. The header is included from where it lies in the reference tree
 * (path given by REF_ACCUM_H on the command line); no reference source is
 * copied. real_accum.h is written to be included after the element type and the
 * arithmetic macros are defined (the reference does so from types/sfloat.h and
 * types/dfloat.h through float_macro.h, which cannot be compiled here because it
 * needs ruby.h); the definitions below are those one-line macros
 * (types/float_macro.h:12-54,84).
 *
 * Build: see oracle/Makefile. Output goes to oracle/_ref/ only.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>
#include <sys/types.h>

typedef REF_DTYPE dtype;

#define m_zero 0.0
#define m_one 1.0
#define m_from_real(x) (x)
#define m_add(x, y) ((x) + (y))
#define m_sub(x, y) ((x) - (y))
#define m_mul(x, y) ((x) * (y))
#define m_div(x, y) ((x) / (y))
#define m_abs(x) fabs(x)
#define m_square(x) ((x) * (x))
#define m_sqrt(x) sqrt(x)
#define m_gt(x, y) ((x) > (y))
#define m_ge(x, y) ((x) >= (y))
#define m_lt(x, y) ((x) < (y))
#define m_le(x, y) ((x) <= (y))

#include REF_ACCUM_H

#define CAT2(a, b) a##b
#define CAT(a, b) CAT2(a, b)

/* value reductions; returns NaN for an unknown name */
double CAT(REF_NAME, _ref_f)(const char *op, size_t n, char *p, ssize_t stride)
{
    dtype mn, mx;
    if (!strcmp(op, "sum")) return f_sum(n, p, stride);
    if (!strcmp(op, "sum_nan")) return f_sum_nan(n, p, stride);
    if (!strcmp(op, "prod")) return f_prod(n, p, stride);
    if (!strcmp(op, "prod_nan")) return f_prod_nan(n, p, stride);
    if (!strcmp(op, "mean")) return f_mean(n, p, stride);
    if (!strcmp(op, "mean_nan")) return f_mean_nan(n, p, stride);
    if (!strcmp(op, "var")) return f_var(n, p, stride);
    if (!strcmp(op, "var_nan")) return f_var_nan(n, p, stride);
    if (!strcmp(op, "stddev")) return f_stddev(n, p, stride);
    if (!strcmp(op, "stddev_nan")) return f_stddev_nan(n, p, stride);
    if (!strcmp(op, "rms")) return f_rms(n, p, stride);
    if (!strcmp(op, "rms_nan")) return f_rms_nan(n, p, stride);
    if (!strcmp(op, "min")) return f_min(n, p, stride);
    if (!strcmp(op, "min_nan")) return f_min_nan(n, p, stride);
    if (!strcmp(op, "max")) return f_max(n, p, stride);
    if (!strcmp(op, "max_nan")) return f_max_nan(n, p, stride);
    if (!strcmp(op, "ptp")) return f_ptp(n, p, stride);
    if (!strcmp(op, "ptp_nan")) return f_ptp_nan(n, p, stride);
    if (!strcmp(op, "minmax_min")) { f_minmax(n, p, stride, &mn, &mx); return mn; }
    if (!strcmp(op, "minmax_max")) { f_minmax(n, p, stride, &mn, &mx); return mx; }
    return NAN;
}

int64_t CAT(REF_NAME, _ref_index_f)(const char *op, size_t n, char *p, ssize_t stride)
{
    if (!strcmp(op, "min_index")) return (int64_t)f_min_index(n, p, stride);
    if (!strcmp(op, "max_index")) return (int64_t)f_max_index(n, p, stride);
    if (!strcmp(op, "min_index_nan")) return (int64_t)f_min_index_nan(n, p, stride);
    if (!strcmp(op, "max_index_nan")) return (int64_t)f_max_index_nan(n, p, stride);
    return -1;
}
