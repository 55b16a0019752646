/*
 * cumo_hip.h -- the C-ABI of the MI355X (gfx950) array-compute library.
 *
 * Everything in this header is `extern "C"`, plain pointers and sizes. The
 * first half reproduces, byte for byte, the launch descriptors and launcher
 * entry points that the Cumo Ruby extension's generated host iterators bind
 * (the reference file:line each one replaces is cited beside it), so that the
 * extension can link this library in place of its own kernel translation
 * units. The second half (`cumo_hip_*`) is what this library adds: the error
 * hook that stands in for the extension's raise, stream selection, the memory
 * pool's C interface and the launch planner's introspection calls. The host
 * launch layer (ndloop) that builds the descriptors from array views is
 * declared in cumo_hip_ndloop.h.
 */
#ifndef CUMO_HIP_H
#define CUMO_HIP_H

#include <stddef.h>
#include <stdint.h>
#include <stdbool.h>
#include <sys/types.h>

#if defined(__cplusplus)
extern "C" {
#endif
/* The library is built with hidden visibility; what this header declares is what it exports. */
#if defined(__GNUC__)
#pragma GCC visibility push(default)
#endif

/* ------------------------------------------------------------------------
 * 1. Launch descriptors (reference: ext/cumo/include/cumo/indexer.h:16-68,
 *    ext/cumo/include/cumo/narray.h:236-240,489-496).
 * ---------------------------------------------------------------------- */
#define CUMO_NA_MAX_DIMENSION 12            /* narray.h:489 */
typedef unsigned int CUMO_BIT_DIGIT;        /* narray.h:492 */
#define CUMO_NB (sizeof(CUMO_BIT_DIGIT)*8)  /* narray.h:494 */

/* stride or index array of one dimension (narray.h:236-240,324-330): a stride
 * is stored as (stride<<1)|1, anything with bit 0 clear is a device pointer to
 * size_t offsets. */
typedef union {
    ssize_t stride;
    size_t *index;
} cumo_stridx_t;
#define CUMO_SDX_IS_STRIDE(x) ((x).stride&0x1)
#define CUMO_SDX_IS_INDEX(x)  (!CUMO_SDX_IS_STRIDE(x))
#define CUMO_SDX_GET_STRIDE(x) ((x).stride>>1)
#define CUMO_SDX_GET_INDEX(x)  ((x).index)
#define CUMO_SDX_SET_STRIDE(x,s) ((x).stride=((s)<<1)|0x1)
#define CUMO_SDX_SET_INDEX(x,idx) ((x).index=idx)

/* indexer.h:16-22 (216 bytes). index[] and raw_index are scratch the
 * reference's kernels write per element; this library never touches them. */
typedef struct {
    unsigned char ndim;
    size_t total_size;
    size_t shape[CUMO_NA_MAX_DIMENSION];
    uint64_t index[CUMO_NA_MAX_DIMENSION];
    uint64_t raw_index;
} cumo_na_indexer_t;

/* indexer.h:28-31 (104 bytes). ptr already includes the view offset; step is a
 * signed byte stride per dimension, 0 for a broadcast dimension. */
typedef struct {
    char* ptr;
    ssize_t step[CUMO_NA_MAX_DIMENSION];
} cumo_na_iarray_t;

/* indexer.h:40-44 (112 bytes). pos and step are in bits. */
typedef struct {
    CUMO_BIT_DIGIT* ptr;
    size_t pos;
    ssize_t step[CUMO_NA_MAX_DIMENSION];
} cumo_na_bit_iarray_t;

/* indexer.h:46-49 */
typedef struct {
    char* ptr;
    cumo_stridx_t stridx[CUMO_NA_MAX_DIMENSION];
} cumo_na_iarray_stridx_t;

/* indexer.h:57-61 */
typedef struct {
    CUMO_BIT_DIGIT* ptr;
    size_t pos;
    cumo_stridx_t stridx[CUMO_NA_MAX_DIMENSION];
} cumo_na_bit_iarray_stridx_t;

/* indexer.h:63-68 (640 bytes). The first out_indexer.ndim dimensions of `in`
 * are the output dimensions, the rest are reduced (indexer.h:189-220). */
typedef struct {
    cumo_na_iarray_t in;
    cumo_na_iarray_t out;
    cumo_na_indexer_t in_indexer;
    cumo_na_indexer_t out_indexer;
} cumo_na_reduction_arg_t;

/* ------------------------------------------------------------------------
 * 2. Runtime glue and device memory (reference:
 *    ext/cumo/include/cumo/cuda/memory_pool.h:15-24,
 *    ext/cumo/include/cumo/template_kernel.h:83-90,
 *    ext/cumo/include/cumo/cuda/runtime.h:59-65, ext/cumo/cuda/runtime.c:16-68).
 *    In the reference these raise a Ruby exception on failure; here a failure
 *    goes to the handler installed with cumo_hip_set_error_handler (which may
 *    longjmp/raise), or is latched for cumo_hip_last_error when none is set.
 * ---------------------------------------------------------------------- */
char* cumo_cuda_runtime_malloc(size_t size);
void  cumo_cuda_runtime_free(char *ptr);
void  cumo_cuda_runtime_free_no_raise(char *ptr);
void  cumo_cuda_runtime_check_kernel_launch(void);
int*  cumo_cuda_runtime_error_flag_ptr(void);
int*  cumo_cuda_runtime_error_flag_new(void);
bool  cumo_cuda_runtime_error_flag_get(int *flag);
size_t* cumo_cuda_runtime_error_item_ptr(void);
size_t* cumo_cuda_runtime_error_item_new(void);

/* ------------------------------------------------------------------------
 * 3. Elementwise launchers. The lists below are expanded into declarations
 *    here and into definitions in the library, so the two cannot drift.
 *    T(type_name, c_type)
 * ---------------------------------------------------------------------- */
#define CUMO_HIP_FLOAT_TYPES(T) T(sfloat, float) T(dfloat, double)
#define CUMO_HIP_INT_TYPES(T)   T(int32, int32_t)

/* binary ops with a scalar form: narray/gen/tmpl/binary_kernel.cu:11,52-81,
 * host declaration narray/gen/tmpl/binary.c:12-15; op list narray/gen/spec.rb:199-207,249-256,268-271 */
#define CUMO_HIP_BINARY_OPS_ALL(X, t, c)   X(t, c, add) X(t, c, sub) X(t, c, mul) X(t, c, div) X(t, c, mod)
#define CUMO_HIP_BINARY_OPS_FLOAT(X, t, c) X(t, c, copysign)
#define CUMO_HIP_BINARY_OPS_INT(X, t, c)   X(t, c, bit_and) X(t, c, bit_or) X(t, c, bit_xor) X(t, c, left_shift) X(t, c, right_shift)

#define CUMO_HIP_DECL_BINARY(t, c, op) \
    void cumo_iter_##t##_##op##_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_iarray_t* a3, cumo_na_indexer_t* indexer, int* divzero); \
    void cumo_iter_##t##_##op##_s_kernel_launch(cumo_na_iarray_t* a1, c sv, cumo_na_iarray_t* a3, cumo_na_indexer_t* indexer, int* divzero, int scalar_is_left);

/* unary ops: narray/gen/tmpl/unary_kernel.cu:14-42, host narray/gen/tmpl/unary.c:3;
 * op list narray/gen/spec.rb:216-219,259,272-277 */
#define CUMO_HIP_UNARY_OPS_ALL(X, t, c)   X(t, c, minus) X(t, c, reciprocal) X(t, c, sign) X(t, c, square)
#define CUMO_HIP_UNARY_OPS_FLOAT(X, t, c) X(t, c, floor) X(t, c, round) X(t, c, ceil) X(t, c, trunc) X(t, c, rint)
#define CUMO_HIP_UNARY_OPS_INT(X, t, c)   X(t, c, bit_not)

#define CUMO_HIP_DECL_UNARY(t, c, op) \
    void cumo_iter_##t##_##op##_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_indexer_t* indexer, int* divzero);

/* abs: narray/gen/tmpl/unary2_kernel.cu:15-41, host narray/gen/tmpl/unary2.c:3 */
#define CUMO_HIP_DECL_ABS(t, c) \
    void cumo_iter_##t##_abs_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_indexer_t* indexer, int* intmin);

/* NMath one-argument functions: narray/gen/tmpl/unary_s_kernel.cu:3-29, host
 * narray/gen/tmpl/unary_s.c:2; list narray/gen/spec.rb:427-457 */
#define CUMO_HIP_MATH_OPS(X, t, c) \
    X(t, c, sqrt) X(t, c, cbrt) X(t, c, log) X(t, c, log2) X(t, c, log10) X(t, c, exp) X(t, c, exp2) X(t, c, exp10) \
    X(t, c, sin) X(t, c, cos) X(t, c, tan) X(t, c, asin) X(t, c, acos) X(t, c, atan) \
    X(t, c, sinh) X(t, c, cosh) X(t, c, tanh) X(t, c, asinh) X(t, c, acosh) X(t, c, atanh) \
    X(t, c, sinc) X(t, c, erf) X(t, c, erfc) X(t, c, log1p) X(t, c, expm1)

#define CUMO_HIP_DECL_MATH(t, c, op) \
    void cumo_iter_##t##_math_s_##op##_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_indexer_t* indexer);

/* NMath two-argument functions: narray/gen/tmpl/binary_s_kernel.cu:7-52, host
 * narray/gen/tmpl/binary_s.c:2-3 */
#define CUMO_HIP_MATH2_OPS(X, t, c) X(t, c, atan2) X(t, c, hypot) X(t, c, ldexp)

#define CUMO_HIP_DECL_MATH2(t, c, op) \
    void cumo_iter_##t##_math_s_##op##_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_iarray_t* a3, cumo_na_indexer_t* indexer); \
    void cumo_iter_##t##_math_s_##op##_s_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a3, cumo_na_indexer_t* indexer, c sv, int scalar_is_left);

/* comparisons into Bit: narray/gen/tmpl/cond_binary_kernel.cu:7-53, host
 * narray/gen/tmpl/cond_binary.c:2-3 */
#define CUMO_HIP_COND_OPS_ALL(X, t, c)   X(t, c, eq) X(t, c, ne) X(t, c, gt) X(t, c, ge) X(t, c, lt) X(t, c, le)
#define CUMO_HIP_COND_OPS_FLOAT(X, t, c) X(t, c, nearly_eq)

#define CUMO_HIP_DECL_COND(t, c, op) \
    void cumo_iter_##t##_##op##_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_bit_iarray_t* a3, cumo_na_indexer_t* indexer); \
    void cumo_iter_##t##_##op##_s_kernel_launch(cumo_na_iarray_t* a1, c sv, cumo_na_bit_iarray_t* a3, cumo_na_indexer_t* indexer, int scalar_is_left);

/* float classification into Bit: narray/gen/tmpl/cond_unary_kernel.cu:3-29,
 * host narray/gen/tmpl/cond_unary.c:2 */
#define CUMO_HIP_COND_UNARY_OPS(X, t, c) X(t, c, isnan) X(t, c, isinf) X(t, c, isposinf) X(t, c, isneginf) X(t, c, isfinite) X(t, c, signbit)

#define CUMO_HIP_DECL_COND_UNARY(t, c, op) \
    void cumo_iter_##t##_##op##_kernel_launch(cumo_na_iarray_t* a1, cumo_na_bit_iarray_t* a2, cumo_na_indexer_t* indexer);

/* fill and 0-dim construction: narray/gen/tmpl/fill_kernel.cu:3-27 (host
 * fill.c:2), narray/gen/tmpl/new_dim0_kernel.cu:2-10 (host new_dim0.c:2);
 * Bit -> number: narray/gen/tmpl/store_bit_kernel.cu:3-30 (host store_bit.c:2) */
#define CUMO_HIP_DECL_FILL(t, c) \
    void cumo_iter_##t##_fill_kernel_launch(cumo_na_iarray_t* a1, cumo_na_indexer_t* indexer, c val); \
    void cumo_##t##_new_dim0_kernel_launch(c *ptr, c x); \
    void cumo_iter_##t##_store_bit_kernel_launch(cumo_na_iarray_stridx_t* a1, cumo_na_bit_iarray_stridx_t* a2, cumo_na_indexer_t* indexer);

/* Bit has no new_dim0 template of its own, so the generator renders the common one for it
 * (gen/cogen.rb:37-39 searches tmpl_bit, then tmpl; tmpl/new_dim0_kernel.cu:2-10 with dtype =
 * BIT_DIGIT): the whole first word of a 0-dim Bit array becomes x. */
void cumo_bit_new_dim0_kernel_launch(unsigned int *ptr, unsigned int x);

CUMO_HIP_BINARY_OPS_ALL(CUMO_HIP_DECL_BINARY, sfloat, float)
CUMO_HIP_BINARY_OPS_ALL(CUMO_HIP_DECL_BINARY, dfloat, double)
CUMO_HIP_BINARY_OPS_ALL(CUMO_HIP_DECL_BINARY, int32, int32_t)
CUMO_HIP_BINARY_OPS_FLOAT(CUMO_HIP_DECL_BINARY, sfloat, float)
CUMO_HIP_BINARY_OPS_FLOAT(CUMO_HIP_DECL_BINARY, dfloat, double)
CUMO_HIP_BINARY_OPS_INT(CUMO_HIP_DECL_BINARY, int32, int32_t)

CUMO_HIP_UNARY_OPS_ALL(CUMO_HIP_DECL_UNARY, sfloat, float)
CUMO_HIP_UNARY_OPS_ALL(CUMO_HIP_DECL_UNARY, dfloat, double)
CUMO_HIP_UNARY_OPS_ALL(CUMO_HIP_DECL_UNARY, int32, int32_t)
CUMO_HIP_UNARY_OPS_FLOAT(CUMO_HIP_DECL_UNARY, sfloat, float)
CUMO_HIP_UNARY_OPS_FLOAT(CUMO_HIP_DECL_UNARY, dfloat, double)
CUMO_HIP_UNARY_OPS_INT(CUMO_HIP_DECL_UNARY, int32, int32_t)

CUMO_HIP_DECL_ABS(sfloat, float)
CUMO_HIP_DECL_ABS(dfloat, double)
CUMO_HIP_DECL_ABS(int32, int32_t)

CUMO_HIP_MATH_OPS(CUMO_HIP_DECL_MATH, sfloat, float)
CUMO_HIP_MATH_OPS(CUMO_HIP_DECL_MATH, dfloat, double)
CUMO_HIP_MATH2_OPS(CUMO_HIP_DECL_MATH2, sfloat, float)
CUMO_HIP_MATH2_OPS(CUMO_HIP_DECL_MATH2, dfloat, double)
/* NMath.frexp: a2 takes the mantissa, a3 the Int32 exponent
 * (narray/gen/tmpl/frexp_kernel.cu:2-35, host narray/gen/tmpl/frexp.c:1) */
void cumo_iter_sfloat_math_s_frexp_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_iarray_t* a3, cumo_na_indexer_t* indexer);
void cumo_iter_dfloat_math_s_frexp_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_iarray_t* a3, cumo_na_indexer_t* indexer);

CUMO_HIP_COND_OPS_ALL(CUMO_HIP_DECL_COND, sfloat, float)
CUMO_HIP_COND_OPS_ALL(CUMO_HIP_DECL_COND, dfloat, double)
CUMO_HIP_COND_OPS_ALL(CUMO_HIP_DECL_COND, int32, int32_t)
CUMO_HIP_COND_OPS_FLOAT(CUMO_HIP_DECL_COND, sfloat, float)
CUMO_HIP_COND_OPS_FLOAT(CUMO_HIP_DECL_COND, dfloat, double)

CUMO_HIP_COND_UNARY_OPS(CUMO_HIP_DECL_COND_UNARY, sfloat, float)
CUMO_HIP_COND_UNARY_OPS(CUMO_HIP_DECL_COND_UNARY, dfloat, double)

CUMO_HIP_DECL_FILL(sfloat, float)
CUMO_HIP_DECL_FILL(dfloat, double)
CUMO_HIP_DECL_FILL(int32, int32_t)

/* divmod: a3 = a1 / a2, a4 = a1 mod a2 (fmod for the float types, C remainder for Int32, where a
 * zero divisor leaves the element unwritten and sets *divzero): narray/gen/tmpl/binary2_kernel.cu:3-42,
 * host binary2.c:2. modf: a2 the fraction, a3 the integral part, both with the argument's sign:
 * narray/gen/tmpl/unary_ret2_kernel.cu:2-35, types/float_macro_kernel.h:51. */
void cumo_iter_sfloat_divmod_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_iarray_t* a3, cumo_na_iarray_t* a4, cumo_na_indexer_t* indexer, int* divzero);
void cumo_iter_dfloat_divmod_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_iarray_t* a3, cumo_na_iarray_t* a4, cumo_na_indexer_t* indexer, int* divzero);
void cumo_iter_int32_divmod_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_iarray_t* a3, cumo_na_iarray_t* a4, cumo_na_indexer_t* indexer, int* divzero);
void cumo_iter_sfloat_modf_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_iarray_t* a3, cumo_na_indexer_t* indexer);
void cumo_iter_dfloat_modf_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_iarray_t* a3, cumo_na_indexer_t* indexer);

/* poly: z = coef[0] + coef[1] x + ... + coef[ncoef-1] x^(ncoef-1) by Horner's rule in the element
 * type, every coefficient an array descriptor over the same indexer (zero steps for a number);
 * ncoef == 0 answers x (narray/gen/tmpl/poly_kernel.cu:3-45, host poly.c:2,18). */
void cumo_iter_sfloat_poly_kernel_launch(cumo_na_iarray_t* x, cumo_na_iarray_t* coef, int ncoef, cumo_na_iarray_t* z, cumo_na_indexer_t* indexer);
void cumo_iter_dfloat_poly_kernel_launch(cumo_na_iarray_t* x, cumo_na_iarray_t* coef, int ncoef, cumo_na_iarray_t* z, cumo_na_indexer_t* indexer);
void cumo_iter_int32_poly_kernel_launch(cumo_na_iarray_t* x, cumo_na_iarray_t* coef, int ncoef, cumo_na_iarray_t* z, cumo_na_indexer_t* indexer);

/* seq: element number i (row-major over the indexer) gets beg + step * (c + i); beg and step come in
 * the element type, in double for Int32 (narray/gen/tmpl/seq_kernel.cu:14-52, host seq.c:1-21,63-68).
 * logseq: base ** seq over one run, strided or through an index array, float types only
 * (logseq_kernel.cu:2-32, host logseq.c). eye: data where row + kofs == column of an n0 x n1 matrix
 * with byte steps s0, s1, zero elsewhere (eye_kernel.cu:2-18, host eye.c:2,42). */
void cumo_iter_sfloat_seq_kernel_launch(cumo_na_iarray_t* a1, cumo_na_indexer_t* indexer, float beg, float step, double c);
void cumo_iter_dfloat_seq_kernel_launch(cumo_na_iarray_t* a1, cumo_na_indexer_t* indexer, double beg, double step, double c);
void cumo_iter_int32_seq_kernel_launch(cumo_na_iarray_t* a1, cumo_na_indexer_t* indexer, double beg, double step, double c);
void cumo_iter_sfloat_logseq_stride_kernel_launch(char* p1, ssize_t s1, float beg, float step, float base, double c, uint64_t n);
void cumo_iter_sfloat_logseq_index_kernel_launch(char* p1, size_t* idx1, float beg, float step, float base, double c, uint64_t n);
void cumo_iter_dfloat_logseq_stride_kernel_launch(char* p1, ssize_t s1, double beg, double step, double base, double c, uint64_t n);
void cumo_iter_dfloat_logseq_index_kernel_launch(char* p1, size_t* idx1, double beg, double step, double base, double c, uint64_t n);
void cumo_iter_sfloat_eye_stride_kernel_launch(char* ptr, ssize_t s0, ssize_t s1, ssize_t kofs, float data, uint64_t n0, uint64_t n1);
void cumo_iter_dfloat_eye_stride_kernel_launch(char* ptr, ssize_t s0, ssize_t s1, ssize_t kofs, double data, uint64_t n0, uint64_t n1);
void cumo_iter_int32_eye_stride_kernel_launch(char* ptr, ssize_t s0, ssize_t s1, ssize_t kofs, int32_t data, uint64_t n0, uint64_t n1);

/* pow: narray/gen/tmpl/pow_kernel.cu:6-36,58-113, host narray/gen/tmpl/pow.c:2-6.
 * A numeric exponent or base rides in as sv; an Int32 exponent takes the
 * repeated-product form (types/float_macro_kernel.h:125-149, int_macro_kernel.h:26-42). */
#define CUMO_HIP_DECL_POW(t, c) \
    void cumo_iter_##t##_pow_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_iarray_t* a3, cumo_na_indexer_t* indexer); \
    void cumo_iter_##t##_pow_s_kernel_launch(cumo_na_iarray_t* a1, c sv, cumo_na_iarray_t* a3, cumo_na_indexer_t* indexer, int scalar_is_left); \
    void cumo_iter_##t##_pow_int32_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_iarray_t* a3, cumo_na_indexer_t* indexer); \
    void cumo_iter_##t##_pow_int32_s_kernel_launch(cumo_na_iarray_t* a1, int32_t sv, cumo_na_iarray_t* a3, cumo_na_indexer_t* indexer); \
    void cumo_iter_##t##_pow_int32_s_left_kernel_launch(c sv_base, cumo_na_iarray_t* a2, cumo_na_iarray_t* a3, cumo_na_indexer_t* indexer);

/* maximum / minimum of two arrays: narray/gen/tmpl/ewcomp_kernel.cu:5-32, host
 * narray/gen/tmpl/ewcomp.c:18; semantics types/real_accum_kernel.h:28-70,
 * xint_macro_kernel.h:54-68 (no iter_ in these names) */
#define CUMO_HIP_DECL_EWCOMP(t, name) \
    void cumo_##t##_##name##_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_iarray_t* a3, cumo_na_indexer_t* indexer);

/* clip: narray/gen/tmpl/clip_kernel.cu:7-44,65-136, host narray/gen/tmpl/clip.c:2-7.
 * The array-bounds form leaves an element with min > max unwritten and sets *invalid. */
#define CUMO_HIP_DECL_CLIP(t, c) \
    void cumo_iter_##t##_clip_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_iarray_t* a3, cumo_na_iarray_t* a4, cumo_na_indexer_t* indexer, int* invalid); \
    void cumo_iter_##t##_clip_s_kernel_launch(cumo_na_iarray_t* a1, c sv_min, c sv_max, cumo_na_iarray_t* a4, cumo_na_indexer_t* indexer); \
    void cumo_iter_##t##_clip_min_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_iarray_t* a3, cumo_na_indexer_t* indexer); \
    void cumo_iter_##t##_clip_min_s_kernel_launch(cumo_na_iarray_t* a1, c sv, cumo_na_iarray_t* a3, cumo_na_indexer_t* indexer); \
    void cumo_iter_##t##_clip_max_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_iarray_t* a3, cumo_na_indexer_t* indexer); \
    void cumo_iter_##t##_clip_max_s_kernel_launch(cumo_na_iarray_t* a1, c sv, cumo_na_iarray_t* a3, cumo_na_indexer_t* indexer);

CUMO_HIP_DECL_POW(sfloat, float)
CUMO_HIP_DECL_POW(dfloat, double)
CUMO_HIP_DECL_POW(int32, int32_t)
CUMO_HIP_DECL_EWCOMP(sfloat, maximum)
CUMO_HIP_DECL_EWCOMP(sfloat, maximum_nan)
CUMO_HIP_DECL_EWCOMP(sfloat, minimum)
CUMO_HIP_DECL_EWCOMP(sfloat, minimum_nan)
CUMO_HIP_DECL_EWCOMP(dfloat, maximum)
CUMO_HIP_DECL_EWCOMP(dfloat, maximum_nan)
CUMO_HIP_DECL_EWCOMP(dfloat, minimum)
CUMO_HIP_DECL_EWCOMP(dfloat, minimum_nan)
CUMO_HIP_DECL_EWCOMP(int32, maximum)
CUMO_HIP_DECL_EWCOMP(int32, minimum)
CUMO_HIP_DECL_CLIP(sfloat, float)
CUMO_HIP_DECL_CLIP(dfloat, double)
CUMO_HIP_DECL_CLIP(int32, int32_t)

/* cumsum / cumprod along one run of n elements with byte steps s1 (input) and s2
 * (result): narray/gen/tmpl/cum_kernel.cu:51-76, host narray/gen/tmpl/cum.c:3.
 * Returns 0 or the runtime's error code, as the reference returns cudaError_t. */
#define CUMO_HIP_DECL_CUM(t, name) \
    int cumo_##t##_##name##_kernel_launch(char *p1, char *p2, ssize_t s1, ssize_t s2, uint64_t n);
CUMO_HIP_DECL_CUM(sfloat, cumsum)
CUMO_HIP_DECL_CUM(sfloat, cumsum_nan)
CUMO_HIP_DECL_CUM(sfloat, cumprod)
CUMO_HIP_DECL_CUM(sfloat, cumprod_nan)
CUMO_HIP_DECL_CUM(dfloat, cumsum)
CUMO_HIP_DECL_CUM(dfloat, cumsum_nan)
CUMO_HIP_DECL_CUM(dfloat, cumprod)
CUMO_HIP_DECL_CUM(dfloat, cumprod_nan)
CUMO_HIP_DECL_CUM(int32, cumsum)
CUMO_HIP_DECL_CUM(int32, cumprod)

/* mulsum: narray/gen/tmpl/accum_binary_kernel.cu:32-110, host
 * narray/gen/tmpl/accum_binary.c:4-5. The reduce form ADDS the sum of the n
 * products onto *p3; the other form does p3[i] += p1[i] * p2[i]. Steps in bytes. */
#define CUMO_HIP_DECL_MULSUM(t, name) \
    void cumo_##t##_##name##_reduce_kernel_launch(char *p1, char *p2, char *p3, ssize_t s1, ssize_t s2, uint64_t n); \
    void cumo_##t##_##name##_kernel_launch(char *p1, char *p2, char *p3, ssize_t s1, ssize_t s2, ssize_t s3, uint64_t n);
CUMO_HIP_DECL_MULSUM(sfloat, mulsum)
CUMO_HIP_DECL_MULSUM(sfloat, mulsum_nan)
CUMO_HIP_DECL_MULSUM(dfloat, mulsum)
CUMO_HIP_DECL_MULSUM(dfloat, mulsum_nan)
CUMO_HIP_DECL_MULSUM(int32, mulsum)

/* typed store / cast, dst = (dst type)src: narray/gen/tmpl/store_from_kernel.cu:3-53,
 * host narray/gen/tmpl/store_from.c:2; pairs narray/gen/spec.rb:122-142.
 * a1 is the destination, a2 the source. int64 appears because Int32#sum
 * answers Int64 (narray/gen/spec.rb:308-319). */
#define CUMO_HIP_STORE_PAIRS(X) \
    X(sfloat, sfloat) X(sfloat, dfloat) X(sfloat, int32) X(sfloat, int64) \
    X(dfloat, sfloat) X(dfloat, dfloat) X(dfloat, int32) X(dfloat, int64) \
    X(int32, sfloat)  X(int32, dfloat)  X(int32, int32)  X(int32, int64)
#define CUMO_HIP_DECL_STORE(dst, src) \
    void cumo_iter_##dst##_store_##src##_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_indexer_t* indexer);
CUMO_HIP_STORE_PAIRS(CUMO_HIP_DECL_STORE)

/* The same-type store between views that may carry index arrays
 * (narray/gen/tmpl/store_from_kernel.cu:19-35, host store_from.c:5,82), and the ingest of a
 * host Array staged in device memory (narray/gen/tmpl/store_array_kernel.cu:2-60, host
 * store_array.c:2-5): element i of the run goes to p1 + idx1[i] or p1 + i*s1 (bytes). */
#define CUMO_HIP_DECL_STORE_STRIDX(t, c) \
    void cumo_iter_##t##_store_##t##_stridx_kernel_launch(cumo_na_iarray_stridx_t* a1, cumo_na_iarray_stridx_t* a2, cumo_na_indexer_t* indexer); \
    void cumo_iter_##t##_store_array_index_kernel_launch(char *p1, size_t *idx1, c* z, uint64_t n); \
    void cumo_iter_##t##_store_array_stride_kernel_launch(char *p1, ssize_t s1, c* z, uint64_t n); \
    void cumo_iter_##t##_store_array_index_scalar_kernel_launch(char *p1, size_t *idx1, c z, uint64_t n); \
    void cumo_iter_##t##_store_array_stride_scalar_kernel_launch(char *p1, ssize_t s1, c z, uint64_t n);
CUMO_HIP_DECL_STORE_STRIDX(sfloat, float)
CUMO_HIP_DECL_STORE_STRIDX(dfloat, double)
CUMO_HIP_DECL_STORE_STRIDX(int32, int32_t)

/* copy of any view, a1 = source, a2 = destination:
 * narray/data_kernel.cu:47-132, host narray/data.c:56,84-92 */
void cumo_iter_copy_bytes_indexer_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_indexer_t* indexer, ssize_t elmsz);

/* ------------------------------------------------------------------------
 * 4. Reduction launchers: narray/gen/tmpl/real_accum_kernel.cu:166-226,
 *    float_accum_kernel.cu:155-206, accum_arg_kernel.cu:117-142,
 *    accum_index_kernel.cu:117-142; host declarations accum.c:8, minmax.c:2-4,
 *    accum_arg.c:5, accum_index.c:5.
 * ---------------------------------------------------------------------- */
#define CUMO_HIP_DECL_REDUCE(t, name) \
    void cumo_##t##_##name##_kernel_launch(cumo_na_reduction_arg_t* arg);
#define CUMO_HIP_DECL_REDUCE_PAIR(t, name) \
    void cumo_##t##_##name##_kernel_launch(cumo_na_reduction_arg_t* arg, cumo_na_iarray_t* out2);

#define CUMO_HIP_REDUCE_OPS_ALL(X, t)   X(t, sum) X(t, prod) X(t, min) X(t, max) X(t, ptp)
#define CUMO_HIP_REDUCE_OPS_FLOAT(X, t) \
    X(t, sum_nan) X(t, prod_nan) X(t, min_nan) X(t, max_nan) X(t, ptp_nan) \
    X(t, mean) X(t, var) X(t, stddev) X(t, rms) \
    X(t, mean_nan) X(t, var_nan) X(t, stddev_nan) X(t, rms_nan)
#define CUMO_HIP_REDUCE_OPS_DOUBLE(X, t) X(t, kahan_sum) X(t, kahan_sum_nan)
#define CUMO_HIP_ARG_OPS_ALL(X, t) \
    X(t, argmin_int32) X(t, argmin_int64) X(t, argmax_int32) X(t, argmax_int64) \
    X(t, min_index_int32) X(t, min_index_int64) X(t, max_index_int32) X(t, max_index_int64)
#define CUMO_HIP_ARG_OPS_FLOAT(X, t) \
    X(t, argmin_nan_int32) X(t, argmin_nan_int64) X(t, argmax_nan_int32) X(t, argmax_nan_int64) \
    X(t, min_index_nan_int32) X(t, min_index_nan_int64) X(t, max_index_nan_int32) X(t, max_index_nan_int64)

CUMO_HIP_REDUCE_OPS_ALL(CUMO_HIP_DECL_REDUCE, sfloat)
CUMO_HIP_REDUCE_OPS_ALL(CUMO_HIP_DECL_REDUCE, dfloat)
CUMO_HIP_REDUCE_OPS_ALL(CUMO_HIP_DECL_REDUCE, int32)
CUMO_HIP_REDUCE_OPS_FLOAT(CUMO_HIP_DECL_REDUCE, sfloat)
CUMO_HIP_REDUCE_OPS_FLOAT(CUMO_HIP_DECL_REDUCE, dfloat)
CUMO_HIP_REDUCE_OPS_DOUBLE(CUMO_HIP_DECL_REDUCE, dfloat)
CUMO_HIP_ARG_OPS_ALL(CUMO_HIP_DECL_REDUCE, sfloat)
CUMO_HIP_ARG_OPS_ALL(CUMO_HIP_DECL_REDUCE, dfloat)
CUMO_HIP_ARG_OPS_ALL(CUMO_HIP_DECL_REDUCE, int32)
CUMO_HIP_ARG_OPS_FLOAT(CUMO_HIP_DECL_REDUCE, sfloat)
CUMO_HIP_ARG_OPS_FLOAT(CUMO_HIP_DECL_REDUCE, dfloat)
CUMO_HIP_DECL_REDUCE_PAIR(sfloat, minmax)
CUMO_HIP_DECL_REDUCE_PAIR(dfloat, minmax)
CUMO_HIP_DECL_REDUCE_PAIR(int32, minmax)
CUMO_HIP_DECL_REDUCE_PAIR(sfloat, minmax_nan)
CUMO_HIP_DECL_REDUCE_PAIR(dfloat, minmax_nan)

/* The SFloat sum for callers that cannot allocate: code under stream capture, tight
 * serving loops, harnesses that forbid hipMalloc. It has no counterpart in the
 * reference, whose split reductions always take their scratch from the memory pool
 * (include/cumo/reduce_kernel.h:493-496). Same descriptors, planner, kernels and
 * result bits as cumo_sfloat_sum_kernel_launch, but the partial sums of a split
 * reduction go to a fixed array of CUMO_HIP_NOALLOC_SCRATCH_BYTES that lives in the
 * library's device image (each GPU the library runs on holds its own copy until the
 * process ends); the call makes no hipMalloc / hipFree and does not touch the pool.
 * Returns CUMO_HIP_OK, or CUMO_HIP_ERROR_ARGUMENT (also latched / handed to the error
 * handler) without launching anything when the partial sums would not fit: a split
 * reduction with more than CUMO_HIP_NOALLOC_SCRATCH_BYTES / 4 partial sums, i.e.
 * outputs x chunks of the reduce axis. Every call on a GPU shares that GPU's array:
 * calls that can overlap on one GPU (different streams or threads) race and must be
 * serialised by the caller. Nothing in the array has to start at zero; it keeps the
 * last call's partial sums. */
#define CUMO_HIP_NOALLOC_SCRATCH_BYTES (256u << 10)
int cumo_hip_sfloat_sum_noalloc_kernel_launch(cumo_na_reduction_arg_t* arg);
/* bytes of the fixed array that this thread's last call of the launcher above handed to its
 * kernels (0: the reduction needed no partial sums, or the call was refused) */
size_t cumo_hip_sfloat_sum_noalloc_scratch_used(void);

/* ------------------------------------------------------------------------
 * 5. Bit launchers: narray/gen/tmpl_bit/binary_kernel.cu:1-52 (host
 *    tmpl_bit/binary.c:1-2), tmpl_bit/unary_kernel.cu (host tmpl_bit/unary.c),
 *    tmpl_bit/bit_count_kernel.cu:4-78 (host tmpl_bit/bit_count.c:4-7).
 *    count_* ADD onto the uint64 the output pointer names, as the reference's
 *    atomicAdd does; ndloop pre-fills it with 0 (narray/ndloop.c:853-860).
 * ---------------------------------------------------------------------- */
#define CUMO_HIP_BIT_BINARY_OPS(X) X(and) X(or) X(xor) X(eq)
#define CUMO_HIP_BIT_UNARY_OPS(X)  X(copy) X(not)
#define CUMO_HIP_DECL_BIT_BINARY(op) \
    void cumo_iter_bit_##op##_kernel_launch(cumo_na_bit_iarray_stridx_t* a1, cumo_na_bit_iarray_stridx_t* a2, cumo_na_bit_iarray_stridx_t* a3, cumo_na_indexer_t* indexer); \
    void cumo_iter_bit_##op##_contiguous_kernel_launch(CUMO_BIT_DIGIT *a1, size_t p1, CUMO_BIT_DIGIT *a2, size_t p2, CUMO_BIT_DIGIT *a3, size_t p3, uint64_t n);
#define CUMO_HIP_DECL_BIT_UNARY(op) \
    void cumo_iter_bit_##op##_kernel_launch(cumo_na_bit_iarray_stridx_t* a1, cumo_na_bit_iarray_stridx_t* a3, cumo_na_indexer_t* indexer); \
    void cumo_iter_bit_##op##_contiguous_kernel_launch(CUMO_BIT_DIGIT *a1, size_t p1, CUMO_BIT_DIGIT *a3, size_t p3, uint64_t n);
#define CUMO_HIP_DECL_BIT_COUNT(name) \
    void cumo_iter_bit_##name##_index_kernel_launch(size_t p1, char *p2, CUMO_BIT_DIGIT *a1, size_t *idx1, uint64_t n); \
    void cumo_iter_bit_##name##_stride_kernel_launch(size_t p1, char *p2, CUMO_BIT_DIGIT *a1, ssize_t s1, uint64_t n); \
    void cumo_iter_bit_##name##_index_stride_kernel_launch(size_t p1, char *p2, CUMO_BIT_DIGIT *a1, size_t *idx1, ssize_t s2, uint64_t n); \
    void cumo_iter_bit_##name##_stride_stride_kernel_launch(size_t p1, char *p2, CUMO_BIT_DIGIT *a1, ssize_t s1, ssize_t s2, uint64_t n);

CUMO_HIP_BIT_BINARY_OPS(CUMO_HIP_DECL_BIT_BINARY)
CUMO_HIP_BIT_UNARY_OPS(CUMO_HIP_DECL_BIT_UNARY)
/* Bit#store(Bit) (narray/gen/tmpl_bit/store_bit.c:1-2, kernels store_bit_kernel.cu:1-47;
 * generated for class Bit by gen/spec.rb:125 `store_from "Bit"`): a1 is the source, a3 the
 * receiver; the contiguous form takes word pointers with bit offsets below 32 and writes
 * only the n bits it names. */
CUMO_HIP_DECL_BIT_UNARY(store_bit)
CUMO_HIP_DECL_BIT_COUNT(count_true)
CUMO_HIP_DECL_BIT_COUNT(count_false)

/* all? / any? (narray/gen/tmpl_bit/bit_reduce_kernel.cu:5-77, host tmpl_bit/bit_reduce.c:1-3;
 * spec.rb:185-186). The result bits start out as 1 (all?) or 0 (any?) -- ndloop fills them
 * with the init value -- and an element that differs flips its result bit; nothing flips it
 * back. elementwise: element i answers result bit p2 + i*s2 (or p2 + idx2[i]); reduce: every
 * element of a strided or indexed run answers the one bit p2; contiguous_reduce: the same for
 * a run of step 1, compared a word at a time. */
#define CUMO_HIP_DECL_BIT_REDUCE(name) \
    void cumo_iter_bit_##name##_elementwise_kernel_launch(CUMO_BIT_DIGIT *a1, size_t p1, ssize_t s1, size_t *idx1, CUMO_BIT_DIGIT *a2, size_t p2, ssize_t s2, size_t *idx2, uint64_t n); \
    void cumo_iter_bit_##name##_reduce_kernel_launch(CUMO_BIT_DIGIT *a1, size_t p1, ssize_t s1, size_t *idx1, CUMO_BIT_DIGIT *a2, size_t p2, uint64_t n); \
    void cumo_iter_bit_##name##_contiguous_reduce_kernel_launch(CUMO_BIT_DIGIT *a1, size_t p1, CUMO_BIT_DIGIT *a2, size_t p2, uint64_t n);
CUMO_HIP_DECL_BIT_REDUCE(all_p)
CUMO_HIP_DECL_BIT_REDUCE(any_p)

/* Bit#fill (narray/gen/tmpl_bit/fill_kernel.cu:2-46, host tmpl_bit/fill.c:1-2): y is 0 or all
 * ones for the contiguous form (a3 = first word of the run, p3 = bit offset in it), its lowest
 * bit for the general form. */
void cumo_iter_bit_fill_kernel_launch(cumo_na_bit_iarray_stridx_t* a3, CUMO_BIT_DIGIT y, cumo_na_indexer_t* indexer);
void cumo_iter_bit_fill_contiguous_kernel_launch(CUMO_BIT_DIGIT *a3, size_t p3, uint64_t n, CUMO_BIT_DIGIT y);

/* number -> Bit, nonzero is 1 (narray/gen/tmpl_bit/store_from_kernel.cu:3-29, host
 * tmpl_bit/store_from.c:2; element rule include/cumo/types/bit_kernel.h:13-19). a1 is the
 * destination. */
#define CUMO_HIP_BIT_STORE_SOURCES(X) X(sfloat) X(dfloat) X(int32) X(int64) X(uint64)
#define CUMO_HIP_DECL_BIT_STORE_FROM(t) \
    void cumo_iter_bit_store_##t##_kernel_launch(cumo_na_bit_iarray_stridx_t* a1, cumo_na_iarray_stridx_t* a2, cumo_na_indexer_t* indexer);
CUMO_HIP_BIT_STORE_SOURCES(CUMO_HIP_DECL_BIT_STORE_FROM)

/* Ingest of a host Array staged in device memory, Bit destination
 * (narray/gen/tmpl_bit/store_array_kernel.cu:2-95, host tmpl_bit/store_array.c:1-5): z is a
 * packed buffer whose bit 0 is the run's first element, or one value for the scalar forms. */
void cumo_iter_bit_store_array_index_kernel_launch(CUMO_BIT_DIGIT *a1, size_t p1, size_t *idx1, CUMO_BIT_DIGIT* z, uint64_t n);
void cumo_iter_bit_store_array_stride_kernel_launch(CUMO_BIT_DIGIT *a1, size_t p1, ssize_t s1, CUMO_BIT_DIGIT* z, uint64_t n);
void cumo_iter_bit_store_array_contiguous_kernel_launch(CUMO_BIT_DIGIT *a1, size_t p1, CUMO_BIT_DIGIT* z, uint64_t n);
void cumo_iter_bit_store_array_index_scalar_kernel_launch(CUMO_BIT_DIGIT *a1, size_t p1, size_t *idx1, CUMO_BIT_DIGIT z, uint64_t n);
void cumo_iter_bit_store_array_stride_scalar_kernel_launch(CUMO_BIT_DIGIT *a1, size_t p1, ssize_t s1, CUMO_BIT_DIGIT z, uint64_t n);

/* Bit#where / Bit#mask compaction: narray/gen/tmpl_bit/where_kernel.cu:83-107 (host
 * tmpl_bit/where.c:10-11) and tmpl_bit/mask_kernel.cu:36-54. The scratch holds two
 * running output cursors (ones, zeros) and up to 1024 block counts; the cursor carries
 * the output position from one run of a view to the next on the device. `out` of where
 * receives count + position as elmsz-byte (4 or 8) integers, `out` of mask the masked
 * array's element positions p2 + j*s2 (or p2 + idx2[j]). */
char *cumo_bit_where_scratch_new(void);
void cumo_bit_where_kernel_launch(CUMO_BIT_DIGIT *a, size_t p, ssize_t s, size_t *idx, uint64_t n, int invert, char *out, size_t elmsz, uint64_t count, char *scratch);
void cumo_bit_mask_kernel_launch(CUMO_BIT_DIGIT *a, size_t p, ssize_t s, size_t *idx, uint64_t n, size_t *out, size_t p2, ssize_t s2, size_t *idx2, char *scratch);

/* Index-array views: arithmetic on device index arrays (narray/index_kernel.cu:87-173,
 * host narray/index.c), the diagonal's index arrays and the 1-D indexed copy
 * (narray/data_kernel.cu:134-164, host narray/data.c), and the gather / scatter
 * between a view with index arrays and a contiguous buffer that ndloop stages such
 * operands through (narray/ndloop_kernel.cu:46-93, host narray/ndloop.c:1251,1316).
 * Index arrays hold byte offsets (size_t). */
void cumo_na_index_aref_nadata_index_stride_kernel_launch(size_t *idx, ssize_t s1, uint64_t n);
void cumo_na_index_aref_naview_index_index_kernel_launch(size_t *idx, size_t *idx1, uint64_t n);
void cumo_na_index_aref_naview_index_stride_last_kernel_launch(size_t *idx, ssize_t s1, size_t last, uint64_t n);
void cumo_na_index_aref_naview_index_stride_kernel_launch(size_t *idx, ssize_t s1, uint64_t n);
void cumo_na_index_aref_naview_index_index_beg_step_kernel_launch(size_t *idx, size_t *idx1, size_t beg, ssize_t step, uint64_t n);
void cumo_na_index_at_nadata_index_stride_add_kernel_launch(size_t *idx, size_t *idx1, ssize_t s1, uint64_t n);
void cumo_na_index_at_nadata_index_beg_step_stride_kernel_launch(size_t *idx, size_t beg, ssize_t step, ssize_t s1, uint64_t n);
void cumo_na_index_at_nadata_index_beg_step_stride_add_kernel_launch(size_t *idx, size_t beg, ssize_t step, ssize_t s1, uint64_t n);
void cumo_na_index_at_naview_index_index_index_add_kernel_launch(size_t *idx, size_t *idx1, size_t *idx2, uint64_t n);
void cumo_na_index_at_naview_index_index_beg_step_add_kernel_launch(size_t *idx, size_t *idx1, size_t beg, ssize_t step, uint64_t n);
void cumo_na_index_at_naview_index_stride_last_add_kernel_launch(size_t *idx, ssize_t s1, size_t last, uint64_t n);
void cumo_iter_copy_bytes_kernel_launch(char *p1, char *p2, ssize_t s1, ssize_t s2, size_t *idx1, size_t *idx2, uint64_t n, ssize_t elmsz);
void cumo_na_diagonal_index_index_kernel_launch(size_t *idx, size_t *idx0, size_t *idx1, size_t k0, size_t k1, uint64_t n);
void cumo_na_diagonal_index_stride_kernel_launch(size_t *idx, size_t *idx0, ssize_t s1, size_t k0, size_t k1, uint64_t n);
void cumo_na_diagonal_stride_index_kernel_launch(size_t *idx, ssize_t s0, size_t *idx1, size_t k0, size_t k1, uint64_t n);
void cumo_ndloop_copy_from_buffer_kernel_launch(cumo_na_iarray_stridx_t *a, cumo_na_indexer_t* indexer, char *buf, size_t elmsz);
void cumo_ndloop_copy_to_buffer_kernel_launch(cumo_na_iarray_stridx_t *a, cumo_na_indexer_t* indexer, char *buf, size_t elmsz);

/* ------------------------------------------------------------------------
 * 6. What this library adds (no counterpart symbol in the reference).
 * ---------------------------------------------------------------------- */

/* Error reporting. The reference raises from inside the launcher
 * (cuda/runtime.c:16-20, cuda/memory_pool.cpp:64-96). A host that can raise
 * installs a handler; it is called with kind and message and may not return
 * (longjmp). With no handler the error is latched per thread. */
enum {
    CUMO_HIP_OK = 0,
    CUMO_HIP_ERROR_RUNTIME = 1,        /* Cumo::CUDA::RuntimeError */
    CUMO_HIP_ERROR_OUT_OF_MEMORY = 2,  /* Cumo::CUDA::OutOfMemoryError */
    CUMO_HIP_ERROR_ARGUMENT = 3,       /* ArgumentError */
    /* raised by the host launch layer (cumo_hip_ndloop.h) */
    CUMO_HIP_ERROR_SHAPE = 4,          /* Cumo::NArray::ShapeError (narray/ndloop.c:508-512, narray/narray.c:1704-1716) */
    CUMO_HIP_ERROR_ZERO_DIVISION = 5,  /* ZeroDivisionError (narray/gen/tmpl/binary.c:120-126) */
    CUMO_HIP_ERROR_TYPE = 6,           /* TypeError / NoMethodError: no such operation for this element type */
    CUMO_HIP_ERROR_VALUE = 7,          /* Cumo::NArray::ValueError (narray/gen/tmpl/unary2.c:61-66) */
    CUMO_HIP_ERROR_DIMENSION = 8,      /* Cumo::NArray::DimensionError (narray/narray.c:1757-1759) */
    CUMO_HIP_ERROR_OPERATION = 9       /* Cumo::NArray::OperationError (narray/gen/tmpl/clip.c:48-51,222) */
};
typedef void (*cumo_hip_error_handler_t)(int kind, int hip_status, const char* message);
void cumo_hip_set_error_handler(cumo_hip_error_handler_t handler);
/* Returns the latched error kind (0 if none) and clears it; message, if not
 * NULL, receives a pointer to a thread-local string. */
int cumo_hip_last_error(const char** message);

/* Kernels that finish in one launch what the reference does in two (a split reduction whose
 * last block folds the partial results, one-pass scans, the one-launch mulsum; the reference's
 * forms are include/cumo/reduce_kernel.h:395-611 and gen/tmpl/cum_kernel.cu:51-76) let a block
 * wait for words that other blocks of the same launch publish, for a bounded number of looks.
 * A wait that runs out cannot produce its result. It is reported the way the reference
 * reports trouble inside a kernel (the pinned flag that the host reads after a device sync,
 * cuda/runtime.c:22-47): the next call that waits for the device -- cumo_hip_synchronize,
 * cumo_hip_memcpy_d2h, cumo_hip_copy_to_host, cumo_cuda_runtime_error_flag_get -- reports
 * CUMO_HIP_ERROR_RUNTIME through the handler / cumo_hip_last_error. This call returns how
 * often it has happened since the process started: counts[0] reductions, counts[1] scans,
 * counts[2] mulsum, counts[3] unused. Returns 0, or -1 when the counts cannot be read.
 * (It waits for the device.) No counterpart in the reference. */
int cumo_hip_wait_give_ups(uint32_t counts[4]);

/* count_true / count_false along axes in one launch (no counterpart in the
 * reference, whose ndloop walks every output on the host and launches one run at a
 * time, narray/ndloop.c:1569-1613 under gen/tmpl_bit/bit_count.c:9-36). The loop is
 * given as kept dimensions then reduced dimensions; input steps and pos are in bits,
 * output steps in bytes; the counts are ADDED onto the uint64 results, or, with
 * `overwrite` set, REPLACE them: the results (out_total contiguous uint64 from `out`,
 * out_step that of a contiguous array) then need not hold zero, and the launcher
 * zeroes them itself where its kernel adds. */
typedef struct {
    int      out_ndim, red_ndim;
    size_t   out_shape[CUMO_NA_MAX_DIMENSION], red_shape[CUMO_NA_MAX_DIMENSION];
    ssize_t  in_out_step[CUMO_NA_MAX_DIMENSION], in_red_step[CUMO_NA_MAX_DIMENSION];
    ssize_t  out_step[CUMO_NA_MAX_DIMENSION];
    CUMO_BIT_DIGIT* in;
    size_t   pos;
    char*    out;
    int      count_false;
    int      overwrite;
} cumo_hip_bit_count_nd_t;
void cumo_hip_bit_count_nd_kernel_launch(const cumo_hip_bit_count_nd_t* counts);
/* *out = the count over one contiguous run of bits, in one launch that neither needs
 * nor reads a zeroed result (the reference zero-fills the result and its launchers add
 * onto it, ndloop.c:853-860 + tmpl_bit/bit_count.c:9-36: two launches). a + pos/32 words,
 * bit pos%32 onwards, n bits. Returns 1 when launched, 0 when the caller has to take
 * the zero-fill + accumulate route. */
int  cumo_hip_bit_count_run_store_kernel_launch(CUMO_BIT_DIGIT* a, size_t pos, uint64_t n, int count_false, uint64_t* out);
/* Bits from counts: bit pos + i of dst = (counts[i] != 0), or (counts[i] == 0) with zero_is_one; n contiguous
 * uint64 counts. What all? / any? along axes make of the counts of clear / set bits along them (no counterpart
 * in the reference, which walks the runs on the host: gen/tmpl_bit/bit_reduce.c:106-146). Bits of dst outside
 * [pos, pos + n) stay as they are. */
void cumo_hip_bit_from_counts_kernel_launch(const uint64_t* counts, uint64_t n, int zero_is_one, CUMO_BIT_DIGIT* dst, size_t pos);
/* all? (all != 0) or any? of each of `rows` runs of n bits, run r at bit pos + r * row_step of `in`, into bit
 * out_pos + r of `out`, in one launch; pos and row_step must be multiples of 32. Returns 1 when launched, 0 when
 * the shape is one the caller should hand to the counts instead (short or few runs, unaligned rows). The
 * reference launches one reduction per run from a walk on the host (gen/tmpl_bit/bit_reduce.c:106-146). Bits of
 * out outside [out_pos, out_pos + rows) stay as they are. */
int  cumo_hip_bit_anyall_rows_kernel_launch(CUMO_BIT_DIGIT* in, size_t pos, uint64_t rows, int64_t row_step, uint64_t n, int all,
                                            CUMO_BIT_DIGIT* out, size_t out_pos);

/* Row-wise softmax and layer normalisation in one pass (no counterpart in the
 * reference, where they are chains of 5 and 6 array operations,
 * bench/transformer_bench.rb:110-124). rows runs of n contiguous elements, row r at
 * in + r * in_row_step; type 0 SFloat, 1 DFloat; mode 0 softmax, 1 layernorm with
 * eps added to the variance (divisor n - 1, as Cumo's var). Returns 1 when
 * launched, 0 when the layout is outside what the kernels take (the caller then
 * composes the chain). */
typedef struct {
    uint64_t rows, n;
    ssize_t  in_row_step, out_row_step;
    char*    in;
    char*    out;
    double   eps;
} cumo_hip_fused_rows_t;
int cumo_hip_fused_rows_kernel_launch(int type, int mode, const cumo_hip_fused_rows_t* rows);

/* Product sums of many rows in one launch (the reference launches
 * cumo_<type>_mulsum_reduce_kernel_launch once per row from a host loop,
 * gen/tmpl/accum_binary.c:20-45): out[r] += sum_i p1[r][i] * p2[r][i] for rows of n
 * contiguous elements, row r of an operand at p + r * row_step (0 repeats the row).
 * type 0 SFloat, 1 DFloat, 2 Int32; nan skips NaN factors. Returns 1 when launched,
 * 0 when the layout is outside what the kernel takes (n not a whole number of
 * 128-bit vectors, operands or row steps not 16-byte aligned). */
typedef struct {
    uint64_t rows, n;
    ssize_t  row_step1, row_step2, out_step;
    char*    p1;
    char*    p2;
    char*    out;
} cumo_hip_mulsum_rows_t;
int cumo_hip_mulsum_rows_kernel_launch(int type, int nan, const cumo_hip_mulsum_rows_t* rows);

/* The compaction of one run for a caller that sizes the result in between (the host
 * iterator of tmpl_bit/where.c:13-28 counts first, reads the count back and allocates):
 * count writes the hits of each block's share of the run into counts[0 ..
 * cumo_hip_bit_where_blocks(n) - 1]; the caller copies them to the host and adds them
 * up; place puts the o-th hit's position in the run (x == NULL; as elmsz-byte integers,
 * 4 or 8) or its element x + j*sx (elmsz 4 or 8; a[mask] without the array of positions
 * that tmpl_bit/mask.c:141-167 makes a view over) at out[o], every block adding up the
 * counts before it. Two launches where a count for the size plus the three of
 * cumo_bit_where_kernel_launch were five. invert: the clear bits are the hits. */
size_t cumo_hip_bit_where_blocks(uint64_t n);
void cumo_hip_bit_where_count_kernel_launch(CUMO_BIT_DIGIT *a, size_t p, ssize_t s, uint64_t n, int invert, uint64_t *counts);
/* count, and the counts in host_counts[0 .. blocks - 1] when the call returns: the kernel also writes
 * them to pinned host memory of the calling thread, and the call waits for the stream (the one
 * synchronisation that sizing the result costs, tmpl_bit/where.c:13-28) instead of queueing a copy
 * behind the kernel. Returns CUMO_HIP_OK or an error kind. */
int  cumo_hip_bit_where_count_to_host(CUMO_BIT_DIGIT *a, size_t p, ssize_t s, uint64_t n, int invert, uint64_t *counts, uint64_t *host_counts);
void cumo_hip_bit_where_place_kernel_launch(CUMO_BIT_DIGIT *a, size_t p, ssize_t s, uint64_t n, int invert, const uint64_t *counts,
                                            const char *x, ssize_t sx, size_t elmsz, char *out);

/* out[i] = the element of a strided view at flat row-major position pos[i] (no
 * counterpart symbol in the reference, where a masked array is a view over an index
 * array, tmpl_bit/mask.c:141-167, read by the index kernels). Elements of 4 or 8
 * bytes, positions of 4 or 8 bytes. */
typedef struct {
    int      ndim;
    uint64_t n;
    size_t   shape[CUMO_NA_MAX_DIMENSION];
    ssize_t  step[CUMO_NA_MAX_DIMENSION];
    char*    in;
    char*    out;
    char*    pos;
    int      pos_elmsz, elmsz;
} cumo_hip_gather_flat_t;
void cumo_hip_gather_flat_kernel_launch(const cumo_hip_gather_flat_t* gather);

/* Many scan runs in one launch (no counterpart in the reference, which calls the
 * run launcher once per run from a loop on the host, narray/gen/tmpl/cum.c:12-46).
 * Run r starts at in + sum_k i_k * ostep_in[k] where (i_0 .. i_{nouter-1}) is r
 * decomposed over oshape, row-major; elements of a run are s_in / s_out bytes apart.
 * type: 0 SFloat, 1 DFloat, 2 Int32. */
typedef struct {
    int      nouter;
    uint64_t rows, n;
    size_t   oshape[CUMO_NA_MAX_DIMENSION];
    ssize_t  ostep_in[CUMO_NA_MAX_DIMENSION], ostep_out[CUMO_NA_MAX_DIMENSION];
    ssize_t  s_in, s_out;
    char*    in;
    char*    out;
} cumo_hip_scan_rows_t;
void cumo_hip_scan_rows_kernel_launch(int type, int prod, int nan, const cumo_hip_scan_rows_t* runs);
/* The same for runs that lie across memory: `cols` neighbouring runs start one
 * element apart (the columns of a matrix scanned down its rows); runs->rows counts
 * the groups of `cols` runs and oshape / ostep_* decompose the group number. */
void cumo_hip_scan_cols_kernel_launch(int type, int prod, int nan, const cumo_hip_scan_rows_t* runs, uint64_t cols);

/* The stream every launcher and the pool use from this host thread. The
 * reference only ever uses the default stream (cuda/memory_pool.cpp:43-44). */
void  cumo_hip_set_stream(void* hip_stream);
void* cumo_hip_get_stream(void);
/* a stream of the default priority that does not synchronise with the null stream, for
 * callers without a HIP binding of their own; destroy resets the current stream to the
 * null stream if it was this one */
void* cumo_hip_stream_create(void);
void  cumo_hip_stream_destroy(void* hip_stream);
/* For a stream the caller created with its own HIP binding and passed to cumo_hip_set_stream:
 * call this before destroying it (it waits for the stream). The library keeps a little state
 * per stream it has seen (one of 64 slots of ticket / hand-over words, the look-back words of
 * one-pass scans, an arena of the pool); a stream that goes away without this call keeps its
 * slot, and once all 64 are taken further streams run split reductions and scans in their
 * slower two-launch forms. cumo_hip_stream_destroy does the same for streams made here. */
void  cumo_hip_stream_release(void* hip_stream);
int   cumo_hip_device_count(void);
void  cumo_hip_synchronize(void);
/* events on the current stream, for callers that time launches */
void* cumo_hip_event_create(void);
void  cumo_hip_event_record(void* event);
float cumo_hip_event_elapsed_ms(void* start, void* stop);   /* waits for stop */
void  cumo_hip_event_destroy(void* event);
/* synchronous copies for host read-back/ingest (extract_cpu, to_a, from_binary) */
void  cumo_hip_memcpy_h2d(void* dst, const void* src, size_t n);
void  cumo_hip_memcpy_d2h(void* dst, const void* src, size_t n);
void  cumo_hip_memset(void* dst, int byte, size_t n);
/* The same copies for any size, with CUMO_HIP_OK or an error kind as the result:
 * pageable host memory moves through a ring of four pinned staging buffers
 * (CUMO_HIP_STAGE_MIB each, default 8) so that the DMA over PCIe overlaps the host-side
 * memcpy, which CUMO_HIP_COPY_THREADS threads share (default 4); pinned host memory
 * goes to the DMA engine directly. Ordered on the current stream after the work
 * already queued; both return when the bytes have arrived. These stand where the
 * reference's host code memcpys from / to managed memory after cudaDeviceSynchronize
 * (narray/narray.c:1455-1460,1514-1518,1551-1557). */
int   cumo_hip_copy_to_host(void* dst_host, const void* src_device, size_t n);
int   cumo_hip_copy_from_host(void* dst_device, const void* src_host, size_t n);

/* Memory pool (replaces cumo::internal::MemoryPool, cuda/memory_pool_impl.hpp:160-435).
 * Returns CUMO_HIP_OK or an error kind; never raises. */
int    cumo_hip_pool_malloc(size_t size, void* hip_stream, void** ptr);
int    cumo_hip_pool_free(void* ptr);                       /* CUMO_HIP_ERROR_ARGUMENT if the pool does not own ptr */
void   cumo_hip_pool_free_all_blocks(void);   /* also drops the scans' kept look-back words (waits for the device if any are held) */
/* device memory the library holds outside the pool's books: the look-back words that each
 * stream keeps from one one-pass scan to the next (at most 64 MiB per stream, sized by the
 * largest scan it has run). free_all_blocks and cumo_hip_stream_release give it back. */
size_t cumo_hip_pool_held_outside_bytes(void);
void   cumo_hip_pool_free_all_blocks_stream(void* hip_stream);
/* files everything the pool holds for a stream (free or in use) under the null stream; the
 * stream must have finished its work. cumo_hip_stream_destroy calls it. */
void   cumo_hip_pool_retire_stream(void* hip_stream);
size_t cumo_hip_pool_n_free_blocks(void);
size_t cumo_hip_pool_used_bytes(void);
size_t cumo_hip_pool_free_bytes(void);
size_t cumo_hip_pool_total_bytes(void);
/* bytes and calls that went to hipMalloc since the process started */
size_t cumo_hip_pool_device_malloc_calls(void);
int    cumo_hip_pool_enable(int on);                        /* returns previous state; CUMO_MEMORY_POOL env sets the default */
/* test hook: cap what the pool may hold from the device (0 = no cap), so that
 * the out-of-memory path can be driven from the host without exhausting HBM */
void   cumo_hip_pool_set_limit(size_t bytes);
/* test hook: back the pool with the host heap (1) or the device (0) so that
 * split/merge/accounting can be exercised without a GPU; only while the pool
 * holds nothing */
int    cumo_hip_pool_use_host_backend(int on);

/* Launch planner introspection: what the elementwise/reduction launchers
 * decide for a given set of descriptors, without launching. Host-only. */
typedef struct {
    int kind;           /* 0 empty, 1 rows (threads along the common fast dim), 2 transpose (LDS tile), 3 generic */
    int ndim;           /* dimensions left after dropping size-1 and merging */
    int vec;            /* elements per 128-bit access, 1 if not vectorised */
    int fast_dim;       /* collapsed dim the threads run along */
    int tr_dim;         /* second tile dim for kind 2, else -1 */
    uint64_t shape[CUMO_NA_MAX_DIMENSION];
    int64_t step[4][CUMO_NA_MAX_DIMENSION];
} cumo_hip_ew_plan_t;
/* elmsz[i] = element size of operand i in bytes, 0 for a Bit operand (steps in bits). */
int cumo_hip_plan_elementwise(const cumo_na_indexer_t* indexer, int n_operands,
                              const cumo_na_iarray_t* const* operands, const int* elmsz,
                              const size_t* bitpos, cumo_hip_ew_plan_t* plan);

typedef struct {
    int kind;           /* 0 empty, 1 row (reduce axis along memory), 2 column (output axis along memory), 3 generic */
    int vec;
    int threads_per_row;     /* kind 1: lanes that share one output */
    int n_split;             /* >1: two-pass, partial accumulators then combine */
    int out_ndim, red_ndim;  /* after merging */
    uint64_t out_total, red_total;
    uint64_t out_shape[CUMO_NA_MAX_DIMENSION], red_shape[CUMO_NA_MAX_DIMENSION];
    int64_t in_out_step[CUMO_NA_MAX_DIMENSION], in_red_step[CUMO_NA_MAX_DIMENSION], out_step[CUMO_NA_MAX_DIMENSION];
} cumo_hip_reduce_plan_t;
int cumo_hip_plan_reduce(const cumo_na_reduction_arg_t* arg, int in_elmsz, int accum_bytes, cumo_hip_reduce_plan_t* plan);

#if defined(__GNUC__)
#pragma GCC visibility pop
#endif
#if defined(__cplusplus)
}
#endif

#endif /* CUMO_HIP_H */
