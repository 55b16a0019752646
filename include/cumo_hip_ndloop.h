/*
 * cumo_hip_ndloop.h -- the host launch layer of the MI355X array-compute library.
 *
 * This is the C interface of the part of the Cumo extension that sits between
 * a method body (`a + b`, `a.sum(axis: 1)`) and the kernel launchers declared
 * in cumo_hip.h:
 *
 *   - ndloop: broadcasting over the operands' views, moving reduce dimensions
 *     last, allocating results from the pool, contracting loop dimensions
 *     (reference: ext/cumo/narray/ndloop.c:339-452,493-595,749-863,870-1168,
 *     1459-1616; user-visible structs ext/cumo/include/cumo/ndloop.h:4-117);
 *   - the marshalling helpers that turn a prepared loop into the launch
 *     descriptors (reference: ext/cumo/include/cumo/indexer.h:114-220);
 *   - the per-operation host iterators and method bodies the reference
 *     generates per type (reference: ext/cumo/narray/gen/tmpl/binary.c:114-209,
 *     unary.c:76-119, unary_s.c:53-79, cond_binary.c:33-98, accum.c:41-100,
 *     accum_arg.c:28-110, store_from.c, fill.c, tmpl_bit/binary.c:17-116,
 *     tmpl_bit/bit_count.c:9-110), here one table-driven function per
 *     operation family, selected by the operation's name.
 *
 * Everything is host code in plain C types; arrays are described by
 * cumo_hip_narray_t (a device pointer plus shape, strides and offset).
 * Errors go through the handler/latch of cumo_hip.h and every function also
 * returns the error kind (CUMO_HIP_OK on success).
 */
#ifndef CUMO_HIP_NDLOOP_H
#define CUMO_HIP_NDLOOP_H

#include "cumo_hip.h"

#if defined(__cplusplus)
extern "C" {
#endif
#if defined(__GNUC__)
#pragma GCC visibility push(default)
#endif

/* Element types on the path (reference: the classes of gen/def/{sfloat,dfloat,
 * int32,int64,uint64,bit}.rb). Int64/UInt64 only appear as results (Int32#sum,
 * arg reductions over more than 2^32-1 elements, Bit#count_true). */
enum {
    CUMO_HIP_SFLOAT = 0,
    CUMO_HIP_DFLOAT = 1,
    CUMO_HIP_INT32  = 2,
    CUMO_HIP_INT64  = 3,
    CUMO_HIP_UINT64 = 4,
    CUMO_HIP_BIT    = 5,
    CUMO_HIP_N_TYPES = 6
};

/* A view of device memory: what cumo_narray_view_t and the data object under
 * it carry (reference: ext/cumo/include/cumo/narray.h:159-188), restricted to
 * stride dimensions (no index arrays).
 *   ptr     start of the buffer. In a RESULT argument ptr == NULL asks the
 *           layer to allocate: it fills type-correct shape, contiguous strides,
 *           offset 0 and a pool pointer the caller releases with
 *           cumo_cuda_runtime_free (reference: ndloop.c:750-863 allocates
 *           results the same way).
 *   offset  of the view's first element from ptr
 *   stride  signed, per dimension; bytes, except Bit where offset and stride
 *           are in bits (reference: narray.h:489-496). */
typedef struct {
    int     type;
    int     ndim;
    char*   ptr;
    ssize_t offset;
    size_t  shape[CUMO_NA_MAX_DIMENSION];
    ssize_t stride[CUMO_NA_MAX_DIMENSION];
} cumo_hip_narray_t;

/* Bytes a contiguous array of this type and element count occupies
 * (Bit: whole 32-bit words; reference: gen/tmpl/alloc_func.c:7-9). */
size_t cumo_hip_na_storage_bytes(int type, size_t n_elements);
/* Fills shape, contiguous strides, offset 0 and allocates ptr from the pool. */
int cumo_hip_na_alloc(cumo_hip_narray_t* a, int type, int ndim, const size_t* shape);

/* ------------------------------------------------------------------------
 * ndloop
 * ---------------------------------------------------------------------- */
#define CUMO_HIP_NDLOOP_MAX_ARGS 4

/* One argument of a prepared loop (reference: cumo_na_loop_args_t +
 * cumo_na_loop_iter_t, ndloop.h:4-20): the element the loop starts at and the
 * step per LOOP dimension, 0 where the argument repeats. */
typedef struct {
    int     type;
    ssize_t elmsz;      /* bytes per element, 0 for Bit */
    char*   ptr;        /* buffer pointer + view offset; for Bit the buffer pointer */
    size_t  bitpos;     /* Bit only: bit offset of the first element */
    ssize_t step[CUMO_NA_MAX_DIMENSION];
} cumo_hip_loop_args_t;

/* What an iterator function receives (reference: cumo_na_loop_t, ndloop.h:23-37). */
typedef struct {
    int    narg;        /* inputs, then results */
    int    ndim;        /* loop dimensions after contraction */
    size_t n[CUMO_NA_MAX_DIMENSION];
    cumo_hip_loop_args_t args[CUMO_HIP_NDLOOP_MAX_ARGS];
    int    reduce_dim;  /* how many trailing loop dimensions are reduced */
    void*  opt_ptr;
    int    status;      /* an iterator sets this to an error kind to fail the call */
} cumo_hip_loop_t;

typedef void (*cumo_hip_iter_func_t)(cumo_hip_loop_t* lp);

#define CUMO_HIP_NDF_FLAT_REDUCE (1u << 6)  /* same bit as CUMO_NDF_FLAT_REDUCE (ndloop.h:48) */
#define CUMO_HIP_NDF_KEEP_DIM    (1u << 3)  /* same bit as CUMO_NDF_KEEP_DIM (ndloop.h:44) */

/* reference: cumo_ndfunc_t, ndloop.h:104-111 */
typedef struct {
    cumo_hip_iter_func_t func;
    unsigned int flag;
    int nin;
    int nout;
    int out_type[2];
} cumo_hip_ndfunc_t;

/* Prepares the loop over `in` (nf->nin views) and `out` (nf->nout views, each
 * either given or to be allocated) and calls nf->func once with it
 * (reference: cumo_na_ndloop3/ndloop_run, ndloop.c:1459-1616).
 *   reduce   bit d set = dimension d of the broadcast shape is reduced
 *            (needs CUMO_HIP_NDF_FLAT_REDUCE); results get those dimensions
 *            removed, or kept with size 1 under CUMO_HIP_NDF_KEEP_DIM.
 * A shape mismatch reports CUMO_HIP_ERROR_SHAPE. When the loop is empty the
 * iterator is not called. */
int cumo_hip_na_ndloop(const cumo_hip_ndfunc_t* nf, const cumo_hip_narray_t* const* in,
                       cumo_hip_narray_t* const* out, unsigned int reduce, void* opt_ptr);

/* The same preparation without the call: fills *lp (and allocates results). */
int cumo_hip_na_ndloop_prepare(const cumo_hip_ndfunc_t* nf, const cumo_hip_narray_t* const* in,
                               cumo_hip_narray_t* const* out, unsigned int reduce, cumo_hip_loop_t* lp);

/* Marshalling a prepared loop into launch descriptors
 * (reference: cumo_na_make_indexer / _iarray / _bit_iarray / _reduction_arg and
 * the stridx forms, indexer.h:114-220). */
void cumo_hip_make_indexer(const cumo_hip_loop_t* lp, cumo_na_indexer_t* indexer);
void cumo_hip_make_iarray(const cumo_hip_loop_t* lp, int arg, cumo_na_iarray_t* a);
void cumo_hip_make_bit_iarray(const cumo_hip_loop_t* lp, int arg, cumo_na_bit_iarray_t* a);
void cumo_hip_make_iarray_stridx(const cumo_hip_loop_t* lp, int arg, cumo_na_iarray_stridx_t* a);
void cumo_hip_make_bit_iarray_stridx(const cumo_hip_loop_t* lp, int arg, cumo_na_bit_iarray_stridx_t* a);
/* args[0] is the input, args[1] the result; the first ndim - reduce_dim loop
 * dimensions are the output's. */
void cumo_hip_make_reduction_arg(const cumo_hip_loop_t* lp, cumo_na_reduction_arg_t* arg);

/* ------------------------------------------------------------------------
 * Operations. `op` is the method name as it appears in the launcher symbols
 * ("add", "minus", "exp", "gt", "sum", "argmax", ...). x and y may differ in
 * type among SFloat/DFloat/Int32: the lower one is cast up first
 * (reference: the upcast tables of gen/def/{sfloat,dfloat,int32}.rb and
 * gen/tmpl/binary.c:184-209). z describes the result; z->ptr == NULL
 * allocates it. An unknown name or an unsupported type reports
 * CUMO_HIP_ERROR_TYPE.
 * ---------------------------------------------------------------------- */

/* z = x op y, element by element with broadcasting. Int32 div/mod read the
 * divide-by-zero flag back after the launch (one stream synchronisation, as
 * gen/tmpl/binary.c:120-126 does) and report CUMO_HIP_ERROR_ZERO_DIVISION. */
int cumo_hip_na_binary(const char* op, const cumo_hip_narray_t* x, const cumo_hip_narray_t* y, cumo_hip_narray_t* z);
/* z = x op sv (or sv op x when scalar_is_left); the scalar rides in the launch. */
int cumo_hip_na_binary_s(const char* op, const cumo_hip_narray_t* x, double sv, int scalar_is_left, cumo_hip_narray_t* z);
/* The same for a number that is a Ruby Float: a float array keeps its type, an Int32 array
 * answers DFloat (reference: the upcast table of gen/def/int32.rb:22-23 through
 * gen/tmpl/binary.c:184-209, which casts the array first; here one launch converts on
 * the way in where the array is one contiguous run). */
int cumo_hip_na_binary_fs(const char* op, const cumo_hip_narray_t* x, double sv, int scalar_is_left, cumo_hip_narray_t* z);
/* z = op(x): minus reciprocal sign square abs floor round ceil trunc rint bit_not.
 * Int32 reciprocal / abs report CUMO_HIP_ERROR_ZERO_DIVISION / CUMO_HIP_ERROR_ARGUMENT
 * for 1/0 and |INT_MIN| (reference: gen/tmpl/unary.c:76-119, unary2.c). */
int cumo_hip_na_unary(const char* op, const cumo_hip_narray_t* x, cumo_hip_narray_t* z);
/* z = x ** y (reference: gen/tmpl/pow.c:117-215): the result has the higher type of
 * the two; an Int32 y takes the repeated-product form. pow_s: x ** sv, or sv ** x
 * when scalar_is_left; sv_is_integer selects the Int32 form as a Ruby Integer does.
 * Int32 ** non-integer reports CUMO_HIP_ERROR_TYPE (cast x first); a non-integer
 * base over an Int32 x answers DFloat. */
int cumo_hip_na_pow(const cumo_hip_narray_t* x, const cumo_hip_narray_t* y, cumo_hip_narray_t* z);
int cumo_hip_na_pow_s(const cumo_hip_narray_t* x, double sv, int sv_is_integer, int scalar_is_left, cumo_hip_narray_t* z);
/* Cumo::<T>.maximum / minimum of two arrays; nan selects the NaN-propagating form
 * (reference: gen/tmpl/ewcomp.c, types/real_accum_kernel.h:28-70). */
int cumo_hip_na_ewcomp(const char* op, const cumo_hip_narray_t* x, const cumo_hip_narray_t* y, int nan, cumo_hip_narray_t* z);
/* x.clip(min, max) (reference: gen/tmpl/clip.c:199-254). lo_kind / hi_kind: 0 absent,
 * 1 the scalar lo_s / hi_s, 2 the array lo_a / hi_a. min > max reports
 * CUMO_HIP_ERROR_OPERATION (two scalars: before anything is written; arrays: after
 * the launch, elements with min > max left unwritten); no bound at all
 * CUMO_HIP_ERROR_ARGUMENT. */
int cumo_hip_na_clip(const cumo_hip_narray_t* x, int lo_kind, double lo_s, const cumo_hip_narray_t* lo_a, int hi_kind,
                     double hi_s, const cumo_hip_narray_t* hi_a, cumo_hip_narray_t* z);
/* Cumo::NMath functions of one and two arguments (reference: gen/tmpl/unary_s.c, binary_s.c). */
int cumo_hip_na_math(const char* op, const cumo_hip_narray_t* x, cumo_hip_narray_t* z);
int cumo_hip_na_math2(const char* op, const cumo_hip_narray_t* x, const cumo_hip_narray_t* y, cumo_hip_narray_t* z);
int cumo_hip_na_math2_s(const char* op, const cumo_hip_narray_t* x, double sv, int scalar_is_left, cumo_hip_narray_t* z);
/* x.divmod(y) -> quotient and remainder with the upcast type of the two (reference: gen/tmpl/binary2.c;
 * Int32 by zero reports CUMO_HIP_ERROR_ZERO_DIVISION after the launch). x.modf -> fraction and integral
 * part, float types only (reference: gen/tmpl/unary_ret2.c). */
int cumo_hip_na_divmod(const cumo_hip_narray_t* x, const cumo_hip_narray_t* y, cumo_hip_narray_t* quot, cumo_hip_narray_t* rem);
int cumo_hip_na_modf(const cumo_hip_narray_t* x, cumo_hip_narray_t* frac, cumo_hip_narray_t* whole);
/* x.poly(a0, ..., an): the ncoef coefficients are arrays of x's type; one element each (numbers) goes
 * out as one launch, anything else as the chain y = x * y + a_k of array operations with broadcasting,
 * which rounds the same way (reference: gen/tmpl/poly.c:38-78). No coefficient answers a copy of x. */
int cumo_hip_na_poly(const cumo_hip_narray_t* x, int ncoef, const cumo_hip_narray_t* const* coef, cumo_hip_narray_t* z);
/* Cumo::NMath.frexp: x = mant * 2**expo, mant of x's float type (DFloat for an Int32 x), expo Int32
 * (reference: gen/tmpl/frexp.c:32-38). */
int cumo_hip_na_frexp(const cumo_hip_narray_t* x, cumo_hip_narray_t* mant, cumo_hip_narray_t* expo);
/* Comparisons and float classification into a Bit result. */
int cumo_hip_na_compare(const char* op, const cumo_hip_narray_t* x, const cumo_hip_narray_t* y, cumo_hip_narray_t* z);
int cumo_hip_na_compare_s(const char* op, const cumo_hip_narray_t* x, double sv, int scalar_is_left, cumo_hip_narray_t* z);
int cumo_hip_na_cond_unary(const char* op, const cumo_hip_narray_t* x, cumo_hip_narray_t* z);
/* dst[...] = src with broadcasting and cast; Bit sources store 0/1, Bit to Bit copies bits
 * (reference: gen/tmpl/store_from.c, store_bit.c, tmpl_bit/store_bit.c). */
int cumo_hip_na_store(cumo_hip_narray_t* dst, const cumo_hip_narray_t* src);
/* dst = contiguous copy of any view of the same type (reference: narray/data.c:84-113). */
int cumo_hip_na_copy(const cumo_hip_narray_t* src, cumo_hip_narray_t* dst);
int cumo_hip_na_fill(cumo_hip_narray_t* dst, double value);
/* dst's elements in row-major order become beg + step * i (reference: gen/tmpl/seq.c:77-107), or
 * base ** (beg + step * i) for logseq (float types; gen/tmpl/logseq.c). */
int cumo_hip_na_seq(cumo_hip_narray_t* dst, double beg, double step);
int cumo_hip_na_logseq(cumo_hip_narray_t* dst, double beg, double step, double base);
/* Every matrix of the last two dimensions of dst gets `element` on the diagonal offset by kofs (above
 * the main one for kofs > 0) and zero elsewhere (reference: gen/tmpl/eye.c:52-107: fewer than two
 * dimensions is a dimension error, an offset beyond the matrix an argument error). */
int cumo_hip_na_eye(cumo_hip_narray_t* dst, double element, ssize_t kofs);

/* Reductions: sum prod min max ptp mean var stddev rms kahan_sum minmax argmin
 * argmax min_index max_index.
 *   reduce    bit d set = reduce dimension d of x; 0 = all dimensions
 *   keepdims  reduced dimensions stay with size 1
 *   nan       the NaN-skipping variant (float types)
 *   z         result; its type is fixed by the operation (Int32#sum -> Int64;
 *             arg reductions -> Int32, or Int64 when x has more than 2^32-1
 *             elements; reference: gen/spec.rb:308-343, gen/tmpl/accum_arg.c:92-110)
 *   z2        second result of minmax, else NULL
 * min/max-like reductions of an empty array report CUMO_HIP_ERROR_ARGUMENT. */
int cumo_hip_na_reduce(const char* op, const cumo_hip_narray_t* x, unsigned int reduce, int keepdims, int nan,
                       cumo_hip_narray_t* z, cumo_hip_narray_t* z2);

/* z = sum over the reduced dimensions of x * y, started from 0 (reference:
 * gen/tmpl/accum_binary.c:62-110); reduce / keepdims / nan as for cumo_hip_na_reduce.
 * The result has the higher type of the two (Int32 stays Int32, wrapping). */
int cumo_hip_na_mulsum(const cumo_hip_narray_t* x, const cumo_hip_narray_t* y, unsigned int reduce, int keepdims, int nan,
                       cumo_hip_narray_t* z);
/* Host read-back and ingest of a view (reference: narray/narray.c:1391-1560
 * from_binary / store_binary / to_binary, gen/tmpl/extract_cpu.c, aref_cpu.c, which
 * touch managed memory from the host). The host side is the view's elements in
 * row-major order, densely packed (Bit: eight to a byte, the first in bit 0). A view
 * that is not contiguous is staged through a contiguous copy on the device.
 *   to_host    host[0,nbytes) = the first nbytes of x; nbytes may not exceed x's size
 *   from_host  x = host[0, x's size); nbytes may be larger, never smaller
 *              ("string is too short to store", narray.c:1507)
 *   extract    out = the element at index[0..ndim) (NULL: the single element of a
 *              one-element array); Bit answers one unsigned char */
int cumo_hip_na_to_host(const cumo_hip_narray_t* x, void* host, size_t nbytes);
int cumo_hip_na_from_host(cumo_hip_narray_t* x, const void* host, size_t nbytes);
int cumo_hip_na_extract(const cumo_hip_narray_t* x, const size_t* index, void* out);

/* op "cumsum" or "cumprod": the running value along the dimensions in `reduce` taken
 * together in row-major order (0 = all); z has x's shape and type (reference:
 * gen/tmpl/cum.c:48-80). nan: NaN elements are skipped (leading ones stay NaN). */
int cumo_hip_na_cum(const char* op, const cumo_hip_narray_t* x, unsigned int reduce, int nan, cumo_hip_narray_t* z);

/* z = the row-major positions of x's set bits (clear bits when invert), as Int32, or
 * Int64 for more than 2^32 - 1 elements (reference: gen/tmpl_bit/where.c:98-127). z
 * normally comes in with ptr == NULL; a given z must be a contiguous 1-D array of that
 * type and exactly as long as the count, or the call fails with a shape error. */
int cumo_hip_na_where(const cumo_hip_narray_t* x, int invert, cumo_hip_narray_t* z);
/* z = the elements of x where mask is set, row-major (reference: gen/tmpl_bit/mask.c:96-167,
 * which answers a view over an index array; here a new array). Shapes must be equal.
 * A given z: as for where, with x's type. */
int cumo_hip_na_mask(const cumo_hip_narray_t* mask, const cumo_hip_narray_t* x, cumo_hip_narray_t* z);

/* Library additions: softmax and layer normalisation along the LAST dimension,
 *   softmax:   e = exp(x - max(x)); e / sum(e)
 *   layernorm: (x - mean(x)) / sqrt(var(x) + eps), var with divisor n - 1 as Cumo's
 * as one launch when rows are contiguous 128-bit-aligned runs of at most 16384
 * SFloat / 4096 DFloat elements, else as the chain of array operations. Every
 * elementwise step is the chain's own; only the order of the two row sums differs. */
int cumo_hip_na_softmax(const cumo_hip_narray_t* x, cumo_hip_narray_t* z);
int cumo_hip_na_layernorm(const cumo_hip_narray_t* x, double eps, cumo_hip_narray_t* z);

/* Bit logic: and or xor eq / copy not (reference: gen/tmpl_bit/binary.c, unary.c). */
int cumo_hip_na_bit_binary(const char* op, const cumo_hip_narray_t* x, const cumo_hip_narray_t* y, cumo_hip_narray_t* z);
int cumo_hip_na_bit_unary(const char* op, const cumo_hip_narray_t* x, cumo_hip_narray_t* z);
/* count_true / count_false into a UInt64 result (reference: gen/tmpl_bit/bit_count.c:9-110). */
int cumo_hip_na_bit_count(const cumo_hip_narray_t* x, unsigned int reduce, int keepdims, int count_false, cumo_hip_narray_t* z);
/* all? / any? along axes into a Bit result; op is "all_p" or "any_p" (reference:
 * gen/tmpl_bit/bit_reduce.c:106-146, spec.rb:185-186). An empty operand leaves the init value
 * (the reference's method answers false for it before the loop, bit_reduce.c:132-134). */
int cumo_hip_na_bit_reduce(const char* op, const cumo_hip_narray_t* x, unsigned int reduce, int keepdims, cumo_hip_narray_t* z);

#if defined(__GNUC__)
#pragma GCC visibility pop
#endif
#if defined(__cplusplus)
}
#endif

#endif /* CUMO_HIP_NDLOOP_H */
