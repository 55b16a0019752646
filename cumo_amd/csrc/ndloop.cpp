// The host launch layer: array views in, launch descriptors out, one launcher
// call per operation.
//
// Replaces, for the stride-view operands of the array hot path,
//   ext/cumo/narray/ndloop.c:339-452,493-595,749-863,870-1168,1459-1616
//     (broadcast, reduce dimensions moved last, result allocation, loop
//     contraction, the single call of the user iterator),
//   ext/cumo/include/cumo/indexer.h:114-220 (cumo_na_make_*), and
//   the host iterators / method bodies the reference generates per type from
//   ext/cumo/narray/gen/tmpl/{binary,unary,unary2,unary_s,binary_s,cond_binary,
//   cond_unary,store_from,store_bit,fill,accum,minmax,accum_arg,accum_index}.c
//   and gen/tmpl_bit/{binary,unary,bit_count}.c.
//
// The reference prepares a loop with one xmalloc and a handful of Ruby calls
// per operation and decomposes nothing itself; the per-element index
// arithmetic is left to the kernels. Here the loop lives in a fixed-size struct
// on the caller's stack, dimensions are merged before the launcher sees them,
// and the per-type method bodies are tables of launcher pointers looked up by
// operation name.
//
// No function here keeps a C++ object with a destructor alive across a call
// that may report an error: the installed handler may leave with longjmp.
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "common.h"
#include "cumo_hip_ndloop.h"

namespace {

using cumo_hip::report_error;

typedef cumo_na_iarray_t IA;
typedef cumo_na_bit_iarray_t BIA;
typedef cumo_na_indexer_t IX;
typedef cumo_hip_narray_t NA;
typedef cumo_hip_loop_t LP;

const int kElmsz[CUMO_HIP_N_TYPES] = {4, 8, 4, 8, 8, 0};
const int kMaxDim = CUMO_NA_MAX_DIMENSION;

int fail(int kind, const char* msg) {
    report_error(kind, 0, msg);
    return kind;
}

inline bool valid_type(int t) { return t >= 0 && t < CUMO_HIP_N_TYPES; }
inline bool is_arith(int t) { return t == CUMO_HIP_SFLOAT || t == CUMO_HIP_DFLOAT || t == CUMO_HIP_INT32; }
inline bool is_float(int t) { return t == CUMO_HIP_SFLOAT || t == CUMO_HIP_DFLOAT; }

size_t total_of(const NA* a) {
    size_t n = 1;
    for (int d = 0; d < a->ndim; d++) n *= a->shape[d];
    return n;
}

// a view whose elements sit in row-major order without gaps (any offset)
bool is_contiguous(const NA* a) {
    ssize_t unit = a->type == CUMO_HIP_BIT ? 1 : kElmsz[a->type];
    ssize_t s = unit;
    for (int d = a->ndim - 1; d >= 0; d--) {
        if (a->shape[d] != 1 && a->stride[d] != s) return false;
        s *= (ssize_t)a->shape[d];
    }
    return true;
}

int check_view(const NA* a, const char* what) {
    if (!a) return fail(CUMO_HIP_ERROR_ARGUMENT, "ndloop: missing array argument");
    if (!valid_type(a->type)) return fail(CUMO_HIP_ERROR_TYPE, "ndloop: unknown element type");
    if (a->ndim < 0 || a->ndim > kMaxDim) return fail(CUMO_HIP_ERROR_DIMENSION, "ndloop: too many dimensions");
    if (a->type == CUMO_HIP_BIT && a->offset < 0) return fail(CUMO_HIP_ERROR_ARGUMENT, "ndloop: negative bit offset");
    (void)what;
    return CUMO_HIP_OK;
}

// Merges and drops loop dimensions inside [lo, hi) and appends what is left at
// position `at`; returns the new end. Two neighbours merge when every argument
// walks them as one run: step[outer] == step[inner] * n[inner]
// (reference: cumo_ndfunc_contract_loop, ndloop.c:870-940; like it, reduce and
// kept dimensions never merge with each other).
int contract_range(LP* lp, const size_t* n, const ssize_t (*step)[kMaxDim], int lo, int hi, int at, bool keep_one) {
    int first = at;
    for (int d = lo; d < hi; d++) {
        if (n[d] == 1) continue;
        if (at > first) {
            int p = at - 1;
            bool merge = true;
            for (int j = 0; j < lp->narg && merge; j++)
                merge = lp->args[j].step[p] == step[j][d] * (ssize_t)n[d];
            if (merge) {
                lp->n[p] *= n[d];
                for (int j = 0; j < lp->narg; j++) lp->args[j].step[p] = step[j][d];
                continue;
            }
        }
        lp->n[at] = n[d];
        for (int j = 0; j < lp->narg; j++) lp->args[j].step[at] = step[j][d];
        at++;
    }
    if (at == first && keep_one) {
        lp->n[at] = 1;
        for (int j = 0; j < lp->narg; j++) lp->args[j].step[at] = 0;
        at++;
    }
    return at;
}

}  // namespace

extern "C" {

size_t cumo_hip_na_storage_bytes(int type, size_t n) {
    if (!valid_type(type)) return 0;
    if (type == CUMO_HIP_BIT) return ((n + 31) / 32) * 4;
    return n * (size_t)kElmsz[type];
}

int cumo_hip_na_alloc(cumo_hip_narray_t* a, int type, int ndim, const size_t* shape) {
    if (!a || !valid_type(type) || ndim < 0 || ndim > kMaxDim) return fail(CUMO_HIP_ERROR_ARGUMENT, "na_alloc: bad arguments");
    a->type = type;
    a->ndim = ndim;
    a->offset = 0;
    a->ptr = NULL;
    ssize_t s = type == CUMO_HIP_BIT ? 1 : kElmsz[type];
    size_t n = 1;
    for (int d = ndim - 1; d >= 0; d--) {
        a->shape[d] = shape[d];
        a->stride[d] = s;
        s *= (ssize_t)shape[d];
        n *= shape[d];
    }
    size_t bytes = cumo_hip_na_storage_bytes(type, n);
    if (bytes) {
        a->ptr = cumo_cuda_runtime_malloc(bytes);  // reports the failure itself
        if (!a->ptr) return CUMO_HIP_ERROR_OUT_OF_MEMORY;
    }
    return CUMO_HIP_OK;
}

int cumo_hip_na_ndloop_prepare(const cumo_hip_ndfunc_t* nf, const cumo_hip_narray_t* const* in,
                               cumo_hip_narray_t* const* out, unsigned int reduce, cumo_hip_loop_t* lp) {
    if (!nf || !lp || nf->nin < 1 || nf->nout < 0 || nf->nout > 2 || nf->nin + nf->nout > CUMO_HIP_NDLOOP_MAX_ARGS)
        return fail(CUMO_HIP_ERROR_ARGUMENT, "ndloop: bad ndfunc");
    const int nin = nf->nin, nout = nf->nout;
    std::memset(lp, 0, sizeof(*lp));
    lp->narg = nin + nout;

    // the loop's rank and shape: operands are aligned at their last dimension
    // and a dimension of size 1 repeats (ndloop.c:493-516)
    int nd = 0;
    for (int j = 0; j < nin; j++) {
        int rc = check_view(in[j], "input");
        if (rc) return rc;
        if (in[j]->ndim > nd) nd = in[j]->ndim;
    }
    size_t bshape[kMaxDim];
    for (int i = 0; i < nd; i++) bshape[i] = 1;
    for (int j = 0; j < nin; j++) {
        int off = nd - in[j]->ndim;
        for (int k = 0; k < in[j]->ndim; k++) {
            size_t n = in[j]->shape[k];
            if (n == 1) continue;
            if (bshape[off + k] == 1) {
                bshape[off + k] = n;
            } else if (bshape[off + k] != n) {
                char msg[128];
                std::snprintf(msg, sizeof(msg), "shape1[%d](=%zu) != shape2[%d](=%zu)", off + k, bshape[off + k], k, n);
                return fail(CUMO_HIP_ERROR_SHAPE, msg);
            }
        }
    }

    // reduce dimensions go last: array [*,+,*,+,*] => loop [*,*,*,+,+] (ndloop.c:421-451)
    if (reduce && !(nf->flag & CUMO_HIP_NDF_FLAT_REDUCE)) return fail(CUMO_HIP_ERROR_ARGUMENT, "ndloop: this operation does not reduce");
    if (nd < 32 && (reduce >> nd)) return fail(CUMO_HIP_ERROR_DIMENSION, "dimension is out of range");
    int trans_map[kMaxDim];
    int nkeep = 0;
    for (int i = 0; i < nd; i++)
        if (!((reduce >> i) & 1u)) trans_map[i] = nkeep++;
    {
        int j = nkeep;
        for (int i = 0; i < nd; i++)
            if ((reduce >> i) & 1u) trans_map[i] = j++;
    }
    size_t n[kMaxDim];
    ssize_t step[CUMO_HIP_NDLOOP_MAX_ARGS][kMaxDim];
    std::memset(step, 0, sizeof(step));
    for (int i = 0; i < nd; i++) n[trans_map[i]] = bshape[i];

    // inputs (ndloop.c:519-595)
    for (int j = 0; j < nin; j++) {
        const NA* a = in[j];
        cumo_hip_loop_args_t* la = &lp->args[j];
        la->type = a->type;
        la->elmsz = kElmsz[a->type];
        if (a->type == CUMO_HIP_BIT) {
            la->ptr = a->ptr;
            la->bitpos = (size_t)a->offset;
        } else {
            la->ptr = a->ptr + a->offset;
        }
        int off = nd - a->ndim;
        for (int k = 0; k < a->ndim; k++) step[j][trans_map[off + k]] = a->shape[k] == 1 ? 0 : a->stride[k];
    }

    // results: the loop's shape without the reduced dimensions, or with them
    // at size 1 under KEEP_DIM (ndloop.c:750-863)
    const bool keep = (nf->flag & CUMO_HIP_NDF_KEEP_DIM) != 0;
    size_t rshape[kMaxDim];
    int rmap[kMaxDim];
    int rnd = 0;
    for (int i = 0; i < nd; i++) {
        bool red = (reduce >> i) & 1u;
        if (red && !keep) {
            rmap[i] = -1;
        } else {
            rshape[rnd] = red ? 1 : bshape[i];
            rmap[i] = rnd++;
        }
    }
    for (int j = 0; j < nout; j++) {
        NA* o = out[j];
        const int type = nf->out_type[j];
        if (!o) return fail(CUMO_HIP_ERROR_ARGUMENT, "ndloop: missing result argument");
        if (o->ptr == NULL) {
            int rc = cumo_hip_na_alloc(o, type, rnd, rshape);
            if (rc) return rc;
        } else {
            int rc = check_view(o, "result");
            if (rc) return rc;
            if (o->type != type) return fail(CUMO_HIP_ERROR_TYPE, "ndloop: result array has the wrong element type");
            bool same = o->ndim == rnd;
            for (int d = 0; same && d < rnd; d++) same = o->shape[d] == rshape[d];
            if (!same) return fail(CUMO_HIP_ERROR_SHAPE, "ndloop: result array has the wrong shape");
        }
        cumo_hip_loop_args_t* la = &lp->args[nin + j];
        la->type = type;
        la->elmsz = kElmsz[type];
        if (type == CUMO_HIP_BIT) {
            la->ptr = o->ptr;
            la->bitpos = (size_t)o->offset;
        } else {
            la->ptr = o->ptr + o->offset;
        }
        for (int i = 0; i < nd; i++) {
            bool red = (reduce >> i) & 1u;
            step[nin + j][trans_map[i]] = (red || rmap[i] < 0 || o->shape[rmap[i]] == 1) ? 0 : o->stride[rmap[i]];
        }
    }

    // contraction, separately for the kept and the reduced dimensions
    int at = contract_range(lp, n, step, 0, nkeep, 0, false);
    int nkept = at;
    // a reducing operation always keeps one reduce dimension, of size 1 if need be
    at = contract_range(lp, n, step, nkeep, nd, at, (nf->flag & CUMO_HIP_NDF_FLAT_REDUCE) != 0);
    lp->reduce_dim = at - nkept;
    if (at == 0) {  // a single element
        lp->n[0] = 1;
        at = 1;
    }
    lp->ndim = at;
    return CUMO_HIP_OK;
}

int cumo_hip_na_ndloop(const cumo_hip_ndfunc_t* nf, const cumo_hip_narray_t* const* in,
                       cumo_hip_narray_t* const* out, unsigned int reduce, void* opt_ptr) {
    cumo_hip_loop_t lp;
    int rc = cumo_hip_na_ndloop_prepare(nf, in, out, reduce, &lp);
    if (rc) return rc;
    lp.opt_ptr = opt_ptr;
    size_t out_total = 1;
    for (int d = 0; d < lp.ndim - lp.reduce_dim; d++) out_total *= lp.n[d];
    if (out_total == 0) return CUMO_HIP_OK;  // nothing to write (template_kernel.h:76-81)
    nf->func(&lp);
    return lp.status;
}

void cumo_hip_make_indexer(const cumo_hip_loop_t* lp, cumo_na_indexer_t* ix) {
    std::memset(ix, 0, sizeof(*ix));
    ix->ndim = (unsigned char)lp->ndim;
    size_t t = 1;
    for (int d = 0; d < lp->ndim; d++) {
        ix->shape[d] = lp->n[d];
        t *= lp->n[d];
    }
    ix->total_size = t;
}

void cumo_hip_make_iarray(const cumo_hip_loop_t* lp, int j, cumo_na_iarray_t* a) {
    std::memset(a, 0, sizeof(*a));
    a->ptr = lp->args[j].ptr;
    for (int d = 0; d < lp->ndim; d++) a->step[d] = lp->args[j].step[d];
}

void cumo_hip_make_bit_iarray(const cumo_hip_loop_t* lp, int j, cumo_na_bit_iarray_t* a) {
    std::memset(a, 0, sizeof(*a));
    a->ptr = (CUMO_BIT_DIGIT*)lp->args[j].ptr;
    a->pos = lp->args[j].bitpos;
    for (int d = 0; d < lp->ndim; d++) a->step[d] = lp->args[j].step[d];
}

void cumo_hip_make_iarray_stridx(const cumo_hip_loop_t* lp, int j, cumo_na_iarray_stridx_t* a) {
    std::memset(a, 0, sizeof(*a));
    a->ptr = lp->args[j].ptr;
    for (int d = 0; d < kMaxDim; d++) CUMO_SDX_SET_STRIDE(a->stridx[d], d < lp->ndim ? lp->args[j].step[d] : 0);
}

void cumo_hip_make_bit_iarray_stridx(const cumo_hip_loop_t* lp, int j, cumo_na_bit_iarray_stridx_t* a) {
    std::memset(a, 0, sizeof(*a));
    a->ptr = (CUMO_BIT_DIGIT*)lp->args[j].ptr;
    a->pos = lp->args[j].bitpos;
    for (int d = 0; d < kMaxDim; d++) CUMO_SDX_SET_STRIDE(a->stridx[d], d < lp->ndim ? lp->args[j].step[d] : 0);
}

void cumo_hip_make_reduction_arg(const cumo_hip_loop_t* lp, cumo_na_reduction_arg_t* arg) {
    std::memset(arg, 0, sizeof(*arg));
    cumo_hip_make_iarray(lp, 0, &arg->in);
    cumo_hip_make_indexer(lp, &arg->in_indexer);
    const int ond = lp->ndim - lp->reduce_dim;
    arg->out.ptr = lp->args[1].ptr;
    arg->out_indexer.ndim = (unsigned char)ond;
    size_t t = 1;
    for (int d = 0; d < ond; d++) {
        arg->out.step[d] = lp->args[1].step[d];
        arg->out_indexer.shape[d] = lp->n[d];
        t *= lp->n[d];
    }
    arg->out_indexer.total_size = t;
}

}  // extern "C"

// ---------------------------------------------------------------------------
// Operation tables: what the reference generates as one C function per type
// and method (gen/spec.rb:199-277,427-457) is one row per method here.
// ---------------------------------------------------------------------------
namespace {

template <class C>
struct BinFns {
    void (*f)(IA*, IA*, IA*, IX*, int*);
    void (*fs)(IA*, C, IA*, IX*, int*, int);
};
struct BinaryRow {
    const char* op;
    BinFns<float> sf;
    BinFns<double> df;
    BinFns<int32_t> i32;
};
#define BIN_FNS(t, op) {cumo_iter_##t##_##op##_kernel_launch, cumo_iter_##t##_##op##_s_kernel_launch}
#define BIN_ROW_ALL(t, c, op) {#op, BIN_FNS(sfloat, op), BIN_FNS(dfloat, op), BIN_FNS(int32, op)},
#define BIN_ROW_FLT(t, c, op) {#op, BIN_FNS(sfloat, op), BIN_FNS(dfloat, op), {nullptr, nullptr}},
#define BIN_ROW_INT(t, c, op) {#op, {nullptr, nullptr}, {nullptr, nullptr}, BIN_FNS(int32, op)},
const BinaryRow kBinary[] = {
    CUMO_HIP_BINARY_OPS_ALL(BIN_ROW_ALL, _, _)
    CUMO_HIP_BINARY_OPS_FLOAT(BIN_ROW_FLT, _, _)
    CUMO_HIP_BINARY_OPS_INT(BIN_ROW_INT, _, _)
};

typedef void (*UnaryFn)(IA*, IA*, IX*, int*);
struct UnaryRow {
    const char* op;
    UnaryFn f[3];  // sfloat, dfloat, int32
};
#define UN_ROW_ALL(t, c, op) {#op, {cumo_iter_sfloat_##op##_kernel_launch, cumo_iter_dfloat_##op##_kernel_launch, cumo_iter_int32_##op##_kernel_launch}},
#define UN_ROW_FLT(t, c, op) {#op, {cumo_iter_sfloat_##op##_kernel_launch, cumo_iter_dfloat_##op##_kernel_launch, nullptr}},
#define UN_ROW_INT(t, c, op) {#op, {nullptr, nullptr, cumo_iter_int32_##op##_kernel_launch}},
const UnaryRow kUnary[] = {
    CUMO_HIP_UNARY_OPS_ALL(UN_ROW_ALL, _, _)
    CUMO_HIP_UNARY_OPS_FLOAT(UN_ROW_FLT, _, _)
    CUMO_HIP_UNARY_OPS_INT(UN_ROW_INT, _, _)
    UN_ROW_ALL(_, _, abs)
};

typedef void (*MathFn)(IA*, IA*, IX*);
struct MathRow {
    const char* op;
    MathFn f[2];
};
#define MATH_ROW(t, c, op) {#op, {cumo_iter_sfloat_math_s_##op##_kernel_launch, cumo_iter_dfloat_math_s_##op##_kernel_launch}},
const MathRow kMath[] = {CUMO_HIP_MATH_OPS(MATH_ROW, _, _)};

struct Math2Row {
    const char* op;
    void (*sf)(IA*, IA*, IA*, IX*);
    void (*sfs)(IA*, IA*, IX*, float, int);
    void (*df)(IA*, IA*, IA*, IX*);
    void (*dfs)(IA*, IA*, IX*, double, int);
};
#define MATH2_ROW(t, c, op) {#op, cumo_iter_sfloat_math_s_##op##_kernel_launch, cumo_iter_sfloat_math_s_##op##_s_kernel_launch, \
                             cumo_iter_dfloat_math_s_##op##_kernel_launch, cumo_iter_dfloat_math_s_##op##_s_kernel_launch},
const Math2Row kMath2[] = {CUMO_HIP_MATH2_OPS(MATH2_ROW, _, _)};

template <class C>
struct CondFns {
    void (*f)(IA*, IA*, BIA*, IX*);
    void (*fs)(IA*, C, BIA*, IX*, int);
};
struct CondRow {
    const char* op;
    CondFns<float> sf;
    CondFns<double> df;
    CondFns<int32_t> i32;
};
#define COND_ROW_ALL(t, c, op) {#op, BIN_FNS(sfloat, op), BIN_FNS(dfloat, op), BIN_FNS(int32, op)},
#define COND_ROW_FLT(t, c, op) {#op, BIN_FNS(sfloat, op), BIN_FNS(dfloat, op), {nullptr, nullptr}},
const CondRow kCond[] = {
    CUMO_HIP_COND_OPS_ALL(COND_ROW_ALL, _, _)
    CUMO_HIP_COND_OPS_FLOAT(COND_ROW_FLT, _, _)
};

typedef void (*CondUnaryFn)(IA*, BIA*, IX*);
struct CondUnaryRow {
    const char* op;
    CondUnaryFn f[2];
};
#define CONDU_ROW(t, c, op) {#op, {cumo_iter_sfloat_##op##_kernel_launch, cumo_iter_dfloat_##op##_kernel_launch}},
const CondUnaryRow kCondUnary[] = {CUMO_HIP_COND_UNARY_OPS(CONDU_ROW, _, _)};

typedef void (*StoreFn)(IA*, IA*, IX*);
// [dst: sfloat dfloat int32][src: sfloat dfloat int32 int64]
#define STORE_ROW(d) {cumo_iter_##d##_store_sfloat_kernel_launch, cumo_iter_##d##_store_dfloat_kernel_launch, \
                      cumo_iter_##d##_store_int32_kernel_launch, cumo_iter_##d##_store_int64_kernel_launch}
const StoreFn kStore[3][4] = {STORE_ROW(sfloat), STORE_ROW(dfloat), STORE_ROW(int32)};

typedef void (*StoreBitFn)(cumo_na_iarray_stridx_t*, cumo_na_bit_iarray_stridx_t*, IX*);
const StoreBitFn kStoreBit[3] = {cumo_iter_sfloat_store_bit_kernel_launch, cumo_iter_dfloat_store_bit_kernel_launch,
                                 cumo_iter_int32_store_bit_kernel_launch};

// number -> Bit, by source type code (sfloat dfloat int32 int64 uint64)
typedef void (*BitStoreFromFn)(cumo_na_bit_iarray_stridx_t*, cumo_na_iarray_stridx_t*, IX*);
const BitStoreFromFn kBitStoreFrom[5] = {cumo_iter_bit_store_sfloat_kernel_launch, cumo_iter_bit_store_dfloat_kernel_launch,
                                         cumo_iter_bit_store_int32_kernel_launch, cumo_iter_bit_store_int64_kernel_launch,
                                         cumo_iter_bit_store_uint64_kernel_launch};

typedef void (*ReduceFn)(cumo_na_reduction_arg_t*);
typedef void (*ReducePairFn)(cumo_na_reduction_arg_t*, IA*);
struct ReduceRow {
    const char* op;
    ReduceFn f[3];      // sfloat, dfloat, int32
    ReduceFn f_nan[3];
    int result;         // 0 same type, 1 the type sum answers (Int32 -> Int64)
};
#define RED3(name) {cumo_sfloat_##name##_kernel_launch, cumo_dfloat_##name##_kernel_launch, cumo_int32_##name##_kernel_launch}
#define RED2(name) {cumo_sfloat_##name##_kernel_launch, cumo_dfloat_##name##_kernel_launch, nullptr}
const ReduceRow kReduce[] = {
    {"sum", RED3(sum), RED2(sum_nan), 1},
    {"prod", RED3(prod), RED2(prod_nan), 1},
    {"min", RED3(min), RED2(min_nan), 0},
    {"max", RED3(max), RED2(max_nan), 0},
    {"ptp", RED3(ptp), RED2(ptp_nan), 0},
    {"mean", RED2(mean), RED2(mean_nan), 0},
    {"var", RED2(var), RED2(var_nan), 0},
    {"stddev", RED2(stddev), RED2(stddev_nan), 0},
    {"rms", RED2(rms), RED2(rms_nan), 0},
    {"kahan_sum", {nullptr, cumo_dfloat_kahan_sum_kernel_launch, nullptr}, {nullptr, cumo_dfloat_kahan_sum_nan_kernel_launch, nullptr}, 0},
};
struct ArgRow {
    const char* op;
    ReduceFn f32[3], f64[3], f32_nan[3], f64_nan[3];
    bool memory_index;  // min_index/max_index: the answer indexes the operand's own flattening
};
#define ARG_ROW(name, mi) {#name, RED3(name##_int32), RED3(name##_int64), RED2(name##_nan_int32), RED2(name##_nan_int64), mi}
const ArgRow kArg[] = {ARG_ROW(argmin, false), ARG_ROW(argmax, false), ARG_ROW(min_index, true), ARG_ROW(max_index, true)};
const ReducePairFn kMinmax[3] = {cumo_sfloat_minmax_kernel_launch, cumo_dfloat_minmax_kernel_launch, cumo_int32_minmax_kernel_launch};
const ReducePairFn kMinmaxNan[3] = {cumo_sfloat_minmax_nan_kernel_launch, cumo_dfloat_minmax_nan_kernel_launch, nullptr};

typedef cumo_na_bit_iarray_stridx_t BSX;
struct BitBinaryRow {
    const char* op;
    void (*f)(BSX*, BSX*, BSX*, IX*);
    void (*fc)(CUMO_BIT_DIGIT*, size_t, CUMO_BIT_DIGIT*, size_t, CUMO_BIT_DIGIT*, size_t, uint64_t);
};
#define BITB_ROW(op) {#op, cumo_iter_bit_##op##_kernel_launch, cumo_iter_bit_##op##_contiguous_kernel_launch},
const BitBinaryRow kBitBinary[] = {CUMO_HIP_BIT_BINARY_OPS(BITB_ROW)};
struct BitUnaryRow {
    const char* op;
    void (*f)(BSX*, BSX*, IX*);
    void (*fc)(CUMO_BIT_DIGIT*, size_t, CUMO_BIT_DIGIT*, size_t, uint64_t);
};
#define BITU_ROW(op) {#op, cumo_iter_bit_##op##_kernel_launch, cumo_iter_bit_##op##_contiguous_kernel_launch},
const BitUnaryRow kBitUnary[] = {CUMO_HIP_BIT_UNARY_OPS(BITU_ROW)};
// Bit#store(Bit) has launchers of its own (gen/tmpl_bit/store_bit.c:1-2)
const BitUnaryRow kBitStoreBit = {"store_bit", cumo_iter_bit_store_bit_kernel_launch, cumo_iter_bit_store_bit_contiguous_kernel_launch};

template <class Row, size_t N>
const Row* find_row(const Row (&rows)[N], const char* op) {
    if (!op) return nullptr;
    for (size_t i = 0; i < N; i++)
        if (std::strcmp(rows[i].op, op) == 0) return &rows[i];
    return nullptr;
}

int no_method(const char* op) {
    char msg[96];
    std::snprintf(msg, sizeof(msg), "undefined operation '%s' for this element type", op ? op : "(null)");
    return fail(CUMO_HIP_ERROR_TYPE, msg);
}

// the higher of two arithmetic types: Int32 < SFloat < DFloat
// (the upcast tables of gen/def/{int32,sfloat,dfloat}.rb)
int upcast(int a, int b) {
    static const int rank[3] = {1, 2, 0};  // indexed by type: sfloat, dfloat, int32
    return rank[a] >= rank[b] ? a : b;
}

void free_tmp(NA* t) {
    if (t->ptr) {
        cumo_cuda_runtime_free(t->ptr);
        t->ptr = NULL;
    }
}

// ---- iterators ---------------------------------------------------------------
struct StoreOpt {
    StoreFn f;
};
void iter_store(LP* lp) {  // args: dst, src (gen/tmpl/store_from.c)
    IA a1, a2;
    IX ix;
    cumo_hip_make_iarray(lp, 0, &a1);
    cumo_hip_make_iarray(lp, 1, &a2);
    cumo_hip_make_indexer(lp, &ix);
    ((StoreOpt*)lp->opt_ptr)->f(&a1, &a2, &ix);
}

// *use = x itself, or a contiguous copy of x in `type` held by tmp
int cast_operand(const NA* x, int type, NA* tmp, const NA** use) {
    tmp->ptr = NULL;
    if (x->type == type) {
        *use = x;
        return CUMO_HIP_OK;
    }
    int rc = cumo_hip_na_alloc(tmp, type, x->ndim, x->shape);
    if (rc) return rc;
    *use = tmp;
    if (total_of(x) == 0) return CUMO_HIP_OK;
    StoreOpt opt = {kStore[type][x->type]};
    cumo_hip_ndfunc_t nf = {iter_store, 0, 2, 0, {0, 0}};
    const NA* in[2] = {tmp, x};
    return cumo_hip_na_ndloop(&nf, in, NULL, 0, &opt);
}

struct BinaryOpt {
    const BinaryRow* row;
    int type;
    bool scalar;
    double sv;
    int left;
    bool checked;   // the launcher reports a data error through the pinned flag
    bool flagged;
};
void iter_binary(LP* lp) {
    BinaryOpt* o = (BinaryOpt*)lp->opt_ptr;
    IA a1, a2, a3;
    IX ix;
    cumo_hip_make_indexer(lp, &ix);
    cumo_hip_make_iarray(lp, 0, &a1);
    int* flag = o->checked ? cumo_cuda_runtime_error_flag_new() : NULL;
    if (o->scalar) {
        cumo_hip_make_iarray(lp, 1, &a3);
        switch (o->type) {
            case CUMO_HIP_SFLOAT: o->row->sf.fs(&a1, (float)o->sv, &a3, &ix, flag, o->left); break;
            case CUMO_HIP_DFLOAT: o->row->df.fs(&a1, o->sv, &a3, &ix, flag, o->left); break;
            default: o->row->i32.fs(&a1, (int32_t)o->sv, &a3, &ix, flag, o->left); break;
        }
    } else {
        cumo_hip_make_iarray(lp, 1, &a2);
        cumo_hip_make_iarray(lp, 2, &a3);
        switch (o->type) {
            case CUMO_HIP_SFLOAT: o->row->sf.f(&a1, &a2, &a3, &ix, flag); break;
            case CUMO_HIP_DFLOAT: o->row->df.f(&a1, &a2, &a3, &ix, flag); break;
            default: o->row->i32.f(&a1, &a2, &a3, &ix, flag); break;
        }
    }
    // the caller reads the flag with a stream synchronisation (gen/tmpl/binary.c:120-126)
    if (flag && cumo_cuda_runtime_error_flag_get(flag)) o->flagged = true;
}

bool binary_has(const BinaryRow* r, int type, bool scalar) {
    switch (type) {
        case CUMO_HIP_SFLOAT: return scalar ? r->sf.fs != nullptr : r->sf.f != nullptr;
        case CUMO_HIP_DFLOAT: return scalar ? r->df.fs != nullptr : r->df.f != nullptr;
        default: return scalar ? r->i32.fs != nullptr : r->i32.f != nullptr;
    }
}

struct UnaryOpt {
    UnaryFn f;
    bool checked, flagged;
};
void iter_unary(LP* lp) {
    UnaryOpt* o = (UnaryOpt*)lp->opt_ptr;
    IA a1, a2;
    IX ix;
    cumo_hip_make_indexer(lp, &ix);
    cumo_hip_make_iarray(lp, 0, &a1);
    cumo_hip_make_iarray(lp, 1, &a2);
    int* flag = o->checked ? cumo_cuda_runtime_error_flag_new() : NULL;
    o->f(&a1, &a2, &ix, flag);
    if (flag && cumo_cuda_runtime_error_flag_get(flag)) o->flagged = true;
}

void iter_math(LP* lp) {
    IA a1, a2;
    IX ix;
    cumo_hip_make_indexer(lp, &ix);
    cumo_hip_make_iarray(lp, 0, &a1);
    cumo_hip_make_iarray(lp, 1, &a2);
    ((MathFn)lp->opt_ptr)(&a1, &a2, &ix);
}

struct Math2Opt {
    const Math2Row* row;
    int type;
    bool scalar;
    double sv;
    int left;
};
void iter_math2(LP* lp) {
    Math2Opt* o = (Math2Opt*)lp->opt_ptr;
    IA a1, a2, a3;
    IX ix;
    cumo_hip_make_indexer(lp, &ix);
    cumo_hip_make_iarray(lp, 0, &a1);
    if (o->scalar) {
        cumo_hip_make_iarray(lp, 1, &a3);
        if (o->type == CUMO_HIP_SFLOAT) o->row->sfs(&a1, &a3, &ix, (float)o->sv, o->left);
        else o->row->dfs(&a1, &a3, &ix, o->sv, o->left);
    } else {
        cumo_hip_make_iarray(lp, 1, &a2);
        cumo_hip_make_iarray(lp, 2, &a3);
        if (o->type == CUMO_HIP_SFLOAT) o->row->sf(&a1, &a2, &a3, &ix);
        else o->row->df(&a1, &a2, &a3, &ix);
    }
}

struct CondOpt {
    const CondRow* row;
    int type;
    bool scalar;
    double sv;
    int left;
};
void iter_cond(LP* lp) {
    CondOpt* o = (CondOpt*)lp->opt_ptr;
    IA a1, a2;
    BIA a3;
    IX ix;
    cumo_hip_make_indexer(lp, &ix);
    cumo_hip_make_iarray(lp, 0, &a1);
    if (o->scalar) {
        cumo_hip_make_bit_iarray(lp, 1, &a3);
        switch (o->type) {
            case CUMO_HIP_SFLOAT: o->row->sf.fs(&a1, (float)o->sv, &a3, &ix, o->left); break;
            case CUMO_HIP_DFLOAT: o->row->df.fs(&a1, o->sv, &a3, &ix, o->left); break;
            default: o->row->i32.fs(&a1, (int32_t)o->sv, &a3, &ix, o->left); break;
        }
    } else {
        cumo_hip_make_iarray(lp, 1, &a2);
        cumo_hip_make_bit_iarray(lp, 2, &a3);
        switch (o->type) {
            case CUMO_HIP_SFLOAT: o->row->sf.f(&a1, &a2, &a3, &ix); break;
            case CUMO_HIP_DFLOAT: o->row->df.f(&a1, &a2, &a3, &ix); break;
            default: o->row->i32.f(&a1, &a2, &a3, &ix); break;
        }
    }
}
bool cond_has(const CondRow* r, int type) {
    switch (type) {
        case CUMO_HIP_SFLOAT: return r->sf.f != nullptr;
        case CUMO_HIP_DFLOAT: return r->df.f != nullptr;
        default: return r->i32.f != nullptr;
    }
}

void iter_cond_unary(LP* lp) {
    IA a1;
    BIA a2;
    IX ix;
    cumo_hip_make_indexer(lp, &ix);
    cumo_hip_make_iarray(lp, 0, &a1);
    cumo_hip_make_bit_iarray(lp, 1, &a2);
    ((CondUnaryFn)lp->opt_ptr)(&a1, &a2, &ix);
}

void iter_store_bit(LP* lp) {  // args: dst (number), src (Bit)  (gen/tmpl/store_bit.c)
    cumo_na_iarray_stridx_t a1;
    BSX a2;
    IX ix;
    cumo_hip_make_indexer(lp, &ix);
    cumo_hip_make_iarray_stridx(lp, 0, &a1);
    cumo_hip_make_bit_iarray_stridx(lp, 1, &a2);
    ((StoreBitFn)lp->opt_ptr)(&a1, &a2, &ix);
}

void iter_bit_store_from(LP* lp) {  // args: dst (Bit), src (number)  (gen/tmpl_bit/store_from.c:56-62)
    BSX a1;
    cumo_na_iarray_stridx_t a2;
    IX ix;
    cumo_hip_make_indexer(lp, &ix);
    cumo_hip_make_bit_iarray_stridx(lp, 0, &a1);
    cumo_hip_make_iarray_stridx(lp, 1, &a2);
    ((BitStoreFromFn)lp->opt_ptr)(&a1, &a2, &ix);
}

void iter_bit_fill(LP* lp) {  // args: dst (Bit); opt: the bit  (gen/tmpl_bit/fill.c:11-40)
    BSX a3;
    IX ix;
    cumo_hip_make_indexer(lp, &ix);
    cumo_hip_make_bit_iarray_stridx(lp, 0, &a3);
    // the launcher itself takes the word-wise form for one run of step 1
    cumo_iter_bit_fill_kernel_launch(&a3, *(const CUMO_BIT_DIGIT*)lp->opt_ptr, &ix);
}

void iter_copy_bytes(LP* lp) {  // args: src, dst  (narray/data.c:84-92)
    IA a1, a2;
    IX ix;
    cumo_hip_make_indexer(lp, &ix);
    cumo_hip_make_iarray(lp, 0, &a1);
    cumo_hip_make_iarray(lp, 1, &a2);
    cumo_iter_copy_bytes_indexer_kernel_launch(&a1, &a2, &ix, lp->args[0].elmsz);
}

struct FillOpt {
    double value;
};
void iter_fill(LP* lp) {
    IA a1;
    IX ix;
    cumo_hip_make_indexer(lp, &ix);
    cumo_hip_make_iarray(lp, 0, &a1);
    double v = ((FillOpt*)lp->opt_ptr)->value;
    switch (lp->args[0].type) {
        case CUMO_HIP_SFLOAT: cumo_iter_sfloat_fill_kernel_launch(&a1, &ix, (float)v); break;
        case CUMO_HIP_DFLOAT: cumo_iter_dfloat_fill_kernel_launch(&a1, &ix, v); break;
        default: cumo_iter_int32_fill_kernel_launch(&a1, &ix, (int32_t)v); break;
    }
}

struct ReduceOpt {
    ReduceFn f;
    ReducePairFn fp;
};
void iter_reduce(LP* lp) {  // gen/tmpl/accum.c:41-45, minmax.c
    ReduceOpt* o = (ReduceOpt*)lp->opt_ptr;
    cumo_na_reduction_arg_t arg;
    cumo_hip_make_reduction_arg(lp, &arg);
    if (o->fp) {
        IA out2;
        std::memset(&out2, 0, sizeof(out2));
        out2.ptr = lp->args[2].ptr;
        for (int d = 0; d < lp->ndim - lp->reduce_dim; d++) out2.step[d] = lp->args[2].step[d];
        o->fp(&arg, &out2);
    } else {
        o->f(&arg);
    }
}

// The flat bit run [pos, pos + n) with step 1 can go to the word kernels.
bool flat_bits(const LP* lp) {
    if (lp->ndim != 1) return false;
    for (int j = 0; j < lp->narg; j++)
        if (lp->args[j].step[0] != 1) return false;
    return true;
}
inline CUMO_BIT_DIGIT* word_ptr(const cumo_hip_loop_args_t& a) { return (CUMO_BIT_DIGIT*)a.ptr + a.bitpos / 32; }

void iter_bit_binary(LP* lp) {  // gen/tmpl_bit/binary.c:17-60
    const BitBinaryRow* r = (const BitBinaryRow*)lp->opt_ptr;
    if (flat_bits(lp)) {
        r->fc(word_ptr(lp->args[0]), lp->args[0].bitpos % 32, word_ptr(lp->args[1]), lp->args[1].bitpos % 32,
              word_ptr(lp->args[2]), lp->args[2].bitpos % 32, lp->n[0]);
        return;
    }
    BSX a1, a2, a3;
    IX ix;
    cumo_hip_make_indexer(lp, &ix);
    cumo_hip_make_bit_iarray_stridx(lp, 0, &a1);
    cumo_hip_make_bit_iarray_stridx(lp, 1, &a2);
    cumo_hip_make_bit_iarray_stridx(lp, 2, &a3);
    r->f(&a1, &a2, &a3, &ix);
}

void iter_bit_unary(LP* lp) {  // gen/tmpl_bit/unary.c
    const BitUnaryRow* r = (const BitUnaryRow*)lp->opt_ptr;
    if (flat_bits(lp)) {
        r->fc(word_ptr(lp->args[0]), lp->args[0].bitpos % 32, word_ptr(lp->args[1]), lp->args[1].bitpos % 32, lp->n[0]);
        return;
    }
    BSX a1, a3;
    IX ix;
    cumo_hip_make_indexer(lp, &ix);
    cumo_hip_make_bit_iarray_stridx(lp, 0, &a1);
    cumo_hip_make_bit_iarray_stridx(lp, 1, &a3);
    r->f(&a1, &a3, &ix);
}

// count_true / count_false: the innermost loop dimension is one launch, the
// outer ones are walked here (gen/tmpl_bit/bit_count.c:9-36 under the
// host-walked loop of ndloop.c:1569-1613).
struct CountOpt {
    bool count_false;
    bool overwrite;  // the results need not hold zero: the launcher sees to it (only the launch for every output at once takes this)
};
void count_walk(const LP* lp, int level, size_t pos, char* optr, bool count_false) {
    const cumo_hip_loop_args_t& in = lp->args[0];
    const cumo_hip_loop_args_t& out = lp->args[1];
    if (level == lp->ndim - 1) {
        const ssize_t s1 = in.step[level], s2 = out.step[level];
        CUMO_BIT_DIGIT* a = (CUMO_BIT_DIGIT*)in.ptr;
        size_t p = pos;
        if (s1 >= 0) {  // CUMO_INIT_PTR_BIT_IDX rebases the word pointer (template.h:41-62)
            a += pos / 32;
            p = pos % 32;
        }
        const uint64_t n = lp->n[level];
        if (s2 == 0) {
            if (count_false) cumo_iter_bit_count_false_stride_kernel_launch(p, optr, a, s1, n);
            else cumo_iter_bit_count_true_stride_kernel_launch(p, optr, a, s1, n);
        } else {
            if (count_false) cumo_iter_bit_count_false_stride_stride_kernel_launch(p, optr, a, s1, s2, n);
            else cumo_iter_bit_count_true_stride_stride_kernel_launch(p, optr, a, s1, s2, n);
        }
        return;
    }
    for (size_t i = 0; i < lp->n[level]; i++)
        count_walk(lp, level + 1, pos + (size_t)((ssize_t)i * in.step[level]), optr + (ssize_t)i * out.step[level], count_false);
}
void iter_bit_count(LP* lp) {
    const bool count_false = ((CountOpt*)lp->opt_ptr)->count_false;
    const int nkeep = lp->ndim - lp->reduce_dim;
    if (nkeep == 0 && lp->reduce_dim == 1) {
        // one run into one counter: the reference's run launcher, whole device on it
        count_walk(lp, 0, lp->args[0].bitpos, lp->args[1].ptr, count_false);
        return;
    }
    // every output in one launch instead of the reference's walk over them on the host
    cumo_hip_bit_count_nd_t d;
    std::memset(&d, 0, sizeof(d));
    d.out_ndim = nkeep;
    d.red_ndim = lp->reduce_dim;
    for (int k = 0; k < nkeep; ++k) {
        d.out_shape[k] = lp->n[k];
        d.in_out_step[k] = lp->args[0].step[k];
        d.out_step[k] = lp->args[1].step[k];
    }
    for (int k = 0; k < lp->reduce_dim; ++k) {
        d.red_shape[k] = lp->n[nkeep + k];
        d.in_red_step[k] = lp->args[0].step[nkeep + k];
    }
    d.in = (CUMO_BIT_DIGIT*)lp->args[0].ptr;
    d.pos = lp->args[0].bitpos;
    d.out = lp->args[1].ptr;
    d.count_false = count_false ? 1 : 0;
    d.overwrite = ((CountOpt*)lp->opt_ptr)->overwrite ? 1 : 0;
    cumo_hip_bit_count_nd_kernel_launch(&d);
}


// ---- pow, maximum/minimum, clip (gen/tmpl/pow.c, ewcomp.c, clip.c) ---------------
typedef void (*Arr3Fn)(IA*, IA*, IA*, IX*);
struct PowFns {
    Arr3Fn pow, pow_int32;
};
#define POW_FNS(t) {cumo_iter_##t##_pow_kernel_launch, cumo_iter_##t##_pow_int32_kernel_launch}
const PowFns kPow[3] = {POW_FNS(sfloat), POW_FNS(dfloat), POW_FNS(int32)};

void iter_arr3(LP* lp) {  // two inputs, one result, no flag
    IA a1, a2, a3;
    IX ix;
    cumo_hip_make_indexer(lp, &ix);
    cumo_hip_make_iarray(lp, 0, &a1);
    cumo_hip_make_iarray(lp, 1, &a2);
    cumo_hip_make_iarray(lp, 2, &a3);
    ((Arr3Fn)lp->opt_ptr)(&a1, &a2, &a3, &ix);
}

struct PowSOpt {
    int type;      // element type of the launcher family
    int form;      // 0: x ** sv, 1: sv ** x, 2: x ** (Int32)sv, 3: sv ** (Int32 array)x
    double sv;
};
void iter_pow_s(LP* lp) {
    const PowSOpt* o = (const PowSOpt*)lp->opt_ptr;
    IA a1, a3;
    IX ix;
    cumo_hip_make_indexer(lp, &ix);
    cumo_hip_make_iarray(lp, 0, &a1);
    cumo_hip_make_iarray(lp, 1, &a3);
    switch (o->type) {
        case CUMO_HIP_SFLOAT:
            if (o->form <= 1) cumo_iter_sfloat_pow_s_kernel_launch(&a1, (float)o->sv, &a3, &ix, o->form);
            else if (o->form == 2) cumo_iter_sfloat_pow_int32_s_kernel_launch(&a1, (int32_t)o->sv, &a3, &ix);
            else cumo_iter_sfloat_pow_int32_s_left_kernel_launch((float)o->sv, &a1, &a3, &ix);
            break;
        case CUMO_HIP_DFLOAT:
            if (o->form <= 1) cumo_iter_dfloat_pow_s_kernel_launch(&a1, o->sv, &a3, &ix, o->form);
            else if (o->form == 2) cumo_iter_dfloat_pow_int32_s_kernel_launch(&a1, (int32_t)o->sv, &a3, &ix);
            else cumo_iter_dfloat_pow_int32_s_left_kernel_launch(o->sv, &a1, &a3, &ix);
            break;
        default:
            if (o->form <= 1) cumo_iter_int32_pow_s_kernel_launch(&a1, (int32_t)o->sv, &a3, &ix, o->form);
            else if (o->form == 2) cumo_iter_int32_pow_int32_s_kernel_launch(&a1, (int32_t)o->sv, &a3, &ix);
            else cumo_iter_int32_pow_int32_s_left_kernel_launch((int32_t)o->sv, &a1, &a3, &ix);
            break;
    }
}

struct EwcompRow {
    const char* op;
    Arr3Fn f[3], fnan[3];
};
const EwcompRow kEwcomp[] = {
    {"maximum", {cumo_sfloat_maximum_kernel_launch, cumo_dfloat_maximum_kernel_launch, cumo_int32_maximum_kernel_launch},
     {cumo_sfloat_maximum_nan_kernel_launch, cumo_dfloat_maximum_nan_kernel_launch, nullptr}},
    {"minimum", {cumo_sfloat_minimum_kernel_launch, cumo_dfloat_minimum_kernel_launch, cumo_int32_minimum_kernel_launch},
     {cumo_sfloat_minimum_nan_kernel_launch, cumo_dfloat_minimum_nan_kernel_launch, nullptr}},
};

struct ClipOpt {
    int type;
    int form;      // 0: two scalars, 1: scalar min, 2: scalar max, 3: array min, 4: array max, 5: two arrays
    double lo, hi;
    bool flagged;
};
void iter_clip(LP* lp) {
    ClipOpt* o = (ClipOpt*)lp->opt_ptr;
    IA a[4];
    IX ix;
    cumo_hip_make_indexer(lp, &ix);
    for (int j = 0; j < lp->narg; ++j) cumo_hip_make_iarray(lp, j, &a[j]);
#define CLIP_CASES(t, c)                                                                              \
    switch (o->form) {                                                                                \
        case 0: cumo_iter_##t##_clip_s_kernel_launch(&a[0], (c)o->lo, (c)o->hi, &a[1], &ix); break;   \
        case 1: cumo_iter_##t##_clip_min_s_kernel_launch(&a[0], (c)o->lo, &a[1], &ix); break;         \
        case 2: cumo_iter_##t##_clip_max_s_kernel_launch(&a[0], (c)o->hi, &a[1], &ix); break;         \
        case 3: cumo_iter_##t##_clip_min_kernel_launch(&a[0], &a[1], &a[2], &ix); break;              \
        case 4: cumo_iter_##t##_clip_max_kernel_launch(&a[0], &a[1], &a[2], &ix); break;              \
        default: {                                                                                    \
            int* flag = cumo_cuda_runtime_error_flag_new();                                           \
            cumo_iter_##t##_clip_kernel_launch(&a[0], &a[1], &a[2], &a[3], &ix, flag);                \
            if (flag && cumo_cuda_runtime_error_flag_get(flag)) o->flagged = true;                    \
        }                                                                                             \
    }
    switch (o->type) {
        case CUMO_HIP_SFLOAT: CLIP_CASES(sfloat, float) break;
        case CUMO_HIP_DFLOAT: CLIP_CASES(dfloat, double) break;
        default: CLIP_CASES(int32, int32_t) break;
    }
#undef CLIP_CASES
}


// ---- mulsum (gen/tmpl/accum_binary.c:8-60): the innermost loop dimension is one
// launch, the others are walked here, as the reference's host-walked loop does.
typedef void (*MulsumReduceFn)(char*, char*, char*, ssize_t, ssize_t, uint64_t);
typedef void (*MulsumEwFn)(char*, char*, char*, ssize_t, ssize_t, ssize_t, uint64_t);
struct MulsumFns {
    MulsumReduceFn red, red_nan;
    MulsumEwFn ew, ew_nan;
};
const MulsumFns kMulsum[3] = {
    {cumo_sfloat_mulsum_reduce_kernel_launch, cumo_sfloat_mulsum_nan_reduce_kernel_launch, cumo_sfloat_mulsum_kernel_launch,
     cumo_sfloat_mulsum_nan_kernel_launch},
    {cumo_dfloat_mulsum_reduce_kernel_launch, cumo_dfloat_mulsum_nan_reduce_kernel_launch, cumo_dfloat_mulsum_kernel_launch,
     cumo_dfloat_mulsum_nan_kernel_launch},
    {cumo_int32_mulsum_reduce_kernel_launch, nullptr, cumo_int32_mulsum_kernel_launch, nullptr},
};
struct MulsumOpt {
    int type;
    bool nan;
};
void mulsum_walk(const LP* lp, int level, char* p1, char* p2, char* p3, const MulsumOpt* o) {
    const int last = lp->ndim - 1;
    if (level == last) {
        const MulsumFns& f = kMulsum[o->type];
        const ssize_t s1 = lp->args[0].step[last], s2 = lp->args[1].step[last], s3 = lp->args[2].step[last];
        if (s3 == 0) (o->nan && f.red_nan ? f.red_nan : f.red)(p1, p2, p3, s1, s2, lp->n[last]);
        else (o->nan && f.ew_nan ? f.ew_nan : f.ew)(p1, p2, p3, s1, s2, s3, lp->n[last]);
        return;
    }
    for (size_t i = 0; i < lp->n[level]; ++i)
        mulsum_walk(lp, level + 1, p1 + (ssize_t)i * lp->args[0].step[level], p2 + (ssize_t)i * lp->args[1].step[level],
                    p3 + (ssize_t)i * lp->args[2].step[level], o);
}

int check_arith(const NA* x) {
    int rc = check_view(x, "operand");
    if (rc) return rc;
    if (!is_arith(x->type)) return fail(CUMO_HIP_ERROR_TYPE, "operand is not SFloat, DFloat or Int32");
    return CUMO_HIP_OK;
}

unsigned all_dims(const NA* x) { return x->ndim ? ((1u << x->ndim) - 1u) : 0u; }

// + - * / of two arrays of different types that have one shape and are one contiguous run each, into a fresh
// result or a given contiguous one of the higher type: one launch that converts on the way in, instead of a cast
// into a temporary array and the higher type's own launch (ew_mixed.hip). *taken says whether it has seen to the
// operation (launched it, or failed to allocate the result: the error kind is returned then).
int mixed_one_launch(const char* op, const NA* x, const NA* y, int up, NA* z, bool* taken) {
    *taken = false;
    int code;
    if (!std::strcmp(op, "add")) code = 0;
    else if (!std::strcmp(op, "sub")) code = 1;
    else if (!std::strcmp(op, "mul")) code = 2;
    else if (!std::strcmp(op, "div") && is_float(up)) code = 3;
    else return CUMO_HIP_OK;
    static const bool off = [] {
        const char* e = std::getenv("CUMO_HIP_MIXED_ONE_LAUNCH");   // =0: always cast first (for tests)
        return e && e[0] == '0';
    }();
    if (off || !z || x->ndim != y->ndim || x->ndim < 1) return CUMO_HIP_OK;
    for (int d = 0; d < x->ndim; d++)
        if (x->shape[d] != y->shape[d]) return CUMO_HIP_OK;
    const size_t n = total_of(x);
    if (n == 0 || !is_contiguous(x) || !is_contiguous(y)) return CUMO_HIP_OK;
    const char* px = x->ptr + x->offset;
    const char* py = y->ptr + y->offset;
    if ((((uintptr_t)px | (uintptr_t)py) & 15u) != 0) return CUMO_HIP_OK;
    const bool fresh = z->ptr == NULL;
    if (!fresh) {
        if (z->type != up || z->ndim != x->ndim || !is_contiguous(z) || (((uintptr_t)(z->ptr + z->offset)) & 15u) != 0) return CUMO_HIP_OK;
        for (int d = 0; d < x->ndim; d++)
            if (z->shape[d] != x->shape[d]) return CUMO_HIP_OK;
    } else {
        const int rc = cumo_hip_na_alloc(z, up, x->ndim, x->shape);
        if (rc != CUMO_HIP_OK) {
            *taken = true;
            return rc;
        }
    }
    if (cumo_hip::mixed_flat_binary(code, x->type, px, y->type, py, z->ptr + z->offset, n)) {
        *taken = true;
        return CUMO_HIP_OK;
    }
    if (fresh) {
        cumo_cuda_runtime_free(z->ptr);
        z->ptr = NULL;
    }
    return CUMO_HIP_OK;
}

// == != > >= < <= of two such arrays into a fresh Bit result (or a given whole contiguous one) the same way
int mixed_compare_one_launch(const char* op, const NA* x, const NA* y, NA* z, bool* taken) {
    *taken = false;
    static const char* const names[6] = {"eq", "ne", "gt", "ge", "lt", "le"};
    int code = -1;
    for (int k = 0; k < 6; k++)
        if (!std::strcmp(op, names[k])) code = k;
    static const bool off = [] {
        const char* e = std::getenv("CUMO_HIP_MIXED_ONE_LAUNCH");
        return e && e[0] == '0';
    }();
    if (code < 0 || off || !z || x->ndim != y->ndim || x->ndim < 1) return CUMO_HIP_OK;
    for (int d = 0; d < x->ndim; d++)
        if (x->shape[d] != y->shape[d]) return CUMO_HIP_OK;
    const size_t n = total_of(x);
    if (n == 0 || !is_contiguous(x) || !is_contiguous(y)) return CUMO_HIP_OK;
    const char* px = x->ptr + x->offset;
    const char* py = y->ptr + y->offset;
    if ((((uintptr_t)px | (uintptr_t)py) & 15u) != 0) return CUMO_HIP_OK;
    const bool fresh = z->ptr == NULL;
    if (!fresh) {
        if (z->type != CUMO_HIP_BIT || z->ndim != x->ndim || z->offset != 0 || !is_contiguous(z) || (((uintptr_t)z->ptr) & 15u) != 0) return CUMO_HIP_OK;
        for (int d = 0; d < x->ndim; d++)
            if (z->shape[d] != x->shape[d]) return CUMO_HIP_OK;
    } else {
        const int rc = cumo_hip_na_alloc(z, CUMO_HIP_BIT, x->ndim, x->shape);
        if (rc != CUMO_HIP_OK) {
            *taken = true;
            return rc;
        }
    }
    if (cumo_hip::mixed_flat_compare(code, x->type, px, y->type, py, reinterpret_cast<CUMO_BIT_DIGIT*>(z->ptr), n)) {
        *taken = true;
        return CUMO_HIP_OK;
    }
    if (fresh) {
        cumo_cuda_runtime_free(z->ptr);
        z->ptr = NULL;
    }
    return CUMO_HIP_OK;
}

}  // namespace

extern "C" {

int cumo_hip_na_binary(const char* op, const cumo_hip_narray_t* x, const cumo_hip_narray_t* y, cumo_hip_narray_t* z) {
    int rc = check_arith(x);
    if (!rc) rc = check_arith(y);
    if (rc) return rc;
    const BinaryRow* row = find_row(kBinary, op);
    const int up = upcast(x->type, y->type);
    if (!row || !binary_has(row, up, false)) return no_method(op);
    if (x->type != y->type) {
        bool taken = false;
        rc = mixed_one_launch(op, x, y, up, z, &taken);
        if (taken) return rc;
    }
    NA tx, ty;
    const NA *ux, *uy;
    rc = cast_operand(x, up, &tx, &ux);
    if (!rc) rc = cast_operand(y, up, &ty, &uy);
    else ty.ptr = NULL;
    if (!rc) {
        BinaryOpt opt = {row, up, false, 0.0, 0, up == CUMO_HIP_INT32 && (!std::strcmp(op, "div") || !std::strcmp(op, "mod")), false};
        cumo_hip_ndfunc_t nf = {iter_binary, 0, 2, 1, {up, 0}};
        const NA* in[2] = {ux, uy};
        NA* out[1] = {z};
        rc = cumo_hip_na_ndloop(&nf, in, out, 0, &opt);
        if (!rc && opt.flagged) rc = CUMO_HIP_ERROR_ZERO_DIVISION;
    }
    free_tmp(&tx);
    free_tmp(&ty);
    if (rc == CUMO_HIP_ERROR_ZERO_DIVISION) return fail(rc, "error in NArray operation");
    return rc;
}

int cumo_hip_na_binary_s(const char* op, const cumo_hip_narray_t* x, double sv, int scalar_is_left, cumo_hip_narray_t* z) {
    int rc = check_arith(x);
    if (rc) return rc;
    const BinaryRow* row = find_row(kBinary, op);
    if (!row || !binary_has(row, x->type, true)) return no_method(op);
    // (an Int32 array divided by one divisor that is not zero rejects nothing: no flag, and no wait for it)
    const bool divides = x->type == CUMO_HIP_INT32 && (!std::strcmp(op, "div") || !std::strcmp(op, "mod"));
    BinaryOpt opt = {row, x->type, true, sv, scalar_is_left ? 1 : 0, divides && (scalar_is_left || (int32_t)sv == 0), false};
    cumo_hip_ndfunc_t nf = {iter_binary, 0, 1, 1, {x->type, 0}};
    const NA* in[1] = {x};
    NA* out[1] = {z};
    rc = cumo_hip_na_ndloop(&nf, in, out, 0, &opt);
    if (!rc && opt.flagged) return fail(CUMO_HIP_ERROR_ZERO_DIVISION, "error in NArray operation");
    return rc;
}

// x op sv for a number that is a Ruby Float: a float array keeps its type, an Int32 array is computed in DFloat
// (the upcast table of gen/def/int32.rb) -- in one launch that converts on the way in where the array is one
// contiguous, aligned run and the operation is + - * /, through a DFloat copy of the array otherwise.
int cumo_hip_na_binary_fs(const char* op, const cumo_hip_narray_t* x, double sv, int scalar_is_left, cumo_hip_narray_t* z) {
    int rc = check_arith(x);
    if (rc) return rc;
    if (x->type != CUMO_HIP_INT32) return cumo_hip_na_binary_s(op, x, sv, scalar_is_left, z);
    const BinaryRow* row = find_row(kBinary, op);
    if (!row || !binary_has(row, CUMO_HIP_DFLOAT, true)) return no_method(op);
    int code = -1;
    if (!std::strcmp(op, "add")) code = 0;
    else if (!std::strcmp(op, "sub")) code = 1;
    else if (!std::strcmp(op, "mul")) code = 2;
    else if (!std::strcmp(op, "div")) code = 3;
    static const bool off = [] {
        const char* e = std::getenv("CUMO_HIP_MIXED_ONE_LAUNCH");
        return e && e[0] == '0';
    }();
    const size_t n = total_of(x);
    if (code >= 0 && !off && z && x->ndim >= 1 && n > 0 && is_contiguous(x) && (((uintptr_t)(x->ptr + x->offset)) & 15u) == 0) {
        const bool fresh = z->ptr == NULL;
        bool fits = true;
        if (!fresh) {
            fits = z->type == CUMO_HIP_DFLOAT && z->ndim == x->ndim && is_contiguous(z) && (((uintptr_t)(z->ptr + z->offset)) & 15u) == 0;
            for (int d = 0; fits && d < x->ndim; d++) fits = z->shape[d] == x->shape[d];
        } else {
            rc = cumo_hip_na_alloc(z, CUMO_HIP_DFLOAT, x->ndim, x->shape);
            if (rc) return rc;
        }
        if (fits) {
            if (cumo_hip::mixed_flat_binary_s(code, x->ptr + x->offset, sv, scalar_is_left != 0, z->ptr + z->offset, n)) return CUMO_HIP_OK;
            if (fresh) {
                cumo_cuda_runtime_free(z->ptr);
                z->ptr = NULL;
            }
        }
    }
    NA tx;
    const NA* ux;
    rc = cast_operand(x, CUMO_HIP_DFLOAT, &tx, &ux);
    if (!rc) rc = cumo_hip_na_binary_s(op, ux, sv, scalar_is_left, z);
    free_tmp(&tx);
    return rc;
}

// x ** y for two arrays (gen/tmpl/pow.c:117-190,200-215): the result has the higher
// type of the two; an Int32 exponent array takes the repeated-product form.
int cumo_hip_na_pow(const cumo_hip_narray_t* x, const cumo_hip_narray_t* y, cumo_hip_narray_t* z) {
    int rc = check_arith(x);
    if (!rc) rc = check_arith(y);
    if (rc) return rc;
    const int up = upcast(x->type, y->type);
    NA tx, ty;
    const NA *ux, *uy;
    ty.ptr = NULL;
    rc = cast_operand(x, up, &tx, &ux);
    Arr3Fn f;
    if (y->type == CUMO_HIP_INT32) {
        uy = y;
        f = kPow[up].pow_int32;
    } else {
        if (!rc) rc = cast_operand(y, up, &ty, &uy);
        f = kPow[up].pow;
    }
    if (!rc) {
        cumo_hip_ndfunc_t nf = {iter_arr3, 0, 2, 1, {up, 0}};
        const NA* in[2] = {ux, uy};
        NA* out[1] = {z};
        rc = cumo_hip_na_ndloop(&nf, in, out, 0, (void*)f);
    }
    free_tmp(&tx);
    free_tmp(&ty);
    return rc;
}

// x ** sv, or sv ** x when scalar_is_left. An integer sv takes the Int32 form as a
// Ruby Integer does (gen/tmpl/pow.c:160-175); a non-integer base over an Int32 array
// answers DFloat, the class a Ruby Float upcasts to.
int cumo_hip_na_pow_s(const cumo_hip_narray_t* x, double sv, int sv_is_integer, int scalar_is_left, cumo_hip_narray_t* z) {
    int rc = check_arith(x);
    if (rc) return rc;
    PowSOpt opt = {x->type, 0, sv};
    int out_type = x->type;
    if (!scalar_is_left) {
        if (sv_is_integer) opt.form = 2;
        else if (x->type == CUMO_HIP_INT32) return fail(CUMO_HIP_ERROR_TYPE, "Int32 ** Float: cast the array to DFloat first");
        else opt.form = 0;
    } else if (x->type == CUMO_HIP_INT32) {
        opt.form = 3;
        if (!sv_is_integer) {
            opt.type = CUMO_HIP_DFLOAT;
            out_type = CUMO_HIP_DFLOAT;
        }
    } else {
        opt.form = 1;
    }
    cumo_hip_ndfunc_t nf = {iter_pow_s, 0, 1, 1, {out_type, 0}};
    const NA* in[1] = {x};
    NA* out[1] = {z};
    return cumo_hip_na_ndloop(&nf, in, out, 0, &opt);
}

// Cumo::<T>.maximum / minimum (gen/tmpl/ewcomp.c:40-75)
int cumo_hip_na_ewcomp(const char* op, const cumo_hip_narray_t* x, const cumo_hip_narray_t* y, int nan, cumo_hip_narray_t* z) {
    int rc = check_arith(x);
    if (!rc) rc = check_arith(y);
    if (rc) return rc;
    const EwcompRow* row = find_row(kEwcomp, op);
    const int up = upcast(x->type, y->type);
    if (!row) return no_method(op);
    Arr3Fn f = (nan && is_float(up)) ? row->fnan[up] : row->f[up];
    NA tx, ty;
    const NA *ux, *uy;
    ty.ptr = NULL;
    rc = cast_operand(x, up, &tx, &ux);
    if (!rc) rc = cast_operand(y, up, &ty, &uy);
    if (!rc) {
        cumo_hip_ndfunc_t nf = {iter_arr3, 0, 2, 1, {up, 0}};
        const NA* in[2] = {ux, uy};
        NA* out[1] = {z};
        rc = cumo_hip_na_ndloop(&nf, in, out, 0, (void*)f);
    }
    free_tmp(&tx);
    free_tmp(&ty);
    return rc;
}

// x.clip(min, max) (gen/tmpl/clip.c:199-254). lo_kind / hi_kind: 0 absent, 1 the
// scalar, 2 the array. The result has x's type; array bounds are cast to it, and a
// scalar bound beside an array bound becomes a 0-dimensional array, as there.
int cumo_hip_na_clip(const cumo_hip_narray_t* x, int lo_kind, double lo_s, const cumo_hip_narray_t* lo_a, int hi_kind,
                     double hi_s, const cumo_hip_narray_t* hi_a, cumo_hip_narray_t* z) {
    int rc = check_arith(x);
    if (rc) return rc;
    if (lo_kind == 0 && hi_kind == 0) return fail(CUMO_HIP_ERROR_ARGUMENT, "min and max are not given");
    const int t = x->type;
    ClipOpt opt = {t, 0, lo_s, hi_s, false};
    NA* out[1] = {z};
    if (lo_kind != 2 && hi_kind != 2) {
        if (lo_kind == 1 && hi_kind == 1) {
            // compared in the element type, as the caller there does after m_num_to_data
            bool bad;
            if (t == CUMO_HIP_SFLOAT) bad = (float)lo_s > (float)hi_s;
            else if (t == CUMO_HIP_DFLOAT) bad = lo_s > hi_s;
            else bad = (int32_t)lo_s > (int32_t)hi_s;
            if (bad) return fail(CUMO_HIP_ERROR_OPERATION, "min is greater than max");
            opt.form = 0;
        } else {
            opt.form = lo_kind == 1 ? 1 : 2;
        }
        cumo_hip_ndfunc_t nf = {iter_clip, 0, 1, 1, {t, 0}};
        const NA* in[1] = {x};
        return cumo_hip_na_ndloop(&nf, in, out, 0, &opt);
    }
    NA tlo, thi;
    tlo.ptr = thi.ptr = NULL;
    const NA *ulo = NULL, *uhi = NULL;
    if (lo_kind == 2) {
        rc = check_arith(lo_a);
        if (!rc) rc = cast_operand(lo_a, t, &tlo, &ulo);
    } else if (lo_kind == 1) {
        rc = cumo_hip_na_alloc(&tlo, t, 0, NULL);
        if (!rc) rc = cumo_hip_na_fill(&tlo, lo_s);
        ulo = &tlo;
    }
    if (!rc) {
        if (hi_kind == 2) {
            rc = check_arith(hi_a);
            if (!rc) rc = cast_operand(hi_a, t, &thi, &uhi);
        } else if (hi_kind == 1) {
            rc = cumo_hip_na_alloc(&thi, t, 0, NULL);
            if (!rc) rc = cumo_hip_na_fill(&thi, hi_s);
            uhi = &thi;
        }
    }
    if (!rc) {
        if (ulo && uhi) {
            opt.form = 5;
            cumo_hip_ndfunc_t nf = {iter_clip, 0, 3, 1, {t, 0}};
            const NA* in[3] = {x, ulo, uhi};
            rc = cumo_hip_na_ndloop(&nf, in, out, 0, &opt);
        } else {
            opt.form = ulo ? 3 : 4;
            cumo_hip_ndfunc_t nf = {iter_clip, 0, 2, 1, {t, 0}};
            const NA* in[2] = {x, ulo ? ulo : uhi};
            rc = cumo_hip_na_ndloop(&nf, in, out, 0, &opt);
        }
    }
    free_tmp(&tlo);
    free_tmp(&thi);
    if (!rc && opt.flagged) return fail(CUMO_HIP_ERROR_OPERATION, "min is greater than max");
    return rc;
}

// x.mulsum(y, axis:, keepdims:, nan:) (gen/tmpl/accum_binary.c:62-110): the sum of the
// products over the reduced dimensions, started from 0. With more inner runs than
// is sensible to launch one by one, the products go through an array of their own
// and the reduction engine (for nan: true that skips a product that is NaN though
// neither factor is, inf * 0, where the run launcher would add it).
int cumo_hip_na_mulsum(const cumo_hip_narray_t* x, const cumo_hip_narray_t* y, unsigned int reduce, int keepdims, int nan,
                       cumo_hip_narray_t* z) {
    int rc = check_arith(x);
    if (!rc) rc = check_arith(y);
    if (rc) return rc;
    const int up = upcast(x->type, y->type);
    const int nd = x->ndim > y->ndim ? x->ndim : y->ndim;
    if (reduce == 0) reduce = nd ? ((1u << nd) - 1u) : 0u;
    NA tx, ty;
    const NA *ux, *uy;
    ty.ptr = NULL;
    rc = cast_operand(x, up, &tx, &ux);
    if (!rc) rc = cast_operand(y, up, &ty, &uy);
    if (!rc) {
        cumo_hip_ndfunc_t nf = {NULL, CUMO_HIP_NDF_FLAT_REDUCE | (keepdims ? CUMO_HIP_NDF_KEEP_DIM : 0u), 2, 1, {up, 0}};
        const NA* in[2] = {ux, uy};
        NA* out[1] = {z};
        LP lp;
        const bool fresh = z->ptr == NULL;
        rc = cumo_hip_na_ndloop_prepare(&nf, in, out, reduce, &lp);
        size_t launches = 1, total = 1;
        for (int d = 0; !rc && d < lp.ndim; ++d) {
            total *= lp.n[d];
            if (d < lp.ndim - 1) launches *= lp.n[d];
        }
        // many short contiguous runs: every row in one launch
        bool rows_done = false;
        if (!rc && total_of(z) != 0 && total != 0 && lp.ndim == 2 && lp.args[2].step[1] == 0 && launches >= 2 &&
            (launches > 1024 || lp.n[1] * (size_t)kElmsz[up] <= (1u << 20)) && lp.args[0].step[1] == (ssize_t)kElmsz[up] &&
            lp.args[1].step[1] == (ssize_t)kElmsz[up]) {
            rc = cumo_hip_na_fill(z, 0.0);
            if (!rc) {
                cumo_hip_mulsum_rows_t g = {lp.n[0], lp.n[1], lp.args[0].step[0], lp.args[1].step[0], lp.args[2].step[0],
                                            lp.args[0].ptr, lp.args[1].ptr, lp.args[2].ptr};
                const int t = up == CUMO_HIP_SFLOAT ? 0 : (up == CUMO_HIP_DFLOAT ? 1 : 2);
                rows_done = cumo_hip_mulsum_rows_kernel_launch(t, nan != 0 && is_float(up), &g) == 1;
            }
        }
        if (!rc && total_of(z) != 0 && !rows_done) {
            if (launches <= 1024 || total == 0) {
                rc = cumo_hip_na_fill(z, 0.0);
                if (!rc && total != 0) {
                    MulsumOpt opt = {up, nan != 0 && is_float(up)};
                    mulsum_walk(&lp, 0, lp.args[0].ptr, lp.args[1].ptr, lp.args[2].ptr, &opt);
                }
            } else {
                NA prod;
                prod.ptr = NULL;
                rc = cumo_hip_na_binary("mul", ux, uy, &prod);
                if (!rc) {
                    // the product has the broadcast shape, so the same dimensions are reduced
                    NA zs = *z;
                    NA sum64;
                    sum64.ptr = NULL;
                    if (up == CUMO_HIP_INT32) {
                        // Int32#sum answers Int64; mulsum stays Int32 (wrapping), so narrow it
                        rc = cumo_hip_na_reduce("sum", &prod, reduce, keepdims, 0, &sum64, NULL);
                        if (!rc) rc = cumo_hip_na_store(&zs, &sum64);
                        free_tmp(&sum64);
                    } else {
                        rc = cumo_hip_na_reduce("sum", &prod, reduce, keepdims, nan && is_float(up), &zs, NULL);
                    }
                }
                free_tmp(&prod);
            }
        }
        if (rc && fresh) free_tmp(z);
    }
    free_tmp(&tx);
    free_tmp(&ty);
    return rc;
}

// x.cumsum / x.cumprod (axis:, nan:) (gen/tmpl/cum.c:48-80): the running sum or
// product along the given dimensions taken together in row-major order (all of them
// when reduce is 0); the result has x's shape and type.
int cumo_hip_na_cum(const char* op, const cumo_hip_narray_t* x, unsigned int reduce, int nan, cumo_hip_narray_t* z) {
    int rc = check_arith(x);
    if (rc) return rc;
    int prod;
    if (op && !std::strcmp(op, "cumsum")) prod = 0;
    else if (op && !std::strcmp(op, "cumprod")) prod = 1;
    else return no_method(op);
    const int nd = x->ndim;
    if (nd < 32 && (reduce >> nd)) return fail(CUMO_HIP_ERROR_DIMENSION, "dimension is out of range");
    if (reduce == 0) reduce = nd ? ((1u << nd) - 1u) : 0u;
    const bool fresh = z->ptr == NULL;
    if (fresh) {
        rc = cumo_hip_na_alloc(z, x->type, nd, x->shape);
        if (rc) return rc;
    } else {
        rc = check_view(z, "result");
        if (rc) return rc;
        bool same = z->type == x->type && z->ndim == nd;
        for (int d = 0; same && d < nd; ++d) same = z->shape[d] == x->shape[d];
        if (!same) return fail(CUMO_HIP_ERROR_SHAPE, "cum: result array has the wrong shape or type");
    }
    if (total_of(x) == 0) return CUMO_HIP_OK;
    const ssize_t es = kElmsz[x->type];

    // the scanned dimensions as one run: each walks its successor's whole extent
    bool one_run = true;
    ssize_t s_in = es, s_out = es;
    size_t n = 1;
    {
        bool first = true;
        for (int d = nd - 1; d >= 0; --d) {
            if (!((reduce >> d) & 1u) || x->shape[d] == 1) continue;
            if (first) {
                s_in = x->stride[d];
                s_out = z->stride[d];
                first = false;
            } else if (x->stride[d] != s_in * (ssize_t)n || z->stride[d] != s_out * (ssize_t)n) {
                one_run = false;
            }
            n *= x->shape[d];
        }
    }
    const NA* src = x;
    NA* dst = z;
    NA tx, tz, zperm;
    tx.ptr = tz.ptr = NULL;
    unsigned int red = reduce;
    if (!one_run) {
        // bring the scanned dimensions together at the end of a contiguous copy, scan
        // that into a contiguous result, and store it back through the same permutation
        NA xperm = *x;
        zperm = *z;
        int k = 0;
        for (int pass = 0; pass < 2; ++pass)
            for (int d = 0; d < nd; ++d)
                if ((((reduce >> d) & 1u) != 0) == (pass == 1)) {
                    xperm.shape[k] = x->shape[d];
                    xperm.stride[k] = x->stride[d];
                    zperm.shape[k] = z->shape[d];
                    zperm.stride[k] = z->stride[d];
                    ++k;
                }
        int nred = 0;
        for (int d = 0; d < nd; ++d) nred += (reduce >> d) & 1u;
        red = ((1u << nred) - 1u) << (nd - nred);
        rc = cumo_hip_na_copy(&xperm, &tx);
        if (!rc) rc = cumo_hip_na_alloc(&tz, x->type, nd, xperm.shape);
        if (rc) {
            free_tmp(&tx);
            if (fresh) free_tmp(z);
            return rc;
        }
        src = &tx;
        dst = &tz;
        n = 1;
        for (int d = nd - nred; d < nd; ++d) n *= src->shape[d];
        s_in = s_out = es;
    }
    cumo_hip_scan_rows_t runs;
    std::memset(&runs, 0, sizeof(runs));
    runs.rows = 1;
    for (int d = 0; d < nd; ++d) {
        if (((red >> d) & 1u) || src->shape[d] == 1) continue;
        runs.oshape[runs.nouter] = src->shape[d];
        runs.ostep_in[runs.nouter] = src->stride[d];
        runs.ostep_out[runs.nouter] = dst->stride[d];
        runs.rows *= src->shape[d];
        ++runs.nouter;
    }
    runs.n = n;
    runs.s_in = s_in;
    runs.s_out = s_out;
    runs.in = src->ptr + src->offset;
    runs.out = dst->ptr + dst->offset;
    const bool use_nan = nan && is_float(x->type);
    if (runs.rows == 1 && n > (1u << 16)) {
        // one long run: the three-launch form
        typedef int (*RunFn)(char*, char*, ssize_t, ssize_t, uint64_t);
        static const RunFn fns[3][4] = {
            {cumo_sfloat_cumsum_kernel_launch, cumo_sfloat_cumsum_nan_kernel_launch, cumo_sfloat_cumprod_kernel_launch, cumo_sfloat_cumprod_nan_kernel_launch},
            {cumo_dfloat_cumsum_kernel_launch, cumo_dfloat_cumsum_nan_kernel_launch, cumo_dfloat_cumprod_kernel_launch, cumo_dfloat_cumprod_nan_kernel_launch},
            {cumo_int32_cumsum_kernel_launch, cumo_int32_cumsum_kernel_launch, cumo_int32_cumprod_kernel_launch, cumo_int32_cumprod_kernel_launch},
        };
        const int st = fns[x->type][prod * 2 + (use_nan ? 1 : 0)](runs.in, runs.out, s_in, s_out, n);
        if (st != 0) {
            cumo_hip::report_hip_error((hipError_t)st, "cumsum/cumprod launch");
            rc = CUMO_HIP_ERROR_RUNTIME;
        }
    } else if (runs.nouter > 0 && s_in != es && runs.ostep_in[runs.nouter - 1] == es && runs.ostep_out[runs.nouter - 1] == es &&
               runs.oshape[runs.nouter - 1] >= 16) {
        // the runs lie across memory: lanes along the contiguous dimension
        const uint64_t cols = runs.oshape[runs.nouter - 1];
        --runs.nouter;
        runs.rows /= cols;
        cumo_hip_scan_cols_kernel_launch(x->type, prod, use_nan ? 1 : 0, &runs, cols);
    } else {
        cumo_hip_scan_rows_kernel_launch(x->type, prod, use_nan ? 1 : 0, &runs);
    }
    if (!rc && !one_run) rc = cumo_hip_na_store(&zperm, &tz);
    free_tmp(&tx);
    free_tmp(&tz);
    if (rc && fresh) free_tmp(z);
    return rc;
}

// softmax / layernorm along the last dimension (library additions). One fused launch
// when the rows are contiguous and fit the row kernels; otherwise the chain of array
// operations a Cumo program would write (bench/transformer_bench.rb:110-124), whose
// results the fused launch matches up to the order of the two row sums.
static int fused_rows(int mode, const cumo_hip_narray_t* x, double eps, cumo_hip_narray_t* z) {
    int rc = check_view(x, "operand");
    if (rc) return rc;
    if (!is_float(x->type)) return fail(CUMO_HIP_ERROR_TYPE, "softmax / layernorm: operand is not SFloat or DFloat");
    if (x->ndim < 1) return fail(CUMO_HIP_ERROR_DIMENSION, "softmax / layernorm need at least one dimension");
    const int nd = x->ndim;
    const size_t n = x->shape[nd - 1];
    const ssize_t es = kElmsz[x->type];
    const bool fresh = z->ptr == NULL;
    if (fresh) {
        rc = cumo_hip_na_alloc(z, x->type, nd, x->shape);
        if (rc) return rc;
    } else {
        rc = check_view(z, "result");
        if (rc) return rc;
        bool same = z->type == x->type && z->ndim == nd;
        for (int d = 0; same && d < nd; ++d) same = z->shape[d] == x->shape[d];
        if (!same) return fail(CUMO_HIP_ERROR_SHAPE, "softmax / layernorm: result array has the wrong shape or type");
    }
    if (total_of(x) == 0) return CUMO_HIP_OK;
    // rows as one uniform step: the outer dimensions of both arrays merge into one
    bool rows_ok = (n == 1 || (x->stride[nd - 1] == es && z->stride[nd - 1] == es));
    size_t rows = 1;
    ssize_t xs = 0, zs = 0;
    {
        bool first = true;
        for (int d = nd - 2; d >= 0 && rows_ok; --d) {
            if (x->shape[d] == 1) continue;
            if (first) {
                xs = x->stride[d];
                zs = z->stride[d];
                first = false;
            } else if (x->stride[d] != xs * (ssize_t)rows || z->stride[d] != zs * (ssize_t)rows) {
                rows_ok = false;
            }
            rows *= x->shape[d];
        }
    }
    if (rows_ok) {
        cumo_hip_fused_rows_t d;
        d.rows = rows;
        d.n = n;
        d.in_row_step = xs;
        d.out_row_step = zs;
        d.in = x->ptr + x->offset;
        d.out = z->ptr + z->offset;
        d.eps = eps;
        if (cumo_hip_fused_rows_kernel_launch(x->type, mode, &d)) return CUMO_HIP_OK;
    }
    // the chain
    const unsigned last = 1u << (nd - 1);
    NA a, b, c, e;
    a.ptr = b.ptr = c.ptr = e.ptr = NULL;
    if (mode == 0) {
        rc = cumo_hip_na_reduce("max", x, last, 1, 0, &a, NULL);
        if (!rc) rc = cumo_hip_na_binary("sub", x, &a, &b);
        if (!rc) rc = cumo_hip_na_math("exp", &b, &c);
        if (!rc) rc = cumo_hip_na_reduce("sum", &c, last, 1, 0, &e, NULL);
        if (!rc) rc = cumo_hip_na_binary("div", &c, &e, z);
    } else {
        NA v2, sd;
        v2.ptr = sd.ptr = NULL;
        rc = cumo_hip_na_reduce("mean", x, last, 1, 0, &a, NULL);
        if (!rc) rc = cumo_hip_na_reduce("var", x, last, 1, 0, &b, NULL);
        if (!rc) rc = cumo_hip_na_binary("sub", x, &a, &c);
        if (!rc) rc = cumo_hip_na_binary_s("add", &b, eps, 0, &v2);
        if (!rc) rc = cumo_hip_na_math("sqrt", &v2, &sd);
        if (!rc) rc = cumo_hip_na_binary("div", &c, &sd, z);
        free_tmp(&v2);
        free_tmp(&sd);
    }
    free_tmp(&a);
    free_tmp(&b);
    free_tmp(&c);
    free_tmp(&e);
    if (rc && fresh) free_tmp(z);
    return rc;
}

int cumo_hip_na_softmax(const cumo_hip_narray_t* x, cumo_hip_narray_t* z) { return fused_rows(0, x, 0.0, z); }
int cumo_hip_na_layernorm(const cumo_hip_narray_t* x, double eps, cumo_hip_narray_t* z) { return fused_rows(1, x, eps, z); }

// ---- Bit#where, Bit#mask (gen/tmpl_bit/where.c:98-127, mask.c:96-167) --------------
namespace {
struct WhereWalk {
    char* out;
    size_t elmsz;
    char* scratch;
    int invert;
    uint64_t count;
};
void where_walk(const LP* lp, int level, size_t pos, WhereWalk* w) {
    const cumo_hip_loop_args_t& in = lp->args[0];
    if (level == lp->ndim - 1) {
        cumo_bit_where_kernel_launch((CUMO_BIT_DIGIT*)in.ptr, pos, in.step[level], NULL, lp->n[level], w->invert, w->out, w->elmsz, w->count, w->scratch);
        w->count += lp->n[level];
        return;
    }
    for (size_t i = 0; i < lp->n[level]; i++) where_walk(lp, level + 1, pos + (size_t)((ssize_t)i * in.step[level]), w);
}
// the 1-D result of where / mask: allocated here, or a caller's array that must be
// exactly as long as the count turns out to be
int result_1d(NA* z, int type, size_t n, bool* allocated) {
    *allocated = false;
    if (!z->ptr) {
        size_t shape1[1] = {n};
        *allocated = true;
        return cumo_hip_na_alloc(z, type, 1, shape1);
    }
    if (z->type != type || z->ndim != 1 || z->shape[0] != n || (n > 1 && z->stride[0] != (ssize_t)kElmsz[type]))
        return fail(CUMO_HIP_ERROR_SHAPE, "the given result must be a contiguous 1-D array of the result's type and exact length");
    return 0;
}
// A mask that walks as one run: its hits are counted block by block, the counts read back
// (the one stream synchronisation) and added up here to size the result, and the same
// counts then place the hits: positions (x == NULL, as itype) or the elements of the run
// (x, sx) of xtype.
int where_single_run(const LP& lp, int invert, int rtype, const char* x, ssize_t sx, NA* z) {
    const cumo_hip_loop_args_t& in = lp.args[0];
    const uint64_t n = lp.n[0];
    const size_t nb = cumo_hip_bit_where_blocks(n);
    uint64_t host_counts[1024];
    if (nb > sizeof(host_counts) / sizeof(host_counts[0])) return fail(CUMO_HIP_ERROR_ARGUMENT, "where: more block counts than expected");
    uint64_t* counts = reinterpret_cast<uint64_t*>(cumo_cuda_runtime_malloc(nb * sizeof(uint64_t)));
    if (!counts) return CUMO_HIP_ERROR_OUT_OF_MEMORY;
    int rc = cumo_hip_bit_where_count_to_host((CUMO_BIT_DIGIT*)in.ptr, in.bitpos, in.step[0], n, invert, counts, host_counts);
    uint64_t n_hit = 0;
    for (size_t b = 0; b < nb; ++b) n_hit += host_counts[b];
    bool allocated = false;
    if (!rc) rc = result_1d(z, rtype, (size_t)n_hit, &allocated);
    if (!rc && n_hit != 0)
        cumo_hip_bit_where_place_kernel_launch((CUMO_BIT_DIGIT*)in.ptr, in.bitpos, in.step[0], n, invert, counts, x, sx, (size_t)kElmsz[rtype],
                                               z->ptr + z->offset);
    cumo_cuda_runtime_free(reinterpret_cast<char*>(counts));
    return rc;
}
}  // namespace

// z = positions (row-major, from 0) of the set bits of x, or of the clear ones when
// invert; Int32, or Int64 for an array of more than 2^32 - 1 elements. The count is
// read back once to size the result (one stream synchronisation, as where.c:13-28).
int cumo_hip_na_where(const cumo_hip_narray_t* x, int invert, cumo_hip_narray_t* z) {
    int rc = check_view(x, "operand");
    if (rc) return rc;
    if (x->type != CUMO_HIP_BIT) return no_method("where");
    if (!z) return fail(CUMO_HIP_ERROR_ARGUMENT, "where: no result descriptor");
    if (total_of(x) != 0) {
        cumo_hip_ndfunc_t nf1 = {NULL, 0, 1, 0, {0, 0}};
        const NA* in1[1] = {x};
        LP lp1;
        if (cumo_hip_na_ndloop_prepare(&nf1, in1, NULL, 0, &lp1) == CUMO_HIP_OK && lp1.ndim == 1)
            return where_single_run(lp1, invert ? 1 : 0, total_of(x) > 4294967295ull ? CUMO_HIP_INT64 : CUMO_HIP_INT32, NULL, 0, z);
    }
    NA cnt;
    cnt.ptr = NULL;
    rc = cumo_hip_na_bit_count(x, 0, 0, invert, &cnt);
    if (rc) return rc;
    uint64_t n_hit = 0;
    rc = cumo_hip_copy_to_host(&n_hit, cnt.ptr + cnt.offset, sizeof(n_hit));
    if (rc) {
        free_tmp(&cnt);
        return rc;
    }
    free_tmp(&cnt);
    const size_t total = total_of(x);
    const int itype = total > 4294967295ull ? CUMO_HIP_INT64 : CUMO_HIP_INT32;
    bool allocated;
    rc = result_1d(z, itype, (size_t)n_hit, &allocated);
    if (rc || n_hit == 0) return rc;
    cumo_hip_ndfunc_t nf = {NULL, 0, 1, 0, {0, 0}};
    const NA* in[1] = {x};
    LP lp;
    rc = cumo_hip_na_ndloop_prepare(&nf, in, NULL, 0, &lp);
    if (!rc) {
        WhereWalk w = {z->ptr + z->offset, (size_t)kElmsz[itype], cumo_bit_where_scratch_new(), invert ? 1 : 0, 0};
        if (!w.scratch) {
            rc = CUMO_HIP_ERROR_OUT_OF_MEMORY;
        } else {
            where_walk(&lp, 0, lp.args[0].bitpos, &w);
            cumo_cuda_runtime_free(w.scratch);
        }
    }
    if (rc && allocated) free_tmp(z);
    return rc;
}

// z = the elements of x where mask is set, in row-major order (mask.c:96-167 returns
// a view over an index array; here the elements are gathered into a new array).
int cumo_hip_na_mask(const cumo_hip_narray_t* mask, const cumo_hip_narray_t* x, cumo_hip_narray_t* z) {
    int rc = check_view(mask, "mask");
    if (!rc) rc = check_view(x, "operand");
    if (rc) return rc;
    if (mask->type != CUMO_HIP_BIT) return no_method("mask");
    if (x->type == CUMO_HIP_BIT) return fail(CUMO_HIP_ERROR_TYPE, "mask: a Bit array cannot be the masked array here");
    bool same = mask->ndim == x->ndim;
    for (int d = 0; same && d < x->ndim; ++d) same = mask->shape[d] == x->shape[d];
    if (!same) return fail(CUMO_HIP_ERROR_SHAPE, "mask and masked arrays must have the same shape");
    if (!z) return fail(CUMO_HIP_ERROR_ARGUMENT, "mask: no result descriptor");
    // mask and masked array walk as one run each (both contiguous, or sliced alike): the
    // elements are compacted directly, without the array of positions in between
    if (total_of(x) != 0) {
        cumo_hip_ndfunc_t nf = {NULL, 0, 2, 0, {0, 0}};
        const NA* in[2] = {mask, x};
        LP lp;
        if (cumo_hip_na_ndloop_prepare(&nf, in, NULL, 0, &lp) == CUMO_HIP_OK && lp.ndim == 1) {
            return where_single_run(lp, 0, x->type, lp.args[1].ptr, lp.args[1].step[0], z);
        }
    }
    NA pos;
    pos.ptr = NULL;
    rc = cumo_hip_na_where(mask, 0, &pos);
    if (rc) return rc;
    bool allocated;
    rc = result_1d(z, x->type, pos.shape[0], &allocated);
    if (!rc && pos.shape[0] != 0) {
        cumo_hip_gather_flat_t g;
        std::memset(&g, 0, sizeof(g));
        g.ndim = x->ndim;
        g.n = pos.shape[0];
        for (int d = 0; d < x->ndim; ++d) {
            g.shape[d] = x->shape[d];
            g.step[d] = x->stride[d];
        }
        g.in = x->ptr + x->offset;
        g.out = z->ptr + z->offset;
        g.pos = pos.ptr;
        g.pos_elmsz = kElmsz[pos.type];
        g.elmsz = kElmsz[x->type];
        cumo_hip_gather_flat_kernel_launch(&g);
    }
    free_tmp(&pos);
    return rc;
}

int cumo_hip_na_unary(const char* op, const cumo_hip_narray_t* x, cumo_hip_narray_t* z) {
    int rc = check_arith(x);
    if (rc) return rc;
    const UnaryRow* row = find_row(kUnary, op);
    if (!row || !row->f[x->type]) return no_method(op);
    const bool is_abs = !std::strcmp(op, "abs");
    UnaryOpt opt = {row->f[x->type], x->type == CUMO_HIP_INT32 && (is_abs || !std::strcmp(op, "reciprocal")), false};
    cumo_hip_ndfunc_t nf = {iter_unary, 0, 1, 1, {x->type, 0}};
    const NA* in[1] = {x};
    NA* out[1] = {z};
    rc = cumo_hip_na_ndloop(&nf, in, out, 0, &opt);
    if (!rc && opt.flagged)
        return is_abs ? fail(CUMO_HIP_ERROR_VALUE, "error in NArray operation") : fail(CUMO_HIP_ERROR_ZERO_DIVISION, "error in NArray operation");
    return rc;
}

int cumo_hip_na_math(const char* op, const cumo_hip_narray_t* x, cumo_hip_narray_t* z) {
    int rc = check_arith(x);
    if (rc) return rc;
    const MathRow* row = find_row(kMath, op);
    if (!row) return no_method(op);
    // an Int32 argument is computed in DFloat (narray/math.c:60-110 picks the math module by upcast)
    const int type = is_float(x->type) ? x->type : CUMO_HIP_DFLOAT;
    NA tx;
    const NA* ux;
    rc = cast_operand(x, type, &tx, &ux);
    if (!rc) {
        cumo_hip_ndfunc_t nf = {iter_math, 0, 1, 1, {type, 0}};
        const NA* in[1] = {ux};
        NA* out[1] = {z};
        rc = cumo_hip_na_ndloop(&nf, in, out, 0, (void*)row->f[type]);
    }
    free_tmp(&tx);
    return rc;
}

int cumo_hip_na_math2(const char* op, const cumo_hip_narray_t* x, const cumo_hip_narray_t* y, cumo_hip_narray_t* z) {
    int rc = check_arith(x);
    if (!rc) rc = check_arith(y);
    if (rc) return rc;
    const Math2Row* row = find_row(kMath2, op);
    if (!row) return no_method(op);
    int up = upcast(x->type, y->type);
    if (!is_float(up)) up = CUMO_HIP_DFLOAT;
    NA tx, ty;
    const NA *ux, *uy;
    rc = cast_operand(x, up, &tx, &ux);
    if (!rc) rc = cast_operand(y, up, &ty, &uy);
    else ty.ptr = NULL;
    if (!rc) {
        Math2Opt opt = {row, up, false, 0.0, 0};
        cumo_hip_ndfunc_t nf = {iter_math2, 0, 2, 1, {up, 0}};
        const NA* in[2] = {ux, uy};
        NA* out[1] = {z};
        rc = cumo_hip_na_ndloop(&nf, in, out, 0, &opt);
    }
    free_tmp(&tx);
    free_tmp(&ty);
    return rc;
}

int cumo_hip_na_math2_s(const char* op, const cumo_hip_narray_t* x, double sv, int scalar_is_left, cumo_hip_narray_t* z) {
    int rc = check_arith(x);
    if (rc) return rc;
    const Math2Row* row = find_row(kMath2, op);
    if (!row) return no_method(op);
    const int type = is_float(x->type) ? x->type : CUMO_HIP_DFLOAT;
    NA tx;
    const NA* ux;
    rc = cast_operand(x, type, &tx, &ux);
    if (!rc) {
        Math2Opt opt = {row, type, true, sv, scalar_is_left ? 1 : 0};
        cumo_hip_ndfunc_t nf = {iter_math2, 0, 1, 1, {type, 0}};
        const NA* in[1] = {ux};
        NA* out[1] = {z};
        rc = cumo_hip_na_ndloop(&nf, in, out, 0, &opt);
    }
    free_tmp(&tx);
    return rc;
}

namespace {
typedef void (*FrexpFn)(IA*, IA*, IA*, IX*);
void iter_frexp(LP* lp) {
    IA a1, a2, a3;
    IX ix;
    cumo_hip_make_indexer(lp, &ix);
    cumo_hip_make_iarray(lp, 0, &a1);
    cumo_hip_make_iarray(lp, 1, &a2);
    cumo_hip_make_iarray(lp, 2, &a3);
    ((FrexpFn)lp->opt_ptr)(&a1, &a2, &a3, &ix);
}
}  // namespace

namespace {
struct DivmodOpt {
    int type;
    bool flagged;
};
void iter_divmod(LP* lp) {
    IA a1, a2, a3, a4;
    IX ix;
    cumo_hip_make_indexer(lp, &ix);
    cumo_hip_make_iarray(lp, 0, &a1);
    cumo_hip_make_iarray(lp, 1, &a2);
    cumo_hip_make_iarray(lp, 2, &a3);
    cumo_hip_make_iarray(lp, 3, &a4);
    DivmodOpt* o = (DivmodOpt*)lp->opt_ptr;
    if (o->type == CUMO_HIP_INT32) {
        int* flag = cumo_cuda_runtime_error_flag_new();
        cumo_iter_int32_divmod_kernel_launch(&a1, &a2, &a3, &a4, &ix, flag);
        if (flag && cumo_cuda_runtime_error_flag_get(flag)) o->flagged = true;
    } else if (o->type == CUMO_HIP_SFLOAT) {
        cumo_iter_sfloat_divmod_kernel_launch(&a1, &a2, &a3, &a4, &ix, NULL);
    } else {
        cumo_iter_dfloat_divmod_kernel_launch(&a1, &a2, &a3, &a4, &ix, NULL);
    }
}
}  // namespace

int cumo_hip_na_divmod(const cumo_hip_narray_t* x, const cumo_hip_narray_t* y, cumo_hip_narray_t* quot, cumo_hip_narray_t* rem) {
    int rc = check_arith(x);
    if (!rc) rc = check_arith(y);
    if (rc) return rc;
    if (!quot || !rem) return fail(CUMO_HIP_ERROR_ARGUMENT, "divmod: two result descriptors are needed");
    const int up = upcast(x->type, y->type);
    NA tx, ty;
    const NA *ux, *uy;
    rc = cast_operand(x, up, &tx, &ux);
    if (!rc) rc = cast_operand(y, up, &ty, &uy);
    else ty.ptr = NULL;
    DivmodOpt opt = {up, false};
    if (!rc) {
        cumo_hip_ndfunc_t nf = {iter_divmod, 0, 2, 2, {up, up}};
        const NA* in[2] = {ux, uy};
        NA* out[2] = {quot, rem};
        rc = cumo_hip_na_ndloop(&nf, in, out, 0, &opt);
    }
    free_tmp(&tx);
    free_tmp(&ty);
    if (!rc && opt.flagged) return fail(CUMO_HIP_ERROR_ZERO_DIVISION, "error in NArray operation");
    return rc;
}

int cumo_hip_na_modf(const cumo_hip_narray_t* x, cumo_hip_narray_t* frac, cumo_hip_narray_t* whole) {
    int rc = check_arith(x);
    if (rc) return rc;
    if (!is_float(x->type)) return no_method("modf");
    if (!frac || !whole) return fail(CUMO_HIP_ERROR_ARGUMENT, "modf: two result descriptors are needed");
    const FrexpFn f = x->type == CUMO_HIP_SFLOAT ? cumo_iter_sfloat_modf_kernel_launch : cumo_iter_dfloat_modf_kernel_launch;
    cumo_hip_ndfunc_t nf = {iter_frexp, 0, 1, 2, {x->type, x->type}};
    const NA* in[1] = {x};
    NA* out[2] = {frac, whole};
    return cumo_hip_na_ndloop(&nf, in, out, 0, (void*)f);
}

namespace {
constexpr int kPolyMaxScalars = 64;
struct PolyOpt {
    int ncoef;
    const NA* const* coef;
};
void iter_poly(LP* lp) {
    IA ax, az, ac[kPolyMaxScalars];
    IX ix;
    cumo_hip_make_indexer(lp, &ix);
    cumo_hip_make_iarray(lp, 0, &ax);
    cumo_hip_make_iarray(lp, 1, &az);
    const PolyOpt* o = (const PolyOpt*)lp->opt_ptr;
    for (int k = 0; k < o->ncoef; ++k) {
        std::memset(&ac[k], 0, sizeof(IA));  // every step 0: the one element repeats
        ac[k].ptr = o->coef[k]->ptr + o->coef[k]->offset;
    }
    switch (lp->args[0].type) {
        case CUMO_HIP_SFLOAT: cumo_iter_sfloat_poly_kernel_launch(&ax, ac, o->ncoef, &az, &ix); break;
        case CUMO_HIP_DFLOAT: cumo_iter_dfloat_poly_kernel_launch(&ax, ac, o->ncoef, &az, &ix); break;
        default: cumo_iter_int32_poly_kernel_launch(&ax, ac, o->ncoef, &az, &ix); break;
    }
}
}  // namespace

int cumo_hip_na_poly(const cumo_hip_narray_t* x, int ncoef, const cumo_hip_narray_t* const* coef, cumo_hip_narray_t* z) {
    int rc = check_arith(x);
    if (rc) return rc;
    if (!z || ncoef < 0 || (ncoef > 0 && !coef)) return fail(CUMO_HIP_ERROR_ARGUMENT, "poly: bad arguments");
    bool scalars = ncoef <= kPolyMaxScalars;
    for (int k = 0; k < ncoef; ++k) {
        rc = check_arith(coef[k]);
        if (rc) return rc;
        if (coef[k]->type != x->type) return fail(CUMO_HIP_ERROR_TYPE, "poly: coefficients must have the array's type");
        if (total_of(coef[k]) != 1) scalars = false;
    }
    if (scalars) {
        PolyOpt opt = {ncoef, coef};
        cumo_hip_ndfunc_t nf = {iter_poly, 0, 1, 1, {x->type, 0}};
        const NA* in[1] = {x};
        NA* out[1] = {z};
        return cumo_hip_na_ndloop(&nf, in, out, 0, &opt);
    }
    if (ncoef == 1) {
        // the constant term alone, spread over the shape x and it make together
        const NA* a0 = coef[0];
        if (!z->ptr) {
            const int nd = x->ndim > a0->ndim ? x->ndim : a0->ndim;
            size_t shape[CUMO_NA_MAX_DIMENSION];
            for (int d = 0; d < nd; ++d) {
                const int dx = d - (nd - x->ndim), da = d - (nd - a0->ndim);
                const size_t nx = dx >= 0 ? x->shape[dx] : 1, na = da >= 0 ? a0->shape[da] : 1;
                if (nx != na && nx != 1 && na != 1) return fail(CUMO_HIP_ERROR_SHAPE, "shape mismatch");
                shape[d] = nx == 1 ? na : nx;
            }
            rc = cumo_hip_na_alloc(z, x->type, nd, shape);
            if (rc) return rc;
            rc = cumo_hip_na_store(z, a0);
            if (rc) free_tmp(z);
            return rc;
        }
        return cumo_hip_na_store(z, a0);
    }
    // Horner as array operations: y = a_n; y = x * y + a_k for k = n-1 .. 0
    NA y, t;
    y.ptr = t.ptr = NULL;
    rc = cumo_hip_na_binary("mul", x, coef[ncoef - 1], &y);
    for (int k = ncoef - 2; k >= 0 && !rc; --k) {
        const bool last = k == 0;
        if (k != ncoef - 2) {
            t.ptr = NULL;
            rc = cumo_hip_na_binary("mul", x, &y, &t);
            free_tmp(&y);
            y = t;
            if (rc) break;
        }
        t.ptr = NULL;
        rc = cumo_hip_na_binary("add", &y, coef[k], last ? z : &t);
        free_tmp(&y);
        if (!last) y = t;
        else y.ptr = NULL;
    }
    if (rc) free_tmp(&y);
    return rc;
}

int cumo_hip_na_frexp(const cumo_hip_narray_t* x, cumo_hip_narray_t* mant, cumo_hip_narray_t* expo) {
    int rc = check_arith(x);
    if (rc) return rc;
    if (!mant || !expo) return fail(CUMO_HIP_ERROR_ARGUMENT, "frexp: two result descriptors are needed");
    const int type = is_float(x->type) ? x->type : CUMO_HIP_DFLOAT;
    NA tx;
    const NA* ux;
    rc = cast_operand(x, type, &tx, &ux);
    if (!rc) {
        const FrexpFn f = type == CUMO_HIP_SFLOAT ? cumo_iter_sfloat_math_s_frexp_kernel_launch : cumo_iter_dfloat_math_s_frexp_kernel_launch;
        cumo_hip_ndfunc_t nf = {iter_frexp, 0, 1, 2, {type, CUMO_HIP_INT32}};
        const NA* in[1] = {ux};
        NA* out[2] = {mant, expo};
        rc = cumo_hip_na_ndloop(&nf, in, out, 0, (void*)f);
    }
    free_tmp(&tx);
    return rc;
}

int cumo_hip_na_compare(const char* op, const cumo_hip_narray_t* x, const cumo_hip_narray_t* y, cumo_hip_narray_t* z) {
    int rc = check_arith(x);
    if (!rc) rc = check_arith(y);
    if (rc) return rc;
    const CondRow* row = find_row(kCond, op);
    const int up = upcast(x->type, y->type);
    if (!row || !cond_has(row, up)) return no_method(op);
    if (x->type != y->type) {
        bool taken = false;
        rc = mixed_compare_one_launch(op, x, y, z, &taken);
        if (taken) return rc;
    }
    NA tx, ty;
    const NA *ux, *uy;
    rc = cast_operand(x, up, &tx, &ux);
    if (!rc) rc = cast_operand(y, up, &ty, &uy);
    else ty.ptr = NULL;
    if (!rc) {
        CondOpt opt = {row, up, false, 0.0, 0};
        cumo_hip_ndfunc_t nf = {iter_cond, 0, 2, 1, {CUMO_HIP_BIT, 0}};
        const NA* in[2] = {ux, uy};
        NA* out[1] = {z};
        rc = cumo_hip_na_ndloop(&nf, in, out, 0, &opt);
    }
    free_tmp(&tx);
    free_tmp(&ty);
    return rc;
}

int cumo_hip_na_compare_s(const char* op, const cumo_hip_narray_t* x, double sv, int scalar_is_left, cumo_hip_narray_t* z) {
    int rc = check_arith(x);
    if (rc) return rc;
    const CondRow* row = find_row(kCond, op);
    if (!row || !cond_has(row, x->type)) return no_method(op);
    CondOpt opt = {row, x->type, true, sv, scalar_is_left ? 1 : 0};
    cumo_hip_ndfunc_t nf = {iter_cond, 0, 1, 1, {CUMO_HIP_BIT, 0}};
    const NA* in[1] = {x};
    NA* out[1] = {z};
    return cumo_hip_na_ndloop(&nf, in, out, 0, &opt);
}

int cumo_hip_na_cond_unary(const char* op, const cumo_hip_narray_t* x, cumo_hip_narray_t* z) {
    int rc = check_arith(x);
    if (rc) return rc;
    const CondUnaryRow* row = find_row(kCondUnary, op);
    if (!row || !is_float(x->type)) return no_method(op);
    cumo_hip_ndfunc_t nf = {iter_cond_unary, 0, 1, 1, {CUMO_HIP_BIT, 0}};
    const NA* in[1] = {x};
    NA* out[1] = {z};
    return cumo_hip_na_ndloop(&nf, in, out, 0, (void*)row->f[x->type]);
}

int cumo_hip_na_store(cumo_hip_narray_t* dst, const cumo_hip_narray_t* src) {
    int rc = check_view(dst, "destination");
    if (!rc) rc = check_view(src, "source");
    if (rc) return rc;
    if (!dst->ptr && total_of(dst)) return fail(CUMO_HIP_ERROR_ARGUMENT, "store: destination has no memory");
    cumo_hip_ndfunc_t nf = {NULL, 0, 2, 0, {0, 0}};
    void* opt = NULL;
    StoreOpt sopt;
    CondOpt copt;
    if (dst->type == CUMO_HIP_BIT && src->type != CUMO_HIP_BIT) {
        if (src->type < 0 || src->type > CUMO_HIP_UINT64) return fail(CUMO_HIP_ERROR_TYPE, "store: unsupported source type");
        nf.func = iter_bit_store_from;  // nonzero is 1 (types/bit_kernel.h:13-19)
        opt = (void*)kBitStoreFrom[src->type];
        // into a whole contiguous Bit array this is the comparison "x != 0", which has the vector kernels
        const CondRow* ne = is_arith(src->type) ? find_row(kCond, "ne") : NULL;
        if (ne && cond_has(ne, src->type) && dst->offset == 0 && is_contiguous(dst)) {
            copt = {ne, src->type, true, 0.0, 0};
            nf.func = iter_cond;  // args: src, dst
            opt = &copt;
        }
    } else if (dst->type == CUMO_HIP_BIT) {
        nf.func = iter_bit_unary;  // args: src, dst
        opt = (void*)&kBitStoreBit;
    } else if (!is_arith(dst->type)) {
        return fail(CUMO_HIP_ERROR_TYPE, "store: destination must be SFloat, DFloat, Int32 or Bit");
    } else if (src->type == CUMO_HIP_BIT) {
        nf.func = iter_store_bit;
        opt = (void*)kStoreBit[dst->type];
    } else if (src->type <= CUMO_HIP_INT64) {
        nf.func = iter_store;
        sopt.f = kStore[dst->type][src->type];
        opt = &sopt;
    } else {
        return fail(CUMO_HIP_ERROR_TYPE, "store: unsupported source type");
    }
    // the loop must have the destination's shape: the source may repeat, the destination may not
    cumo_hip_loop_t lp;
    const NA* in[2] = {dst, src};
    if (nf.func == iter_bit_unary || nf.func == iter_cond) {
        in[0] = src;
        in[1] = dst;
    }
    rc = cumo_hip_na_ndloop_prepare(&nf, in, NULL, 0, &lp);
    if (rc) return rc;
    size_t total = 1, dtotal = total_of(dst);
    for (int d = 0; d < lp.ndim; d++) total *= lp.n[d];
    if (total != dtotal || src->ndim > dst->ndim) return fail(CUMO_HIP_ERROR_SHAPE, "store: source cannot be broadcast to the destination");
    if (total == 0) return CUMO_HIP_OK;
    lp.opt_ptr = opt;
    nf.func(&lp);
    return lp.status;
}

int cumo_hip_na_copy(const cumo_hip_narray_t* src, cumo_hip_narray_t* dst) {
    int rc = check_view(src, "source");
    if (rc) return rc;
    const NA* in[1] = {src};
    NA* out[1] = {dst};
    if (src->type == CUMO_HIP_BIT) {
        cumo_hip_ndfunc_t nf = {iter_bit_unary, 0, 1, 1, {CUMO_HIP_BIT, 0}};
        return cumo_hip_na_ndloop(&nf, in, out, 0, (void*)find_row(kBitUnary, "copy"));
    }
    cumo_hip_ndfunc_t nf = {iter_copy_bytes, 0, 1, 1, {src->type, 0}};
    return cumo_hip_na_ndloop(&nf, in, out, 0, NULL);
}

// ---- host read-back and ingest (narray/narray.c:1391-1560 to_binary / from_binary /
// store_binary, gen/tmpl/extract_cpu.c, gen/tmpl/aref_cpu.c): the reference reads and
// writes managed memory after a device synchronisation; here the bytes cross by an
// explicit transfer, staged through a contiguous copy when the view is not contiguous
namespace {
// bytes of the view's elements laid out row-major (Bit: whole bytes)
size_t packed_bytes(const NA* a) {
    const size_t n = total_of(a);
    return a->type == CUMO_HIP_BIT ? (n + 7) / 8 : n * (size_t)kElmsz[a->type];
}
// a view whose bytes already lie as the transfer wants them
bool directly_addressable(const NA* a) { return is_contiguous(a) && (a->type != CUMO_HIP_BIT || a->offset % 8 == 0); }
char* first_byte(const NA* a) { return a->ptr + (a->type == CUMO_HIP_BIT ? a->offset / 8 : a->offset); }
}  // namespace

// host[0, nbytes) = the first nbytes of x's elements in row-major order
int cumo_hip_na_to_host(const cumo_hip_narray_t* x, void* host, size_t nbytes) {
    int rc = check_view(x, "source");
    if (rc) return rc;
    if (nbytes > packed_bytes(x)) return fail(CUMO_HIP_ERROR_ARGUMENT, "to_host: more bytes asked for than the array holds");
    if (nbytes == 0) return CUMO_HIP_OK;
    if (!host) return fail(CUMO_HIP_ERROR_ARGUMENT, "to_host: no host memory given");
    if (directly_addressable(x)) return cumo_hip_copy_to_host(host, first_byte(x), nbytes);
    NA tmp;
    tmp.ptr = NULL;
    rc = cumo_hip_na_copy(x, &tmp);  // the dup of narray.c:1543
    if (!rc) rc = cumo_hip_copy_to_host(host, tmp.ptr, nbytes);
    free_tmp(&tmp);
    return rc;
}

// x's elements in row-major order = host[0, nbytes); nbytes must cover the whole view
int cumo_hip_na_from_host(cumo_hip_narray_t* x, const void* host, size_t nbytes) {
    int rc = check_view(x, "destination");
    if (rc) return rc;
    const size_t need = packed_bytes(x);
    if (nbytes < need) return fail(CUMO_HIP_ERROR_ARGUMENT, "string is too short to store");
    if (need == 0) return CUMO_HIP_OK;
    if (!host) return fail(CUMO_HIP_ERROR_ARGUMENT, "from_host: no host memory given");
    if (!x->ptr) return fail(CUMO_HIP_ERROR_ARGUMENT, "from_host: destination has no memory");
    if (directly_addressable(x) && (x->type != CUMO_HIP_BIT || total_of(x) % 8 == 0)) return cumo_hip_copy_from_host(first_byte(x), host, need);
    NA tmp;
    tmp.ptr = NULL;
    rc = cumo_hip_na_alloc(&tmp, x->type, x->ndim, x->shape);
    if (!rc) rc = cumo_hip_copy_from_host(tmp.ptr, host, need);
    if (!rc) rc = cumo_hip_na_store(x, &tmp);
    free_tmp(&tmp);
    return rc;
}

// out = the element at index[0 .. ndim) (NULL: the only element of a one-element
// array), as the element type; for Bit one unsigned char, 0 or 1
int cumo_hip_na_extract(const cumo_hip_narray_t* x, const size_t* index, void* out) {
    int rc = check_view(x, "source");
    if (rc) return rc;
    if (!out) return fail(CUMO_HIP_ERROR_ARGUMENT, "extract: no host memory given");
    ssize_t off = x->offset;
    if (index) {
        for (int d = 0; d < x->ndim; ++d) {
            if (index[d] >= x->shape[d]) return fail(CUMO_HIP_ERROR_ARGUMENT, "index out of range");
            off += (ssize_t)index[d] * x->stride[d];
        }
    } else if (total_of(x) != 1) {
        return fail(CUMO_HIP_ERROR_SHAPE, "not a single-element array");
    }
    if (x->type == CUMO_HIP_BIT) {
        CUMO_BIT_DIGIT w = 0;
        rc = cumo_hip_copy_to_host(&w, x->ptr + (off / 32) * 4, sizeof(w));
        if (!rc) *(unsigned char*)out = (unsigned char)((w >> (off % 32)) & 1u);
        return rc;
    }
    return cumo_hip_copy_to_host(out, x->ptr + off, (size_t)kElmsz[x->type]);
}

int cumo_hip_na_fill(cumo_hip_narray_t* dst, double value) {
    if (dst && dst->type == CUMO_HIP_BIT) {
        int rcb = check_view(dst, "destination");
        if (rcb) return rcb;
        // reference: gen/tmpl_bit/fill.c:27-36
        if (value != 0.0 && value != 1.0) return fail(CUMO_HIP_ERROR_ARGUMENT, "invalid value for Bit");
        CUMO_BIT_DIGIT y = value != 0.0 ? ~(CUMO_BIT_DIGIT)0 : 0;
        cumo_hip_ndfunc_t nfb = {iter_bit_fill, 0, 1, 0, {0, 0}};
        const NA* inb[1] = {dst};
        return cumo_hip_na_ndloop(&nfb, inb, NULL, 0, &y);
    }
    int rc = check_arith(dst);
    if (rc) return rc;
    FillOpt opt = {value};
    cumo_hip_ndfunc_t nf = {iter_fill, 0, 1, 0, {0, 0}};
    const NA* in[1] = {dst};
    return cumo_hip_na_ndloop(&nf, in, NULL, 0, &opt);
}

namespace {
struct SeqOpt {
    double beg, step;
};
void iter_seq(LP* lp) {
    IA a1;
    IX ix;
    cumo_hip_make_indexer(lp, &ix);
    cumo_hip_make_iarray(lp, 0, &a1);
    const SeqOpt* g = (const SeqOpt*)lp->opt_ptr;
    switch (lp->args[0].type) {
        case CUMO_HIP_SFLOAT: cumo_iter_sfloat_seq_kernel_launch(&a1, &ix, (float)g->beg, (float)g->step, 0.0); break;
        case CUMO_HIP_DFLOAT: cumo_iter_dfloat_seq_kernel_launch(&a1, &ix, g->beg, g->step, 0.0); break;
        default: cumo_iter_int32_seq_kernel_launch(&a1, &ix, g->beg, g->step, 0.0); break;
    }
}
// one run at a time, the count carried from run to run (logseq.c walks the array the same way)
struct LogseqWalk {
    int type;
    double beg, step, base, count;
};
void logseq_walk(const LP* lp, int level, char* p, LogseqWalk* w) {
    const cumo_hip_loop_args_t& a = lp->args[0];
    if (level == lp->ndim - 1) {
        const uint64_t n = lp->n[level];
        if (w->type == CUMO_HIP_SFLOAT)
            cumo_iter_sfloat_logseq_stride_kernel_launch(p, a.step[level], (float)w->beg, (float)w->step, (float)w->base, w->count, n);
        else
            cumo_iter_dfloat_logseq_stride_kernel_launch(p, a.step[level], w->beg, w->step, w->base, w->count, n);
        w->count += (double)n;
        return;
    }
    for (size_t i = 0; i < lp->n[level]; i++) logseq_walk(lp, level + 1, p + (ssize_t)i * a.step[level], w);
}
}  // namespace

int cumo_hip_na_seq(cumo_hip_narray_t* dst, double beg, double step) {
    int rc = check_arith(dst);
    if (rc) return rc;
    SeqOpt opt = {beg, step};
    cumo_hip_ndfunc_t nf = {iter_seq, 0, 1, 0, {0, 0}};
    const NA* in[1] = {dst};
    return cumo_hip_na_ndloop(&nf, in, NULL, 0, &opt);
}

int cumo_hip_na_logseq(cumo_hip_narray_t* dst, double beg, double step, double base) {
    int rc = check_arith(dst);
    if (rc) return rc;
    if (!is_float(dst->type)) return no_method("logseq");
    if (total_of(dst) == 0) return CUMO_HIP_OK;
    cumo_hip_ndfunc_t nf = {NULL, 0, 1, 0, {0, 0}};
    const NA* in[1] = {dst};
    LP lp;
    rc = cumo_hip_na_ndloop_prepare(&nf, in, NULL, 0, &lp);
    if (rc) return rc;
    LogseqWalk w = {dst->type, beg, step, base, 0.0};
    logseq_walk(&lp, 0, lp.args[0].ptr, &w);
    return CUMO_HIP_OK;
}

int cumo_hip_na_eye(cumo_hip_narray_t* dst, double element, ssize_t kofs) {
    int rc = check_arith(dst);
    if (rc) return rc;
    const int nd = dst->ndim;
    if (nd < 2) return fail(CUMO_HIP_ERROR_DIMENSION, "less than 2-d array");
    if (kofs >= 0 ? (size_t)kofs >= dst->shape[nd - 1] : (size_t)(-kofs) >= dst->shape[nd - 2])
        return fail(CUMO_HIP_ERROR_ARGUMENT, "invalid diagonal offset for the size of the matrix");
    if (total_of(dst) == 0) return CUMO_HIP_OK;
    // the leading dimensions walk on the host, a launch per matrix (eye.c is a user loop over the last two)
    size_t idx[CUMO_NA_MAX_DIMENSION] = {0};
    for (;;) {
        ssize_t off = dst->offset;
        for (int d = 0; d < nd - 2; ++d) off += (ssize_t)idx[d] * dst->stride[d];
        char* p = dst->ptr + off;
        const ssize_t s0 = dst->stride[nd - 2], s1 = dst->stride[nd - 1];
        const uint64_t n0 = dst->shape[nd - 2], n1 = dst->shape[nd - 1];
        switch (dst->type) {
            case CUMO_HIP_SFLOAT: cumo_iter_sfloat_eye_stride_kernel_launch(p, s0, s1, kofs, (float)element, n0, n1); break;
            case CUMO_HIP_DFLOAT: cumo_iter_dfloat_eye_stride_kernel_launch(p, s0, s1, kofs, element, n0, n1); break;
            default: cumo_iter_int32_eye_stride_kernel_launch(p, s0, s1, kofs, (int32_t)element, n0, n1); break;
        }
        int d = nd - 3;
        for (; d >= 0; --d) {
            if (++idx[d] < dst->shape[d]) break;
            idx[d] = 0;
        }
        if (d < 0) break;
    }
    return CUMO_HIP_OK;
}

int cumo_hip_na_reduce(const char* op, const cumo_hip_narray_t* x, unsigned int reduce, int keepdims, int nan,
                       cumo_hip_narray_t* z, cumo_hip_narray_t* z2) {
    int rc = check_arith(x);
    if (rc) return rc;
    if (!op) return no_method(op);
    // narray/narray.c:1704-1716
    if (total_of(x) == 0) return fail(CUMO_HIP_ERROR_SHAPE, "cannot reduce empty NArray");
    if (x->ndim < 32 && (reduce >> x->ndim)) return fail(CUMO_HIP_ERROR_DIMENSION, "dimension is out of range");
    if (!reduce) reduce = all_dims(x);
    const bool use_nan = nan && is_float(x->type);
    const unsigned flag = CUMO_HIP_NDF_FLAT_REDUCE | (keepdims ? CUMO_HIP_NDF_KEEP_DIM : 0u);
    ReduceOpt opt = {nullptr, nullptr};
    int out_type = x->type;
    const NA* src = x;
    NA tmp;
    tmp.ptr = NULL;
    int nout = 1;

    if (!std::strcmp(op, "minmax")) {
        opt.fp = use_nan ? kMinmaxNan[x->type] : kMinmax[x->type];
        if (!opt.fp || !z2) return no_method(op);
        nout = 2;
    } else if (const ArgRow* arow = find_row(kArg, op)) {
        // an Int64 answer only when Int32 cannot hold every index (gen/tmpl/accum_arg.c:92-110)
        const bool wide = total_of(x) > 0xffffffffull;
        out_type = wide ? CUMO_HIP_INT64 : CUMO_HIP_INT32;
        opt.f = use_nan ? (wide ? arow->f64_nan : arow->f32_nan)[x->type] : (wide ? arow->f64 : arow->f32)[x->type];
        if (!opt.f) return no_method(op);
        if (arow->memory_index && !is_contiguous(x)) {
            // the answer counts along the view's own row-major order: work on a
            // contiguous copy (gen/tmpl/accum_index.c:118-126)
            rc = cumo_hip_na_copy(x, &tmp);
            if (rc) return rc;
            src = &tmp;
        }
    } else if (const ReduceRow* row = find_row(kReduce, op)) {
        opt.f = use_nan ? row->f_nan[x->type] : row->f[x->type];
        if (!opt.f) return no_method(op);
        if (row->result == 1 && x->type == CUMO_HIP_INT32) out_type = CUMO_HIP_INT64;  // gen/spec.rb:308-319
    } else {
        return no_method(op);
    }
    cumo_hip_ndfunc_t nf = {iter_reduce, flag, 1, nout, {out_type, out_type}};
    const NA* in[1] = {src};
    NA* out[2] = {z, z2};
    rc = cumo_hip_na_ndloop(&nf, in, out, reduce, &opt);
    free_tmp(&tmp);
    return rc;
}

int cumo_hip_na_bit_binary(const char* op, const cumo_hip_narray_t* x, const cumo_hip_narray_t* y, cumo_hip_narray_t* z) {
    int rc = check_view(x, "operand");
    if (!rc) rc = check_view(y, "operand");
    if (rc) return rc;
    const BitBinaryRow* row = find_row(kBitBinary, op);
    if (!row || x->type != CUMO_HIP_BIT || y->type != CUMO_HIP_BIT) return no_method(op);
    cumo_hip_ndfunc_t nf = {iter_bit_binary, 0, 2, 1, {CUMO_HIP_BIT, 0}};
    const NA* in[2] = {x, y};
    NA* out[1] = {z};
    return cumo_hip_na_ndloop(&nf, in, out, 0, (void*)row);
}

int cumo_hip_na_bit_unary(const char* op, const cumo_hip_narray_t* x, cumo_hip_narray_t* z) {
    int rc = check_view(x, "operand");
    if (rc) return rc;
    const BitUnaryRow* row = find_row(kBitUnary, op);
    if (!row || x->type != CUMO_HIP_BIT) return no_method(op);
    cumo_hip_ndfunc_t nf = {iter_bit_unary, 0, 1, 1, {CUMO_HIP_BIT, 0}};
    const NA* in[1] = {x};
    NA* out[1] = {z};
    return cumo_hip_na_ndloop(&nf, in, out, 0, (void*)row);
}

int cumo_hip_na_bit_count(const cumo_hip_narray_t* x, unsigned int reduce, int keepdims, int count_false, cumo_hip_narray_t* z) {
    int rc = check_view(x, "operand");
    if (rc) return rc;
    if (x->type != CUMO_HIP_BIT) return no_method(count_false ? "count_false" : "count_true");
    if (x->ndim < 32 && (reduce >> x->ndim)) return fail(CUMO_HIP_ERROR_DIMENSION, "dimension is out of range");
    if (!reduce) reduce = all_dims(x);
    const unsigned flag = CUMO_HIP_NDF_FLAT_REDUCE | (keepdims ? CUMO_HIP_NDF_KEEP_DIM : 0u);
    cumo_hip_ndfunc_t nf = {iter_bit_count, flag, 1, 1, {CUMO_HIP_UINT64, 0}};
    const NA* in[1] = {x};
    NA* out[1] = {z};
    if (z && z->ptr && !is_contiguous(z)) return fail(CUMO_HIP_ERROR_ARGUMENT, "bit count: the result array must be contiguous");
    cumo_hip_loop_t lp;
    rc = cumo_hip_na_ndloop_prepare(&nf, in, out, reduce, &lp);
    if (rc) return rc;
    // one contiguous run into one counter: a single launch that stores the count
    if (total_of(x) != 0 && lp.ndim == 1 && lp.reduce_dim == 1 && lp.args[0].step[0] == 1 && total_of(z) == 1) {
        CUMO_BIT_DIGIT* a = (CUMO_BIT_DIGIT*)lp.args[0].ptr + lp.args[0].bitpos / 32;
        if (cumo_hip_bit_count_run_store_kernel_launch(a, lp.args[0].bitpos % 32, lp.n[0], count_false != 0, (uint64_t*)lp.args[1].ptr))
            return CUMO_HIP_OK;
    }
    // the launchers add onto the result: start from 0 (ndloop.c:853-860). The launch that takes every
    // output at once zeroes the results itself where its kernel adds, and not where it stores.
    const bool at_once = total_of(x) != 0 && !(lp.ndim - lp.reduce_dim == 0 && lp.reduce_dim == 1);
    size_t zbytes = total_of(z) * 8;
    if (zbytes && !at_once) cumo_hip_memset(z->ptr + z->offset, 0, zbytes);
    if (total_of(x) == 0) return CUMO_HIP_OK;
    CountOpt opt = {count_false != 0, at_once};
    lp.opt_ptr = &opt;
    iter_bit_count(&lp);
    return lp.status;
}

// all? / any? along axes into a Bit result (reference: gen/tmpl_bit/bit_reduce.c:5-146). The
// result starts out as the init bit (1 for all?, 0 for any?) and the launchers flip it. The
// reference walks every dimension but the innermost on the host and launches once per run;
// so does this for up to 32 runs. With more runs it takes the counts along the same axes
// instead (one launch, whatever the shape): any? = (count_true != 0), all? = !(count_false != 0).
int cumo_hip_na_bit_reduce(const char* op, const cumo_hip_narray_t* x, unsigned int reduce, int keepdims, cumo_hip_narray_t* z) {
    int rc = check_view(x, "operand");
    if (rc) return rc;
    if (!op || (std::strcmp(op, "all_p") != 0 && std::strcmp(op, "any_p") != 0)) return no_method(op ? op : "(null)");
    const bool all = op[1] == 'l';
    if (x->type != CUMO_HIP_BIT) return no_method(all ? "all?" : "any?");
    if (x->ndim < 32 && (reduce >> x->ndim)) return fail(CUMO_HIP_ERROR_DIMENSION, "dimension is out of range");
    if (!reduce) reduce = all_dims(x);
    const unsigned flag = CUMO_HIP_NDF_FLAT_REDUCE | (keepdims ? CUMO_HIP_NDF_KEEP_DIM : 0u);
    cumo_hip_ndfunc_t nf = {NULL, flag, 1, 1, {CUMO_HIP_BIT, 0}};
    const NA* in[1] = {x};
    NA* out[1] = {z};
    cumo_hip_loop_t lp;
    rc = cumo_hip_na_ndloop_prepare(&nf, in, out, reduce, &lp);
    if (rc) return rc;
    if (total_of(z) == 0) return CUMO_HIP_OK;
    size_t runs = 1;
    for (int d = 0; d + 1 < lp.ndim; d++) runs *= lp.n[d];
    const bool by_counts = total_of(x) != 0 && (lp.ndim == 0 || runs > 32);  // (every bit of the result gets written then)
    if (!by_counts) {
        rc = cumo_hip_na_fill(z, all ? 1.0 : 0.0);
        if (rc || total_of(x) == 0) return rc;
    }
    if (by_counts && lp.reduce_dim == 1 && lp.ndim >= 2 && lp.args[0].step[lp.ndim - 1] == 1) {
        // rows that start on words, results that are consecutive bits: one launch from the rows to the packed bits
        const int nkeep = lp.ndim - 1;
        bool rows_ok = true;
        uint64_t nrows = lp.n[nkeep - 1];
        for (int d = nkeep - 2; d >= 0 && rows_ok; d--) {
            rows_ok = lp.args[0].step[d] == lp.args[0].step[d + 1] * (ssize_t)lp.n[d + 1];
            nrows *= lp.n[d];
        }
        ssize_t zs = 1;
        for (int d = nkeep - 1; d >= 0 && rows_ok; d--) {
            rows_ok = lp.args[1].step[d] == zs;
            zs *= (ssize_t)lp.n[d];
        }
        if (rows_ok && cumo_hip_bit_anyall_rows_kernel_launch((CUMO_BIT_DIGIT*)lp.args[0].ptr, lp.args[0].bitpos, nrows, lp.args[0].step[nkeep - 1],
                                                              lp.n[lp.ndim - 1], all ? 1 : 0, (CUMO_BIT_DIGIT*)lp.args[1].ptr, lp.args[1].bitpos))
            return CUMO_HIP_OK;
    }
    if (by_counts) {
        NA counts;
        std::memset(&counts, 0, sizeof(counts));
        rc = cumo_hip_na_bit_count(x, reduce, keepdims, all ? 1 : 0, &counts);
        if (!rc && is_contiguous(z) && is_contiguous(&counts) && z->offset >= 0 && total_of(&counts) == total_of(z)) {
            // any? = some bit set, all? = no bit clear: packed from the counts in one launch
            cumo_hip_bit_from_counts_kernel_launch((const uint64_t*)(counts.ptr + counts.offset), total_of(z), all ? 1 : 0, (CUMO_BIT_DIGIT*)z->ptr,
                                                   (size_t)z->offset);
            free_tmp(&counts);
            return CUMO_HIP_OK;
        }
        if (!rc) rc = cumo_hip_na_store(z, &counts);  // nonzero -> 1
        free_tmp(&counts);
        if (!rc && all) rc = cumo_hip_na_bit_unary("not", z, z);
        return rc;
    }
    CUMO_BIT_DIGIT* a1 = (CUMO_BIT_DIGIT*)lp.args[0].ptr;
    CUMO_BIT_DIGIT* a2 = (CUMO_BIT_DIGIT*)lp.args[1].ptr;
    const int last = lp.ndim - 1;
    const ssize_t s1 = lp.args[0].step[last], s2 = lp.args[1].step[last];
    const uint64_t n = lp.n[last];
    size_t idx[CUMO_NA_MAX_DIMENSION] = {0};
    for (size_t r = 0; r < runs; r++) {
        ssize_t p1 = (ssize_t)lp.args[0].bitpos, p2 = (ssize_t)lp.args[1].bitpos;
        for (int d = 0; d < last; d++) {
            p1 += (ssize_t)idx[d] * lp.args[0].step[d];
            p2 += (ssize_t)idx[d] * lp.args[1].step[d];
        }
        if (s2 != 0) {
            if (all) cumo_iter_bit_all_p_elementwise_kernel_launch(a1, (size_t)p1, s1, NULL, a2, (size_t)p2, s2, NULL, n);
            else cumo_iter_bit_any_p_elementwise_kernel_launch(a1, (size_t)p1, s1, NULL, a2, (size_t)p2, s2, NULL, n);
        } else if (s1 == 1) {
            if (all) cumo_iter_bit_all_p_contiguous_reduce_kernel_launch(a1, (size_t)p1, a2, (size_t)p2, n);
            else cumo_iter_bit_any_p_contiguous_reduce_kernel_launch(a1, (size_t)p1, a2, (size_t)p2, n);
        } else {
            if (all) cumo_iter_bit_all_p_reduce_kernel_launch(a1, (size_t)p1, s1, NULL, a2, (size_t)p2, n);
            else cumo_iter_bit_any_p_reduce_kernel_launch(a1, (size_t)p1, s1, NULL, a2, (size_t)p2, n);
        }
        for (int d = last - 1; d >= 0; d--) {
            if (++idx[d] < lp.n[d]) break;
            idx[d] = 0;
        }
    }
    return CUMO_HIP_OK;
}

}  // extern "C"
