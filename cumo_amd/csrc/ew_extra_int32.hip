// Int32 pow, maximum/minimum and clip launchers (reference: narray/gen/tmpl/pow.c:2-6,
// ewcomp.c:18, clip.c:2-7; semantics types/int_macro_kernel.h:26-42,
// xint_macro_kernel.h:21-22,54-68).
#include "ew_kernels.h"
#include "ew_ops.h"
#include "ew_clip3.h"
#include "ew_ret2.h"

using namespace cumo_hip;

// ---- pow: the Int32 exponent forms are the same function for an Int32 base -----------
extern "C" void cumo_iter_int32_pow_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_iarray_t* a3,
                                                  cumo_na_indexer_t* indexer) {
    ew_launch(OpIPow{}, a1, a2, a3, nullptr, indexer, (int32_t)0, 0, nullptr);
}
extern "C" void cumo_iter_int32_pow_s_kernel_launch(cumo_na_iarray_t* a1, int32_t sv, cumo_na_iarray_t* a3,
                                                    cumo_na_indexer_t* indexer, int scalar_is_left) {
    if (scalar_is_left) {
        OpIPowLeft op;
        op.base = sv;
        ew_launch(op, a1, nullptr, a3, nullptr, indexer, (int32_t)0, 0, nullptr);
    } else {
        OpIPowS op;
        op.p = sv;
        ew_launch(op, a1, nullptr, a3, nullptr, indexer, (int32_t)0, 0, nullptr);
    }
}
extern "C" void cumo_iter_int32_pow_int32_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_iarray_t* a3,
                                                        cumo_na_indexer_t* indexer) {
    ew_launch(OpIPow{}, a1, a2, a3, nullptr, indexer, (int32_t)0, 0, nullptr);
}
extern "C" void cumo_iter_int32_pow_int32_s_kernel_launch(cumo_na_iarray_t* a1, int32_t sv, cumo_na_iarray_t* a3,
                                                          cumo_na_indexer_t* indexer) {
    OpIPowS op;
    op.p = sv;
    ew_launch(op, a1, nullptr, a3, nullptr, indexer, (int32_t)0, 0, nullptr);
}
extern "C" void cumo_iter_int32_pow_int32_s_left_kernel_launch(int32_t sv_base, cumo_na_iarray_t* a2, cumo_na_iarray_t* a3,
                                                               cumo_na_indexer_t* indexer) {
    OpIPowLeft op;
    op.base = sv_base;
    ew_launch(op, a2, nullptr, a3, nullptr, indexer, (int32_t)0, 0, nullptr);
}

// ---- maximum / minimum (no NaN forms for an integer type) ------------------------------
extern "C" void cumo_int32_maximum_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_iarray_t* a3,
                                                 cumo_na_indexer_t* indexer) {
    ew_launch(OpMaximum<int32_t>{}, a1, a2, a3, nullptr, indexer, (int32_t)0, 0, nullptr);
}
extern "C" void cumo_int32_minimum_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_iarray_t* a3,
                                                 cumo_na_indexer_t* indexer) {
    ew_launch(OpMinimum<int32_t>{}, a1, a2, a3, nullptr, indexer, (int32_t)0, 0, nullptr);
}

// ---- divmod (reference: narray/gen/tmpl/binary2.c:2; a zero divisor raises the flag) ---------
extern "C" void cumo_iter_int32_divmod_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_iarray_t* a3,
                                                     cumo_na_iarray_t* a4, cumo_na_indexer_t* indexer, int* divzero) {
    const cumo_na_iarray_t* arr[4] = {a1, a2, a3, a4};
    ret2_launch(OpDivmodI{}, arr, indexer, divzero);
}

// ---- clip ---------------------------------------------------------------------------------
extern "C" void cumo_iter_int32_clip_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_iarray_t* a3,
                                                   cumo_na_iarray_t* a4, cumo_na_indexer_t* indexer, int* invalid) {
    clip3_launch<int32_t>(a1, a2, a3, a4, indexer, invalid);
}
extern "C" void cumo_iter_int32_clip_s_kernel_launch(cumo_na_iarray_t* a1, int32_t sv_min, int32_t sv_max, cumo_na_iarray_t* a4,
                                                     cumo_na_indexer_t* indexer) {
    OpClipS<int32_t> op;
    op.lo = sv_min;
    op.hi = sv_max;
    ew_launch(op, a1, nullptr, a4, nullptr, indexer, (int32_t)0, 0, nullptr);
}
extern "C" void cumo_iter_int32_clip_min_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_iarray_t* a3,
                                                       cumo_na_indexer_t* indexer) {
    ew_launch(OpClipMin<int32_t>{}, a1, a2, a3, nullptr, indexer, (int32_t)0, 0, nullptr);
}
extern "C" void cumo_iter_int32_clip_min_s_kernel_launch(cumo_na_iarray_t* a1, int32_t sv, cumo_na_iarray_t* a3,
                                                         cumo_na_indexer_t* indexer) {
    ew_launch(OpClipMin<int32_t>{}, a1, nullptr, a3, nullptr, indexer, sv, 1, nullptr);
}
extern "C" void cumo_iter_int32_clip_max_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, cumo_na_iarray_t* a3,
                                                       cumo_na_indexer_t* indexer) {
    ew_launch(OpClipMax<int32_t>{}, a1, a2, a3, nullptr, indexer, (int32_t)0, 0, nullptr);
}
extern "C" void cumo_iter_int32_clip_max_s_kernel_launch(cumo_na_iarray_t* a1, int32_t sv, cumo_na_iarray_t* a3,
                                                         cumo_na_indexer_t* indexer) {
    ew_launch(OpClipMax<int32_t>{}, a1, nullptr, a3, nullptr, indexer, sv, 1, nullptr);
}
