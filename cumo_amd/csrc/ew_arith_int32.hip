// Int32 arithmetic launchers (reference: narray/gen/tmpl/binary.c:12-15,
// unary.c:3, unary2.c:3; semantics types/xint_macro_kernel.h, int_macro_kernel.h).
#include "ew_kernels.h"
#include "ew_ops.h"

using namespace cumo_hip;

#define CUMO_DEF_BINARY(name, OP)                                                                                    \
    extern "C" void cumo_iter_int32_##name##_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2,               \
                                                           cumo_na_iarray_t* a3, cumo_na_indexer_t* indexer,         \
                                                           int* divzero) {                                           \
        ew_launch(OP{}, a1, a2, a3, nullptr, indexer, (int32_t)0, 0, divzero);                                       \
    }                                                                                                                \
    extern "C" void cumo_iter_int32_##name##_s_kernel_launch(cumo_na_iarray_t* a1, int32_t sv, cumo_na_iarray_t* a3, \
                                                             cumo_na_indexer_t* indexer, int* divzero,               \
                                                             int scalar_is_left) {                                   \
        ew_launch(OP{}, a1, nullptr, a3, nullptr, indexer, sv, scalar_is_left ? 2 : 1, divzero);                     \
    }

#define CUMO_DEF_UNARY(name, OP)                                                                          \
    extern "C" void cumo_iter_int32_##name##_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2,    \
                                                           cumo_na_indexer_t* indexer, int* flag) {       \
        ew_launch(OP{}, a1, nullptr, a2, nullptr, indexer, (int32_t)0, 0, flag);                          \
    }

CUMO_DEF_BINARY(add, OpIAdd)
CUMO_DEF_BINARY(sub, OpISub)
CUMO_DEF_BINARY(mul, OpIMul)
// div, mod: the array forms and the form with the scalar on the left as the others; an array by one divisor that is not
// zero goes by multiplication (OpIDivBy), nothing there can be rejected
#define CUMO_DEF_DIVISION(name, OP, OPBY)                                                                            \
    extern "C" void cumo_iter_int32_##name##_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2,               \
                                                           cumo_na_iarray_t* a3, cumo_na_indexer_t* indexer,         \
                                                           int* divzero) {                                           \
        ew_launch(OP{}, a1, a2, a3, nullptr, indexer, (int32_t)0, 0, divzero);                                       \
    }                                                                                                                \
    extern "C" void cumo_iter_int32_##name##_s_kernel_launch(cumo_na_iarray_t* a1, int32_t sv, cumo_na_iarray_t* a3, \
                                                             cumo_na_indexer_t* indexer, int* divzero,               \
                                                             int scalar_is_left) {                                   \
        if (!scalar_is_left && sv != 0) {                                                                            \
            OPBY op;                                                                                                 \
            op.d = sv;                                                                                               \
            op.magic = div31_make(sv < 0 ? 0u - (uint32_t)sv : (uint32_t)sv);                                        \
            ew_launch(op, a1, nullptr, a3, nullptr, indexer, (int32_t)0, 0, nullptr);                                \
            return;                                                                                                  \
        }                                                                                                            \
        ew_launch(OP{}, a1, nullptr, a3, nullptr, indexer, sv, scalar_is_left ? 2 : 1, divzero);                     \
    }
CUMO_DEF_DIVISION(div, OpIDiv, OpIDivBy)
CUMO_DEF_DIVISION(mod, OpIMod, OpIModBy)
CUMO_DEF_BINARY(bit_and, OpIAnd)
CUMO_DEF_BINARY(bit_or, OpIOr)
CUMO_DEF_BINARY(bit_xor, OpIXor)
CUMO_DEF_BINARY(left_shift, OpIShl)
CUMO_DEF_BINARY(right_shift, OpIShr)

CUMO_DEF_UNARY(minus, OpIMinus)
CUMO_DEF_UNARY(reciprocal, OpIReciprocal)
CUMO_DEF_UNARY(sign, OpISign)
CUMO_DEF_UNARY(square, OpISquare)
CUMO_DEF_UNARY(bit_not, OpINot)
CUMO_DEF_UNARY(abs, OpIAbs)
