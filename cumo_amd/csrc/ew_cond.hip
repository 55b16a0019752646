// Comparison and classification launchers, results packed into Bit
// (reference: narray/gen/tmpl/cond_binary.c:2-3, cond_unary.c:2).
#include "ew_kernels.h"
#include "ew_ops.h"

using namespace cumo_hip;

#define CUMO_DEF_COND(t, c, name, OP)                                                                               \
    extern "C" void cumo_iter_##t##_##name##_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2,              \
                                                           cumo_na_bit_iarray_t* a3, cumo_na_indexer_t* indexer) {  \
        ew_launch(OP<c>{}, a1, a2, nullptr, a3, indexer, (c)0, 0, nullptr);                                         \
    }                                                                                                               \
    extern "C" void cumo_iter_##t##_##name##_s_kernel_launch(cumo_na_iarray_t* a1, c sv, cumo_na_bit_iarray_t* a3,  \
                                                             cumo_na_indexer_t* indexer, int scalar_is_left) {      \
        ew_launch(OP<c>{}, a1, nullptr, nullptr, a3, indexer, sv, scalar_is_left ? 2 : 1, nullptr);                 \
    }

#define CUMO_DEF_COND_UNARY(t, c, name, OP)                                                                         \
    extern "C" void cumo_iter_##t##_##name##_kernel_launch(cumo_na_iarray_t* a1, cumo_na_bit_iarray_t* a2,          \
                                                           cumo_na_indexer_t* indexer) {                            \
        ew_launch(OP<c>{}, a1, nullptr, nullptr, a2, indexer, (c)0, 0, nullptr);                                    \
    }

#define CUMO_DEF_COND_ALL(t, c)      \
    CUMO_DEF_COND(t, c, eq, OpEq)    \
    CUMO_DEF_COND(t, c, ne, OpNe)    \
    CUMO_DEF_COND(t, c, gt, OpGt)    \
    CUMO_DEF_COND(t, c, ge, OpGe)    \
    CUMO_DEF_COND(t, c, lt, OpLt)    \
    CUMO_DEF_COND(t, c, le, OpLe)

#define CUMO_DEF_COND_FLOAT(t, c)                   \
    CUMO_DEF_COND(t, c, nearly_eq, OpNearlyEq)      \
    CUMO_DEF_COND_UNARY(t, c, isnan, OpIsNan)       \
    CUMO_DEF_COND_UNARY(t, c, isinf, OpIsInf)       \
    CUMO_DEF_COND_UNARY(t, c, isposinf, OpIsPosInf) \
    CUMO_DEF_COND_UNARY(t, c, isneginf, OpIsNegInf) \
    CUMO_DEF_COND_UNARY(t, c, isfinite, OpIsFinite) \
    CUMO_DEF_COND_UNARY(t, c, signbit, OpSignbit)

CUMO_DEF_COND_ALL(sfloat, float)
CUMO_DEF_COND_ALL(dfloat, double)
CUMO_DEF_COND_ALL(int32, int32_t)
CUMO_DEF_COND_FLOAT(sfloat, float)
CUMO_DEF_COND_FLOAT(dfloat, double)
