// Host-side launch planning: turns the reference's per-launch descriptors
// (shape + per-operand byte steps, include/cumo_hip.h) into the few numbers a
// kernel needs, so that no kernel decomposes a flat index per element the way
// cumo_na_indexer_set_dim does (reference: ext/cumo/include/cumo/indexer.h:228-300).
//
// Nothing here touches the device; the tests drive it on a CPU-only machine.
#ifndef CUMO_HIP_PLAN_H
#define CUMO_HIP_PLAN_H

#include <stdint.h>
#include <stddef.h>
#include "cumo_hip.h"

namespace cumo_hip {

constexpr int kMaxDim = CUMO_NA_MAX_DIMENSION;
constexpr int kMaxOperands = 4;

struct EwOperand {
    const char* ptr;      // element 0 of the view (word pointer for a Bit operand)
    const ssize_t* step;  // per input dimension; bytes, or bits for a Bit operand
    int elmsz;            // bytes; 0 marks a Bit operand
    size_t bitpos;        // Bit operand: position of element 0 in bits
};

enum { EW_EMPTY = 0, EW_ROWS = 1, EW_TRANSPOSE = 2 };

struct EwPlan {
    int kind;
    int ndim;       // collapsed dims; the fast dim is last, for EW_TRANSPOSE the second tile dim is ndim-2
    int vec;        // elements per thread per access (1, 2 or 4)
    int vec_loose;  // the same when inputs only need their element's alignment (global loads of 128 bits
                    // work on any 4-byte boundary); the result still starts on a boundary of the access
    int fast_dim;   // which collapsed dim (before the final permutation) became last
    int tr_dim;     // ditto for the transpose partner, -1 otherwise
    uint64_t total;
    uint64_t shape[kMaxDim];
    int64_t step[kMaxOperands][kMaxDim];
};

// nops operands, the last one is the one written.
void plan_elementwise(int ndim, const size_t* shape, int nops, const EwOperand* ops, EwPlan* plan);

enum { RED_EMPTY = 0, RED_ROW = 1, RED_COL = 2, RED_GENERIC = 3 };

struct ReducePlan {
    int kind;
    int vec;               // elements per access along the contiguous axis
    int threads_per_row;   // RED_ROW: lanes sharing one output (power of two, <= 256)
    int n_split;           // > 1: the reduce axis is cut into n_split chunks and combined by a second launch
    int local_split_bits;  // RED_COL: 2^bits lanes of a block share an output's reduce axis and combine through LDS
    int red_tail;          // only when the caller allowed it: RED_ROW, elements of the axis past its last whole vector;
                           // RED_COL, outputs past the last whole vector of outputs
    int out_ndim, red_ndim;
    uint64_t out_total, red_total;
    uint64_t out_shape[kMaxDim], red_shape[kMaxDim];
    int64_t in_out_step[kMaxDim];  // input byte steps over the output dims
    int64_t in_red_step[kMaxDim];  // input byte steps over the reduce dims
    int64_t out_step[kMaxDim];     // output byte steps over the output dims
    int64_t out2_step[kMaxDim];    // second output (minmax)
};

// in_elmsz: bytes per input element. accum_bytes: sizeof the accumulator, which
// sizes the scratch of a split reduction. out2 may be NULL.
// allow_tail: a contiguous reduce axis (or, with the outputs along memory, their one dimension) need not be a
// whole number of vectors (red_tail says what is left over); for callers whose kernels see to the rest.
void plan_reduce(const cumo_na_reduction_arg_t* arg, const cumo_na_iarray_t* out2, int in_elmsz, int accum_bytes,
                 ReducePlan* plan, bool allow_tail = false);

// number of compute units the planner sizes grids for
constexpr int kNumCU = 256;

}  // namespace cumo_hip

#endif
