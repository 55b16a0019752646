// One instance of the split row reduction, for tests/test_emitted_ordering.py: compiled to
// assembly (device side only), never linked or run.
#include "reduce_kernels.h"
#include "reduce_impls.h"

using namespace cumo_hip;

template __global__ void cumo_hip::red_srow_split_kernel<SumImpl<float, float, false, false>, 4, false>(RedSParams, SumImpl<float, float, false, false>);
