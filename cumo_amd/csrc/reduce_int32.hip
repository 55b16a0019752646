// Int32 reduction launchers (reference: narray/gen/tmpl/accum.c:8, minmax.c:2,
// accum_arg.c:5, accum_index.c:5). sum and prod answer Int64
// (narray/gen/spec.rb:308-319).
#include "reduce_kernels.h"
#include "reduce_impls.h"

using namespace cumo_hip;

#define CUMO_RED(name) extern "C" void cumo_int32_##name##_kernel_launch(cumo_na_reduction_arg_t* arg)

typedef int32_t T;

CUMO_RED(sum) { reduce_launch(arg, nullptr, SumImpl<T, int64_t, false, false>{0}, 0); }
CUMO_RED(prod) { reduce_launch(arg, nullptr, SumImpl<T, int64_t, true, false>{0}, 0); }
CUMO_RED(min) { reduce_launch(arg, nullptr, ValueExtremeImpl<T, false>{}, 1); }
CUMO_RED(max) { reduce_launch(arg, nullptr, ValueExtremeImpl<T, true>{}, 1); }
CUMO_RED(ptp) { reduce_launch(arg, nullptr, MinMaxValueImpl<T>{1}, 0); }
CUMO_RED(argmin_int32) { reduce_launch(arg, nullptr, ArgImpl<T, false, false>{4}, 1); }
CUMO_RED(argmin_int64) { reduce_launch(arg, nullptr, ArgImpl<T, false, false>{8}, 1); }
CUMO_RED(argmax_int32) { reduce_launch(arg, nullptr, ArgImpl<T, true, false>{4}, 1); }
CUMO_RED(argmax_int64) { reduce_launch(arg, nullptr, ArgImpl<T, true, false>{8}, 1); }
CUMO_RED(min_index_int32) { reduce_launch(arg, nullptr, ArgImpl<T, false, false>{4}, 2); }
CUMO_RED(min_index_int64) { reduce_launch(arg, nullptr, ArgImpl<T, false, false>{8}, 2); }
CUMO_RED(max_index_int32) { reduce_launch(arg, nullptr, ArgImpl<T, true, false>{4}, 2); }
CUMO_RED(max_index_int64) { reduce_launch(arg, nullptr, ArgImpl<T, true, false>{8}, 2); }
extern "C" void cumo_int32_minmax_kernel_launch(cumo_na_reduction_arg_t* arg, cumo_na_iarray_t* out2) {
    reduce_launch(arg, out2, MinMaxValueImpl<T>{0}, 0);
}
