// Same-type store between views that may carry index arrays, and ingest of a host
// array staged in device memory (store_array).
//
// Replaces the stridx kernel of ext/cumo/narray/gen/tmpl/store_from_kernel.cu:19-35
// (host declaration store_from.c:5; only the same-type store is reachable with an
// index array, through store_array's own loop) and
// narray/gen/tmpl/store_array_kernel.cu:2-60 (host store_array.c:2-5), under the
// reference's symbols. Neither is a bandwidth path: one element per lane, four
// elements in flight per lane for the staged copies.
#include "bit_common.h"

using namespace cumo_hip;

namespace {

template <class T>
__global__ __launch_bounds__(kBlock) void store_stridx_kernel(cumo_na_iarray_stridx_t a1, cumo_na_iarray_stridx_t a2, BitNd nd) {
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < nd.total; i += (uint64_t)gridDim.x * kBlock) {
        *reinterpret_cast<T*>(a1.ptr + stridx_offset(a1.stridx, nd, i)) = *reinterpret_cast<const T*>(a2.ptr + stridx_offset(a2.stridx, nd, i));
    }
}

// p1 + idx1[i] (idx1 given) or p1 + i * s1 takes z[i], or the one value z0
template <class T, bool SCALAR>
__global__ __launch_bounds__(kBlock) void store_array_kernel(char* p1, int64_t s1, const size_t* idx1, const T* z, T z0, uint64_t n) {
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (uint64_t)gridDim.x * kBlock) {
        const int64_t off = idx1 ? (int64_t)idx1[i] : (int64_t)i * s1;
        *reinterpret_cast<T*>(p1 + off) = SCALAR ? z0 : z[i];
    }
}

template <class T, bool SCALAR>
void launch_store_array(char* p1, ssize_t s1, size_t* idx1, T* z, T z0, uint64_t n) {
    if (n == 0) return;
    hipLaunchKernelGGL((store_array_kernel<T, SCALAR>), dim3(grid_for(n)), dim3(kBlock), 0, current_stream(), p1, (int64_t)s1, (const size_t*)idx1,
                       (const T*)z, z0, n);
    cumo_cuda_runtime_check_kernel_launch();
}

}  // namespace

#define CUMO_DEF_STORE_STRIDX(t, c)                                                                                               \
    extern "C" void cumo_iter_##t##_store_##t##_stridx_kernel_launch(cumo_na_iarray_stridx_t* a1, cumo_na_iarray_stridx_t* a2,    \
                                                                     cumo_na_indexer_t* indexer) {                                \
        if (indexer->total_size == 0) return;                                                                                     \
        BitNd nd = make_nd(indexer);                                                                                              \
        hipLaunchKernelGGL((store_stridx_kernel<c>), dim3(grid_for(nd.total)), dim3(kBlock), 0, current_stream(), *a1, *a2, nd);  \
        cumo_cuda_runtime_check_kernel_launch();                                                                                  \
    }                                                                                                                             \
    extern "C" void cumo_iter_##t##_store_array_index_kernel_launch(char* p1, size_t* idx1, c* z, uint64_t n) {                   \
        launch_store_array<c, false>(p1, 0, idx1, z, (c)0, n);                                                                    \
    }                                                                                                                             \
    extern "C" void cumo_iter_##t##_store_array_stride_kernel_launch(char* p1, ssize_t s1, c* z, uint64_t n) {                    \
        launch_store_array<c, false>(p1, s1, nullptr, z, (c)0, n);                                                                \
    }                                                                                                                             \
    extern "C" void cumo_iter_##t##_store_array_index_scalar_kernel_launch(char* p1, size_t* idx1, c z, uint64_t n) {             \
        launch_store_array<c, true>(p1, 0, idx1, nullptr, z, n);                                                                  \
    }                                                                                                                             \
    extern "C" void cumo_iter_##t##_store_array_stride_scalar_kernel_launch(char* p1, ssize_t s1, c z, uint64_t n) {              \
        launch_store_array<c, true>(p1, s1, nullptr, nullptr, z, n);                                                              \
    }
CUMO_DEF_STORE_STRIDX(sfloat, float)
CUMO_DEF_STORE_STRIDX(dfloat, double)
CUMO_DEF_STORE_STRIDX(int32, int32_t)
