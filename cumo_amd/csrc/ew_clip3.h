// clip against two array bounds: the one elementwise operation with three
// inputs (reference: narray/gen/tmpl/clip_kernel.cu:7-24). An element whose
// lower bound exceeds its upper bound is left unwritten and raises the flag.
// Rare enough to get the plain form: one element per thread, its position
// decomposed over the loop dimensions.
#ifndef CUMO_HIP_EW_CLIP3_H
#define CUMO_HIP_EW_CLIP3_H

#include "common.h"

namespace cumo_hip {

struct Clip3Params {
    int ndim;
    uint64_t total;
    uint64_t shape[CUMO_NA_MAX_DIMENSION];
    int64_t step[4][CUMO_NA_MAX_DIMENSION];
    char* ptr[4];
    int* invalid;
};

template <class T>
__global__ __launch_bounds__(256) void clip3_kernel(Clip3Params p) {
    for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < p.total; i += (uint64_t)gridDim.x * 256) {
        uint64_t r = i;
        int64_t off[4] = {0, 0, 0, 0};
        for (int d = p.ndim - 1; d >= 0; --d) {
            const uint64_t n = p.shape[d];
            const uint64_t q = r / n;
            const int64_t k = (int64_t)(r - q * n);
            r = q;
#pragma unroll
            for (int a = 0; a < 4; ++a) off[a] += k * p.step[a][d];
        }
        T x = *reinterpret_cast<const T*>(p.ptr[0] + off[0]);
        const T lo = *reinterpret_cast<const T*>(p.ptr[1] + off[1]);
        const T hi = *reinterpret_cast<const T*>(p.ptr[2] + off[2]);
        if (lo > hi) {
            if (p.invalid) *p.invalid = 1;
            continue;
        }
        if (x < lo) x = lo;
        if (x > hi) x = hi;
        *reinterpret_cast<T*>(p.ptr[3] + off[3]) = x;
    }
}

template <class T>
static void clip3_launch(const cumo_na_iarray_t* a1, const cumo_na_iarray_t* a2, const cumo_na_iarray_t* a3,
                         const cumo_na_iarray_t* a4, const cumo_na_indexer_t* indexer, int* invalid) {
    if (indexer->total_size == 0) return;
    Clip3Params p;
    p.ndim = indexer->ndim;
    p.total = indexer->total_size;
    const cumo_na_iarray_t* arr[4] = {a1, a2, a3, a4};
    for (int d = 0; d < CUMO_NA_MAX_DIMENSION; ++d) {
        p.shape[d] = d < indexer->ndim ? indexer->shape[d] : 1;
        for (int a = 0; a < 4; ++a) p.step[a][d] = d < indexer->ndim ? arr[a]->step[d] : 0;
    }
    for (int a = 0; a < 4; ++a) p.ptr[a] = arr[a]->ptr;
    p.invalid = invalid;
    uint64_t grid = (p.total + 255) / 256;
    if (grid > 65536) grid = 65536;
    hipLaunchKernelGGL((clip3_kernel<T>), dim3((unsigned)grid), dim3(256), 0, current_stream(), p);
    cumo_cuda_runtime_check_kernel_launch();
}

}  // namespace cumo_hip

#endif
