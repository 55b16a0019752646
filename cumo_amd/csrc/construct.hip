// Arrays made from a formula: seq (beg + step * i over the row-major element number i),
// logseq (base ** seq) and eye (a value on one diagonal, zero elsewhere).
//
// Replaces narray/gen/tmpl/seq_kernel.cu, logseq_kernel.cu and eye_kernel.cu of the
// reference with the same launcher symbols and arguments. The arithmetic is the
// reference's f_seq (types/float_macro_kernel.h:151-154, xint_macro_kernel.h:49-52):
// the float types compute beg + step * c in double and round once to the element type,
// Int32 computes in double and converts through a signed 64-bit integer.
#include "common.h"

#include <type_traits>

namespace cumo_hip {
namespace {

struct SeqParams {
    int ndim;
    uint64_t total;
    uint64_t shape[CUMO_NA_MAX_DIMENSION];
    int64_t step[CUMO_NA_MAX_DIMENSION];
    char* ptr;
};

template <class T>
__device__ __forceinline__ T seq_value(double beg, double step, double c) {
    const double v = beg + step * c;
    if (std::is_integral<T>::value) return (T)(int64_t)v;
    return (T)v;
}

// S: the type beg and step arrive in (the element type, or double for Int32)
template <class T, class S>
__global__ __launch_bounds__(256) void seq_kernel(SeqParams p, S beg, S step, double c) {
    for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < p.total; i += (uint64_t)gridDim.x * 256) {
        int64_t off;
        if (p.ndim == 1) {
            off = (int64_t)i * p.step[0];
        } else {
            uint64_t r = i;
            off = 0;
            for (int d = p.ndim - 1; d >= 0; --d) {
                const uint64_t n = p.shape[d];
                const uint64_t q = r / n;
                off += (int64_t)(r - q * n) * p.step[d];
                r = q;
            }
        }
        *reinterpret_cast<T*>(p.ptr + off) = seq_value<T>((double)beg, (double)step, c + (double)i);
    }
}

template <class T, class S>
void seq_launch(const cumo_na_iarray_t* a1, const cumo_na_indexer_t* indexer, S beg, S step, double c) {
    if (indexer->total_size == 0) return;
    SeqParams p;
    p.ndim = indexer->ndim < 1 ? 1 : indexer->ndim;
    p.total = indexer->total_size;
    for (int d = 0; d < CUMO_NA_MAX_DIMENSION; ++d) {
        p.shape[d] = d < indexer->ndim ? indexer->shape[d] : 1;
        p.step[d] = d < indexer->ndim ? a1->step[d] : 0;
    }
    p.ptr = a1->ptr;
    uint64_t grid = (p.total + 255) / 256;
    if (grid > 65536) grid = 65536;
    hipLaunchKernelGGL((seq_kernel<T, S>), dim3((unsigned)grid), dim3(256), 0, current_stream(), p, beg, step, c);
    cumo_cuda_runtime_check_kernel_launch();
}

// out = base ** x with x = the seq value rounded to the element type first
// (logseq_kernel.cu:5-15; m_pow is the double pow on the promoted arguments, stored once)
template <class T>
__global__ __launch_bounds__(256) void logseq_kernel(char* p1, int64_t s1, const size_t* idx1, T beg, T step, T base, double c, uint64_t n) {
    for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256) {
        const T x = seq_value<T>((double)beg, (double)step, c + (double)i);
        char* dst = idx1 ? p1 + idx1[i] : p1 + (int64_t)i * s1;
        *reinterpret_cast<T*>(dst) = (T)pow((double)base, (double)x);
    }
}

template <class T>
void logseq_launch(char* p1, ssize_t s1, size_t* idx1, T beg, T step, T base, double c, uint64_t n) {
    if (n == 0) return;
    uint64_t grid = (n + 255) / 256;
    if (grid > 65536) grid = 65536;
    hipLaunchKernelGGL((logseq_kernel<T>), dim3((unsigned)grid), dim3(256), 0, current_stream(), p1, (int64_t)s1, (const size_t*)idx1, beg, step, base,
                       c, n);
    cumo_cuda_runtime_check_kernel_launch();
}

// eye_kernel.cu:2-9; rows of n1 elements, a row's elements to consecutive lanes
template <class T>
__global__ __launch_bounds__(256) void eye_kernel(char* ptr, int64_t s0, int64_t s1, int64_t kofs, T data, uint64_t n1, uint64_t n) {
    for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256) {
        const uint64_t i0 = i / n1;
        const uint64_t i1 = i - i0 * n1;
        *reinterpret_cast<T*>(ptr + (int64_t)i0 * s0 + (int64_t)i1 * s1) = (i0 + (uint64_t)kofs == i1) ? data : (T)0;
    }
}

template <class T>
void eye_launch(char* ptr, ssize_t s0, ssize_t s1, ssize_t kofs, T data, uint64_t n0, uint64_t n1) {
    const uint64_t n = n0 * n1;
    if (n == 0) return;
    uint64_t grid = (n + 255) / 256;
    if (grid > 65536) grid = 65536;
    hipLaunchKernelGGL((eye_kernel<T>), dim3((unsigned)grid), dim3(256), 0, current_stream(), ptr, (int64_t)s0, (int64_t)s1, (int64_t)kofs, data, n1, n);
    cumo_cuda_runtime_check_kernel_launch();
}

}  // namespace
}  // namespace cumo_hip

using namespace cumo_hip;

extern "C" {

void cumo_iter_sfloat_seq_kernel_launch(cumo_na_iarray_t* a1, cumo_na_indexer_t* indexer, float beg, float step, double c) {
    seq_launch<float, float>(a1, indexer, beg, step, c);
}
void cumo_iter_dfloat_seq_kernel_launch(cumo_na_iarray_t* a1, cumo_na_indexer_t* indexer, double beg, double step, double c) {
    seq_launch<double, double>(a1, indexer, beg, step, c);
}
void cumo_iter_int32_seq_kernel_launch(cumo_na_iarray_t* a1, cumo_na_indexer_t* indexer, double beg, double step, double c) {
    seq_launch<int32_t, double>(a1, indexer, beg, step, c);
}

void cumo_iter_sfloat_logseq_stride_kernel_launch(char* p1, ssize_t s1, float beg, float step, float base, double c, uint64_t n) {
    logseq_launch<float>(p1, s1, nullptr, beg, step, base, c, n);
}
void cumo_iter_sfloat_logseq_index_kernel_launch(char* p1, size_t* idx1, float beg, float step, float base, double c, uint64_t n) {
    logseq_launch<float>(p1, 0, idx1, beg, step, base, c, n);
}
void cumo_iter_dfloat_logseq_stride_kernel_launch(char* p1, ssize_t s1, double beg, double step, double base, double c, uint64_t n) {
    logseq_launch<double>(p1, s1, nullptr, beg, step, base, c, n);
}
void cumo_iter_dfloat_logseq_index_kernel_launch(char* p1, size_t* idx1, double beg, double step, double base, double c, uint64_t n) {
    logseq_launch<double>(p1, 0, idx1, beg, step, base, c, n);
}

void cumo_iter_sfloat_eye_stride_kernel_launch(char* ptr, ssize_t s0, ssize_t s1, ssize_t kofs, float data, uint64_t n0, uint64_t n1) {
    eye_launch<float>(ptr, s0, s1, kofs, data, n0, n1);
}
void cumo_iter_dfloat_eye_stride_kernel_launch(char* ptr, ssize_t s0, ssize_t s1, ssize_t kofs, double data, uint64_t n0, uint64_t n1) {
    eye_launch<double>(ptr, s0, s1, kofs, data, n0, n1);
}
void cumo_iter_int32_eye_stride_kernel_launch(char* ptr, ssize_t s0, ssize_t s1, ssize_t kofs, int32_t data, uint64_t n0, uint64_t n1) {
    eye_launch<int32_t>(ptr, s0, s1, kofs, data, n0, n1);
}

}  // extern "C"
