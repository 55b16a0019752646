// Typed store/cast, view copy, fill and 0-dim construction
// (reference: narray/gen/tmpl/store_from_kernel.cu:3-53, narray/data_kernel.cu:47-132,
// narray/gen/tmpl/fill_kernel.cu:3-27, narray/gen/tmpl/new_dim0_kernel.cu:2-10).
#include "ew_kernels.h"
#include "ew_ops.h"

#include <cstring>

using namespace cumo_hip;

typedef float sfloat_c;
typedef double dfloat_c;
typedef int32_t int32_c;
typedef int64_t int64_c;

// a1 is the destination, a2 the source
#define CUMO_DEF_STORE(dst, src)                                                                             \
    extern "C" void cumo_iter_##dst##_store_##src##_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2, \
                                                                  cumo_na_indexer_t* indexer) {              \
        ew_launch(OpCast<dst##_c, src##_c>{}, a2, nullptr, a1, nullptr, indexer, (src##_c)0, 0, nullptr);    \
    }
CUMO_HIP_STORE_PAIRS(CUMO_DEF_STORE)

struct bytes16 {
    uint64_t lo, hi;
};

// a1 is the source, a2 the destination. A copy never looks at the element, so
// it is a cast between same-sized unsigned words; an odd element size becomes
// one more dimension of bytes.
extern "C" void cumo_iter_copy_bytes_indexer_kernel_launch(cumo_na_iarray_t* a1, cumo_na_iarray_t* a2,
                                                           cumo_na_indexer_t* indexer, ssize_t elmsz) {
    switch (elmsz) {
    case 1: ew_launch(OpCast<uint8_t, uint8_t>{}, a1, nullptr, a2, nullptr, indexer, (uint8_t)0, 0, nullptr); return;
    case 2: ew_launch(OpCast<uint16_t, uint16_t>{}, a1, nullptr, a2, nullptr, indexer, (uint16_t)0, 0, nullptr); return;
    case 4: ew_launch(OpCast<uint32_t, uint32_t>{}, a1, nullptr, a2, nullptr, indexer, (uint32_t)0, 0, nullptr); return;
    case 8: ew_launch(OpCast<uint64_t, uint64_t>{}, a1, nullptr, a2, nullptr, indexer, (uint64_t)0, 0, nullptr); return;
    default: break;
    }
    if (elmsz <= 0) return;
    if (indexer->ndim >= CUMO_NA_MAX_DIMENSION) {
        report_error(CUMO_HIP_ERROR_ARGUMENT, 0, "copy: element size needs a dimension more than the descriptor holds");
        return;
    }
    cumo_na_indexer_t ix = *indexer;
    cumo_na_iarray_t s = *a1, d = *a2;
    ix.shape[ix.ndim] = (size_t)elmsz;
    s.step[ix.ndim] = 1;
    d.step[ix.ndim] = 1;
    ix.ndim += 1;
    ix.total_size *= (size_t)elmsz;
    ew_launch(OpCast<uint8_t, uint8_t>{}, &s, nullptr, &d, nullptr, &ix, (uint8_t)0, 0, nullptr);
}

template <class T>
__global__ void set_one_kernel(T* ptr, T x) {
    *ptr = x;
}

#define CUMO_DEF_FILL(t, c)                                                                                      \
    extern "C" void cumo_iter_##t##_fill_kernel_launch(cumo_na_iarray_t* a1, cumo_na_indexer_t* indexer, c val) { \
        OpFill<c> op;                                                                                            \
        op.value = val;                                                                                          \
        ew_launch(op, nullptr, nullptr, a1, nullptr, indexer, (c)0, 0, nullptr);                                 \
    }                                                                                                            \
    extern "C" void cumo_##t##_new_dim0_kernel_launch(c* ptr, c x) {                                             \
        hipLaunchKernelGGL((set_one_kernel<c>), dim3(1), dim3(1), 0, current_stream(), ptr, x);                  \
        cumo_cuda_runtime_check_kernel_launch();                                                                 \
    }
CUMO_DEF_FILL(sfloat, float)
CUMO_DEF_FILL(dfloat, double)
CUMO_DEF_FILL(int32, int32_t)

// the common new_dim0 template rendered for Bit: one whole word
extern "C" void cumo_bit_new_dim0_kernel_launch(unsigned int* ptr, unsigned int x) {
    hipLaunchKernelGGL((set_one_kernel<unsigned int>), dim3(1), dim3(1), 0, current_stream(), ptr, x);
    cumo_cuda_runtime_check_kernel_launch();
}

// A fill kernel rather than hipMemsetAsync, so that a caller may capture it.
extern "C" void cumo_hip_memset(void* dst, int byte, size_t n) {
    if (n == 0) return;
    cumo_na_iarray_t a;
    cumo_na_indexer_t ix;
    std::memset(&a, 0, sizeof(a));
    std::memset(&ix, 0, sizeof(ix));
    OpFill<uint8_t> op;
    op.value = (uint8_t)byte;
    if (((uintptr_t)dst % 4) == 0 && (n % 4) == 0) {
        OpFill<uint32_t> op4;
        op4.value = 0x01010101u * (uint8_t)byte;
        a.ptr = (char*)dst;
        a.step[0] = 4;
        ix.ndim = 1;
        ix.total_size = n / 4;
        ix.shape[0] = n / 4;
        ew_launch(op4, nullptr, nullptr, &a, nullptr, &ix, (uint32_t)0, 0, nullptr);
        return;
    }
    a.ptr = (char*)dst;
    a.step[0] = 1;
    ix.ndim = 1;
    ix.total_size = n;
    ix.shape[0] = n;
    ew_launch(op, nullptr, nullptr, &a, nullptr, &ix, (uint8_t)0, 0, nullptr);
}
