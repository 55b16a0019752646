// The rest of the Bit template set: all? / any?, fill, number -> Bit store, and
// ingest of a packed host buffer (store_array).
//
// Replaces ext/cumo/narray/gen/tmpl_bit/{bit_reduce,fill,store_from,store_array}_kernel.cu
// of the reference, under the same launcher symbols and argument lists
// (tmpl_bit/bit_reduce.c:1-3, fill.c:1-2, store_from.c:2, store_array.c:1-5).
// The reference's kernels take one thread per bit and two atomics per stored bit
// (template_kernel.h:26-35). Here every contiguous run is handled a 32-bit word at a
// time (a wave's ballot packs the bits of a number -> Bit store; masked word compares
// answer all? / any?), and atomics are left for the words a run shares with its
// neighbours and for strided or indexed destinations.
#include "bit_common.h"

using namespace cumo_hip;

namespace {

__device__ __forceinline__ uint64_t bit_pos(uint64_t p, int64_t s, const size_t* idx, uint64_t i) {
    return idx ? (p + idx[i]) : (uint64_t)((int64_t)p + (int64_t)i * s);
}

// mask of the bits of word w that belong to the run [p, p + n)
__device__ __forceinline__ uint32_t run_mask(uint64_t p, uint64_t n, uint64_t w) {
    const uint64_t lo_bit = w << 5, end = p + n;
    if (lo_bit + 32 <= p || lo_bit >= end) return 0u;
    const unsigned lo = p > lo_bit ? (unsigned)(p - lo_bit) : 0u;
    const unsigned hi = end - lo_bit >= 32 ? 32u : (unsigned)(end - lo_bit);
    return low_bits(hi) & ~low_bits(lo);
}

// word w of the destination takes `bits` under `mask`; words that lie wholly inside the
// run are plain stores, the run's edge words may be shared with other writers
__device__ __forceinline__ void store_word_masked(CUMO_BIT_DIGIT* a, uint64_t w, uint32_t bits, uint32_t mask) {
    if (mask == 0xffffffffu) {
        a[w] = bits;
    } else if (mask) {
        atomicOr(&a[w], bits & mask);
        atomicAnd(&a[w], bits | ~mask);
    }
}

// ---- all? / any? ---------------------------------------------------------------
// INIT is the bit the result starts from (1 for all?, 0 for any?); an element that
// differs from it flips the result, and nothing ever flips it back.
template <int INIT>
__device__ __forceinline__ void flip_result(CUMO_BIT_DIGIT* a2, uint64_t q2) {
    if (INIT) atomicAnd(&a2[q2 >> 5], ~(1u << (q2 & 31)));
    else atomicOr(&a2[q2 >> 5], 1u << (q2 & 31));
}

template <int INIT>
__global__ __launch_bounds__(kBlock) void bit_reduce_elementwise_kernel(const CUMO_BIT_DIGIT* a1, uint64_t p1, int64_t s1, const size_t* idx1,
                                                                        CUMO_BIT_DIGIT* a2, uint64_t p2, int64_t s2, const size_t* idx2, uint64_t n) {
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (uint64_t)gridDim.x * kBlock) {
        if (load_bit(a1, bit_pos(p1, s1, idx1, i)) != (uint32_t)INIT) flip_result<INIT>(a2, bit_pos(p2, s2, idx2, i));
    }
}

// every element answers the same result bit: a block folds its lanes to one flag
template <int INIT>
__global__ __launch_bounds__(kBlock) void bit_reduce_gather_kernel(const CUMO_BIT_DIGIT* a1, uint64_t p1, int64_t s1, const size_t* idx1,
                                                                   CUMO_BIT_DIGIT* a2, uint64_t p2, uint64_t n) {
    int flip = 0;
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (uint64_t)gridDim.x * kBlock)
        flip |= load_bit(a1, bit_pos(p1, s1, idx1, i)) != (uint32_t)INIT;
    if (__syncthreads_or(flip) && threadIdx.x == 0) flip_result<INIT>(a2, p2);
}

// a1 is 16-byte aligned (the launcher moves the pointer back); 128-bit loads, edge words masked
template <int INIT>
__global__ __launch_bounds__(kBlock) void bit_reduce_words_kernel(const CUMO_BIT_DIGIT* a1, uint64_t p1, CUMO_BIT_DIGIT* a2, uint64_t p2, uint64_t n) {
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    const uint32_t init_word = INIT ? 0xffffffffu : 0u;
    const uint64_t w1 = (p1 + n + 31) >> 5;
    const uint64_t v0 = (p1 >> 5) >> 2, v1 = (w1 + 3) >> 2;
    int flip = 0;
    for (uint64_t v = v0 + (uint64_t)blockIdx.x * kBlock + threadIdx.x; v < v1; v += (uint64_t)gridDim.x * kBlock) {
        const uint64_t w = v << 2;
        if (w >= (p1 >> 5) + 1 && w + 4 < w1) {  // four whole words of the run
            const u4 x = *reinterpret_cast<const u4*>(a1 + w);
            flip |= ((x.x ^ init_word) | (x.y ^ init_word) | (x.z ^ init_word) | (x.w ^ init_word)) != 0;
        } else {
            for (uint64_t k = w; k < w + 4 && k < w1; ++k) {
                const uint32_t m = run_mask(p1, n, k);
                if (m) flip |= ((a1[k] ^ init_word) & m) != 0;
            }
        }
    }
    if (__syncthreads_or(flip) && threadIdx.x == 0) flip_result<INIT>(a2, p2);
}

template <int INIT>
void launch_reduce_elementwise(CUMO_BIT_DIGIT* a1, size_t p1, ssize_t s1, size_t* idx1, CUMO_BIT_DIGIT* a2, size_t p2, ssize_t s2, size_t* idx2,
                               uint64_t n) {
    if (n == 0) return;
    hipLaunchKernelGGL((bit_reduce_elementwise_kernel<INIT>), dim3(grid_for(n)), dim3(kBlock), 0, current_stream(), (const CUMO_BIT_DIGIT*)a1,
                       (uint64_t)p1, (int64_t)s1, (const size_t*)idx1, a2, (uint64_t)p2, (int64_t)s2, (const size_t*)idx2, n);
    cumo_cuda_runtime_check_kernel_launch();
}

template <int INIT>
void launch_reduce_words(CUMO_BIT_DIGIT* a1, size_t p1, CUMO_BIT_DIGIT* a2, size_t p2, uint64_t n) {
    if (n == 0) return;
    // whole 128-bit vectors: move the word pointer back to a 16-byte boundary
    const uintptr_t back = ((uintptr_t)a1 & 15) / sizeof(CUMO_BIT_DIGIT);
    a1 -= back;
    p1 += back * 32;
    const uint64_t vecs = ((p1 + n + 31) / 32 + 3) / 4 - (p1 / 32) / 4;
    hipLaunchKernelGGL((bit_reduce_words_kernel<INIT>), dim3(grid_for(vecs)), dim3(kBlock), 0, current_stream(), (const CUMO_BIT_DIGIT*)a1,
                       (uint64_t)p1, a2, (uint64_t)p2, n);
    cumo_cuda_runtime_check_kernel_launch();
}

template <int INIT>
void launch_reduce_gather(CUMO_BIT_DIGIT* a1, size_t p1, ssize_t s1, size_t* idx1, CUMO_BIT_DIGIT* a2, size_t p2, uint64_t n) {
    if (n == 0) return;
    if (!idx1 && s1 == 1) {
        launch_reduce_words<INIT>(a1, p1, a2, p2, n);
        return;
    }
    hipLaunchKernelGGL((bit_reduce_gather_kernel<INIT>), dim3(grid_for(n)), dim3(kBlock), 0, current_stream(), (const CUMO_BIT_DIGIT*)a1, (uint64_t)p1,
                       (int64_t)s1, (const size_t*)idx1, a2, (uint64_t)p2, n);
    cumo_cuda_runtime_check_kernel_launch();
}

// ---- counts -> bits -----------------------------------------------------------------
// bit i of the run that starts at bit `pos` of dst = (counts[i] != 0), or (counts[i] == 0) with
// zero_is_one: what all? / any? along axes make of the counts of clear / set bits. The bits of the
// run's first and last word that lie outside it stay.
__global__ __launch_bounds__(kBlock) void bit_from_counts_kernel(const uint64_t* counts, uint64_t n, int zero_is_one, CUMO_BIT_DIGIT* dst, uint64_t pos) {
    // lane t of the grid owns bit t of dst (pos < 32): a wave's ballot packs 64 of them, and the lanes at 0 and 32 store the two words
    const uint64_t span = pos + n;
    const uint64_t rounds = (span + (uint64_t)gridDim.x * kBlock - 1) / ((uint64_t)gridDim.x * kBlock);
    for (uint64_t r = 0; r < rounds; ++r) {
        const uint64_t q = (r * gridDim.x + blockIdx.x) * (uint64_t)kBlock + threadIdx.x;  // whole waves stay together
        bool on = false;
        if (q >= pos && q < span) on = (counts[q - pos] == 0) == (zero_is_one != 0);
        const uint64_t ballot = __ballot(on);
        const unsigned lane = threadIdx.x & 63;
        if ((lane & 31) == 0) {
            const uint64_t w = q >> 5;
            store_word_masked(dst, w, (uint32_t)(ballot >> lane), run_mask(pos, n, w));
        }
    }
}

// ---- fill --------------------------------------------------------------------------
__global__ __launch_bounds__(kBlock) void bit_fill_words_kernel(CUMO_BIT_DIGIT* a3, uint64_t p3, uint64_t n, uint32_t word) {
    const uint64_t w0 = p3 >> 5, w1 = (p3 + n + 31) >> 5;
    for (uint64_t w = w0 + (uint64_t)blockIdx.x * kBlock + threadIdx.x; w < w1; w += (uint64_t)gridDim.x * kBlock)
        store_word_masked(a3, w, word, run_mask(p3, n, w));
}

__global__ __launch_bounds__(kBlock) void bit_fill_generic_kernel(cumo_na_bit_iarray_stridx_t a3, uint32_t bit, BitNd nd) {
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < nd.total; i += (uint64_t)gridDim.x * kBlock)
        store_bit_atomic(a3.ptr, a3.pos + (uint64_t)stridx_offset(a3.stridx, nd, i), bit);
}

void launch_fill_words(CUMO_BIT_DIGIT* a3, size_t p3, uint64_t n, CUMO_BIT_DIGIT y) {
    if (n == 0) return;
    const uint32_t word = (y & 1u) ? 0xffffffffu : 0u;
    hipLaunchKernelGGL(bit_fill_words_kernel, dim3(grid_for((p3 % 32 + n + 31) / 32)), dim3(kBlock), 0, current_stream(), a3, (uint64_t)p3, n, word);
    cumo_cuda_runtime_check_kernel_launch();
}

// ---- number -> Bit (nonzero is 1: types/bit_kernel.h:13-19) ---------------------------
// The destination is one run of step 1 and the source one run of elements: lane t of the
// grid owns absolute bit position (p1 rounded down to a word) + t, a wave's ballot packs 64
// of them, and the lanes at 0 and 32 store the two words.
template <class T>
__global__ __launch_bounds__(kBlock) void bit_store_from_run_kernel(CUMO_BIT_DIGIT* a1, uint64_t p1, const char* src, int64_t s2, uint64_t n) {
    const uint64_t base = p1 & ~(uint64_t)31;
    const uint64_t span = (p1 - base) + n;
    const uint64_t rounds = (span + (uint64_t)gridDim.x * kBlock - 1) / ((uint64_t)gridDim.x * kBlock);
    for (uint64_t r = 0; r < rounds; ++r) {
        const uint64_t t = (r * gridDim.x + blockIdx.x) * (uint64_t)kBlock + threadIdx.x;  // whole waves stay together
        const uint64_t q = base + t;
        const bool mine = q >= p1 && q < p1 + n;
        bool on = false;
        if (mine) on = *reinterpret_cast<const T*>(src + (int64_t)(q - p1) * s2) != (T)0;
        const uint64_t ballot = __ballot(on);
        const unsigned lane = threadIdx.x & 63;
        if ((lane & 31) == 0) {
            const uint64_t w = q >> 5;
            store_word_masked(a1, w, (uint32_t)(ballot >> lane), run_mask(p1, n, w));
        }
    }
}

template <class T>
__global__ __launch_bounds__(kBlock) void bit_store_from_generic_kernel(cumo_na_bit_iarray_stridx_t a1, cumo_na_iarray_stridx_t a2, BitNd nd) {
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < nd.total; i += (uint64_t)gridDim.x * kBlock) {
        const T x = *reinterpret_cast<const T*>(a2.ptr + stridx_offset(a2.stridx, nd, i));
        store_bit_atomic(a1.ptr, a1.pos + (uint64_t)stridx_offset(a1.stridx, nd, i), x != (T)0 ? 1u : 0u);
    }
}

template <class T>
void launch_store_from(cumo_na_bit_iarray_stridx_t* a1, cumo_na_iarray_stridx_t* a2, cumo_na_indexer_t* indexer) {
    const uint64_t n = indexer->total_size;
    if (n == 0) return;
    hipStream_t st = current_stream();
    if (indexer->ndim == 1 && CUMO_SDX_IS_STRIDE(a1->stridx[0]) && CUMO_SDX_GET_STRIDE(a1->stridx[0]) == 1 && CUMO_SDX_IS_STRIDE(a2->stridx[0])) {
        const uint64_t span = a1->pos % 32 + n;
        hipLaunchKernelGGL((bit_store_from_run_kernel<T>), dim3(grid_for(span)), dim3(kBlock), 0, st, a1->ptr, (uint64_t)a1->pos, (const char*)a2->ptr,
                           (int64_t)CUMO_SDX_GET_STRIDE(a2->stridx[0]), n);
    } else {
        BitNd nd = make_nd(indexer);
        hipLaunchKernelGGL((bit_store_from_generic_kernel<T>), dim3(grid_for(n)), dim3(kBlock), 0, st, *a1, *a2, nd);
    }
    cumo_cuda_runtime_check_kernel_launch();
}

// ---- store_array: bits of a packed staging buffer (bit 0 first) into a run ----------------
__global__ __launch_bounds__(kBlock) void bit_store_array_scatter_kernel(CUMO_BIT_DIGIT* a1, uint64_t p1, int64_t s1, const size_t* idx1,
                                                                         const CUMO_BIT_DIGIT* z, uint32_t scalar, int use_scalar, uint64_t n) {
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (uint64_t)gridDim.x * kBlock) {
        const uint32_t y = use_scalar ? (scalar & 1u) : load_bit(z, i);
        store_bit_atomic(a1, bit_pos(p1, s1, idx1, i), y);
    }
}

__global__ __launch_bounds__(kBlock) void bit_store_array_words_kernel(CUMO_BIT_DIGIT* a1, uint64_t p1, const CUMO_BIT_DIGIT* z, uint64_t n) {
    const uint64_t w0 = p1 >> 5, w1 = (p1 + n + 31) >> 5, nz = (n + 31) >> 5;
    for (uint64_t w = w0 + (uint64_t)blockIdx.x * kBlock + threadIdx.x; w < w1; w += (uint64_t)gridDim.x * kBlock) {
        // staging bit of this word's bit 0 (negative inside the first word)
        const uint32_t x = bits_at(z, (int64_t)(w << 5) - (int64_t)p1, nz);
        store_word_masked(a1, w, x, run_mask(p1, n, w));
    }
}

void launch_store_array_scatter(CUMO_BIT_DIGIT* a1, size_t p1, ssize_t s1, size_t* idx1, CUMO_BIT_DIGIT* z, CUMO_BIT_DIGIT scalar, int use_scalar,
                                uint64_t n) {
    if (n == 0) return;
    if (use_scalar && !idx1 && s1 == 1) {
        launch_fill_words(a1 + p1 / 32, p1 % 32, n, scalar);
        return;
    }
    hipLaunchKernelGGL(bit_store_array_scatter_kernel, dim3(grid_for(n)), dim3(kBlock), 0, current_stream(), a1, (uint64_t)p1, (int64_t)s1,
                       (const size_t*)idx1, (const CUMO_BIT_DIGIT*)z, (uint32_t)scalar, use_scalar, n);
    cumo_cuda_runtime_check_kernel_launch();
}

}  // namespace

#define CUMO_DEF_BIT_REDUCE(name, INIT)                                                                                            \
    extern "C" void cumo_iter_bit_##name##_elementwise_kernel_launch(CUMO_BIT_DIGIT* a1, size_t p1, ssize_t s1, size_t* idx1,      \
                                                                     CUMO_BIT_DIGIT* a2, size_t p2, ssize_t s2, size_t* idx2,      \
                                                                     uint64_t n) {                                                 \
        launch_reduce_elementwise<INIT>(a1, p1, s1, idx1, a2, p2, s2, idx2, n);                                                    \
    }                                                                                                                              \
    extern "C" void cumo_iter_bit_##name##_reduce_kernel_launch(CUMO_BIT_DIGIT* a1, size_t p1, ssize_t s1, size_t* idx1,           \
                                                                CUMO_BIT_DIGIT* a2, size_t p2, uint64_t n) {                       \
        launch_reduce_gather<INIT>(a1, p1, s1, idx1, a2, p2, n);                                                                   \
    }                                                                                                                              \
    extern "C" void cumo_iter_bit_##name##_contiguous_reduce_kernel_launch(CUMO_BIT_DIGIT* a1, size_t p1, CUMO_BIT_DIGIT* a2,      \
                                                                           size_t p2, uint64_t n) {                                \
        launch_reduce_words<INIT>(a1, p1, a2, p2, n);                                                                              \
    }
CUMO_DEF_BIT_REDUCE(all_p, 1)
CUMO_DEF_BIT_REDUCE(any_p, 0)

extern "C" void cumo_iter_bit_fill_kernel_launch(cumo_na_bit_iarray_stridx_t* a3, CUMO_BIT_DIGIT y, cumo_na_indexer_t* indexer) {
    if (indexer->total_size == 0) return;
    if (indexer->ndim == 1 && CUMO_SDX_IS_STRIDE(a3->stridx[0]) && CUMO_SDX_GET_STRIDE(a3->stridx[0]) == 1) {
        launch_fill_words(a3->ptr + a3->pos / 32, a3->pos % 32, indexer->total_size, y);
        return;
    }
    BitNd nd = make_nd(indexer);
    hipLaunchKernelGGL(bit_fill_generic_kernel, dim3(grid_for(nd.total)), dim3(kBlock), 0, current_stream(), *a3, (uint32_t)(y & 1u), nd);
    cumo_cuda_runtime_check_kernel_launch();
}

// y is all ones or zero here (tmpl_bit/fill.c:27-36); only its lowest bit is looked at
extern "C" void cumo_iter_bit_fill_contiguous_kernel_launch(CUMO_BIT_DIGIT* a3, size_t p3, uint64_t n, CUMO_BIT_DIGIT y) {
    launch_fill_words(a3, p3, n, y);
}

#define CUMO_DEF_BIT_STORE_FROM(t, c)                                                                                          \
    extern "C" void cumo_iter_bit_store_##t##_kernel_launch(cumo_na_bit_iarray_stridx_t* a1, cumo_na_iarray_stridx_t* a2,      \
                                                            cumo_na_indexer_t* indexer) {                                      \
        launch_store_from<c>(a1, a2, indexer);                                                                                 \
    }
CUMO_DEF_BIT_STORE_FROM(sfloat, float)
CUMO_DEF_BIT_STORE_FROM(dfloat, double)
CUMO_DEF_BIT_STORE_FROM(int32, int32_t)
CUMO_DEF_BIT_STORE_FROM(int64, int64_t)
CUMO_DEF_BIT_STORE_FROM(uint64, uint64_t)

extern "C" void cumo_iter_bit_store_array_index_kernel_launch(CUMO_BIT_DIGIT* a1, size_t p1, size_t* idx1, CUMO_BIT_DIGIT* z, uint64_t n) {
    launch_store_array_scatter(a1, p1, 0, idx1, z, 0, 0, n);
}
extern "C" void cumo_iter_bit_store_array_stride_kernel_launch(CUMO_BIT_DIGIT* a1, size_t p1, ssize_t s1, CUMO_BIT_DIGIT* z, uint64_t n) {
    launch_store_array_scatter(a1, p1, s1, nullptr, z, 0, 0, n);
}
extern "C" void cumo_iter_bit_store_array_contiguous_kernel_launch(CUMO_BIT_DIGIT* a1, size_t p1, CUMO_BIT_DIGIT* z, uint64_t n) {
    if (n == 0) return;
    hipLaunchKernelGGL(bit_store_array_words_kernel, dim3(grid_for((p1 % 32 + n + 31) / 32)), dim3(kBlock), 0, current_stream(), a1, (uint64_t)p1,
                       (const CUMO_BIT_DIGIT*)z, n);
    cumo_cuda_runtime_check_kernel_launch();
}
extern "C" void cumo_iter_bit_store_array_index_scalar_kernel_launch(CUMO_BIT_DIGIT* a1, size_t p1, size_t* idx1, CUMO_BIT_DIGIT z, uint64_t n) {
    launch_store_array_scatter(a1, p1, 0, idx1, nullptr, z, 1, n);
}
extern "C" void cumo_iter_bit_store_array_stride_scalar_kernel_launch(CUMO_BIT_DIGIT* a1, size_t p1, ssize_t s1, CUMO_BIT_DIGIT z, uint64_t n) {
    launch_store_array_scatter(a1, p1, s1, nullptr, nullptr, z, 1, n);
}

extern "C" void cumo_hip_bit_from_counts_kernel_launch(const uint64_t* counts, uint64_t n, int zero_is_one, CUMO_BIT_DIGIT* dst, size_t pos) {
    if (n == 0) return;
    dst += pos / 32;
    pos %= 32;
    hipLaunchKernelGGL(bit_from_counts_kernel, dim3(grid_for(pos + n)), dim3(kBlock), 0, current_stream(), counts, n, zero_is_one, dst,
                       (uint64_t)pos);
    cumo_cuda_runtime_check_kernel_launch();
}
