// Bit (1 bit per element, LSB first in 32-bit words) kernels: logical ops,
// count_true / count_false, Bit -> number.
//
// Replaces ext/cumo/narray/gen/tmpl_bit/{binary,unary,bit_count}_kernel.cu and
// narray/gen/tmpl/store_bit_kernel.cu of the reference. count_* there is one
// thread per bit and one 64-bit global atomicAdd per set bit
// (tmpl_bit/bit_count_kernel.cu:15-24); here a contiguous run is counted by
// popcount over whole words, reduced across the wave with shuffles and across
// the block through LDS, and each block adds its total once. Integer addition
// commutes, so the answer does not depend on the order the blocks arrive in.
#include "bit_common.h"

#include <cstring>
#include <mutex>
#include <unordered_map>

using namespace cumo_hip;

namespace {

// counting ends in one atomic add per block on a single word, so fewer, longer
// blocks: one per compute unit
constexpr unsigned kCountGridCap = kNumCU;

enum { B_AND, B_OR, B_XOR, B_EQ, B_COPY, B_NOT };

template <int OP>
__device__ __forceinline__ uint32_t bit_apply(uint32_t x, uint32_t y) {
    switch (OP) {
    case B_AND: return x & y;
    case B_OR: return x | y;
    case B_XOR: return x ^ y;
    case B_EQ: return ~(x ^ y);
    case B_COPY: return x;
    default: return ~x;
    }
}

// z[p3 + i] = op(x[p1 + i], y[p2 + i]) for i in [0, n): one output word per thread
template <int OP, bool BINARY>
__global__ __launch_bounds__(kBlock) void bit_contiguous_kernel(const CUMO_BIT_DIGIT* a1, uint64_t p1, const CUMO_BIT_DIGIT* a2,
                                                                uint64_t p2, CUMO_BIT_DIGIT* a3, uint64_t p3, uint64_t n) {
    const uint64_t nw1 = (p1 + n + 31) >> 5, nw2 = (p2 + n + 31) >> 5, nw3 = (p3 + n + 31) >> 5;
    for (uint64_t w = (uint64_t)blockIdx.x * kBlock + threadIdx.x; w < nw3; w += (uint64_t)gridDim.x * kBlock) {
        // element index of bit 0 of this output word (negative inside the first word)
        const int64_t e0 = (int64_t)(w << 5) - (int64_t)p3;
        const uint32_t x = bits_at(a1, e0 + (int64_t)p1, nw1);
        const uint32_t y = BINARY ? bits_at(a2, e0 + (int64_t)p2, nw2) : 0u;
        const uint32_t z = bit_apply<OP>(x, y);
        const unsigned lo = (w == 0) ? (unsigned)p3 : 0u;
        const uint64_t endbit = p3 + n;
        const unsigned hi = ((w + 1) << 5) <= endbit ? 32u : (unsigned)(endbit - (w << 5));
        const uint32_t mask = low_bits(hi) & ~low_bits(lo);
        // one thread owns a word, so the shared edge words need no atomic
        if (mask == 0xffffffffu) a3[w] = z;
        else a3[w] = (z & mask) | (a3[w] & ~mask);
    }
}

template <int OP, bool BINARY>
__global__ __launch_bounds__(kBlock) void bit_generic_kernel(cumo_na_bit_iarray_stridx_t a1, cumo_na_bit_iarray_stridx_t a2,
                                                             cumo_na_bit_iarray_stridx_t a3, BitNd nd) {
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < nd.total; i += (uint64_t)gridDim.x * kBlock) {
        const uint32_t x = load_bit(a1.ptr, a1.pos + (uint64_t)stridx_offset(a1.stridx, nd, i));
        const uint32_t y = BINARY ? load_bit(a2.ptr, a2.pos + (uint64_t)stridx_offset(a2.stridx, nd, i)) : 0u;
        store_bit_atomic(a3.ptr, a3.pos + (uint64_t)stridx_offset(a3.stridx, nd, i), bit_apply<OP>(x, y) & 1u);
    }
}

template <class T>
__global__ __launch_bounds__(kBlock) void store_bit_kernel(cumo_na_iarray_stridx_t dst, cumo_na_bit_iarray_stridx_t src, BitNd nd) {
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < nd.total; i += (uint64_t)gridDim.x * kBlock) {
        const uint32_t x = load_bit(src.ptr, src.pos + (uint64_t)stridx_offset(src.stridx, nd, i));
        *reinterpret_cast<T*>(dst.ptr + stridx_offset(dst.stridx, nd, i)) = (T)x;
    }
}

// ---- counting -------------------------------------------------------------------
__device__ __forceinline__ uint64_t block_sum_u64(uint64_t v) {
    __shared__ uint64_t wave_sum[kBlock / 64];
    for (unsigned d = 32; d > 0; d >>= 1) {
        const uint32_t lo = __shfl_down((uint32_t)v, d);
        const uint32_t hi = __shfl_down((uint32_t)(v >> 32), d);
        v += ((uint64_t)hi << 32) | lo;
    }
    if ((threadIdx.x & 63) == 0) wave_sum[threadIdx.x >> 6] = v;
    __syncthreads();
    uint64_t t = 0;
    if (threadIdx.x == 0) {
        for (int w = 0; w < kBlock / 64; ++w) t += wave_sum[w];
    }
    return t;  // valid in thread 0
}

// bits [p1, p1 + n) of a, step 1: whole words, edges masked
template <bool COUNT_FALSE>
__global__ __launch_bounds__(kBlock) void bit_count_words_kernel(const CUMO_BIT_DIGIT* a, uint64_t p1, uint64_t n, unsigned long long* out) {
    const uint64_t w0 = p1 >> 5;
    const uint64_t endbit = p1 + n;
    const uint64_t w1 = (endbit + 31) >> 5;
    uint64_t c = 0;
    for (uint64_t w = w0 + (uint64_t)blockIdx.x * kBlock + threadIdx.x; w < w1; w += (uint64_t)gridDim.x * kBlock) {
        uint32_t x = a[w];
        if (COUNT_FALSE) x = ~x;
        const unsigned lo = (w == w0) ? (unsigned)(p1 & 31) : 0u;
        const unsigned hi = ((w + 1) << 5) <= endbit ? 32u : (unsigned)(endbit - (w << 5));
        x &= low_bits(hi) & ~low_bits(lo);
        c += (uint64_t)__popc(x);
    }
    const uint64_t t = block_sum_u64(c);
    if (threadIdx.x == 0 && t) atomicAdd(out, (unsigned long long)t);
}

// The same count in one launch that needs no zeroed result: every block adds its total
// and a "one more block done" mark to a ticket word with ONE atomic (count in the low
// 44 bits, blocks done above them), so the block whose atomic answers "all others were
// here before me" also holds the grand total, stores it and puts the ticket back to 0.
// Nothing but that single word is shared between blocks, so no fence is needed.
// Lanes read 128 bits; the words of the run's first and last vector are masked one by one.
constexpr int kTicketSlots = 64;
constexpr int kTicketShift = 44;
__device__ unsigned long long g_count_ticket[kTicketSlots];

template <bool COUNT_FALSE>
__global__ __launch_bounds__(kBlock) void bit_count_words_store_kernel(const CUMO_BIT_DIGIT* a, uint64_t p1, uint64_t n, unsigned long long* ticket,
                                                                       unsigned long long* out) {
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    const uint64_t endbit = p1 + n;
    const uint64_t w0 = p1 >> 5, w1 = (endbit + 31) >> 5;  // a is 16-byte aligned
    const uint64_t v0 = w0 >> 2, v1 = (w1 + 3) >> 2;
    uint64_t c = 0;
    const uint64_t stride = (uint64_t)gridDim.x * kBlock;
    uint64_t v = v0 + (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    // four interior vectors per lane in flight
    for (; v > v0 && v + 3 * stride + 1 < v1 - 1; v += 4 * stride) {
        u4 x[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) x[u] = *reinterpret_cast<const u4*>(a + ((v + u * stride) << 2));
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (COUNT_FALSE) x[u] = ~x[u];
            c += (uint64_t)(__popc(x[u].x) + __popc(x[u].y) + __popc(x[u].z) + __popc(x[u].w));
        }
    }
    for (; v < v1; v += stride) {
        const uint64_t w = v << 2;
        if (w >= w0 + 1 && w + 4 < w1) {  // four whole words of the run
            u4 x = *reinterpret_cast<const u4*>(a + w);
            if (COUNT_FALSE) x = ~x;
            c += (uint64_t)(__popc(x.x) + __popc(x.y) + __popc(x.z) + __popc(x.w));
        } else {
            for (uint64_t k = (w < w0 ? w0 : w); k < w + 4 && k < w1; ++k) {
                uint32_t x = a[k];
                if (COUNT_FALSE) x = ~x;
                const unsigned lo = (k == w0) ? (unsigned)(p1 & 31) : 0u;
                const unsigned hi = ((k + 1) << 5) <= endbit ? 32u : (unsigned)(endbit - (k << 5));
                x &= low_bits(hi) & ~low_bits(lo);
                c += (uint64_t)__popc(x);
            }
        }
    }
    const uint64_t t = block_sum_u64(c);
    if (threadIdx.x == 0) {
        const unsigned long long mine = (1ull << kTicketShift) | (unsigned long long)t;
        const unsigned long long before = atomicAdd(ticket, mine);
        if ((before >> kTicketShift) == (unsigned long long)gridDim.x - 1) {
            *out = (before + mine) & ((1ull << kTicketShift) - 1);
            atomicExch(ticket, 0ull);
        }
    }
}

// any stride or an index array, all into one counter
template <bool COUNT_FALSE>
__global__ __launch_bounds__(kBlock) void bit_count_gather_kernel(const CUMO_BIT_DIGIT* a, uint64_t p1, int64_t s1, const size_t* idx1,
                                                                  uint64_t n, unsigned long long* out) {
    uint64_t c = 0;
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (uint64_t)gridDim.x * kBlock) {
        const uint64_t pos = idx1 ? (p1 + idx1[i]) : (uint64_t)((int64_t)p1 + (int64_t)i * s1);
        const uint32_t x = load_bit(a, pos);
        c += COUNT_FALSE ? (x == 0) : (x != 0);
    }
    const uint64_t t = block_sum_u64(c);
    if (threadIdx.x == 0 && t) atomicAdd(out, (unsigned long long)t);
}

// element i goes to its own counter at p2 + i*s2 (s2 != 0), so nothing is shared
template <bool COUNT_FALSE>
__global__ __launch_bounds__(kBlock) void bit_count_scatter_kernel(const CUMO_BIT_DIGIT* a, uint64_t p1, int64_t s1, const size_t* idx1,
                                                                   char* p2, int64_t s2, uint64_t n) {
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (uint64_t)gridDim.x * kBlock) {
        const uint64_t pos = idx1 ? (p1 + idx1[i]) : (uint64_t)((int64_t)p1 + (int64_t)i * s1);
        const uint32_t x = load_bit(a, pos);
        if (COUNT_FALSE ? (x == 0) : (x != 0)) *reinterpret_cast<uint64_t*>(p2 + (int64_t)i * s2) += 1;
    }
}

template <int OP, bool BINARY>
void launch_contiguous(CUMO_BIT_DIGIT* a1, size_t p1, CUMO_BIT_DIGIT* a2, size_t p2, CUMO_BIT_DIGIT* a3, size_t p3, uint64_t n) {
    if (n == 0) return;
    const uint64_t nw3 = (p3 + n + 31) >> 5;
    hipLaunchKernelGGL((bit_contiguous_kernel<OP, BINARY>), dim3(grid_for(nw3)), dim3(kBlock), 0, current_stream(), a1, (uint64_t)p1, a2,
                       (uint64_t)p2, a3, (uint64_t)p3, n);
    cumo_cuda_runtime_check_kernel_launch();
}

bool flat_stride1(const cumo_na_bit_iarray_stridx_t* a, int ndim) {
    return ndim == 1 && CUMO_SDX_IS_STRIDE(a->stridx[0]) && CUMO_SDX_GET_STRIDE(a->stridx[0]) == 1;
}

template <int OP, bool BINARY>
void launch_generic(cumo_na_bit_iarray_stridx_t* a1, cumo_na_bit_iarray_stridx_t* a2, cumo_na_bit_iarray_stridx_t* a3,
                    cumo_na_indexer_t* indexer) {
    if (indexer->total_size == 0) return;
    // the host iterator already routes the flat case to the word kernel
    // (tmpl_bit/binary.c:17-31); do the same for callers that do not
    if (flat_stride1(a1, indexer->ndim) && (!BINARY || flat_stride1(a2, indexer->ndim)) && flat_stride1(a3, indexer->ndim)) {
        launch_contiguous<OP, BINARY>(a1->ptr + a1->pos / 32, a1->pos % 32, BINARY ? a2->ptr + a2->pos / 32 : nullptr,
                                      BINARY ? a2->pos % 32 : 0, a3->ptr + a3->pos / 32, a3->pos % 32, indexer->total_size);
        return;
    }
    BitNd nd = make_nd(indexer);
    hipLaunchKernelGGL((bit_generic_kernel<OP, BINARY>), dim3(grid_for(nd.total)), dim3(kBlock), 0, current_stream(), *a1,
                       BINARY ? *a2 : *a1, *a3, nd);
    cumo_cuda_runtime_check_kernel_launch();
}

template <bool COUNT_FALSE>
void launch_count(size_t p1, char* p2, CUMO_BIT_DIGIT* a1, ssize_t s1, size_t* idx1, ssize_t s2, uint64_t n) {
    if (n == 0) return;
    hipStream_t st = current_stream();
    if (s2 != 0) {
        hipLaunchKernelGGL((bit_count_scatter_kernel<COUNT_FALSE>), dim3(grid_for(n)), dim3(kBlock), 0, st, a1, (uint64_t)p1, (int64_t)s1, idx1,
                           p2, (int64_t)s2, n);
    } else if (!idx1 && s1 == 1) {
        hipLaunchKernelGGL((bit_count_words_kernel<COUNT_FALSE>), dim3(grid_for((n + 31) / 32 + 1, kCountGridCap)), dim3(kBlock), 0, st, a1, (uint64_t)p1, n,
                           (unsigned long long*)p2);
    } else {
        hipLaunchKernelGGL((bit_count_gather_kernel<COUNT_FALSE>), dim3(grid_for(n, kCountGridCap * 4)), dim3(kBlock), 0, st, a1, (uint64_t)p1,
                           (int64_t)s1, idx1, n, (unsigned long long*)p2);
    }
    cumo_cuda_runtime_check_kernel_launch();
}

// count_true / count_false along axes, every output in one launch. A work item is
// one run of bits (the innermost reduced dimension) of one output; a wave takes an
// item, its lanes share the run (whole masked words when the run is contiguous,
// single bits otherwise) and the wave's total is added to the output's counter.
// The counters are integers, so the order of the additions cannot show.
struct BitCountNd {
    int out_ndim, red_ndim;
    uint64_t out_total, red_outer, n_last;
    uint64_t out_shape[CUMO_NA_MAX_DIMENSION], red_shape[CUMO_NA_MAX_DIMENSION];
    int64_t in_out_step[CUMO_NA_MAX_DIMENSION], in_red_step[CUMO_NA_MAX_DIMENSION];  // bits
    int64_t out_step[CUMO_NA_MAX_DIMENSION];                                         // bytes
    const CUMO_BIT_DIGIT* in;
    uint64_t pos;
    char* out;
};

template <bool COUNT_FALSE>
__global__ __launch_bounds__(kBlock) void bit_count_nd_kernel(BitCountNd p) {
    const unsigned lane = threadIdx.x & 63;
    const uint64_t wave0 = ((uint64_t)blockIdx.x * kBlock + threadIdx.x) >> 6;
    const uint64_t n_waves = ((uint64_t)gridDim.x * kBlock) >> 6;
    const uint64_t items = p.out_total * p.red_outer;
    const int64_t s_last = p.red_ndim > 0 ? p.in_red_step[p.red_ndim - 1] : 0;
    for (uint64_t item = wave0; item < items; item += n_waves) {
        uint64_t o = item / p.red_outer, r = item - o * p.red_outer;
        int64_t bit = (int64_t)p.pos, ooff = 0;
        for (int d = p.out_ndim - 1; d >= 0; --d) {
            const uint64_t m = p.out_shape[d];
            const uint64_t q = o / m;
            const int64_t k = (int64_t)(o - q * m);
            o = q;
            bit += k * p.in_out_step[d];
            ooff += k * p.out_step[d];
        }
        for (int d = p.red_ndim - 2; d >= 0; --d) {
            const uint64_t m = p.red_shape[d];
            const uint64_t q = r / m;
            bit += (int64_t)(r - q * m) * p.in_red_step[d];
            r = q;
        }
        uint64_t c = 0;
        if (s_last == 1) {
            const uint64_t p1 = (uint64_t)bit, endbit = p1 + p.n_last;
            const uint64_t w0 = p1 >> 5, w1 = (endbit + 31) >> 5;
            for (uint64_t w = w0 + lane; w < w1; w += 64) {
                uint32_t x = p.in[w];
                if (COUNT_FALSE) x = ~x;
                const unsigned lo = (w == w0) ? (unsigned)(p1 & 31) : 0u;
                const unsigned hi = ((w + 1) << 5) <= endbit ? 32u : (unsigned)(endbit - (w << 5));
                x &= low_bits(hi) & ~low_bits(lo);
                c += (uint64_t)__popc(x);
            }
        } else {
            for (uint64_t i = lane; i < p.n_last; i += 64) {
                const uint64_t q = (uint64_t)(bit + (int64_t)i * s_last);
                const uint32_t b = (p.in[q >> 5] >> (q & 31)) & 1u;
                c += COUNT_FALSE ? (b ^ 1u) : b;
            }
        }
        for (unsigned d = 32; d > 0; d >>= 1) {
            const uint32_t lo = __shfl_down((uint32_t)c, d);
            const uint32_t hi = __shfl_down((uint32_t)(c >> 32), d);
            c += ((uint64_t)hi << 32) | lo;
        }
        if (lane == 0 && c) atomicAdd(reinterpret_cast<unsigned long long*>(p.out + ooff), (unsigned long long)c);
    }
}


}  // namespace

#define CUMO_DEF_BIT_BINARY(name, OP)                                                                                         \
    extern "C" void cumo_iter_bit_##name##_kernel_launch(cumo_na_bit_iarray_stridx_t* a1, cumo_na_bit_iarray_stridx_t* a2,    \
                                                         cumo_na_bit_iarray_stridx_t* a3, cumo_na_indexer_t* indexer) {       \
        launch_generic<OP, true>(a1, a2, a3, indexer);                                                                        \
    }                                                                                                                         \
    extern "C" void cumo_iter_bit_##name##_contiguous_kernel_launch(CUMO_BIT_DIGIT* a1, size_t p1, CUMO_BIT_DIGIT* a2,        \
                                                                    size_t p2, CUMO_BIT_DIGIT* a3, size_t p3, uint64_t n) {   \
        launch_contiguous<OP, true>(a1, p1, a2, p2, a3, p3, n);                                                               \
    }
#define CUMO_DEF_BIT_UNARY(name, OP)                                                                                          \
    extern "C" void cumo_iter_bit_##name##_kernel_launch(cumo_na_bit_iarray_stridx_t* a1, cumo_na_bit_iarray_stridx_t* a3,    \
                                                         cumo_na_indexer_t* indexer) {                                        \
        launch_generic<OP, false>(a1, nullptr, a3, indexer);                                                                  \
    }                                                                                                                         \
    extern "C" void cumo_iter_bit_##name##_contiguous_kernel_launch(CUMO_BIT_DIGIT* a1, size_t p1, CUMO_BIT_DIGIT* a3,        \
                                                                    size_t p3, uint64_t n) {                                  \
        launch_contiguous<OP, false>(a1, p1, nullptr, 0, a3, p3, n);                                                          \
    }
CUMO_DEF_BIT_BINARY(and, B_AND)
CUMO_DEF_BIT_BINARY(or, B_OR)
CUMO_DEF_BIT_BINARY(xor, B_XOR)
CUMO_DEF_BIT_BINARY(eq, B_EQ)
CUMO_DEF_BIT_UNARY(copy, B_COPY)
CUMO_DEF_BIT_UNARY(not, B_NOT)

#define CUMO_DEF_BIT_COUNT(name, CF)                                                                                          \
    extern "C" void cumo_iter_bit_##name##_index_kernel_launch(size_t p1, char* p2, CUMO_BIT_DIGIT* a1, size_t* idx1,         \
                                                               uint64_t n) {                                                  \
        launch_count<CF>(p1, p2, a1, 0, idx1, 0, n);                                                                          \
    }                                                                                                                         \
    extern "C" void cumo_iter_bit_##name##_stride_kernel_launch(size_t p1, char* p2, CUMO_BIT_DIGIT* a1, ssize_t s1,          \
                                                                uint64_t n) {                                                 \
        launch_count<CF>(p1, p2, a1, s1, nullptr, 0, n);                                                                      \
    }                                                                                                                         \
    extern "C" void cumo_iter_bit_##name##_index_stride_kernel_launch(size_t p1, char* p2, CUMO_BIT_DIGIT* a1, size_t* idx1,  \
                                                                      ssize_t s2, uint64_t n) {                               \
        launch_count<CF>(p1, p2, a1, 0, idx1, s2, n);                                                                         \
    }                                                                                                                         \
    extern "C" void cumo_iter_bit_##name##_stride_stride_kernel_launch(size_t p1, char* p2, CUMO_BIT_DIGIT* a1, ssize_t s1,   \
                                                                       ssize_t s2, uint64_t n) {                              \
        launch_count<CF>(p1, p2, a1, s1, nullptr, s2, n);                                                                     \
    }
CUMO_DEF_BIT_COUNT(count_true, false)
CUMO_DEF_BIT_COUNT(count_false, true)

#define CUMO_DEF_STORE_BIT(t, c)                                                                                              \
    extern "C" void cumo_iter_##t##_store_bit_kernel_launch(cumo_na_iarray_stridx_t* a1, cumo_na_bit_iarray_stridx_t* a2,     \
                                                            cumo_na_indexer_t* indexer) {                                     \
        if (indexer->total_size == 0) return;                                                                                 \
        BitNd nd = make_nd(indexer);                                                                                          \
        hipLaunchKernelGGL((store_bit_kernel<c>), dim3(grid_for(nd.total)), dim3(kBlock), 0, current_stream(), *a1, *a2, nd); \
        cumo_cuda_runtime_check_kernel_launch();                                                                              \
    }
CUMO_DEF_STORE_BIT(sfloat, float)
CUMO_DEF_STORE_BIT(dfloat, double)
CUMO_DEF_STORE_BIT(int32, int32_t)

// *out = the number of set (or clear) bits of the contiguous run [pos, pos + n) of a, in
// one launch and without a zeroed result. Returns 1 when launched, 0 when it cannot be
// (more streams in use than there are ticket words, or a run too long for the ticket):
// the caller then zeroes the result and uses the accumulating launcher.
extern "C" int cumo_hip_bit_count_run_store_kernel_launch(CUMO_BIT_DIGIT* a, size_t pos, uint64_t n, int count_false, uint64_t* out) {
    static std::mutex mu;
    static unsigned long long* tickets = nullptr;
    if (n == 0 || n >= (1ull << kTicketShift)) return 0;
    hipStream_t st = current_stream();
    const int slot = stream_slot(st);  // the stream's own ticket word; given back when the stream is destroyed
    if (slot < 0 || slot >= kTicketSlots) return 0;
    {
        std::lock_guard<std::mutex> lk(mu);
        if (!tickets) {
            void* p = nullptr;
            if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_count_ticket)) != hipSuccess) {
                (void)hipGetLastError();
                return 0;
            }
            tickets = (unsigned long long*)p;
        }
    }
    // whole 128-bit vectors: move the word pointer back to a 16-byte boundary
    const uintptr_t back = ((uintptr_t)a & 15) / sizeof(CUMO_BIT_DIGIT);
    a -= back;
    pos += back * 32;
    const uint64_t vecs = ((pos + n + 31) / 32 + 3) / 4 - (pos / 32) / 4;
    uint64_t grid = (vecs + kBlock - 1) / kBlock;
    if (grid > 128) grid = 128;  // every block ends in one returning atomic on the same word
    if (grid == 0) grid = 1;
    if (count_false)
        hipLaunchKernelGGL((bit_count_words_store_kernel<true>), dim3((unsigned)grid), dim3(kBlock), 0, st, (const CUMO_BIT_DIGIT*)a, (uint64_t)pos, n,
                           tickets + slot, (unsigned long long*)out);
    else
        hipLaunchKernelGGL((bit_count_words_store_kernel<false>), dim3((unsigned)grid), dim3(kBlock), 0, st, (const CUMO_BIT_DIGIT*)a, (uint64_t)pos, n,
                           tickets + slot, (unsigned long long*)out);
    cumo_cuda_runtime_check_kernel_launch();
    return 1;
}

extern "C" void cumo_hip_bit_count_nd_kernel_launch(const cumo_hip_bit_count_nd_t* d) {
    if (!d) return;
    BitCountNd p;
    std::memset(&p, 0, sizeof(p));
    p.out_ndim = d->out_ndim;
    p.red_ndim = d->red_ndim;
    p.out_total = 1;
    p.red_outer = 1;
    for (int k = 0; k < d->out_ndim; ++k) {
        p.out_shape[k] = d->out_shape[k];
        p.in_out_step[k] = d->in_out_step[k];
        p.out_step[k] = d->out_step[k];
        p.out_total *= d->out_shape[k];
    }
    for (int k = 0; k < d->red_ndim; ++k) {
        p.red_shape[k] = d->red_shape[k];
        p.in_red_step[k] = d->in_red_step[k];
        if (k < d->red_ndim - 1) p.red_outer *= d->red_shape[k];
    }
    p.n_last = d->red_ndim > 0 ? d->red_shape[d->red_ndim - 1] : 1;
    if (d->red_ndim == 0) {
        // nothing is reduced: every element is a run of one bit
        p.red_ndim = 1;
        p.red_shape[0] = 1;
        p.in_red_step[0] = 1;
    }
    p.in = d->in;
    p.pos = d->pos;
    p.out = d->out;
    const uint64_t items = p.out_total * p.red_outer;
    if (items == 0 || p.n_last == 0) return;
    uint64_t grid = (items * 64 + kBlock - 1) / kBlock;
    if (grid > 256u * 32u) grid = 256u * 32u;
    if (d->count_false)
        hipLaunchKernelGGL((bit_count_nd_kernel<true>), dim3((unsigned)grid), dim3(kBlock), 0, current_stream(), p);
    else
        hipLaunchKernelGGL((bit_count_nd_kernel<false>), dim3((unsigned)grid), dim3(kBlock), 0, current_stream(), p);
    cumo_cuda_runtime_check_kernel_launch();
}
