// mulsum: the sum of products of two runs (the inner product under Cumo's dot).
//
// Replaces narray/gen/tmpl/accum_binary_kernel.cu of the reference (a grid of up to
// 1024 blocks of 512 threads with a nine-level LDS tree each, then one block over
// the partials). Here a block takes one contiguous chunk of the run, lanes read 128
// bits from both operands when both are contiguous and keep four independent
// accumulators, lanes combine with wave64 shuffles and the four waves through LDS;
// the partials of the blocks are folded in index order by a second launch, which
// also adds onto what the result already holds, as the reference does
// (accum_binary_kernel.cu:46-47,63). No atomics: the answer does not depend on
// scheduling. Products and sums are in the element type, unfused, as the macros
// write them (types/real_accum_kernel.h:6-10, xint_macro_kernel.h:44).
#include "common.h"
#include "wait_ctl.h"

namespace cumo_hip {
namespace {

constexpr int kMsBlock = 256;
constexpr int kMsMaxGrid = 2048;

template <class T> struct ms_is_int { static constexpr bool value = false; };
template <> struct ms_is_int<int32_t> { static constexpr bool value = true; };

template <class T, bool NANF>
__device__ __forceinline__ void ms_fold(T x, T y, T& acc) {
    if constexpr (ms_is_int<T>::value) {
        acc = (T)((uint32_t)acc + (uint32_t)x * (uint32_t)y);
    } else {
        if (NANF && (x != x || y != y)) return;
        acc = x * y + acc;
    }
}
template <class T>
__device__ __forceinline__ T ms_add(T a, T b) {
    if constexpr (ms_is_int<T>::value) return (T)((uint32_t)a + (uint32_t)b);
    else return a + b;
}

template <class T>
__device__ __forceinline__ T ms_shfl_down(T v, unsigned d) {
    if constexpr (sizeof(T) == 8) {
        union { T t; uint32_t w[2]; } a, b;
        a.t = v;
        b.w[0] = __shfl_down(a.w[0], d);
        b.w[1] = __shfl_down(a.w[1], d);
        return b.t;
    } else {
        union { T t; uint32_t w; } a, b;
        a.t = v;
        b.w = __shfl_down(a.w, d);
        return b.t;
    }
}

// the block's total in thread 0
template <class T>
__device__ __forceinline__ T ms_block_sum(T acc) {
    __shared__ T wave_acc[kMsBlock / 64];
    for (unsigned d = 32; d > 0; d >>= 1) acc = ms_add(acc, ms_shfl_down(acc, d));
    if ((threadIdx.x & 63) == 0) wave_acc[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < kMsBlock / 64; ++w) acc = ms_add(acc, wave_acc[w]);
    }
    return acc;
}

// VEC > 1: both runs contiguous and 16-byte aligned at every chunk start
// NT: non-temporal loads, for runs that do not fit the last-level cache anyway
template <class T, bool NANF, int VEC, bool NT>
__global__ __launch_bounds__(kMsBlock) void mulsum_partial_kernel(const char* p1, const char* p2, int64_t s1, int64_t s2, uint64_t n,
                                                                  uint64_t chunk, T* partial, T* out, uint64_t* words, uint32_t launch,
                                                                  WaitCtl* wait) {
    constexpr int W = (int)(sizeof(T) / 4);
    uint32_t block = blockIdx.x;
    if (words) {
        // One launch for the whole sum: block 0 reads nothing of the operands; it waits for the other
        // blocks' totals, which arrive as 64-bit words {launch number, 32 bits of the total} written
        // with agent-scope atomic stores, folds them in index order and adds onto the result.
        if (block == 0) {
            const uint32_t n_parts = gridDim.x - 1;
            T acc = T();
            for (uint32_t i = threadIdx.x; i < n_parts; i += kMsBlock) {
                union { T t; uint32_t w[W]; } u;
#pragma unroll
                for (int k = 0; k < W; ++k) {
                    const uint64_t* slot = words + (size_t)i * W + k;
                    uint64_t x = __hip_atomic_load(slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    uint32_t looks = 0;
                    const uint32_t limit = wait_limit(wait, 1u << 24);
                    while ((uint32_t)(x >> 32) != launch) {
                        if (++looks > limit) {
                            wait_gave_up(wait, WAIT_MULSUM);  // the total is not valid; the host is told
                            break;
                        }
                        __builtin_amdgcn_s_sleep(4);
                        x = __hip_atomic_load(slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                    u.w[k] = (uint32_t)x;
                }
                acc = ms_add(acc, u.t);
            }
            acc = ms_block_sum<T>(acc);
            if (threadIdx.x == 0) *out = ms_add(*out, acc);
            return;
        }
        block -= 1;
    }
    const uint64_t begin = (uint64_t)block * chunk;
    uint64_t end = begin + chunk;
    if (end > n) end = n;
    T acc[4] = {T(), T(), T(), T()};
    if constexpr (VEC > 1) {
        typedef uint32_t u4 __attribute__((ext_vector_type(4)));
        union V { u4 q; T t[VEC]; __device__ V() {} };
        const uint64_t stride = (uint64_t)kMsBlock * VEC;
        uint64_t i = begin + (uint64_t)threadIdx.x * VEC;
        // whole vectors, four per lane and operand in flight
        for (; i + 3 * stride + VEC <= end; i += 4 * stride) {
            V a[4], b[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const u4* pa = reinterpret_cast<const u4*>(p1 + (i + u * stride) * sizeof(T));
                const u4* pb = reinterpret_cast<const u4*>(p2 + (i + u * stride) * sizeof(T));
                a[u].q = NT ? __builtin_nontemporal_load(pa) : *pa;
                b[u].q = NT ? __builtin_nontemporal_load(pb) : *pb;
            }
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int j = 0; j < VEC; ++j) ms_fold<T, NANF>(a[u].t[j], b[u].t[j], acc[u]);
        }
        for (; i < end; i += stride) {
            if (i + VEC <= end) {
                V a, b;
                a.q = *reinterpret_cast<const u4*>(p1 + i * sizeof(T));
                b.q = *reinterpret_cast<const u4*>(p2 + i * sizeof(T));
#pragma unroll
                for (int j = 0; j < VEC; ++j) ms_fold<T, NANF>(a.t[j], b.t[j], acc[0]);
            } else {
                for (uint64_t k = i; k < end; ++k)
                    ms_fold<T, NANF>(reinterpret_cast<const T*>(p1)[k], reinterpret_cast<const T*>(p2)[k], acc[0]);
            }
        }
    } else {
        uint64_t i = begin + threadIdx.x;
        for (; i + 3 * kMsBlock < end; i += 4 * kMsBlock) {
            T a[4], b[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                a[u] = *reinterpret_cast<const T*>(p1 + (int64_t)(i + u * kMsBlock) * s1);
                b[u] = *reinterpret_cast<const T*>(p2 + (int64_t)(i + u * kMsBlock) * s2);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) ms_fold<T, NANF>(a[u], b[u], acc[u]);
        }
        for (; i < end; i += kMsBlock)
            ms_fold<T, NANF>(*reinterpret_cast<const T*>(p1 + (int64_t)i * s1), *reinterpret_cast<const T*>(p2 + (int64_t)i * s2), acc[0]);
    }
    T tot = ms_add(ms_add(acc[0], acc[1]), ms_add(acc[2], acc[3]));
    tot = ms_block_sum<T>(tot);
    if (threadIdx.x == 0) {
        if (words) {
            union { T t; uint32_t w[W]; } u;
            u.t = tot;
#pragma unroll
            for (int k = 0; k < W; ++k)
                __hip_atomic_store(words + (size_t)block * W + k, ((uint64_t)launch << 32) | u.w[k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else if (partial) {
            partial[block] = tot;
        } else {
            *out = ms_add(*out, tot);
        }
    }
}

template <class T>
__global__ __launch_bounds__(kMsBlock) void mulsum_combine_kernel(const T* partial, uint64_t n, T* out) {
    T acc = T();
    for (uint64_t i = threadIdx.x; i < n; i += kMsBlock) acc = ms_add(acc, partial[i]);
    acc = ms_block_sum<T>(acc);
    if (threadIdx.x == 0) *out = ms_add(*out, acc);
}

template <class T, bool NANF>
__global__ __launch_bounds__(kMsBlock) void mulsum_elementwise_kernel(const char* p1, const char* p2, char* p3, int64_t s1, int64_t s2, int64_t s3,
                                                                      uint64_t n) {
    for (uint64_t i = (uint64_t)blockIdx.x * kMsBlock + threadIdx.x; i < n; i += (uint64_t)gridDim.x * kMsBlock) {
        T* z = reinterpret_cast<T*>(p3 + (int64_t)i * s3);
        T acc = *z;
        ms_fold<T, NANF>(*reinterpret_cast<const T*>(p1 + (int64_t)i * s1), *reinterpret_cast<const T*>(p2 + (int64_t)i * s2), acc);
        *z = acc;
    }
}


// One product sum per row, many rows in one launch: LPR lanes share a row whose two
// runs are contiguous (aligned as their elements are), four vectors per operand in flight per
// lane, four accumulators, then a butterfly over the lanes of the row (and the four
// waves through LDS when a block shares the row). The order is fixed by the layout.
struct MulsumRows {
    uint64_t rows, n;
    int64_t step1, step2, step3;  // bytes from one row to the next
    const char *p1, *p2;
    char* out;
};

template <class T, bool NANF, int LPR, bool NT>
__global__ __launch_bounds__(kMsBlock) void mulsum_rows_kernel(MulsumRows g) {
    constexpr int VEC = 16 / (int)sizeof(T);
    constexpr int RPB = kMsBlock / LPR;
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    union V { u4 q; T t[VEC]; __device__ V() {} };
    const uint32_t lane = threadIdx.x % LPR;
    const uint64_t nvec = g.n / VEC;
    const uint64_t n_blocks = (g.rows + RPB - 1) / RPB;
    for (uint64_t rb = blockIdx.x; rb < n_blocks; rb += gridDim.x) {
        const uint64_t row = rb * RPB + threadIdx.x / LPR;
        const bool ok = row < g.rows;
        const uint64_t r = ok ? row : 0;  // surplus lanes redo row 0 and store nothing
        const u4* a4 = reinterpret_cast<const u4*>(g.p1 + (int64_t)r * g.step1);
        const u4* b4 = reinterpret_cast<const u4*>(g.p2 + (int64_t)r * g.step2);
        T acc[4] = {T(), T(), T(), T()};
        uint64_t v = lane;
        for (; v + 3 * LPR < nvec; v += 4 * LPR) {
            V a[4], b[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                a[u].q = NT ? __builtin_nontemporal_load(a4 + v + u * LPR) : a4[v + u * LPR];
                b[u].q = NT ? __builtin_nontemporal_load(b4 + v + u * LPR) : b4[v + u * LPR];
            }
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int j = 0; j < VEC; ++j) ms_fold<T, NANF>(a[u].t[j], b[u].t[j], acc[u]);
        }
        for (; v < nvec; v += LPR) {
            V a, b;
            a.q = a4[v];
            b.q = b4[v];
#pragma unroll
            for (int j = 0; j < VEC; ++j) ms_fold<T, NANF>(a.t[j], b.t[j], acc[0]);
        }
        // what the row has past its last whole vector (fewer than VEC elements)
        if (lane == 0) {
            const T* a1 = reinterpret_cast<const T*>(a4);
            const T* b1 = reinterpret_cast<const T*>(b4);
            for (uint64_t e = nvec * VEC; e < g.n; ++e) ms_fold<T, NANF>(a1[e], b1[e], acc[1]);
        }
        T tot = ms_add(ms_add(acc[0], acc[1]), ms_add(acc[2], acc[3]));
        if constexpr (LPR <= 64) {
#pragma unroll
            for (unsigned d = LPR >> 1; d > 0; d >>= 1) tot = ms_add(tot, ms_shfl_down(tot, d));
        } else {
            __syncthreads();  // the LDS slots of the previous row have been read
            tot = ms_block_sum<T>(tot);
        }
        if (lane == 0 && ok) {
            T* z = reinterpret_cast<T*>(g.out + (int64_t)row * g.step3);
            *z = ms_add(*z, tot);
        }
    }
}

template <class T, bool NANF>
bool mulsum_rows_launch(const cumo_hip_mulsum_rows_t* d) {
    constexpr int VEC = 16 / (int)sizeof(T);
    // rows need their element's alignment only (a 128-bit load works on any 4-byte boundary) and may end in
    // part of a vector, which the row's first lane folds element by element
    if (d->n < (uint64_t)VEC * 16) return false;
    if (((uintptr_t)d->p1 | (uintptr_t)d->p2 | (uintptr_t)d->row_step1 | (uintptr_t)d->row_step2) % sizeof(T)) return false;
    if (((uintptr_t)d->out | (uintptr_t)d->out_step) % sizeof(T)) return false;
    MulsumRows g = {d->rows, d->n, (int64_t)d->row_step1, (int64_t)d->row_step2, (int64_t)d->out_step, d->p1, d->p2, d->out};
    const uint64_t nvec = d->n / VEC;
    const int lpr = nvec <= 64 ? 16 : (nvec <= 256 ? 64 : 256);
    const uint64_t rpb = kMsBlock / lpr;
    uint64_t grid = (d->rows + rpb - 1) / rpb;
    if (grid > 256u * 64u) grid = 256u * 64u;
    // both operands streamed once and larger than the last-level cache together
    const bool nt = d->row_step1 != 0 && d->row_step2 != 0 && stream_past_caches(2 * d->rows * d->n * sizeof(T));
    hipStream_t stream = current_stream();
#define MS_ROWS(L, N) hipLaunchKernelGGL((mulsum_rows_kernel<T, NANF, L, N>), dim3((unsigned)grid), dim3(kMsBlock), 0, stream, g)
    if (lpr == 16) { if (nt) MS_ROWS(16, true); else MS_ROWS(16, false); }
    else if (lpr == 64) { if (nt) MS_ROWS(64, true); else MS_ROWS(64, false); }
    else { if (nt) MS_ROWS(256, true); else MS_ROWS(256, false); }
#undef MS_ROWS
    cumo_cuda_runtime_check_kernel_launch();
    return true;
}

template <class T, bool NANF>
void mulsum_reduce_launch(char* p1, char* p2, char* p3, ssize_t s1, ssize_t s2, uint64_t n) {
    hipStream_t stream = current_stream();
    constexpr int VEC = 16 / (int)sizeof(T);
    // a block's chunk: at least 16 KiB per operand, a whole number of 4-vector rounds
    const uint64_t round = (uint64_t)kMsBlock * VEC * 4;
    uint64_t grid = (n + 4 * round - 1) / (4 * round);
    if (grid == 0) grid = 1;
    if (grid > (uint64_t)kMsMaxGrid) grid = kMsMaxGrid;
    uint64_t chunk = (n + grid - 1) / grid;
    chunk = ((chunk + round - 1) / round) * round;
    grid = n ? (n + chunk - 1) / chunk : 1;
    const bool vec = s1 == (ssize_t)sizeof(T) && s2 == (ssize_t)sizeof(T) && ((uintptr_t)p1 % 16) == 0 && ((uintptr_t)p2 % 16) == 0;
    // several blocks: their totals go to the stream's hand-over words and block 0 of the same launch
    // folds them (not while the stream is being captured: a replayed launch would carry the same
    // launch number again), else to scratch from the pool and a second launch
    T* partial = nullptr;
    uint64_t* words = nullptr;
    WaitCtl* wait = nullptr;
    uint32_t launch = 0;
    if (grid > 1) {
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(stream, &capturing) != hipSuccess) {
            (void)hipGetLastError();
            capturing = hipStreamCaptureStatusActive;
        }
        if (capturing == hipStreamCaptureStatusNone && grid * (sizeof(T) / 4) <= 8192 && (wait = wait_ctl()) != nullptr)
            words = red_handover_words(stream_slot(stream), &launch);
        if (!words) {
            partial = reinterpret_cast<T*>(cumo_cuda_runtime_malloc(sizeof(T) * grid));
            if (!partial) return;
        }
    }
    const bool nt = stream_past_caches(2 * n * sizeof(T));
    const dim3 g((unsigned)(words ? grid + 1 : grid)), b(kMsBlock);
    T* out = reinterpret_cast<T*>(p3);
    if (vec && nt) hipLaunchKernelGGL((mulsum_partial_kernel<T, NANF, VEC, true>), g, b, 0, stream, p1, p2, (int64_t)s1, (int64_t)s2, n, chunk, partial, out, words, launch, wait);
    else if (vec) hipLaunchKernelGGL((mulsum_partial_kernel<T, NANF, VEC, false>), g, b, 0, stream, p1, p2, (int64_t)s1, (int64_t)s2, n, chunk, partial, out, words, launch, wait);
    else hipLaunchKernelGGL((mulsum_partial_kernel<T, NANF, 1, false>), g, b, 0, stream, p1, p2, (int64_t)s1, (int64_t)s2, n, chunk, partial, out, words, launch, wait);
    if (partial) {
        hipLaunchKernelGGL((mulsum_combine_kernel<T>), dim3(1), dim3(kMsBlock), 0, stream, (const T*)partial, grid, out);
        cumo_cuda_runtime_free(reinterpret_cast<char*>(partial));
    }
    cumo_cuda_runtime_check_kernel_launch();
}

template <class T, bool NANF>
void mulsum_elementwise_launch(char* p1, char* p2, char* p3, ssize_t s1, ssize_t s2, ssize_t s3, uint64_t n) {
    if (n == 0) return;
    uint64_t grid = (n + kMsBlock - 1) / kMsBlock;
    if (grid > 65536) grid = 65536;
    hipLaunchKernelGGL((mulsum_elementwise_kernel<T, NANF>), dim3((unsigned)grid), dim3(kMsBlock), 0, current_stream(), p1, p2, p3, (int64_t)s1,
                       (int64_t)s2, (int64_t)s3, n);
    cumo_cuda_runtime_check_kernel_launch();
}

}  // namespace
}  // namespace cumo_hip

using namespace cumo_hip;

extern "C" {

#define CUMO_DEF_MULSUM(t, c, name, NANF)                                                                                  \
    void cumo_##t##_##name##_reduce_kernel_launch(char* p1, char* p2, char* p3, ssize_t s1, ssize_t s2, uint64_t n) {      \
        mulsum_reduce_launch<c, NANF>(p1, p2, p3, s1, s2, n);                                                              \
    }                                                                                                                      \
    void cumo_##t##_##name##_kernel_launch(char* p1, char* p2, char* p3, ssize_t s1, ssize_t s2, ssize_t s3, uint64_t n) { \
        mulsum_elementwise_launch<c, NANF>(p1, p2, p3, s1, s2, s3, n);                                                     \
    }
CUMO_DEF_MULSUM(sfloat, float, mulsum, false)
CUMO_DEF_MULSUM(sfloat, float, mulsum_nan, true)
CUMO_DEF_MULSUM(dfloat, double, mulsum, false)
CUMO_DEF_MULSUM(dfloat, double, mulsum_nan, true)
CUMO_DEF_MULSUM(int32, int32_t, mulsum, false)

// type: 0 SFloat, 1 DFloat, 2 Int32. out[r] += sum over the row of p1 * p2, for every
// row in one launch. Returns 1 when launched, 0 when the layout is outside what the
// kernel takes (rows not a whole number of 128-bit vectors, or not 16-byte aligned):
// the caller then launches the rows one by one.
int cumo_hip_mulsum_rows_kernel_launch(int type, int nan, const cumo_hip_mulsum_rows_t* d) {
    if (!d || d->rows == 0 || d->n == 0) return 1;
    bool ok = false;
    if (type == 0) ok = nan ? mulsum_rows_launch<float, true>(d) : mulsum_rows_launch<float, false>(d);
    else if (type == 1) ok = nan ? mulsum_rows_launch<double, true>(d) : mulsum_rows_launch<double, false>(d);
    else if (type == 2) ok = mulsum_rows_launch<int32_t, false>(d);
    return ok ? 1 : 0;
}

}  // extern "C"
