// Bit#where and Bit#mask: the positions of the set (or clear) bits of a run,
// compacted in ascending order.
//
// Replaces narray/gen/tmpl_bit/where_kernel.cu and mask_kernel.cu of the reference
// with the same launcher ABI and the same scratch layout (two running cursors, then
// up to 1024 block counts), so that the host iterators (tmpl_bit/where.c:34-52,
// mask.c) bind unchanged: a cursor in the scratch carries the output position from
// one run of a view to the next on the device, and nothing is read back.
//
// Three launches per run: every block counts the set bits of its contiguous range
// of 32-bit chunks; one block turns the counts into output positions (and advances
// the cursor); every block walks its range again, 256 chunks a round: an exclusive
// scan over the block places each chunk's hits in a list in LDS, and consecutive
// lanes then write the list out, so the stores of a wave are adjacent. Blocks are 256
// threads (4 wave64): the scan inside a block is a wave scan by DPP steps plus four LDS
// slots.
// A contiguous run reads whole words (two per chunk when the run starts inside a
// word); strided and index-array runs gather bit by bit.
#include "common.h"
#include "div31.h"

#include <type_traits>

#include <cstring>

namespace cumo_hip {
namespace {

constexpr int kWhBlock = 256;
constexpr uint64_t kWhMaxBlocks = 1024;  // the scratch holds this many block counts (where_kernel.cu:11)

// the 32 bits [c*32, c*32+32) of the run, bits beyond n cleared
__device__ __forceinline__ uint32_t wh_chunk(const CUMO_BIT_DIGIT* a, uint64_t p, int64_t s, const size_t* idx, uint64_t n, uint64_t c,
                                             int contiguous, int invert) {
    const uint64_t first = c * 32;
    const uint64_t left = n - first;
    const uint32_t valid = left >= 32 ? 0xffffffffu : ((1u << left) - 1u);
    uint32_t z;
    if (contiguous) {
        const uint64_t q = p + first;
        const uint64_t w = q >> 5;
        const unsigned sh = (unsigned)(q & 31);
        z = a[w] >> sh;
        // the second word only exists when the chunk reaches into it
        if (sh && (uint64_t)(32 - sh) < left) z |= a[w + 1] << (32 - sh);
    } else {
        z = 0;
        const unsigned m = left >= 32 ? 32u : (unsigned)left;
        for (unsigned k = 0; k < m; ++k) {
            const uint64_t q = idx ? (p + idx[first + k]) : (uint64_t)((int64_t)p + (int64_t)(first + k) * s);
            z |= ((a[q >> 5] >> (q & 31)) & 1u) << k;
        }
    }
    if (invert) z = ~z;
    return z & valid;
}

// exclusive scan of one value per thread over the block; *total gets the block's sum
// in every thread. Two barriers; safe to call again right away.
__device__ __forceinline__ uint64_t wh_block_exscan(uint64_t v, uint64_t* total) {
    __shared__ uint64_t wave_sum[kWhBlock / 64];
    const unsigned lane = threadIdx.x & 63;
    uint64_t inc = v;
    for (unsigned d = 1; d < 64; d <<= 1) {
        const uint32_t lo = __shfl_up((uint32_t)inc, d);
        const uint32_t hi = __shfl_up((uint32_t)(inc >> 32), d);
        if (lane >= d) inc += ((uint64_t)hi << 32) | lo;
    }
    __syncthreads();  // the slots may still be read from the previous call
    if (lane == 63) wave_sum[threadIdx.x >> 6] = inc;
    __syncthreads();
    uint64_t before = 0, all = 0;
    for (unsigned w = 0; w < kWhBlock / 64; ++w) {
        if (w < (threadIdx.x >> 6)) before += wave_sum[w];
        all += wave_sum[w];
    }
    *total = all;
    return before + inc - v;
}

// A barrier for the LDS traffic only: loads from global memory that were sent ahead stay
// in flight across it (__syncthreads() waits for them as well).
__device__ __forceinline__ void wh_lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// inclusive scan over the 64 lanes of a wave: four shifts within the rows of 16 lanes,
// then lane 15 of a row into the next row and lane 31 into the upper half
__device__ __forceinline__ uint32_t wh_wave_scan(uint32_t v) {
    int x = (int)v;
    x += __builtin_amdgcn_update_dpp(0, x, 0x111, 0xf, 0xf, true);   // row_shr:1
    x += __builtin_amdgcn_update_dpp(0, x, 0x112, 0xf, 0xf, true);   // row_shr:2
    x += __builtin_amdgcn_update_dpp(0, x, 0x114, 0xf, 0xf, true);   // row_shr:4
    x += __builtin_amdgcn_update_dpp(0, x, 0x118, 0xf, 0xf, true);   // row_shr:8
    x += __builtin_amdgcn_update_dpp(0, x, 0x142, 0xa, 0xf, false);  // row_bcast:15 into rows 1 and 3
    x += __builtin_amdgcn_update_dpp(0, x, 0x143, 0xc, 0xf, false);  // row_bcast:31 into rows 2 and 3
    return (uint32_t)x;
}

// exclusive scan of one small value per thread over the block (the sum fits 32 bits); *total
// gets the block's sum in every thread. Two LDS-only barriers; safe to call again right away.
__device__ __forceinline__ uint32_t wh_block_exscan32(uint32_t v, uint32_t* total) {
    __shared__ uint32_t wave_sum32[kWhBlock / 64];
    const uint32_t inc = wh_wave_scan(v);
    wh_lds_barrier();  // the slots may still be read from the previous call
    if ((threadIdx.x & 63) == 63) wave_sum32[threadIdx.x >> 6] = inc;
    wh_lds_barrier();
    uint32_t before = 0, all = 0;
#pragma unroll
    for (unsigned w = 0; w < kWhBlock / 64; ++w) {
        const uint32_t ws = wave_sum32[w];
        before += (w < (threadIdx.x >> 6)) ? ws : 0u;
        all += ws;
    }
    *total = all;
    return before + inc - v;
}

__global__ __launch_bounds__(kWhBlock) void where_count_kernel(const CUMO_BIT_DIGIT* a, uint64_t p, int64_t s, const size_t* idx, uint64_t n,
                                                               int contiguous, int invert, uint64_t nchunks, uint64_t cpb, uint64_t* block_sums,
                                                               uint64_t* host_sums) {
    uint64_t start = (uint64_t)blockIdx.x * cpb;
    if (start > nchunks) start = nchunks;
    const uint64_t end = (nchunks - start < cpb) ? nchunks : start + cpb;
    uint64_t cnt = 0;
    for (uint64_t c = start + threadIdx.x; c < end; c += kWhBlock) cnt += (uint64_t)__popc(wh_chunk(a, p, s, idx, n, c, contiguous, invert));
    uint64_t total;
    wh_block_exscan(cnt, &total);
    if (threadIdx.x == 0) {
        block_sums[blockIdx.x] = total;
        // a copy straight into the caller's pinned host memory: the host then only has to wait for
        // the stream, not for a copy queued behind the kernel
        if (host_sums) host_sums[blockIdx.x] = total;
    }
}

// block_sums[b] becomes the output position of block b's first hit; *running moves on
__global__ __launch_bounds__(kWhBlock) void where_scan_kernel(uint64_t* block_sums, uint64_t nblocks, uint64_t* running) {
    uint64_t acc = *running;
    for (uint64_t t0 = 0; t0 < nblocks; t0 += kWhBlock) {
        const uint64_t t = t0 + threadIdx.x;
        const uint64_t v = t < nblocks ? block_sums[t] : 0;
        uint64_t total;
        const uint64_t pre = wh_block_exscan(v, &total);
        if (t < nblocks) block_sums[t] = acc + pre;
        acc += total;
    }
    __syncthreads();  // every thread has read *running before it is rewritten
    if (threadIdx.x == 0) *running = acc;
}

// MODE 0: out[o] = count + position in the run, as ES-byte integers (where).
// MODE 1: out[o] = the masked array's element position p2 + j*s2 (or p2 + idx2[j]), as size_t (mask; ES 8).
// MODE 2: out[o] = the masked array's element itself, ES (4 or 8) bytes read at p2 + j*s2 where p2 is
//         its address (the compaction the reference reaches through a view over the positions of mode 1).
// COUNTS: block_sums holds the blocks' plain counts (no scan launch ran): the block adds up
// the counts of the blocks before it.
template <int MODE, int ES, bool COUNTS>
__global__ __launch_bounds__(kWhBlock) void where_scatter_kernel(const CUMO_BIT_DIGIT* a, uint64_t p, int64_t s, const size_t* idx, uint64_t n,
                                                                 int contiguous, int invert, uint64_t nchunks, uint64_t cpb, char* out,
                                                                 uint64_t count, size_t p2, int64_t s2, const size_t* idx2,
                                                                 const uint64_t* block_sums) {
    typedef typename std::conditional<ES == 4, uint32_t, uint64_t>::type E;
    uint64_t start = (uint64_t)blockIdx.x * cpb;
    if (start > nchunks) start = nchunks;
    const uint64_t end = (nchunks - start < cpb) ? nchunks : start + cpb;
    // hits of one round (256 chunks, up to 8192 bits) are listed in LDS by their bit
    // position within the round, then written out by consecutive lanes
    __shared__ uint16_t hit[kWhBlock * 32];
    uint64_t off;
    if (COUNTS) {
        uint64_t before = 0;
        for (uint64_t t = threadIdx.x; t < blockIdx.x; t += kWhBlock) before += block_sums[t];
        wh_block_exscan(before, &off);
    } else {
        off = block_sums[blockIdx.x];
    }
    // the next round's bits are loaded before this round's are placed
    uint32_t znext = start + threadIdx.x < end ? wh_chunk(a, p, s, idx, n, start + threadIdx.x, contiguous, invert) : 0u;
    for (uint64_t c0 = start; c0 < end; c0 += kWhBlock) {
        uint32_t z = znext;
        const uint64_t cn = c0 + kWhBlock + threadIdx.x;
        znext = cn < end ? wh_chunk(a, p, s, idx, n, cn, contiguous, invert) : 0u;
        uint32_t total;
        // the first barrier inside the scan also ends the previous round's reads of hit[]
        uint32_t o = wh_block_exscan32((uint32_t)__popc(z), &total);
        const uint32_t mine = threadIdx.x * 32;
        while (z) {
            hit[o++] = (uint16_t)(mine + (unsigned)__builtin_ctz(z));
            z &= z - 1;
        }
        wh_lds_barrier();
        const uint64_t j0 = c0 * 32;             // the round's first bit, and where its hits go
        E* const dst = reinterpret_cast<E*>(out) + off;
#pragma unroll 4
        for (uint32_t k = threadIdx.x; k < total; k += kWhBlock) {
            const uint32_t h = hit[k];
            if (MODE == 2) {
                dst[k] = *reinterpret_cast<const E*>(reinterpret_cast<const char*>(p2) + (int64_t)(j0 + h) * s2);
            } else if (MODE == 1) {
                const uint64_t j = j0 + h;
                dst[k] = (E)(idx2 ? (p2 + idx2[j]) : (size_t)((int64_t)p2 + (int64_t)j * s2));
            } else {
                dst[k] = (E)(count + j0) + (E)h;
            }
        }
        off += total;
    }
}

// a run of n bits as 32-bit chunks shared out over the blocks, a contiguous range each
struct WhGeometry {
    uint64_t nchunks, nblocks, cpb;
};
WhGeometry wh_geometry(uint64_t n) {
    WhGeometry g;
    g.nchunks = (n + 31) / 32;
    g.nblocks = (g.nchunks + kWhBlock - 1) / kWhBlock;
    if (g.nblocks > kWhMaxBlocks) g.nblocks = kWhMaxBlocks;
    g.cpb = g.nblocks ? (g.nchunks + g.nblocks - 1) / g.nblocks : 0;
    return g;
}

template <int MODE>
void where_launch(CUMO_BIT_DIGIT* a, size_t p, ssize_t s, size_t* idx, uint64_t n, int invert, char* out, size_t elmsz, uint64_t count, size_t p2,
                  ssize_t s2, size_t* idx2, uint64_t* running, uint64_t* block_sums) {
    if (n == 0) return;  // a grid of no blocks is an invalid launch
    const WhGeometry g = wh_geometry(n);
    const uint64_t nchunks = g.nchunks, nblocks = g.nblocks, cpb = g.cpb;
    const int contiguous = (idx == nullptr && s == 1) ? 1 : 0;
    hipStream_t st = current_stream();
    hipLaunchKernelGGL(where_count_kernel, dim3((unsigned)nblocks), dim3(kWhBlock), 0, st, a, (uint64_t)p, (int64_t)s, (const size_t*)idx, n, contiguous,
                       invert, nchunks, cpb, block_sums, (uint64_t*)nullptr);
    hipLaunchKernelGGL(where_scan_kernel, dim3(1), dim3(kWhBlock), 0, st, block_sums, nblocks, running);
#define WH_SCATTER(ES)                                                                                                                      \
    hipLaunchKernelGGL((where_scatter_kernel<MODE, ES, false>), dim3((unsigned)nblocks), dim3(kWhBlock), 0, st, a, (uint64_t)p, (int64_t)s,     \
                       (const size_t*)idx, n, contiguous, invert, nchunks, cpb, out, count, p2, (int64_t)s2, (const size_t*)idx2,               \
                       (const uint64_t*)block_sums)
    if (elmsz == 4) {
        if constexpr (MODE != 1) WH_SCATTER(4);
    } else {
        WH_SCATTER(8);
    }
#undef WH_SCATTER
    cumo_cuda_runtime_check_kernel_launch();
}

// a tiny fill instead of a memset node, so that a caller may capture the stream
__global__ void where_zero_kernel(uint64_t* p) {
    if (threadIdx.x < 2) p[threadIdx.x] = 0;
}

// z[i] = the element of x at flat (row-major) position pos[i]
struct GatherParams {
    int ndim;
    uint64_t n;
    uint64_t shape[CUMO_NA_MAX_DIMENSION];
    Div31 div[CUMO_NA_MAX_DIMENSION];
    int64_t step[CUMO_NA_MAX_DIMENSION];
    const char* in;
    char* out;
    const char* pos;
};
// PW, EW: bytes per position and per element (4 or 8). SMALL: the view has fewer than
// 2^31 elements, so a position splits over the dimensions with 32-bit multiplies.
template <int PW, int EW, bool SMALL>
__global__ __launch_bounds__(256) void gather_flat_kernel(GatherParams g) {
    typedef typename std::conditional<PW == 4, uint32_t, uint64_t>::type P;
    typedef typename std::conditional<EW == 4, uint32_t, uint64_t>::type E;
    for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < g.n; i += (uint64_t)gridDim.x * 256) {
        const uint64_t r0 = (uint64_t)reinterpret_cast<const P*>(g.pos)[i];
        int64_t off = 0;
        if (SMALL) {
            uint32_t r = (uint32_t)r0;
            for (int d = g.ndim - 1; d > 0; --d) {
                const uint32_t q = div31(r, g.div[d]);
                off += (int64_t)(r - q * (uint32_t)g.shape[d]) * g.step[d];
                r = q;
            }
            off += (int64_t)r * g.step[0];
        } else {
            uint64_t r = r0;
            for (int d = g.ndim - 1; d > 0; --d) {
                const uint64_t m = g.shape[d];
                const uint64_t q = r / m;
                off += (int64_t)(r - q * m) * g.step[d];
                r = q;
            }
            off += (int64_t)r * g.step[0];
        }
        reinterpret_cast<E*>(g.out)[i] = *reinterpret_cast<const E*>(g.in + off);
    }
}

}  // namespace
}  // namespace cumo_hip

using namespace cumo_hip;

extern "C" {

// reference: where_kernel.cu:83-89
char* cumo_bit_where_scratch_new(void) {
    char* scratch = cumo_cuda_runtime_malloc((2 + kWhMaxBlocks) * sizeof(uint64_t));
    if (!scratch) return nullptr;
    hipLaunchKernelGGL(where_zero_kernel, dim3(1), dim3(64), 0, current_stream(), reinterpret_cast<uint64_t*>(scratch));
    cumo_cuda_runtime_check_kernel_launch();
    return scratch;
}

// reference: where_kernel.cu:91-107
void cumo_bit_where_kernel_launch(CUMO_BIT_DIGIT* a, size_t p, ssize_t s, size_t* idx, uint64_t n, int invert, char* out, size_t elmsz, uint64_t count,
                                  char* scratch) {
    uint64_t* running = reinterpret_cast<uint64_t*>(scratch) + (invert ? 1 : 0);
    where_launch<0>(a, p, s, idx, n, invert, out, elmsz, count, 0, 0, nullptr, running, reinterpret_cast<uint64_t*>(scratch) + 2);
}

// reference: mask_kernel.cu:36-54
void cumo_bit_mask_kernel_launch(CUMO_BIT_DIGIT* a, size_t p, ssize_t s, size_t* idx, uint64_t n, size_t* out, size_t p2, ssize_t s2, size_t* idx2,
                                 char* scratch) {
    where_launch<1>(a, p, s, idx, n, 0, reinterpret_cast<char*>(out), sizeof(size_t), 0, p2, s2, idx2, reinterpret_cast<uint64_t*>(scratch),
                       reinterpret_cast<uint64_t*>(scratch) + 2);
}

// The same compaction for a caller that sizes the result in between: the blocks' counts of one run
// (cumo_hip_bit_where_blocks(n) of them, every one written), which the caller reads back and adds
// up, then the placement, where every block adds up the counts before it. Two launches instead of
// a count for the size plus the three above.
size_t cumo_hip_bit_where_blocks(uint64_t n) { return (size_t)wh_geometry(n).nblocks; }

void cumo_hip_bit_where_count_kernel_launch(CUMO_BIT_DIGIT* a, size_t p, ssize_t s, uint64_t n, int invert, uint64_t* counts) {
    if (n == 0) return;
    const WhGeometry g = wh_geometry(n);
    hipLaunchKernelGGL(where_count_kernel, dim3((unsigned)g.nblocks), dim3(kWhBlock), 0, current_stream(), a, (uint64_t)p, (int64_t)s,
                       (const size_t*)nullptr, n, s == 1 ? 1 : 0, invert, g.nchunks, g.cpb, counts, (uint64_t*)nullptr);
    cumo_cuda_runtime_check_kernel_launch();
}

// The same, and the counts on the host when the call returns (it waits for the stream): the kernel
// writes them into pinned host memory of the calling thread as well, so no copy is queued behind
// it. host_counts: cumo_hip_bit_where_blocks(n) words of ordinary host memory.
int cumo_hip_bit_where_count_to_host(CUMO_BIT_DIGIT* a, size_t p, ssize_t s, uint64_t n, int invert, uint64_t* counts, uint64_t* host_counts) {
    if (n == 0) return CUMO_HIP_OK;
    const WhGeometry g = wh_geometry(n);
    static thread_local uint64_t* pinned = nullptr;   // kWhMaxBlocks words, kept for the thread's lifetime
    if (pinned == nullptr) {
        void* m = nullptr;
        if (!hip_ok(hipHostMalloc(&m, kWhMaxBlocks * sizeof(uint64_t), hipHostMallocMapped | hipHostMallocPortable), "hipHostMalloc")) return CUMO_HIP_ERROR_RUNTIME;
        pinned = static_cast<uint64_t*>(m);
    }
    hipStream_t st = current_stream();
    hipLaunchKernelGGL(where_count_kernel, dim3((unsigned)g.nblocks), dim3(kWhBlock), 0, st, a, (uint64_t)p, (int64_t)s, (const size_t*)nullptr, n,
                       s == 1 ? 1 : 0, invert, g.nchunks, g.cpb, counts, pinned);
    cumo_cuda_runtime_check_kernel_launch();
    if (!hip_ok(hipStreamSynchronize(st), "hipStreamSynchronize")) return CUMO_HIP_ERROR_RUNTIME;
    if (!wait_trouble_check()) return CUMO_HIP_ERROR_RUNTIME;
    std::memcpy(host_counts, pinned, g.nblocks * sizeof(uint64_t));
    return CUMO_HIP_OK;
}

// x == NULL: out[o] = the position in the run of the o-th hit, as an elmsz-byte integer (4 or 8);
// otherwise out[o] = the element (elmsz 4 or 8 bytes) at x + j*sx of the o-th hit j.
void cumo_hip_bit_where_place_kernel_launch(CUMO_BIT_DIGIT* a, size_t p, ssize_t s, uint64_t n, int invert, const uint64_t* counts, const char* x,
                                            ssize_t sx, size_t elmsz, char* out) {
    if (n == 0) return;
    const WhGeometry g = wh_geometry(n);
    const int contiguous = s == 1 ? 1 : 0;
    hipStream_t st = current_stream();
#define WH_PLACE(MODE, ES, P2, S2)                                                                                                     \
    hipLaunchKernelGGL((where_scatter_kernel<MODE, ES, true>), dim3((unsigned)g.nblocks), dim3(kWhBlock), 0, st, a, (uint64_t)p, (int64_t)s, \
                       (const size_t*)nullptr, n, contiguous, invert, g.nchunks, g.cpb, out, (uint64_t)0, (size_t)(P2), (int64_t)(S2),      \
                       (const size_t*)nullptr, counts)
    if (x) {
        if (elmsz == 4) WH_PLACE(2, 4, (uintptr_t)x, sx);
        else WH_PLACE(2, 8, (uintptr_t)x, sx);
    } else {
        if (elmsz == 4) WH_PLACE(0, 4, 0, 0);
        else WH_PLACE(0, 8, 0, 0);
    }
#undef WH_PLACE
    cumo_cuda_runtime_check_kernel_launch();
}

void cumo_hip_gather_flat_kernel_launch(const cumo_hip_gather_flat_t* d) {
    if (!d || d->n == 0) return;
    GatherParams g;
    std::memset(&g, 0, sizeof(g));
    // dimensions that follow one another in memory count as one; size-1 dimensions drop out
    uint64_t total = 1;
    int nd = 0;
    for (int k = 0; k < d->ndim && k < CUMO_NA_MAX_DIMENSION; ++k) {
        total *= d->shape[k];
        if (d->shape[k] == 1) continue;
        if (nd > 0 && g.step[nd - 1] == (int64_t)d->step[k] * (int64_t)d->shape[k]) {
            g.shape[nd - 1] *= d->shape[k];
            g.step[nd - 1] = d->step[k];
        } else {
            g.shape[nd] = d->shape[k];
            g.step[nd] = d->step[k];
            ++nd;
        }
    }
    if (nd == 0) {
        g.shape[0] = 1;
        nd = 1;
    }
    g.ndim = nd;
    const bool small = total < (1ull << 31);
    if (small) {
        for (int k = 0; k < nd; ++k) g.div[k] = div31_make((uint32_t)g.shape[k]);
    }
    g.n = d->n;
    g.in = d->in;
    g.out = d->out;
    g.pos = d->pos;
    uint64_t grid = (d->n + 255) / 256;
    if (grid > 65536) grid = 65536;
    hipStream_t st = current_stream();
#define WH_GATHER(PW, EW)                                                                                              \
    do {                                                                                                               \
        if (small) hipLaunchKernelGGL((gather_flat_kernel<PW, EW, true>), dim3((unsigned)grid), dim3(256), 0, st, g);  \
        else hipLaunchKernelGGL((gather_flat_kernel<PW, EW, false>), dim3((unsigned)grid), dim3(256), 0, st, g);       \
    } while (0)
    if (d->pos_elmsz == 4 && d->elmsz == 4) WH_GATHER(4, 4);
    else if (d->pos_elmsz == 4) WH_GATHER(4, 8);
    else if (d->elmsz == 4) WH_GATHER(8, 4);
    else WH_GATHER(8, 8);
#undef WH_GATHER
    cumo_cuda_runtime_check_kernel_launch();
}

}  // extern "C"
