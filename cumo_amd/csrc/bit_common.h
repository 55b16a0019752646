// Device and host helpers shared by the Bit kernels (bit.hip, bit_store.hip): bits are
// packed LSB first in 32-bit words (reference: ext/cumo/include/cumo/narray.h:489-496,
// include/cumo/template.h:110-138); positions and steps are in bits.
#ifndef CUMO_HIP_BIT_COMMON_H
#define CUMO_HIP_BIT_COMMON_H

#include "common.h"
#include "plan.h"

#include <cstring>

namespace {

using namespace cumo_hip;

constexpr int kBlock = 256;
constexpr unsigned kGridCap = kNumCU * 8;

__device__ __forceinline__ uint32_t low_bits(unsigned n) { return n >= 32 ? 0xffffffffu : ((1u << n) - 1u); }

// 32 bits of `a` starting at absolute bit position q (q may be negative at the
// front edge or run past the end; bits outside [0, 32*nw) read as 0)
__device__ __forceinline__ uint32_t bits_at(const CUMO_BIT_DIGIT* a, int64_t q, uint64_t nw) {
    const int64_t w = q >> 5;  // floor
    const unsigned sh = (unsigned)(q & 31);
    uint32_t lo = (w >= 0 && (uint64_t)w < nw) ? a[w] : 0u;
    if (sh == 0) return lo;
    uint32_t hi = (w + 1 >= 0 && (uint64_t)(w + 1) < nw) ? a[w + 1] : 0u;
    return (lo >> sh) | (hi << (32 - sh));
}

struct BitNd {
    int ndim;
    uint64_t total;
    uint64_t shape[kMaxDim];
};

// bit position / byte offset of flat element i of an operand that is strided or
// indexed per dimension
__device__ __forceinline__ int64_t stridx_offset(const cumo_stridx_t* sdx, const BitNd& nd, uint64_t i) {
    int64_t off = 0;
    for (int d = nd.ndim - 1; d >= 0; --d) {
        uint64_t k;
        if (d == 0) {
            k = i;
        } else {
            const uint64_t q = i / nd.shape[d];
            k = i - q * nd.shape[d];
            i = q;
        }
        const cumo_stridx_t s = sdx[d];
        if (s.stride & 1) off += (s.stride >> 1) * (int64_t)k;
        else off += (int64_t)s.index[k];
    }
    return off;
}

__device__ __forceinline__ uint32_t load_bit(const CUMO_BIT_DIGIT* a, uint64_t pos) { return (a[pos >> 5] >> (pos & 31)) & 1u; }

__device__ __forceinline__ void store_bit_atomic(CUMO_BIT_DIGIT* a, uint64_t pos, uint32_t v) {
    const uint32_t bit = 1u << (pos & 31);
    if (v) atomicOr(&a[pos >> 5], bit);
    else atomicAnd(&a[pos >> 5], ~bit);
}

inline unsigned grid_for(uint64_t items, unsigned cap = kGridCap) {
    uint64_t g = (items + kBlock - 1) / kBlock;
    if (g > cap) g = cap;
    if (g == 0) g = 1;
    return (unsigned)g;
}

inline BitNd make_nd(const cumo_na_indexer_t* indexer) {
    BitNd nd;
    std::memset(&nd, 0, sizeof(nd));
    nd.ndim = indexer->ndim;
    nd.total = indexer->total_size;
    for (int d = 0; d < indexer->ndim; ++d) nd.shape[d] = indexer->shape[d];
    return nd;
}

}  // namespace

#endif
