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
#include "div31.h"

#include <cstdlib>
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

// 128 bits of `a` from bit position q on (q >= 0): one 128-bit load from a 4-byte boundary and, when q is not
// at the start of a word, the word after it, funnel-shifted. Nothing that looks at a loaded word sits under a
// branch: that would make the caller wait for one operand's words before it asks for the next operand's. The
// caller has checked that all the bits are there. Every lane of a wave that is switched on calls it together.
struct Raw128 {
    uint32_t v __attribute__((ext_vector_type(4)));
    uint32_t e;
    unsigned sh;
    bool own;  // the fifth word is the lane's own load (e); otherwise it is the next lane's first word
};
// what the next lane (within a row of sixteen) holds in `x`; `otherwise` where there is no such lane or it is switched off
__device__ __forceinline__ uint32_t next_lane(uint32_t x, uint32_t otherwise) {
    return (uint32_t)__builtin_amdgcn_update_dpp((int)otherwise, (int)x, 0x101 /* row_shl:1 */, 0xf, 0xf, false);
}
template <bool NT>
__device__ __forceinline__ Raw128 raw128_load(const CUMO_BIT_DIGIT* a, uint64_t q) {
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    Raw128 r;
    const uint64_t w = q >> 5;
    r.sh = (unsigned)(q & 31);
    r.v = NT ? __builtin_nontemporal_load(reinterpret_cast<const u4*>(a + w)) : *reinterpret_cast<const u4*>(a + w);
    // The word after the four is the first of the next lane's four when that lane reads the 128 bits that follow
    // these; a lane whose neighbour reads elsewhere (or is the last of its sixteen, or sits this out) loads the
    // word itself. A load per lane would cost the memory pipeline a fifth of what the vectors cost it.
    const uint64_t q_after = q + 128;
    const uint32_t qlo = (uint32_t)q, qhi = (uint32_t)(q >> 32);
    r.own = next_lane(qlo, qlo) != (uint32_t)q_after || next_lane(qhi, ~qhi) != (uint32_t)(q_after >> 32);
    r.e = 0;
    if (r.sh != 0 && r.own) r.e = a[w + 4];
    return r;
}
// (kept apart from the loads so that a caller can ask for all its operands' words before it shifts the first)
__device__ __forceinline__ uint4 raw128_bits(const Raw128& r) {
    const uint32_t from_next = next_lane(r.v.x, 0u);
    const uint32_t e = r.own ? r.e : from_next;
    return make_uint4(__builtin_amdgcn_alignbit(r.v.y, r.v.x, r.sh), __builtin_amdgcn_alignbit(r.v.z, r.v.y, r.sh),
                      __builtin_amdgcn_alignbit(r.v.w, r.v.z, r.sh), __builtin_amdgcn_alignbit(e, r.v.w, r.sh));
}
template <bool NT>
__device__ __forceinline__ uint4 bits128_at(const CUMO_BIT_DIGIT* a, uint64_t q) {
    return raw128_bits(raw128_load<NT>(a, q));
}

// The same, four output words per lane. The output vectors are the 16-byte aligned ones (`lead` = words
// between the boundary before a3 and a3); a vector whose words all lie inside the run away from its
// first and last word goes as a whole, the words of the others one by one as above.
template <int OP, bool BINARY, bool NT>
__global__ __launch_bounds__(kBlock) void bit_contiguous_vec_kernel(const CUMO_BIT_DIGIT* a1, uint64_t p1, const CUMO_BIT_DIGIT* a2, uint64_t p2,
                                                                    CUMO_BIT_DIGIT* a3, uint64_t p3, uint64_t n, unsigned lead) {
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    const uint64_t nw1 = (p1 + n + 31) >> 5, nw2 = (p2 + n + 31) >> 5, nw3 = (p3 + n + 31) >> 5;
    const uint64_t nvec = (nw3 + lead + 3) >> 2;
    const uint64_t endbit = p3 + n;
    for (uint64_t v = (uint64_t)blockIdx.x * kBlock + threadIdx.x; v < nvec; v += (uint64_t)gridDim.x * kBlock) {
        const int64_t w0 = (int64_t)(v << 2) - (int64_t)lead;
        if (w0 >= 1 && (uint64_t)w0 + 4 <= nw3 - 1) {
            const uint64_t e0 = ((uint64_t)w0 << 5) - p3;
            const uint4 x = bits128_at<NT>(a1, e0 + p1);
            uint4 y = make_uint4(0u, 0u, 0u, 0u);
            if (BINARY) y = bits128_at<NT>(a2, e0 + p2);
            u4 z;
            z.x = bit_apply<OP>(x.x, y.x);
            z.y = bit_apply<OP>(x.y, y.y);
            z.z = bit_apply<OP>(x.z, y.z);
            z.w = bit_apply<OP>(x.w, y.w);
            if (NT) __builtin_nontemporal_store(z, reinterpret_cast<u4*>(a3 + w0));
            else *reinterpret_cast<u4*>(a3 + w0) = z;
            continue;
        }
        for (int64_t ww = w0 < 0 ? 0 : w0; ww < w0 + 4 && (uint64_t)ww < nw3; ++ww) {
            const uint64_t w = (uint64_t)ww;
            const int64_t e0 = (int64_t)(w << 5) - (int64_t)p3;
            const uint32_t x = bits_at(a1, e0 + (int64_t)p1, nw1);
            const uint32_t y = BINARY ? bits_at(a2, e0 + (int64_t)p2, nw2) : 0u;
            const uint32_t z = bit_apply<OP>(x, y);
            const unsigned lo = (w == 0) ? (unsigned)p3 : 0u;
            const unsigned hi = ((w + 1) << 5) <= endbit ? 32u : (unsigned)(endbit - (w << 5));
            const uint32_t mask = low_bits(hi) & ~low_bits(lo);
            if (mask == 0xffffffffu) a3[w] = z;
            else a3[w] = (z & mask) | (a3[w] & ~mask);
        }
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

// Views whose innermost dimension runs along the bits (step 1) in every operand and that use no index
// array: a lane takes four words of one result row, as a vector where the row has all four to itself.
// nw1 / nw2: words of a1 / a2 up to the last bit the view reaches (nothing past them is read). A
// row's first and last word may be shared with its neighbours in memory, so those two are changed
// with atomics; the words between them belong to the row alone.
struct BitRowsOp {
    int ndim;
    uint64_t items, chunks, inner;   // chunks: lanes per row, each with four of the result words the row can span
    uint64_t shape[kMaxDim];
    int64_t s1[kMaxDim], s2[kMaxDim], s3[kMaxDim];  // bit steps of the outer dimensions
    uint64_t nw1, nw2;
};

template <int OP, bool BINARY>
__global__ __launch_bounds__(kBlock) void bit_rows_kernel(const CUMO_BIT_DIGIT* a1, uint64_t p1, const CUMO_BIT_DIGIT* a2, uint64_t p2,
                                                          CUMO_BIT_DIGIT* a3, uint64_t p3, BitRowsOp nd) {
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    for (uint64_t item = (uint64_t)blockIdx.x * kBlock + threadIdx.x; item < nd.items; item += (uint64_t)gridDim.x * kBlock) {
        uint64_t q = item / nd.chunks;
        const uint64_t k = (item - q * nd.chunks) * 4;  // a lane takes four words of the row
        int64_t q1 = (int64_t)p1, q2 = (int64_t)p2, q3 = (int64_t)p3;
        for (int d = nd.ndim - 2; d >= 0; --d) {
            uint64_t i = q;
            if (d > 0) {
                const uint64_t up = q / nd.shape[d];
                i = q - up * nd.shape[d];
                q = up;
            }
            q1 += (int64_t)i * nd.s1[d];
            q2 += (int64_t)i * nd.s2[d];
            q3 += (int64_t)i * nd.s3[d];
        }
        const uint64_t w_first = (uint64_t)q3 >> 5, w_last = ((uint64_t)q3 + nd.inner - 1) >> 5;
        const uint64_t w0 = w_first + k;
        if (w0 > w_last) continue;
        const int64_t e00 = (int64_t)(w0 << 5) - q3;  // the row's element at bit 0 of the lane's first word (negative in the row's first word)
        // four words that the row has to itself, whose inputs (five words each when they start inside a word) are all there
        if (w0 > w_first && w0 + 3 < w_last && (((uint64_t)(q1 + e00)) >> 5) + 5 <= nd.nw1 &&
            (!BINARY || (((uint64_t)(q2 + e00)) >> 5) + 5 <= nd.nw2)) {
            const uint4 x = bits128_at<false>(a1, (uint64_t)(q1 + e00));
            uint4 y = make_uint4(0u, 0u, 0u, 0u);
            if (BINARY) y = bits128_at<false>(a2, (uint64_t)(q2 + e00));
            u4 z;
            z.x = bit_apply<OP>(x.x, y.x);
            z.y = bit_apply<OP>(x.y, y.y);
            z.z = bit_apply<OP>(x.z, y.z);
            z.w = bit_apply<OP>(x.w, y.w);
            *reinterpret_cast<u4*>(a3 + w0) = z;
            continue;
        }
        for (uint64_t w = w0; w < w0 + 4 && w <= w_last; ++w) {
            const int64_t e0 = (int64_t)(w << 5) - q3;
            const uint32_t x = bits_at(a1, q1 + e0, nd.nw1);
            const uint32_t y = BINARY ? bits_at(a2, q2 + e0, nd.nw2) : 0u;
            const uint32_t z = bit_apply<OP>(x, y);
            const unsigned lo = (w == w_first) ? (unsigned)((uint64_t)q3 & 31) : 0u;
            const unsigned hi = (w == w_last) ? (unsigned)(((uint64_t)q3 + nd.inner - 1) & 31) + 1u : 32u;
            const uint32_t mask = low_bits(hi) & ~low_bits(lo);
            if (w != w_first && w != w_last) {
                a3[w] = z;
            } else {
                atomicAnd(&a3[w], ~mask);
                atomicOr(&a3[w], z & mask);
            }
        }
    }
}

// The same views when the result's rows follow one another without a gap (a fresh result always does): the
// result is then one run of bits, and a lane takes one 16-byte aligned vector of its words, wherever the rows
// fall in it. It finds the row and the column of the vector's first bit (one multiplication by the reciprocal of
// the row length, corrected by at most one) and reads 128 bits of each source from there; a vector that a row
// ends in, or whose sources end within reach, is put together word by word from the two rows it spans (rows are
// at least 128 bits long here). Stores are whole aligned vectors but for the run's first and last word.
constexpr int kFlatOuter = 6;
struct BitFlatRows {
    int nouter;                  // outer dimensions after merging, outermost first
    uint32_t rows;
    uint32_t shape[kFlatOuter];
    Div31 dv[kFlatOuter];
    int64_t s1[kFlatOuter], s2[kFlatOuter];
    uint64_t inner, total, nw1, nw2;
    double inv_inner;
};

__device__ __forceinline__ void flat_row_col(const BitFlatRows& nd, uint64_t e, uint32_t& r, uint64_t& c) {
    uint64_t q = (uint64_t)((double)e * nd.inv_inner);  // within one of e / inner: e < 2^52
    int64_t rem = (int64_t)e - (int64_t)(q * nd.inner);
    if (rem < 0) {
        --q;
        rem += (int64_t)nd.inner;
    } else if (rem >= (int64_t)nd.inner) {
        ++q;
        rem -= (int64_t)nd.inner;
    }
    r = (uint32_t)q;
    c = (uint64_t)rem;
}

__device__ __forceinline__ void flat_row_pos(const BitFlatRows& nd, uint32_t r, int64_t& q1, int64_t& q2) {
    uint32_t q = r;
    for (int d = nd.nouter - 1; d > 0; --d) {
        const uint32_t up = div31(q, nd.dv[d]);
        const uint32_t i = q - up * nd.shape[d];
        q = up;
        q1 += (int64_t)i * nd.s1[d];
        q2 += (int64_t)i * nd.s2[d];
    }
    q1 += (int64_t)q * nd.s1[0];
    q2 += (int64_t)q * nd.s2[0];
}

// 32 bits of both sources for the result's elements e ... e + 31 (bit b = element e + b; bits of elements outside
// [0, total) come out as anything: the caller masks them)
template <bool BINARY>
__device__ __forceinline__ void flat_src_words(const CUMO_BIT_DIGIT* a1, uint64_t p1, const CUMO_BIT_DIGIT* a2, uint64_t p2, const BitFlatRows& nd,
                                               int64_t e, uint32_t& x, uint32_t& y) {
    const uint64_t ec = e < 0 ? 0 : (uint64_t)e;
    const unsigned shift = (unsigned)(ec - (uint64_t)e);  // e + shift = ec
    x = y = 0;
    if (ec >= nd.total) return;
    uint32_t r;
    uint64_t c;
    flat_row_col(nd, ec, r, c);
    int64_t q1 = (int64_t)p1, q2 = (int64_t)p2;
    flat_row_pos(nd, r, q1, q2);
    x = bits_at(a1, q1 + (int64_t)c, nd.nw1);
    if (BINARY) y = bits_at(a2, q2 + (int64_t)c, nd.nw2);
    const uint64_t avail = nd.inner - c;
    if (avail < 32) {
        const uint32_t keep = low_bits((unsigned)avail);
        x &= keep;
        y &= keep;
        if (r + 1 < nd.rows) {
            int64_t n1 = (int64_t)p1, n2 = (int64_t)p2;
            flat_row_pos(nd, r + 1, n1, n2);
            x |= bits_at(a1, n1, nd.nw1) << avail;
            if (BINARY) y |= bits_at(a2, n2, nd.nw2) << avail;
        }
    }
    x <<= shift;
    y <<= shift;
}

template <int OP, bool BINARY, bool NT>
__global__ __launch_bounds__(kBlock) void bit_rows_flat_kernel(const CUMO_BIT_DIGIT* a1, uint64_t p1, const CUMO_BIT_DIGIT* a2, uint64_t p2,
                                                               CUMO_BIT_DIGIT* a3, uint64_t p3, unsigned lead, BitFlatRows nd) {
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    const uint64_t nw3 = (p3 + nd.total + 31) >> 5;
    const uint64_t nvec = (nw3 + lead + 3) >> 2;
    const uint64_t endbit = p3 + nd.total;
    // the row and column of a lane's vector come from a division once; from then on they move by what the grid's
    // step is in rows and columns (the two lanes whose order is changed below divide every time)
    bool have_rc = false;
    uint32_t r = 0;
    uint64_t c = 0;
    const uint64_t step_bits = ((uint64_t)gridDim.x * kBlock) << 7;
    const uint32_t step_r = (uint32_t)(step_bits / nd.inner);
    const uint64_t step_c = step_bits - (uint64_t)step_r * nd.inner;
    for (uint64_t it = (uint64_t)blockIdx.x * kBlock + threadIdx.x; it < nvec; it += (uint64_t)gridDim.x * kBlock) {
        if (have_rc) {
            r += step_r;
            c += step_c;
            if (c >= nd.inner) {
                c -= nd.inner;
                ++r;
            }
        }
        // the run's last vector goes first (with the first one, in the launch's first wave): the two are put together word by
        // word, a chain of loads that would otherwise stand alone at the end of the launch
        const uint64_t v = it == 0 ? nvec - 1 : it - 1;
        const int64_t w0 = (int64_t)(v << 2) - (int64_t)lead;
        const bool whole = w0 >= 1 && (uint64_t)w0 + 4 <= nw3 - 1;
        if (whole) {
            if (!have_rc) {
                flat_row_col(nd, ((uint64_t)w0 << 5) - p3, r, c);
                have_rc = it >= 2;
            }
            int64_t q1 = (int64_t)p1, q2 = (int64_t)p2;
            flat_row_pos(nd, r, q1, q2);
            q1 += (int64_t)c;
            q2 += (int64_t)c;
            bool ok = ((uint64_t)q1 >> 5) + 5 <= nd.nw1 && (!BINARY || ((uint64_t)q2 >> 5) + 5 <= nd.nw2);
            // a row ends inside the vector: its first `mine` bits are row r's, the rest the start of row r + 1, read as the
            // 128 bits that have that start at bit `mine`
            const bool split = c + 128 > nd.inner;
            const unsigned mine = split ? (unsigned)(nd.inner - c) : 128u;
            int64_t n1 = (int64_t)p1, n2 = (int64_t)p2;
            if (split) {
                flat_row_pos(nd, r + 1, n1, n2);
                n1 -= (int64_t)mine;
                n2 -= (int64_t)mine;
                ok = ok && n1 >= 0 && ((uint64_t)n1 >> 5) + 5 <= nd.nw1 && (!BINARY || (n2 >= 0 && ((uint64_t)n2 >> 5) + 5 <= nd.nw2));
            }
            if (ok) {
                // every load of the vector is asked for before the first is looked at
                const Raw128 rx = raw128_load<NT>(a1, (uint64_t)q1);
                Raw128 none;
                none.v = 0;
                none.e = 0;
                none.sh = 0;
                none.own = true;
                Raw128 ry = none, rxn = none, ryn = none;  // (not copies of rx: a copy would wait for its words)
                if (BINARY) ry = raw128_load<NT>(a2, (uint64_t)q2);
                if (split) {
                    rxn = raw128_load<NT>(a1, (uint64_t)n1);
                    if (BINARY) ryn = raw128_load<NT>(a2, (uint64_t)n2);
                }
                uint4 x = raw128_bits(rx);
                uint4 y = BINARY ? raw128_bits(ry) : make_uint4(0u, 0u, 0u, 0u);
                if (split) {
                    const uint4 xn = raw128_bits(rxn);
                    const uint32_t m0 = low_bits(mine), m1 = mine > 32 ? low_bits(mine - 32) : 0u, m2 = mine > 64 ? low_bits(mine - 64) : 0u,
                                   m3 = mine > 96 ? low_bits(mine - 96) : 0u;
                    x = make_uint4((x.x & m0) | (xn.x & ~m0), (x.y & m1) | (xn.y & ~m1), (x.z & m2) | (xn.z & ~m2), (x.w & m3) | (xn.w & ~m3));
                    if (BINARY) {
                        const uint4 yn = raw128_bits(ryn);
                        y = make_uint4((y.x & m0) | (yn.x & ~m0), (y.y & m1) | (yn.y & ~m1), (y.z & m2) | (yn.z & ~m2), (y.w & m3) | (yn.w & ~m3));
                    }
                }
                u4 z;
                z.x = bit_apply<OP>(x.x, y.x);
                z.y = bit_apply<OP>(x.y, y.y);
                z.z = bit_apply<OP>(x.z, y.z);
                z.w = bit_apply<OP>(x.w, y.w);
                if (NT) __builtin_nontemporal_store(z, reinterpret_cast<u4*>(a3 + w0));
                else *reinterpret_cast<u4*>(a3 + w0) = z;
                continue;
            }
        }
        for (int64_t ww = w0 < 0 ? 0 : w0; ww < w0 + 4 && (uint64_t)ww < nw3; ++ww) {
            const uint64_t w = (uint64_t)ww;
            uint32_t x, y;
            flat_src_words<BINARY>(a1, p1, a2, p2, nd, (int64_t)(w << 5) - (int64_t)p3, x, y);
            const uint32_t z = bit_apply<OP>(x, y);
            const unsigned lo = (w == 0) ? (unsigned)p3 : 0u;
            const unsigned hi = ((w + 1) << 5) <= endbit ? 32u : (unsigned)(endbit - (w << 5));
            const uint32_t mask = low_bits(hi) & ~low_bits(lo);
            if (mask == 0xffffffffu) a3[w] = z;
            else a3[w] = (z & mask) | (a3[w] & ~mask);
        }
    }
}

// The most blocks a launch of the vector kernels gets. A lane per vector, in blocks that come and go, keeps memory
// busier than fewer blocks whose lanes loop (measured on 64 and 256 MiB operands: 0.73 -> 0.74 and 0.70 -> 0.80 of
// peak for a & b, more where the sources are shifted), so the bound only guards the grid's size.
// CUMO_HIP_BIT_VEC_GRID (read once) sets it in blocks per compute unit.
unsigned bit_vec_grid_cap() {
    static int64_t cap = -1;
    if (cap < 0) {
        const char* e = std::getenv("CUMO_HIP_BIT_VEC_GRID");
        const long mult = e ? std::atol(e) : 0;
        cap = mult >= 1 && mult <= (1 << 14) ? (int64_t)kNumCU * mult : (int64_t)1 << 22;
    }
    return (unsigned)cap;
}

// the flat form of the row kernel, for operands bit_rows_launch has vetted (strides only, innermost step 1,
// no position below zero); false when the result's rows do not follow one another or the shape is outside its limits
template <int OP, bool BINARY>
bool bit_rows_flat_launch(cumo_na_bit_iarray_stridx_t* const* ops, const cumo_na_indexer_t* indexer, const uint64_t* reach) {
    const int n = indexer->ndim;
    const uint64_t inner = indexer->shape[n - 1];
    if (inner < 128) return false;
    uint64_t rows = 1;
    int64_t want = (int64_t)inner;
    for (int d = n - 2; d >= 0; --d) {
        if ((int64_t)CUMO_SDX_GET_STRIDE(ops[2]->stridx[d]) != want && indexer->shape[d] != 1) return false;
        want *= (int64_t)indexer->shape[d];
        rows *= indexer->shape[d];
    }
    if (rows == 0 || rows >= (1ull << 31) || rows * inner >= (1ull << 52)) return false;
    BitFlatRows nd;
    std::memset(&nd, 0, sizeof(nd));
    // outer dimensions, merged where both sources step through two of them as through one
    int m = 0;
    for (int d = 0; d < n - 1; ++d) {
        if (indexer->shape[d] == 1) continue;
        const int64_t t1 = (int64_t)CUMO_SDX_GET_STRIDE(ops[0]->stridx[d]), t2 = (int64_t)CUMO_SDX_GET_STRIDE(ops[1]->stridx[d]);
        if (m > 0 && nd.s1[m - 1] == t1 * (int64_t)indexer->shape[d] && nd.s2[m - 1] == t2 * (int64_t)indexer->shape[d]) {
            nd.shape[m - 1] *= (uint32_t)indexer->shape[d];
            nd.s1[m - 1] = t1;
            nd.s2[m - 1] = t2;
            continue;
        }
        if (m == kFlatOuter) return false;
        nd.shape[m] = (uint32_t)indexer->shape[d];
        nd.s1[m] = t1;
        nd.s2[m] = t2;
        ++m;
    }
    if (m == 0) {  // a single row
        nd.shape[0] = 1;
        m = 1;
    }
    for (int d = 0; d < m; ++d) nd.dv[d] = div31_make(nd.shape[d]);
    nd.nouter = m;
    nd.rows = (uint32_t)rows;
    nd.inner = inner;
    nd.total = rows * inner;
    nd.inv_inner = 1.0 / (double)inner;
    nd.nw1 = reach[0];
    nd.nw2 = reach[1];
    CUMO_BIT_DIGIT* a3 = ops[2]->ptr + ops[2]->pos / 32;
    const uint64_t p3 = ops[2]->pos % 32;
    const uint64_t nw3 = (p3 + nd.total + 31) >> 5;
    const unsigned lead = (unsigned)(((uintptr_t)a3 % 16) / sizeof(CUMO_BIT_DIGIT));
    const dim3 g(grid_for((nw3 + lead + 3) / 4, bit_vec_grid_cap())), b(kBlock);
    if (stream_past_caches(nw3 * 4 * (BINARY ? 3 : 2)))
        hipLaunchKernelGGL((bit_rows_flat_kernel<OP, BINARY, true>), g, b, 0, current_stream(), (const CUMO_BIT_DIGIT*)ops[0]->ptr, (uint64_t)ops[0]->pos,
                           (const CUMO_BIT_DIGIT*)ops[1]->ptr, (uint64_t)ops[1]->pos, a3, p3, lead, nd);
    else
        hipLaunchKernelGGL((bit_rows_flat_kernel<OP, BINARY, false>), g, b, 0, current_stream(), (const CUMO_BIT_DIGIT*)ops[0]->ptr, (uint64_t)ops[0]->pos,
                           (const CUMO_BIT_DIGIT*)ops[1]->ptr, (uint64_t)ops[1]->pos, a3, p3, lead, nd);
    cumo_cuda_runtime_check_kernel_launch();
    return true;
}

// launches the row form when the operands allow it; false: the caller uses the bit-by-bit kernel
template <int OP, bool BINARY>
bool bit_rows_launch(cumo_na_bit_iarray_stridx_t* a1, cumo_na_bit_iarray_stridx_t* a2, cumo_na_bit_iarray_stridx_t* a3, cumo_na_indexer_t* indexer) {
    const int n = indexer->ndim;
    if (n < 2 || n > kMaxDim || force_wide_indices() || indexer->shape[n - 1] < 32) return false;
    cumo_na_bit_iarray_stridx_t* ops[3] = {a1, BINARY ? a2 : a1, a3};
    BitRowsOp nd;
    std::memset(&nd, 0, sizeof(nd));
    uint64_t reach[3];
    for (int j = 0; j < 3; ++j) {
        int64_t lowest = (int64_t)ops[j]->pos, highest = (int64_t)ops[j]->pos;
        for (int d = 0; d < n; ++d) {
            if (!CUMO_SDX_IS_STRIDE(ops[j]->stridx[d])) return false;
            const int64_t st = (int64_t)CUMO_SDX_GET_STRIDE(ops[j]->stridx[d]);
            if (d == n - 1 && st != 1) return false;
            const int64_t span = st * (int64_t)(indexer->shape[d] - 1);
            if (span < 0) lowest += span;
            else highest += span;
        }
        if (lowest < 0) return false;  // (bit positions are computed unsigned)
        // a result row that lies across another's words in memory (a repeated or reversed-overlapping view) is not taken
        if (j == 2) {
            for (int d = 0; d < n - 1; ++d) {
                const int64_t st = (int64_t)CUMO_SDX_GET_STRIDE(a3->stridx[d]);
                if ((st < 0 ? -st : st) < (int64_t)indexer->shape[n - 1]) return false;
            }
        }
        reach[j] = ((uint64_t)highest + 32) >> 5;
    }
    nd.ndim = n;
    nd.inner = indexer->shape[n - 1];
    nd.chunks = ((nd.inner + 31) / 32 + 1 + 3) / 4;  // lanes a row can need: four of its words each
    nd.items = nd.chunks;
    for (int d = 0; d < n; ++d) {
        nd.shape[d] = indexer->shape[d];
        if (d < n - 1) {
            nd.items *= indexer->shape[d];
            nd.s1[d] = (int64_t)CUMO_SDX_GET_STRIDE(ops[0]->stridx[d]);
            nd.s2[d] = (int64_t)CUMO_SDX_GET_STRIDE(ops[1]->stridx[d]);
            nd.s3[d] = (int64_t)CUMO_SDX_GET_STRIDE(ops[2]->stridx[d]);
        }
    }
    nd.nw1 = reach[0];
    nd.nw2 = reach[1];
    if (bit_rows_flat_launch<OP, BINARY>(ops, indexer, reach)) return true;
    hipLaunchKernelGGL((bit_rows_kernel<OP, BINARY>), dim3(grid_for(nd.items, kNumCU * 32)), dim3(kBlock), 0, current_stream(),
                       (const CUMO_BIT_DIGIT*)ops[0]->ptr, (uint64_t)ops[0]->pos, (const CUMO_BIT_DIGIT*)ops[1]->ptr, (uint64_t)ops[1]->pos, a3->ptr,
                       (uint64_t)a3->pos, nd);
    cumo_cuda_runtime_check_kernel_launch();
    return true;
}

template <class T>
__global__ __launch_bounds__(kBlock) void store_bit_kernel(cumo_na_iarray_stridx_t dst, cumo_na_bit_iarray_stridx_t src, BitNd nd) {
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < nd.total; i += (uint64_t)gridDim.x * kBlock) {
        const uint32_t x = load_bit(src.ptr, src.pos + (uint64_t)stridx_offset(src.stridx, nd, i));
        *reinterpret_cast<T*>(dst.ptr + stridx_offset(dst.stridx, nd, i)) = (T)x;
    }
}

// Bit -> number where both run along the innermost dimension (bit step 1, element step sizeof(T)) and
// no dimension goes through an index array: a lane takes four neighbouring elements of a row, reads the
// one or two words that hold their bits and stores them as 128-bit vectors (which need the element's
// alignment only). s_src (bits) and s_dst (bytes) are the steps of the outer dimensions.
struct BitRowsNd {
    int ndim;
    uint64_t items, chunks;          // work items; chunks of four elements in a row
    uint64_t shape[kMaxDim];
    int64_t s_src[kMaxDim], s_dst[kMaxDim];
};

template <class T, bool NT>
__global__ __launch_bounds__(kBlock) void store_bit_rows_kernel(char* dst, const CUMO_BIT_DIGIT* src, uint64_t pos, BitRowsNd nd) {
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    const uint64_t inner = nd.shape[nd.ndim - 1];
    for (uint64_t item = (uint64_t)blockIdx.x * kBlock + threadIdx.x; item < nd.items; item += (uint64_t)gridDim.x * kBlock) {
        uint64_t c = item;
        int64_t bit = (int64_t)pos, off = 0;
        if (nd.ndim > 1) {
            uint64_t q = item / nd.chunks;
            c = item - q * nd.chunks;
            for (int d = nd.ndim - 2; d >= 0; --d) {
                uint64_t k = q;
                if (d > 0) {
                    const uint64_t q2 = q / nd.shape[d];
                    k = q - q2 * nd.shape[d];
                    q = q2;
                }
                bit += (int64_t)k * nd.s_src[d];
                off += (int64_t)k * nd.s_dst[d];
            }
        }
        const uint64_t e0 = c * 4;
        const unsigned cnt = inner - e0 >= 4 ? 4u : (unsigned)(inner - e0);
        const uint64_t b0 = (uint64_t)bit + e0;
        const unsigned sh = (unsigned)(b0 & 31);
        // (both words loaded with no branch between them: the second from the first's address when it is not needed)
        const uint32_t lo = src[b0 >> 5];
        const uint32_t hi = src[(b0 >> 5) + (sh + cnt > 32 ? 1 : 0)];
        uint32_t x = lo >> sh;
        if (sh != 0) x |= hi << (32 - sh);
        T* out = reinterpret_cast<T*>(dst + off) + e0;
        if (cnt == 4) {
            union V {
                u4 q[sizeof(T) / 4];
                T v[4];
                __device__ V() {}
            } t;
#pragma unroll
            for (int j = 0; j < 4; ++j) t.v[j] = (T)((x >> j) & 1u);
#pragma unroll
            for (int k = 0; k < (int)(sizeof(T) / 4); ++k) {
                if (NT) __builtin_nontemporal_store(t.q[k], reinterpret_cast<u4*>(out) + k);
                else reinterpret_cast<u4*>(out)[k] = t.q[k];
            }
        } else {
            for (unsigned j = 0; j < cnt; ++j) out[j] = (T)((x >> j) & 1u);
        }
    }
}

// launches the row form when the operands allow it; false: the caller uses the element-wise kernel
template <class T>
bool store_bit_rows_launch(cumo_na_iarray_stridx_t* a1, cumo_na_bit_iarray_stridx_t* a2, cumo_na_indexer_t* indexer) {
    const int n = indexer->ndim;
    if (n < 1 || n > kMaxDim || force_wide_indices()) return false;
    for (int d = 0; d < n; ++d)
        if (!CUMO_SDX_IS_STRIDE(a1->stridx[d]) || !CUMO_SDX_IS_STRIDE(a2->stridx[d])) return false;
    if (CUMO_SDX_GET_STRIDE(a1->stridx[n - 1]) != (ssize_t)sizeof(T) || CUMO_SDX_GET_STRIDE(a2->stridx[n - 1]) != 1) return false;
    if (((uintptr_t)a1->ptr % alignof(T)) != 0 || indexer->shape[n - 1] < 16) return false;
    BitRowsNd nd;
    std::memset(&nd, 0, sizeof(nd));
    nd.ndim = n;
    nd.chunks = (indexer->shape[n - 1] + 3) / 4;
    nd.items = nd.chunks;
    int64_t lowest = 0;
    for (int d = 0; d < n; ++d) {
        nd.shape[d] = indexer->shape[d];
        if (d < n - 1) {
            nd.items *= indexer->shape[d];
            nd.s_src[d] = (int64_t)CUMO_SDX_GET_STRIDE(a2->stridx[d]);
            nd.s_dst[d] = (int64_t)CUMO_SDX_GET_STRIDE(a1->stridx[d]);
            if ((nd.s_dst[d] % (int64_t)alignof(T)) != 0) return false;
            if (nd.s_src[d] < 0) lowest += nd.s_src[d] * (int64_t)(indexer->shape[d] - 1);
        }
    }
    if ((int64_t)a2->pos + lowest < 0) return false;  // (bit positions are computed unsigned)
    const bool nt = stream_past_caches((uint64_t)indexer->total_size * sizeof(T));
    const dim3 g(grid_for(nd.items, kNumCU * 32)), b(kBlock);
    if (nt) hipLaunchKernelGGL((store_bit_rows_kernel<T, true>), g, b, 0, current_stream(), a1->ptr, (const CUMO_BIT_DIGIT*)a2->ptr, (uint64_t)a2->pos, nd);
    else hipLaunchKernelGGL((store_bit_rows_kernel<T, false>), g, b, 0, current_stream(), a1->ptr, (const CUMO_BIT_DIGIT*)a2->ptr, (uint64_t)a2->pos, nd);
    cumo_cuda_runtime_check_kernel_launch();
    return true;
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
    if (nw3 >= 64 && p1 < 32 && p2 < 32 && p3 < 32) {
        const unsigned lead = (unsigned)(((uintptr_t)a3 % 16) / sizeof(CUMO_BIT_DIGIT));
        const dim3 g(grid_for((nw3 + lead + 3) / 4, bit_vec_grid_cap())), b(kBlock);
        if (stream_past_caches(nw3 * 4 * (BINARY ? 3 : 2)))
            hipLaunchKernelGGL((bit_contiguous_vec_kernel<OP, BINARY, true>), g, b, 0, current_stream(), a1, (uint64_t)p1, a2, (uint64_t)p2, a3,
                               (uint64_t)p3, n, lead);
        else
            hipLaunchKernelGGL((bit_contiguous_vec_kernel<OP, BINARY, false>), g, b, 0, current_stream(), a1, (uint64_t)p1, a2, (uint64_t)p2, a3,
                               (uint64_t)p3, n, lead);
        cumo_cuda_runtime_check_kernel_launch();
        return;
    }
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
    if (bit_rows_launch<OP, BINARY>(a1, a2, a3, indexer)) return;
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
            // four words per lane (a 128-bit load from a 4-byte boundary), two such loads in flight
            typedef uint32_t u4 __attribute__((ext_vector_type(4)));
            for (uint64_t wa = w0 + 4 * lane; wa < w1; wa += 512) {
                u4 t[2];
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const uint64_t w = wa + 256 * u;
                    if (w + 4 <= w1) {
                        t[u] = *reinterpret_cast<const u4*>(p.in + w);
                    } else {
                        t[u].x = w < w1 ? p.in[w] : 0u;
                        t[u].y = w + 1 < w1 ? p.in[w + 1] : 0u;
                        t[u].z = w + 2 < w1 ? p.in[w + 2] : 0u;
                        t[u].w = 0u;
                    }
                }
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const uint64_t w = wa + 256 * u;
                    const uint32_t xs[4] = {t[u].x, t[u].y, t[u].z, t[u].w};
                    if (w > w0 && w + 4 < w1) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) c += (uint64_t)__popc(COUNT_FALSE ? ~xs[j] : xs[j]);
                    } else {
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const uint64_t k = w + j;
                            if (k >= w1) continue;
                            uint32_t x = COUNT_FALSE ? ~xs[j] : xs[j];
                            const unsigned lo = (k == w0) ? (unsigned)(p1 & 31) : 0u;
                            const unsigned hi = ((k + 1) << 5) <= endbit ? 32u : (unsigned)(endbit - (k << 5));
                            x &= low_bits(hi) & ~low_bits(lo);
                            c += (uint64_t)__popc(x);
                        }
                    }
                }
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

// Counts down columns: the kept dimension that runs along the bits (step 1) has `cols` outputs, the one
// reduced dimension steps `s_red` bits, and an optional outer kept dimension steps s_outer bits /
// o_outer bytes. A block of 1024 lanes has 32 x 32 neighbouring columns of one outer position and a
// stretch of the rows, a thirty-second of it per group of 32 lanes; a lane owns 32 columns: it reads
// their word row by row (two words where the row does not start on a word; eight rows' loads go out
// before the first is waited for, with no branch between them) and counts every column in byte-wide
// counters, four to a register (column j of the 32 sits in counter j / 8 of register j % 8), moved to
// 32-bit counters before a byte could overflow. The groups add their totals up in LDS, and the block
// adds the sums onto the 64-bit results, one atomic per column that has any.
constexpr int kCountColsBlock = 1024;
constexpr int kCountColsRows = 8;   // rows a lane has in flight

struct BitCountCols {
    const CUMO_BIT_DIGIT* in;
    char* out;
    uint64_t pos;
    uint32_t cols, chunks, chunk_blocks, rows, rows_per_wave, row_parts, n_outer;
    int64_t s_red, s_outer, o_outer, o_col;
};

template <bool COUNT_FALSE>
__global__ __launch_bounds__(kCountColsBlock) void bit_count_cols_kernel(BitCountCols p) {
    __shared__ uint32_t sums[32][32];
    // half a wave has 32 neighbouring chunks of columns (128 bytes of a row), the other half the same chunks of another stretch of rows
    const unsigned lane = threadIdx.x & 31, group = threadIdx.x >> 5;
    const uint32_t cb = blockIdx.x % p.chunk_blocks;
    const uint32_t b2 = blockIdx.x / p.chunk_blocks;
    const uint32_t part = b2 % p.row_parts;
    const uint32_t o = b2 / p.row_parts;
    for (unsigned i = threadIdx.x; i < 32 * 32; i += kCountColsBlock) (&sums[0][0])[i] = 0u;
    __syncthreads();
    const uint32_t c = cb * 32u + lane;
    if (c < p.chunks) {
        const uint64_t first_row = ((uint64_t)part * 32 + group) * p.rows_per_wave;
        const uint32_t r0 = first_row < p.rows ? (uint32_t)first_row : p.rows;
        const uint32_t r1 = r0 + p.rows_per_wave < p.rows ? r0 + p.rows_per_wave : p.rows;
        const unsigned cnt = p.cols - c * 32u >= 32u ? 32u : p.cols - c * 32u;
        const uint32_t keep = low_bits(cnt);
        const int64_t first = (int64_t)p.pos + (int64_t)o * p.s_outer + (int64_t)c * 32;
        uint32_t total[32];
#pragma unroll
        for (int j = 0; j < 32; ++j) total[j] = 0u;
        for (uint32_t ra = r0; ra < r1; ra += 240) {
            const uint32_t rb = ra + 240 < r1 ? ra + 240 : r1;
            uint32_t bytes[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) bytes[k] = 0u;
            for (uint32_t r = ra; r < rb; r += kCountColsRows) {
                // every load of the step goes out before anything waits for one: no branch between them (the
                // word after a row's word is loaded whether needed or not, from the same address when not)
                uint32_t x[kCountColsRows], lo[kCountColsRows], hi[kCountColsRows];
                unsigned shs[kCountColsRows];
#pragma unroll
                for (int u = 0; u < kCountColsRows; ++u) {
                    const uint32_t rr = r + u < rb ? r + u : rb - 1;
                    const uint64_t q = (uint64_t)(first + (int64_t)rr * p.s_red);
                    shs[u] = (unsigned)(q & 31);
                    const uint64_t w = q >> 5;
                    lo[u] = p.in[w];
                    hi[u] = p.in[w + (shs[u] + cnt > 32 ? 1 : 0)];
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = 0; u < kCountColsRows; ++u) {
                    uint32_t w = lo[u] >> shs[u];
                    if (shs[u] != 0) w |= hi[u] << (32 - shs[u]);
                    if (COUNT_FALSE) w = ~w;
                    x[u] = (r + u < rb) ? (w & keep) : 0u;
                }
#pragma unroll
                for (int u = 0; u < kCountColsRows; ++u) {
#pragma unroll
                    for (int k = 0; k < 8; ++k) bytes[k] += (x[u] >> k) & 0x01010101u;
                }
            }
#pragma unroll
            for (int j = 0; j < 32; ++j) total[j] += (bytes[j & 7] >> (8 * (j >> 3))) & 0xffu;
        }
        if (r0 < r1) {
#pragma unroll
            for (int j = 0; j < 32; ++j)
                if (total[j] != 0u) atomicAdd(&sums[j][lane], total[j]);
        }
    }
    __syncthreads();
    for (unsigned i = threadIdx.x; i < 32 * 32; i += kCountColsBlock) {
        // consecutive threads, consecutive columns
        const unsigned l = i >> 5, j = i & 31;
        const uint32_t col = (cb * 32u + l) * 32u + j;
        const uint32_t v = sums[j][l];
        if (col < p.cols && v != 0u)
            atomicAdd(reinterpret_cast<unsigned long long*>(p.out + (int64_t)o * p.o_outer + (int64_t)col * p.o_col), (unsigned long long)v);
    }
}

// launches the column form when the loop allows it; false: the caller uses the general kernel
bool bit_count_cols_launch(const cumo_hip_bit_count_nd_t* d) {
    if (d->red_ndim != 1 || d->out_ndim < 1 || d->out_ndim > 2 || force_wide_indices()) return false;
    const int L = d->out_ndim - 1;
    if (d->in_out_step[L] != 1 || d->in_red_step[0] <= 0 || d->out_shape[L] < 64 || d->red_shape[0] < 2) return false;
    if (d->out_shape[L] >= 0x7fffffffull || d->red_shape[0] >= 0x7fffffffull) return false;
    if (L == 1 && (d->in_out_step[0] < 0 || d->out_shape[0] >= 0x10000ull)) return false;
    BitCountCols p;
    std::memset(&p, 0, sizeof(p));
    p.in = d->in;
    p.out = d->out;
    p.pos = d->pos;
    p.cols = (uint32_t)d->out_shape[L];
    p.chunks = (p.cols + 31u) / 32u;
    p.chunk_blocks = (p.chunks + 31u) / 32u;
    p.rows = (uint32_t)d->red_shape[0];
    p.n_outer = L == 1 ? (uint32_t)d->out_shape[0] : 1u;
    p.s_red = d->in_red_step[0];
    p.s_outer = L == 1 ? d->in_out_step[0] : 0;
    p.o_outer = L == 1 ? d->out_step[0] : 0;
    p.o_col = d->out_step[L];
    // a block for every compute unit where the rows allow it (with two, the atomics at the end double and
    // [16384,32768] takes 28 us instead of 25), stretches of 32 rows or more per lane
    const uint64_t across = (uint64_t)p.chunk_blocks * p.n_outer;
    uint64_t parts = ((uint64_t)kNumCU + across - 1) / across;
    const uint64_t most = ((uint64_t)p.rows + 32 * 32 - 1) / (32 * 32);
    if (parts > most) parts = most;
    if (parts < 1) parts = 1;
    p.rows_per_wave = (uint32_t)(((uint64_t)p.rows + parts * 32 - 1) / (parts * 32));
    p.row_parts = (uint32_t)(((uint64_t)p.rows + (uint64_t)p.rows_per_wave * 32 - 1) / ((uint64_t)p.rows_per_wave * 32));
    const uint64_t blocks = across * p.row_parts;
    if (blocks > 0x7fffffffull) return false;
    const dim3 g((unsigned)blocks), b(kCountColsBlock);
    if (d->count_false) hipLaunchKernelGGL((bit_count_cols_kernel<true>), g, b, 0, current_stream(), p);
    else hipLaunchKernelGGL((bit_count_cols_kernel<false>), g, b, 0, current_stream(), p);
    cumo_cuda_runtime_check_kernel_launch();
    return true;
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
// Bit#store(Bit): the same word-wise / per-bit copy as `copy`, with the receiver as a3
// (narray/gen/tmpl_bit/store_bit.c:1-2, store_bit_kernel.cu:21,38)
CUMO_DEF_BIT_UNARY(store_bit, B_COPY)

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
        if (store_bit_rows_launch<c>(a1, a2, indexer)) return;                                                                \
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
    // a long run goes through the reduction kernels (2^29 bits: 21 us with the ticket kernel on 512 blocks)
    if (bit_count_run_reduce(a, pos, n, count_false, out)) return 1;
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
    // every block ends in one returning atomic on the same word, which serialise: 128 blocks, and more
    // (up to 512) only where every lane still has sixteen vectors to read
    uint64_t most = vecs / ((uint64_t)kBlock * 16);
    if (most < 128) most = 128;
    if (most > 512) most = 512;
    if (grid > most) grid = most;
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
    // (counts of whole-word rows can be stored; every other kernel adds, onto results that hold zero)
    const int L = d->out_ndim - 1;
    const bool down_columns = d->red_ndim == 1 && d->out_ndim >= 1 && d->in_out_step[L] == 1;
    if (!down_columns && bit_count_rows_reduce(d)) return;
    if (down_columns && bit_count_cols_words_launch(d)) return;   // rows on word boundaries: one launch, no zero-fill
    if (d->overwrite) {
        size_t outs = 1;
        for (int k = 0; k < d->out_ndim; ++k) outs *= d->out_shape[k];
        if (outs) cumo_hip_memset(d->out, 0, outs * 8);
    }
    if (bit_count_cols_launch(d)) return;
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
