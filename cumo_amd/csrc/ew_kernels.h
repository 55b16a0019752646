// Elementwise kernels for gfx950 and the launcher template that drives them.
//
// These replace every expansion of the reference's elementwise templates
// (ext/cumo/narray/gen/tmpl/{binary,unary,unary2,unary_s,binary_s,cond_binary,
// cond_unary,store_from,fill}_kernel.cu). The reference expands each template
// once per ndim 0..8 and decomposes a flat index with 64-bit divides per
// element; here there are four kernels:
//
//  ew_flat_kernel       every operand is one contiguous run (or the scalar): one
//                       128-bit access per lane, one 4 KiB tile per block.
//  ew_rows2_kernel      rows x inner, every operand contiguous or constant along
//                       inner and free to repeat along rows (matrix with row
//                       vector, column vector or scalar): the same tile shape
//                       with 32-bit index arithmetic.
//  ew_rows_kernel       the general form. Lanes run along the one dimension every
//                       operand walks fastest (or is broadcast along); the other
//                       dimensions are decomposed once per row per thread, never
//                       per element. Strided and ragged rows, any number of
//                       dimensions, Bit results.
//  ew_transpose_kernel  an input walks a different dimension fastest than the
//                       output does (a transposed view): a 64-wide tile goes
//                       through LDS so that both the read and the write are
//                       along memory.
//
// A Bit result is written by whole 32-bit words assembled across lanes;
// only words shared with a neighbouring row fall back to atomics
// (the reference does two atomics per element: include/cumo/template_kernel.h:26-35).
#ifndef CUMO_HIP_EW_KERNELS_H
#define CUMO_HIP_EW_KERNELS_H

#include "common.h"
#include "plan.h"
#include "div31.h"
#include "ew_ops.h"

#include <cstdlib>
#include <type_traits>
#include <cstring>

namespace cumo_hip {

// An operator that reads the LDS tables of ew_ops.h declares USES_TABLES; every kernel here fills them first.
template <class O, class = void> struct op_uses_tables { static constexpr bool value = false; };
template <class O> struct op_uses_tables<O, decltype((void)O::USES_TABLES)> { static constexpr bool value = O::USES_TABLES; };
template <class O, class = void> struct op_uses_pair_table { static constexpr bool value = false; };
template <class O> struct op_uses_pair_table<O, decltype((void)O::USES_PAIR_TABLE)> { static constexpr bool value = O::USES_PAIR_TABLE; };
template <class O, class = void> struct op_uses_pow_pair_tables { static constexpr bool value = false; };
template <class O> struct op_uses_pow_pair_tables<O, decltype((void)O::USES_POW_PAIR_TABLES)> { static constexpr bool value = O::USES_POW_PAIR_TABLES; };
template <class O, class = void> struct op_uses_erfc_tables { static constexpr bool value = false; };
template <class O> struct op_uses_erfc_tables<O, decltype((void)O::USES_ERFC_TABLES)> { static constexpr bool value = O::USES_ERFC_TABLES; };
template <class O, class = void> struct op_is_heavy { static constexpr bool value = false; };
template <class O> struct op_is_heavy<O, decltype((void)O::HEAVY)> { static constexpr bool value = O::HEAVY; };
// Vectors a lane of the flat kernel takes: two for the functions with long chains of dependent operations (their
// elements are evaluated side by side), one for everything else.
template <class Op> struct ew_flat_vectors_per_lane {
    static constexpr int value = op_is_heavy<Op>::value ? 2 : 1;
};
template <class Op> struct op_fills_tables {
    static constexpr bool value = op_uses_tables<Op>::value || op_uses_pair_table<Op>::value || op_uses_pow_pair_tables<Op>::value ||
                                  op_uses_erfc_tables<Op>::value;
};
template <class Op>
__device__ __forceinline__ void ew_op_prepare() {
    if constexpr (op_uses_tables<Op>::value) float_tables_prepare();
    if constexpr (op_uses_pair_table<Op>::value) exp_pair_table_prepare();
    if constexpr (op_uses_pow_pair_tables<Op>::value) pow_pair_tables_prepare();
    if constexpr (op_uses_erfc_tables<Op>::value) erfc_tables_prepare();
}

constexpr int kEwBlock = 256;
constexpr int kEwUnroll = 4;

struct EwKParams {
    uint64_t inner;      // extent of the fast dim
    uint64_t rows;       // product of the other dims
    uint64_t col_tiles;  // tiles along the fast dim
    uint64_t n_tiles;
    int small_tiles;     // n_tiles < 2^32
    int nouter;
    int tx_bits;         // 2^tx_bits lanes along the fast dim, the rest of the block along rows
    int use_scalar;      // 0: both inputs are arrays, 1: y = sv, 2: x = sv
    int small_rows;      // rows < 2^32: decompose with 32-bit divides
    int* flag;           // pinned host word for rejected elements (may be NULL)
    uint64_t out_bitpos; // Bit output: position of element 0
    uint64_t oshape[kMaxDim - 1];
    int64_t ostep[3][kMaxDim - 1];  // [in1, in2, out]; bits for a Bit output
    int64_t istep[3];
    char* ptr[3];
};

template <class T, int N>
struct alignas((sizeof(T) * N) > 16 ? 16 : (sizeof(T) * N)) VecT {
    T v[N];
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// VEC elements of T as raw 128/64/32-bit accesses. NT marks the access
// non-temporal: streamed data that is touched once should not displace what the
// caches hold. It has to be a compile-time choice: behind a run-time branch the
// compiler merges the two forms and the marking is lost.
template <class T, int VEC, bool NT>
__device__ __forceinline__ void raw_load(const char* p, T (&out)[VEC]) {
    constexpr int BYTES = (int)sizeof(T) * VEC;
    union U {
        T t[VEC];
        u32x4 q[BYTES >= 16 ? BYTES / 16 : 1];
        u32x2 d;
        uint32_t w;
        __device__ U() {}
    } u;
    if constexpr (BYTES % 16 == 0) {
#pragma unroll
        for (int k = 0; k < BYTES / 16; ++k) {
            const u32x4* src = reinterpret_cast<const u32x4*>(p) + k;
            u.q[k] = NT ? __builtin_nontemporal_load(src) : *src;
        }
    } else if constexpr (BYTES == 8) {
        const u32x2* src = reinterpret_cast<const u32x2*>(p);
        u.d = NT ? __builtin_nontemporal_load(src) : *src;
    } else if constexpr (BYTES == 4) {
        const uint32_t* src = reinterpret_cast<const uint32_t*>(p);
        u.w = NT ? __builtin_nontemporal_load(src) : *src;
    } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) u.t[j] = reinterpret_cast<const T*>(p)[j];
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j) out[j] = u.t[j];
}

// A 128-bit store for tiles that are written once, far apart from one another, by an operation
// too large for the caches: non-temporal AND written through at device scope (`nt sc1`), so the
// second-level cache does not collect the partly written lines of many rows before it lets them
// go. Measured on the transposed 8192 x 4096 SFloat copy, every launch on fresh operands: 47.2 us
// with `nt` alone, 46.3 us with `nt sc1` (plain stores: 50.9 us); a contiguous stream gains
// nothing from it (43.5 us either way for 128 MiB -> 128 MiB). No builtin spells the pair.
template <class T, int VEC>
__device__ __forceinline__ void raw_store_scattered_stream(char* p, const T (&in)[VEC]) {
    static_assert(sizeof(T) * VEC == 16, "one 128-bit store");
    union U {
        T t[VEC];
        u32x4 q;
        __device__ U() {}
    } u;
#pragma unroll
    for (int j = 0; j < VEC; ++j) u.t[j] = in[j];
    asm volatile("global_store_dwordx4 %0, %1, off nt sc1" ::"v"(p), "v"(u.q) : "memory");
}

template <class T, int VEC, bool NT>
__device__ __forceinline__ void raw_store(char* p, const T (&in)[VEC]) {
    constexpr int BYTES = (int)sizeof(T) * VEC;
    union U {
        T t[VEC];
        u32x4 q[BYTES >= 16 ? BYTES / 16 : 1];
        u32x2 d;
        uint32_t w;
        __device__ U() {}
    } u;
#pragma unroll
    for (int j = 0; j < VEC; ++j) u.t[j] = in[j];
    if constexpr (BYTES % 16 == 0) {
#pragma unroll
        for (int k = 0; k < BYTES / 16; ++k) {
            u32x4* dst = reinterpret_cast<u32x4*>(p) + k;
            if (NT) __builtin_nontemporal_store(u.q[k], dst);
            else *dst = u.q[k];
        }
    } else if constexpr (BYTES == 8) {
        u32x2* dst = reinterpret_cast<u32x2*>(p);
        if (NT) __builtin_nontemporal_store(u.d, dst);
        else *dst = u.d;
    } else if constexpr (BYTES == 4) {
        uint32_t* dst = reinterpret_cast<uint32_t*>(p);
        if (NT) __builtin_nontemporal_store(u.w, dst);
        else *dst = u.w;
    } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) reinterpret_cast<T*>(p)[j] = u.t[j];
    }
}

template <class T, int VEC, bool NT>
__device__ __forceinline__ void ew_load(const char* base, int64_t istep, int64_t col, T (&out)[VEC]) {
    if (istep == 0) {
        T v = *reinterpret_cast<const T*>(base);
#pragma unroll
        for (int j = 0; j < VEC; ++j) out[j] = v;
    } else if (VEC > 1 && istep < 0) {
        // the row runs backwards in memory: the vector that ends at this column's element, turned round
        T rev[VEC];
        raw_load<T, VEC, NT>(base - (col + (VEC - 1)) * (int64_t)sizeof(T), rev);
#pragma unroll
        for (int j = 0; j < VEC; ++j) out[j] = rev[VEC - 1 - j];
    } else if (VEC > 1) {
        const char* p = base + col * (int64_t)sizeof(T);
        raw_load<T, VEC, NT>(p, out);
    } else {
        out[0] = *reinterpret_cast<const T*>(base + col * istep);
    }
}

// Stores the VEC result bits of every lane of the wave. Every lane of the
// wave must call it (inactive lanes with active == false).
//   P      bit position of the lane's first bit
//   bits   the lane's results, bit j = element j
//   vmask  which of them exist
template <int VEC>
__device__ __forceinline__ void ew_store_bits(CUMO_BIT_DIGIT* base, uint64_t P, uint32_t bits, uint32_t vmask, bool active) {
    constexpr unsigned G = 32 / VEC;  // lanes per word
    const unsigned lane = __lane_id();
    const unsigned want_sh = (lane % G) * VEC;
    const uint64_t actmask = __ballot(active);
    if (actmask == 0) return;
    const uint64_t word = P >> 5;
    const unsigned gbase = lane & ~(G - 1);
    const uint64_t gmask = (actmask >> gbase) & ((1ull << G) - 1);
    const int leader = gmask ? (int)(gbase + __builtin_ctzll(gmask)) : (int)lane;
    const uint32_t lw_lo = __shfl((uint32_t)word, leader);
    const uint32_t lw_hi = __shfl((uint32_t)(word >> 32), leader);
    const bool fits = !active || (((unsigned)(P & 31) == want_sh) && lw_lo == (uint32_t)word && lw_hi == (uint32_t)(word >> 32));
    const bool fast = __ballot(!fits) == 0;
    if (fast) {
        uint32_t w = active ? ((bits & vmask) << want_sh) : 0u;
        uint32_t m = active ? (vmask << want_sh) : 0u;
#pragma unroll
        for (unsigned d = 1; d < G; d <<= 1) {
            w |= __shfl_xor(w, d);
            m |= __shfl_xor(m, d);
        }
        if (active && (int)lane == leader) {
            if (m == 0xffffffffu) {
                base[word] = w;
            } else {
                // the rest of the word belongs to a neighbouring row or to elements
                // outside the view
                atomicAnd(&base[word], ~m);
                atomicOr(&base[word], w);
            }
        }
    } else if (active) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            if ((vmask >> j) & 1u) {
                const uint64_t q = P + j;
                const uint32_t bit = 1u << (q & 31);
                if ((bits >> j) & 1u) atomicOr(&base[q >> 5], bit);
                else atomicAnd(&base[q >> 5], ~bit);
            }
        }
    }
}

// The vector form of a Bit row. The launcher only picks it when every row starts
// on a word boundary and a word's 32/VEC lanes sit in one row. Lane k of a group of
// 32/VEC lanes holds bits [k*VEC, k*VEC+VEC) of the group's word; the word is
// gathered into the group's first lane with DPP row shifts (lane i reads lane i+d
// of its 16-lane row): plain vector ALU, no trip through LDS.
template <int VEC>
__device__ __forceinline__ uint32_t ew_gather_word(uint32_t bits) {
    constexpr unsigned G = 32 / VEC;
    uint32_t w = bits;
    w |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)w, 0x101, 0xf, 0xf, true) << VEC;
    w |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)w, 0x102, 0xf, 0xf, true) << (2 * VEC);
    w |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)w, 0x104, 0xf, 0xf, true) << (4 * VEC);
    if constexpr (G > 8) w |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)w, 0x108, 0xf, 0xf, true) << (8 * VEC);
    return w;
}

template <int NOPS>
__device__ __forceinline__ void ew_row_offsets(const EwKParams& p, uint64_t row, int64_t (&off)[3]) {
    off[0] = off[1] = off[2] = 0;
    if (p.nouter == 0) return;
    if (p.small_rows) {
        uint32_t r = (uint32_t)row;
        for (int d = p.nouter - 1; d >= 1; --d) {
            const uint32_t n = (uint32_t)p.oshape[d];
            const uint32_t q = r / n;
            const uint32_t i = r - q * n;
            r = q;
            off[0] += (int64_t)i * p.ostep[0][d];
            if (NOPS > 2) off[1] += (int64_t)i * p.ostep[1][d];
            off[2] += (int64_t)i * p.ostep[2][d];
        }
        off[0] += (int64_t)r * p.ostep[0][0];
        if (NOPS > 2) off[1] += (int64_t)r * p.ostep[1][0];
        off[2] += (int64_t)r * p.ostep[2][0];
    } else {
        uint64_t r = row;
        for (int d = p.nouter - 1; d >= 1; --d) {
            const uint64_t n = p.oshape[d];
            const uint64_t q = r / n;
            const uint64_t i = r - q * n;
            r = q;
            off[0] += (int64_t)i * p.ostep[0][d];
            if (NOPS > 2) off[1] += (int64_t)i * p.ostep[1][d];
            off[2] += (int64_t)i * p.ostep[2][d];
        }
        off[0] += (int64_t)r * p.ostep[0][0];
        if (NOPS > 2) off[1] += (int64_t)r * p.ostep[1][0];
        off[2] += (int64_t)r * p.ostep[2][0];
    }
}

// Op contract:
//   typedef A, B (input element types), R (output element type; uint32_t 0/1 for BIT_OUT), S (scalar type)
//   static constexpr int NIN (0, 1 or 2); static constexpr bool BIT_OUT, CHECKED
//   __device__ bool operator()(A x, B y, R& z) const   -- false: reject the element (do not store, raise flag)
template <class Op, int VEC>
__global__ __launch_bounds__(kEwBlock) void ew_rows_kernel(EwKParams p, Op op, typename Op::S sv) {
    ew_op_prepare<Op>();
    typedef typename Op::A A;
    typedef typename Op::B B;
    typedef typename Op::R R;
    constexpr int NIN = Op::NIN;
    constexpr bool TWO = (NIN == 2);
    constexpr int UNR = kEwUnroll;

    const unsigned TX = 1u << p.tx_bits;
    const unsigned TY = kEwBlock >> p.tx_bits;
    const unsigned tx = threadIdx.x & (TX - 1);
    const unsigned ty = threadIdx.x >> p.tx_bits;
    const uint64_t tile_cols = (uint64_t)TX * VEC * UNR;
    const int64_t inner = (int64_t)p.inner;
    const bool two_arrays = TWO && p.use_scalar == 0;

    for (uint64_t tile = blockIdx.x; tile < p.n_tiles; tile += gridDim.x) {
        uint64_t rt, ct;
        if (p.col_tiles == 1) {
            rt = tile;
            ct = 0;
        } else if (p.small_tiles) {
            const uint32_t q = (uint32_t)tile / (uint32_t)p.col_tiles;
            rt = q;
            ct = (uint32_t)tile - q * (uint32_t)p.col_tiles;
        } else {
            rt = tile / p.col_tiles;
            ct = tile - rt * p.col_tiles;
        }
        const uint64_t row = rt * TY + ty;
        const bool row_ok = row < p.rows;
        int64_t off[3];
        ew_row_offsets<TWO ? 3 : 2>(p, row_ok ? row : 0, off);

        int64_t lead = 0;
        if (Op::BIT_OUT && VEC == 1) lead = (int64_t)((p.out_bitpos + (uint64_t)off[2]) & 31);
        // Typed results: a wave's lanes sit side by side, unroll steps a whole lane
        // row apart. Vector Bit results: the 32/VEC lanes of a word sit side by side
        // and the unroll steps are the NEXT words, so that a group's first lane ends
        // up with UNR consecutive words and stores them as one 128-bit access.
        constexpr bool BITVEC = Op::BIT_OUT && VEC > 1;
        constexpr int64_t G = BITVEC ? 32 / VEC : 1;
        const int64_t col0 = BITVEC ? (int64_t)(ct * tile_cols) + (int64_t)(tx / G) * (32 * UNR) + (int64_t)(tx % G) * VEC
                                    : (int64_t)(ct * tile_cols) + (int64_t)tx * VEC - lead;
        const int64_t ustep = BITVEC ? 32 : (int64_t)TX * VEC;

        const char* b0 = p.ptr[0] + off[0];
        const char* b1 = p.ptr[1] + off[1];

        A xv[UNR][VEC];
        B yv[UNR][VEC];
        int nval[UNR];  // how many of the VEC elements exist
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            const int64_t col = col0 + (int64_t)u * ustep;
            int nv = 0;
            if (row_ok && col >= 0 && col < inner) nv = (col + VEC <= inner) ? VEC : (int)(inner - col);
            nval[u] = nv;
            if (nv == VEC) {
                if (NIN >= 1) ew_load<A, VEC, false>(b0, p.istep[0], col, xv[u]);
                if (two_arrays) ew_load<B, VEC, false>(b1, p.istep[1], col, yv[u]);
            } else if (nv > 0) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    if (j < nv) {
                        if (NIN >= 1) xv[u][j] = *reinterpret_cast<const A*>(b0 + (col + j) * p.istep[0]);
                        if (two_arrays) yv[u][j] = *reinterpret_cast<const B*>(b1 + (col + j) * p.istep[1]);
                    }
                }
            }
        }

        uint32_t words[UNR];
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            const int64_t col = col0 + (int64_t)u * ustep;
            const int nv = nval[u];
            R zv[VEC];
            uint32_t okmask = 0;
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                if (j < nv) {
                    A x = (NIN >= 1) ? xv[u][j] : A();
                    B y = B();
                    if (TWO) {
                        if (p.use_scalar == 0) y = yv[u][j];
                        else if (p.use_scalar == 1) y = (B)sv;
                        else { y = (B)x; x = (A)sv; }
                    }
                    R z = R();
                    if (op(x, y, z)) okmask |= 1u << j;
                    zv[j] = z;
                }
            }
            if (Op::BIT_OUT) {
                uint32_t bits = 0;
#pragma unroll
                for (int j = 0; j < VEC; ++j) if (j < nv && zv[j]) bits |= 1u << j;
                const uint64_t P = p.out_bitpos + (uint64_t)off[2] + (uint64_t)(col * p.istep[2]);
                if constexpr (VEC > 1) {
                    words[u] = ew_gather_word<VEC>(bits);
                } else {
                    ew_store_bits<VEC>(reinterpret_cast<CUMO_BIT_DIGIT*>(p.ptr[2]), P, bits, nv > 0 ? 1u : 0u, nv > 0);
                }
            } else if (nv > 0) {
                char* o = p.ptr[2] + off[2];
                const uint32_t full = (1u << VEC) - 1u;
                if (Op::CHECKED && okmask != ((nv >= VEC) ? full : ((1u << nv) - 1u))) {
                    if (p.flag) *p.flag = 1;
                }
                if (VEC > 1 && nv == VEC && okmask == full && p.istep[2] != 0) {
                    raw_store<R, VEC, false>(o + col * (int64_t)sizeof(R), zv);
                } else {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) {
                        if (j < nv && ((okmask >> j) & 1u)) *reinterpret_cast<R*>(o + (col + j) * p.istep[2]) = zv[j];
                    }
                }
            }
        }
        if constexpr (BITVEC) {
            // the first lane of each group holds UNR consecutive words
            if ((tx % G) == 0 && nval[0] > 0) {
                CUMO_BIT_DIGIT* base = reinterpret_cast<CUMO_BIT_DIGIT*>(p.ptr[2]);
                const uint64_t P0 = p.out_bitpos + (uint64_t)off[2] + (uint64_t)col0;
                const int64_t left0 = inner - col0;  // elements of this row from the group's first bit on
                CUMO_BIT_DIGIT* dst = base + (P0 >> 5);
                static_assert(UNR == 4, "a lane group stores four words as one access");
                if (left0 >= 32 * UNR && (reinterpret_cast<uintptr_t>(dst) & 15) == 0) {
                    *reinterpret_cast<u32x4*>(dst) = u32x4{words[0], words[1], words[2], words[3]};
                } else {
#pragma unroll
                    for (int u = 0; u < UNR; ++u) {
                        const int64_t left = left0 - 32 * u;
                        if (left >= 32) {
                            dst[u] = words[u];
                        } else if (left > 0) {
                            // a row's last, partly used word: its other bits are not ours
                            const uint32_t m = (1u << left) - 1u;
                            atomicAnd(&dst[u], ~m);
                            atomicOr(&dst[u], words[u] & m);
                        }
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Flat kernel: every operand is one contiguous run (or the scalar). One 128-bit
// access per lane, one 4 KiB tile per block, nothing to decompose.
// NT: loads and stores are non-temporal.
// ---------------------------------------------------------------------------
// Ops that cost many instructions per element declare HEAVY: a lane then takes two
// vectors, a block apart, so that one vector's loads are in flight while the other
// is computed (measured on the SFloat exp of 2^27 elements: 168 us against 178 us;
// for a plain copy the single vector is ahead, 164 us against 175 us).
// Ops that declare HAS_RARE offer fast / rare / slow beside operator() (see ew_ops.h).
template <class O, class = void> struct op_has_rare { static constexpr bool value = false; };
template <class O> struct op_has_rare<O, decltype((void)O::HAS_RARE)> { static constexpr bool value = O::HAS_RARE; };

// Flat over a two-dimensional array whose rows are not a whole number of vectors: one input and
// the result are each one contiguous run (so their 128-bit accesses stay whole and aligned whatever
// the row length), the other input is addressed by row and column of each element - the operand
// that repeats along the rows (matrix + row vector), is constant along them (matrix - column
// vector) or is any other two-dimensional view. Rows of an odd length otherwise go element by
// element through the general kernel (DFloat 4096 x 4095 + 1 x 4095: 57.5 us; this way 44 us).
// Both inputs have one type; cheap ops only. n < 2^31.
struct EwPeriod {
    uint32_t period;      // row length in elements
    Div31 div;
    int64_t s_outer, s_inner;  // the addressed operand's byte steps per row and per column
    int first;            // 1: the addressed operand is the op's first input
    // three dimensions (outer x mid x inner): rows are numbered outer * mid + mid position, and the
    // addressed operand steps s_outer per mid position and s_outermost per outer position; mid 0 = two dimensions
    uint32_t mid;
    Div31 div_mid;
    int64_t s_outermost;
};

// byte offset of row q of the addressed operand
__device__ __forceinline__ int64_t ew_period_row(const EwPeriod& pr, uint32_t q) {
    if (pr.mid == 0) return (int64_t)q * pr.s_outer;
    const uint32_t o = div31(q, pr.div_mid);
    return (int64_t)o * pr.s_outermost + (int64_t)(q - o * pr.mid) * pr.s_outer;
}

template <class Op, int VEC, bool NT>
__global__ __launch_bounds__(kEwBlock) void ew_flat_period_kernel(const char* __restrict__ pfull, const char* __restrict__ pper,
                                                                  char* __restrict__ pz, uint32_t n, EwPeriod pr, int* flag, Op op) {
    ew_op_prepare<Op>();
    typedef typename Op::A A;
    typedef typename Op::R R;
    static_assert(Op::NIN == 2, "two inputs");
    const uint32_t i = (blockIdx.x * (uint32_t)kEwBlock + threadIdx.x) * VEC;
    if (i >= n) return;
    const uint32_t q = div31(i, pr.div);
    const uint32_t r = i - q * pr.period;
    const uint32_t cnt = n - i < (uint32_t)VEC ? n - i : (uint32_t)VEC;
    A fv[VEC], pv[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) { fv[j] = A(); pv[j] = A(); }
    if (cnt == VEC) {
        raw_load<A, VEC, NT>(pfull + (uint64_t)i * sizeof(A), fv);
    } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j)
            if ((uint32_t)j < cnt) fv[j] = reinterpret_cast<const A*>(pfull)[i + j];
    }
    // the vector lies inside one row nearly always: then the addressed operand gives one (unaligned)
    // 128-bit load where it is contiguous along the row, one element where it is constant along it
    const char* prow = pper + ew_period_row(pr, q);
    if (cnt == VEC && r + VEC <= pr.period && pr.s_inner == (int64_t)sizeof(A)) {
        raw_load<A, VEC, false>(prow + (int64_t)r * (int64_t)sizeof(A), pv);
    } else if (cnt == VEC && r + VEC <= pr.period && pr.s_inner == 0) {
        const A v = *reinterpret_cast<const A*>(prow);
#pragma unroll
        for (int j = 0; j < VEC; ++j) pv[j] = v;
    } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            uint32_t rr = r + j, qq = q;
            if (rr >= pr.period) { rr -= pr.period; ++qq; }
            if ((uint32_t)j < cnt) pv[j] = *reinterpret_cast<const A*>(pper + ew_period_row(pr, qq) + (int64_t)rr * pr.s_inner);
        }
    }
    R zv[VEC];
    bool ok = true;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
        zv[j] = R();
        const A x = pr.first ? pv[j] : fv[j];
        const A y = pr.first ? fv[j] : pv[j];
        bool okj = true;
        if ((uint32_t)j < cnt) okj = op(x, y, zv[j]);
        ok = ok && okj;
    }
    if (cnt == VEC && (!Op::CHECKED || ok)) {
        raw_store<R, VEC, NT>(pz + (uint64_t)i * sizeof(R), zv);
        return;
    }
    // the run's last, ragged vector, or a vector with a rejected element: one by one
    if (Op::CHECKED && !ok && flag) *flag = 1;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
        if ((uint32_t)j >= cnt) continue;
        R zz = R();
        const A x = pr.first ? pv[j] : fv[j];
        const A y = pr.first ? fv[j] : pv[j];
        if (op(x, y, zz)) reinterpret_cast<R*>(pz)[i + j] = zz;
    }
}

// The same with every input addressed by row and column: a unary function of a slice whose rows are not whole
// vectors (NMath.exp(x[true, 1..-1])), two such slices (x[true, 1..-1] - x[true, 0..-2]), a slice and the scalar,
// into a result that is one run. A lane takes an aligned vector of the result; where the vector lies inside one row
// (nearly always) each input gives one 128-bit load from wherever the slice puts it, or one element where the input
// is constant along the rows; the vector that spans two rows goes element by element. These shapes otherwise went
// element by element altogether (SFloat 4096 x 4095 exp of a slice: 55 us).
struct EwAddressed {
    const char* in[2];
    char* out;
    uint32_t n, period, mid;
    Div31 div, div_mid;
    int64_t s_outer[2], s_inner[2], s_outermost[2];
};

__device__ __forceinline__ int64_t ew_addressed_row(const EwAddressed& p, int sl, uint32_t q) {
    if (p.mid == 0) return (int64_t)q * p.s_outer[sl];
    const uint32_t o = div31(q, p.div_mid);
    return (int64_t)o * p.s_outermost[sl] + (int64_t)(q - o * p.mid) * p.s_outer[sl];
}

template <class T, int VEC>
__device__ __forceinline__ void ew_addressed_fetch(const EwAddressed& p, int sl, uint32_t q, uint32_t r, uint32_t cnt, bool inside, T (&v)[VEC]) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) v[j] = T();
    const char* prow = p.in[sl] + ew_addressed_row(p, sl, q);
    if (inside && p.s_inner[sl] == (int64_t)sizeof(T)) {
        raw_load<T, VEC, false>(prow + (int64_t)r * (int64_t)sizeof(T), v);
    } else if (inside && p.s_inner[sl] == 0) {
        const T one = *reinterpret_cast<const T*>(prow);
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = one;
    } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            uint32_t rr = r + j, qq = q;
            if (rr >= p.period) { rr -= p.period; ++qq; }
            if ((uint32_t)j < cnt) v[j] = *reinterpret_cast<const T*>(p.in[sl] + ew_addressed_row(p, sl, qq) + (int64_t)rr * p.s_inner[sl]);
        }
    }
}

template <class Op, int VEC, bool NT>
__global__ __launch_bounds__(kEwBlock) void ew_flat_addressed_kernel(EwAddressed p, int use_scalar, int* flag, Op op, typename Op::S sv) {
    ew_op_prepare<Op>();
    typedef typename Op::A A;
    typedef typename Op::B B;
    typedef typename Op::R R;
    constexpr bool TWO = Op::NIN == 2;
    const uint32_t i = (blockIdx.x * (uint32_t)kEwBlock + threadIdx.x) * VEC;
    if (i >= p.n) return;
    const uint32_t q = div31(i, p.div);
    const uint32_t r = i - q * p.period;
    const uint32_t cnt = p.n - i < (uint32_t)VEC ? p.n - i : (uint32_t)VEC;
    const bool inside = cnt == VEC && r + VEC <= p.period;
    A xv[VEC];
    B yv[VEC];
    ew_addressed_fetch<A, VEC>(p, 0, q, r, cnt, inside, xv);
    if (TWO && use_scalar == 0) {
        ew_addressed_fetch<B, VEC>(p, 1, q, r, cnt, inside, yv);
    } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) yv[j] = B();
    }
    R zv[VEC];
    bool okv[VEC];
    bool ok = true;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
        A x = xv[j];
        B y = yv[j];
        if (TWO) {
            if (use_scalar == 1) y = (B)sv;
            else if (use_scalar == 2) { y = (B)x; x = (A)sv; }
        }
        zv[j] = R();
        okv[j] = op(x, y, zv[j]);
        ok = ok && (okv[j] || (uint32_t)j >= cnt);
    }
    if (cnt == VEC && (!Op::CHECKED || ok)) {
        raw_store<R, VEC, NT>(p.out + (uint64_t)i * sizeof(R), zv);
        return;
    }
    // the run's last, ragged vector, or a vector with a rejected element: one by one
    if (Op::CHECKED && !ok && flag) *flag = 1;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
        if ((uint32_t)j < cnt && okv[j]) reinterpret_cast<R*>(p.out)[i + j] = zv[j];
    }
}

template <class Op, int VEC, bool NT>
__global__ __launch_bounds__(kEwBlock) void ew_flat_kernel(const char* __restrict__ px, const char* __restrict__ py,
                                                           char* __restrict__ pz, uint64_t n, int use_scalar, int* flag, Op op,
                                                           typename Op::S sv) {
    typedef typename Op::A A;
    typedef typename Op::B B;
    typedef typename Op::R R;
    constexpr int NIN = Op::NIN;
    constexpr bool TWO = (NIN == 2);
    constexpr int UNR = ew_flat_vectors_per_lane<Op>::value;
    // An operator with tables to fill takes several tiles per block (the launcher's grid is smaller than the number
    // of tiles; tile t goes to block t mod the grid), so that one filling serves them all; every other operator
    // gets a block per tile and runs the body once.
    constexpr bool LOOPS = op_fills_tables<Op>::value;
    if (TWO && (use_scalar & 4)) {
        // the scalar operand is an array of one element (x - x.mean): py points at it, the rest is the scalar form
        sv = *reinterpret_cast<const typename Op::S*>(py);
        use_scalar &= 3;
    }
    const uint64_t tiles = LOOPS ? (n + (uint64_t)(kEwBlock * UNR * VEC) - 1) / (uint64_t)(kEwBlock * UNR * VEC) : 0;
    uint64_t tile = blockIdx.x;
    bool first_tile = true;
    do {
    const uint64_t i0 = (tile * (kEwBlock * UNR) + threadIdx.x) * VEC;
    const bool two_arrays = TWO && use_scalar == 0;
    A xv[UNR][VEC];
    B yv[UNR][VEC];
    bool whole[UNR];
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
        const uint64_t i = i0 + (uint64_t)u * (kEwBlock * VEC);
        whole[u] = i + VEC <= n;
#pragma unroll
        for (int j = 0; j < VEC; ++j) { xv[u][j] = A(); yv[u][j] = B(); }
        if (whole[u]) {
            if (NIN >= 1) raw_load<A, VEC, NT>(px + i * sizeof(A), xv[u]);
            if (two_arrays) raw_load<B, VEC, NT>(py + i * sizeof(B), yv[u]);
        }
    }
    // Every vector is evaluated, loaded or not (an absent one holds zeros and is not stored):
    // with no branch around the arithmetic the compiler interleaves the elements of all the
    // lane's vectors, which the long dependent chains of the NMath functions need.
    // (the tables of an operator that reads them are filled after the first tile's loads have gone out)
    if (first_tile) ew_op_prepare<Op>();
    first_tile = false;
    R zv[UNR][VEC];
    bool ok[UNR];
    if constexpr (op_has_rare<Op>::value) {
        // the arithmetic for every element first, then one loop (not unrolled: the out-of-line
        // answer is called from one place, after the arithmetic has let go of its registers)
        // over the lane's elements if any of them is of the rare kind
        A xe[UNR * VEC];
        B ye[UNR * VEC];
        bool any = false;
        // which operand the scalar stands for is the same for every element: with it known at compile time
        // (three copies of the arithmetic under one uniform switch) the scalar's share of the arithmetic is
        // done once and no element selects its operands. Only where the arithmetic is what bounds the kernel.
        auto arithmetic = [&](auto mode) {
            constexpr int SM = decltype(mode)::value;
#pragma unroll
            for (int u = 0; u < UNR; ++u) {
                ok[u] = true;
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    A x = xv[u][j];
                    B y = B();
                    if (TWO) {
                        const int sm = SM >= 0 ? SM : use_scalar;
                        if (sm == 0) y = yv[u][j];
                        else if (sm == 1) y = (B)sv;
                        else { y = (B)x; x = (A)sv; }
                    }
                    xe[u * VEC + j] = x;
                    ye[u * VEC + j] = y;
                    op.fast(x, y, zv[u][j]);
                    any = any || op.rare(x, y);
                }
            }
        };
        if constexpr (TWO && (op_uses_tables<Op>::value || op_uses_pow_pair_tables<Op>::value)) {
            if (use_scalar == 0) arithmetic(std::integral_constant<int, 0>{});
            else if (use_scalar == 1) arithmetic(std::integral_constant<int, 1>{});
            else arithmetic(std::integral_constant<int, 2>{});
        } else {
            arithmetic(std::integral_constant<int, -1>{});
        }
        if (any) {
#pragma clang loop unroll(disable)
            for (int e = 0; e < UNR * VEC; ++e) {
                A x = xe[0];
                B y = ye[0];
#pragma unroll
                for (int q = 1; q < UNR * VEC; ++q) {
                    x = (e == q) ? xe[q] : x;
                    y = (e == q) ? ye[q] : y;
                }
                if (op.rare(x, y)) {
                    const R r = op.slow(x, y);
#pragma unroll
                    for (int q = 0; q < UNR * VEC; ++q) zv[q / VEC][q % VEC] = (e == q) ? r : zv[q / VEC][q % VEC];
                }
            }
        }
    } else {
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            ok[u] = true;
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                A x = (NIN >= 1) ? xv[u][j] : A();
                B y = B();
                if (TWO) {
                    if (use_scalar == 0) y = yv[u][j];
                    else if (use_scalar == 1) y = (B)sv;
                    else { y = (B)x; x = (A)sv; }
                }
                zv[u][j] = R();
                ok[u] = op(x, y, zv[u][j]) && ok[u];
            }
        }
    }
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
        const uint64_t i = i0 + (uint64_t)u * (kEwBlock * VEC);
        if (whole[u] && (!Op::CHECKED || ok[u])) {
            raw_store<R, VEC, NT>(pz + i * sizeof(R), zv[u]);
            continue;
        }
        if (i >= n) continue;
        // the last, ragged vector of the run, or a vector with a rejected element: one by one
        const int nv = whole[u] ? VEC : (int)(n - i);
        for (int j = 0; j < nv; ++j) {
            A x = (NIN >= 1) ? reinterpret_cast<const A*>(px)[i + j] : A();
            B y = B();
            if (TWO) {
                if (use_scalar == 0) y = reinterpret_cast<const B*>(py)[i + j];
                else if (use_scalar == 1) y = (B)sv;
                else { y = (B)x; x = (A)sv; }
            }
            R z = R();
            if (op(x, y, z)) reinterpret_cast<R*>(pz)[i + j] = z;
            else if (flag) *flag = 1;
        }
    }
    tile += gridDim.x;
    } while (LOOPS && tile < tiles);
}

// ---------------------------------------------------------------------------
// Flat kernel for a Bit result: every input is one contiguous run (or the scalar)
// and the result's first bit is the first bit of a 128-bit unit. The 32/VEC lanes
// of a group take four consecutive words: per step each lane loads one vector, the
// group's word is gathered in its first lane with DPP row shifts, and the first
// lane stores the four words as one access. Nothing between the four loads of a
// lane depends on data, so they go out back to back. Only the run's last group can
// be ragged; it sets or clears its bits one by one.
// ---------------------------------------------------------------------------
template <class Op, int VEC, bool NT>
__global__ __launch_bounds__(kEwBlock) void ew_flat_bit_kernel(const char* __restrict__ px, const char* __restrict__ py,
                                                               CUMO_BIT_DIGIT* __restrict__ pz, uint64_t n, int use_scalar, Op op,
                                                               typename Op::S sv) {
    ew_op_prepare<Op>();
    typedef typename Op::A A;
    typedef typename Op::B B;
    constexpr int NIN = Op::NIN;
    constexpr bool TWO = (NIN == 2);
    constexpr int UNR = 4;
    constexpr unsigned G = 32 / VEC;
    if (TWO && (use_scalar & 4)) {
        // the scalar operand is an array of one element: py points at it, the rest is the scalar form
        sv = *reinterpret_cast<const typename Op::S*>(py);
        use_scalar &= 3;
    }
    const uint64_t lane = (uint64_t)blockIdx.x * kEwBlock + threadIdx.x;
    const uint64_t group = lane / G;
    const unsigned k = (unsigned)(lane % G);
    const uint64_t first = group * (32 * UNR);  // the group's first element
    if (first >= n) return;
    const bool two_arrays = TWO && use_scalar == 0;
    const uint64_t e0 = first + (uint64_t)k * VEC;
    if (first + 32 * UNR <= n) {
        A xv[UNR][VEC];
        B yv[UNR][VEC];
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            if (NIN >= 1) raw_load<A, VEC, NT>(px + (e0 + 32 * u) * sizeof(A), xv[u]);
            if (two_arrays) raw_load<B, VEC, NT>(py + (e0 + 32 * u) * sizeof(B), yv[u]);
        }
        uint32_t words[UNR];
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            uint32_t bits = 0;
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                A x = (NIN >= 1) ? xv[u][j] : A();
                B y = B();
                if (TWO) {
                    if (use_scalar == 0) y = yv[u][j];
                    else if (use_scalar == 1) y = (B)sv;
                    else { y = (B)x; x = (A)sv; }
                }
                uint32_t z = 0;
                op(x, y, z);
                bits |= (z ? 1u : 0u) << j;
            }
            words[u] = ew_gather_word<VEC>(bits);
        }
        if (k == 0) *reinterpret_cast<u32x4*>(pz + group * UNR) = u32x4{words[0], words[1], words[2], words[3]};
        return;
    }
    // the ragged end: at most 32 * UNR - 1 elements in the whole launch
    for (int u = 0; u < UNR; ++u) {
        for (int j = 0; j < VEC; ++j) {
            const uint64_t e = e0 + 32 * u + j;
            if (e >= n) continue;
            A x = (NIN >= 1) ? reinterpret_cast<const A*>(px)[e] : A();
            B y = B();
            if (TWO) {
                if (use_scalar == 0) y = reinterpret_cast<const B*>(py)[e];
                else if (use_scalar == 1) y = (B)sv;
                else { y = (B)x; x = (A)sv; }
            }
            uint32_t z = 0;
            op(x, y, z);
            const uint32_t bit = 1u << (e & 31);
            if (z) atomicOr(&pz[e >> 5], bit);
            else atomicAnd(&pz[e >> 5], ~bit);
        }
    }
}

// The same over a contiguous matrix (op) a second two-dimensional operand that is addressed by row
// and column (a row vector, a column vector, a view): the matrix and the bits are each one run, so
// this takes `matrix > row` for any row length (it went through the general row kernel: SFloat
// [8192,4096] > [1,4096] 30.6 us, [8192,4095] 100 us). Both inputs of one type; n < 2^31.
template <class Op, int VEC, bool NT>
__global__ __launch_bounds__(kEwBlock) void ew_flat_bit_period_kernel(const char* __restrict__ pfull, const char* __restrict__ pper,
                                                                      CUMO_BIT_DIGIT* __restrict__ pz, uint32_t n, EwPeriod pr, Op op) {
    ew_op_prepare<Op>();
    typedef typename Op::A A;
    static_assert(Op::NIN == 2, "two inputs");
    constexpr int UNR = 4;
    constexpr unsigned G = 32 / VEC;
    const uint32_t lane = blockIdx.x * (uint32_t)kEwBlock + threadIdx.x;
    const uint32_t group = lane / G;
    const unsigned k = lane % G;
    const uint64_t first64 = (uint64_t)group * (32 * UNR);  // the group's first element
    if (first64 >= n) return;
    const uint32_t first = (uint32_t)first64;
    const uint32_t e0 = first + k * VEC;
    auto addressed = [&](uint32_t e, int j) -> A {
        const uint32_t q = div31(e + j, pr.div);
        const uint32_t r = e + j - q * pr.period;
        return *reinterpret_cast<const A*>(pper + ew_period_row(pr, q) + (int64_t)r * pr.s_inner);
    };
    if (first64 + 32 * UNR <= n) {
        A fv[UNR][VEC], pv[UNR][VEC];
#pragma unroll
        for (int u = 0; u < UNR; ++u) raw_load<A, VEC, NT>(pfull + (uint64_t)(e0 + 32 * u) * sizeof(A), fv[u]);
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            const uint32_t e = e0 + 32 * u;
            const uint32_t q = div31(e, pr.div);
            const uint32_t r = e - q * pr.period;
            const char* prow = pper + ew_period_row(pr, q);
            if (r + VEC <= pr.period && pr.s_inner == (int64_t)sizeof(A)) {
                raw_load<A, VEC, false>(prow + (int64_t)r * (int64_t)sizeof(A), pv[u]);
            } else if (r + VEC <= pr.period && pr.s_inner == 0) {
                const A v = *reinterpret_cast<const A*>(prow);
#pragma unroll
                for (int j = 0; j < VEC; ++j) pv[u][j] = v;
            } else {
#pragma unroll
                for (int j = 0; j < VEC; ++j) pv[u][j] = addressed(e, j);
            }
        }
        uint32_t words[UNR];
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            uint32_t bits = 0;
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const A x = pr.first ? pv[u][j] : fv[u][j];
                const A y = pr.first ? fv[u][j] : pv[u][j];
                uint32_t z = 0;
                op(x, y, z);
                bits |= (z ? 1u : 0u) << j;
            }
            words[u] = ew_gather_word<VEC>(bits);
        }
        if (k == 0) *reinterpret_cast<u32x4*>(pz + (size_t)group * UNR) = u32x4{words[0], words[1], words[2], words[3]};
        return;
    }
    // the ragged end: at most 32 * UNR - 1 elements in the whole launch
    for (int u = 0; u < UNR; ++u) {
        for (int j = 0; j < VEC; ++j) {
            const uint64_t e = (uint64_t)e0 + 32 * u + j;
            if (e >= n) continue;
            const A f = reinterpret_cast<const A*>(pfull)[e];
            const A a = addressed((uint32_t)e, 0);
            uint32_t z = 0;
            op(pr.first ? a : f, pr.first ? f : a, z);
            const uint32_t bit = 1u << (e & 31);
            if (z) atomicOr(&pz[e >> 5], bit);
            else atomicAnd(&pz[e >> 5], ~bit);
        }
    }
}

// The same with every input addressed by row and column (see ew_flat_addressed_kernel): a comparison of a slice whose
// rows are not whole vectors with the scalar or with another slice (x[true, 1..-1] > x[true, 0..-2]; v[1..-1] > v[0..-2]
// of one dimension is one row), the bits one run. These went element by element: SFloat [8192,4095] of [8192,4096]
// `> 0` 100 us.
template <class Op, int VEC, bool NT>
__global__ __launch_bounds__(kEwBlock) void ew_flat_bit_addressed_kernel(EwAddressed p, CUMO_BIT_DIGIT* __restrict__ pz, int use_scalar, Op op,
                                                                         typename Op::S sv) {
    ew_op_prepare<Op>();
    typedef typename Op::A A;
    typedef typename Op::B B;
    constexpr bool TWO = Op::NIN == 2;
    constexpr int UNR = 4;
    constexpr unsigned G = 32 / VEC;
    const uint32_t lane = blockIdx.x * (uint32_t)kEwBlock + threadIdx.x;
    const uint32_t group = lane / G;
    const unsigned k = lane % G;
    const uint64_t first64 = (uint64_t)group * (32 * UNR);  // the group's first element
    if (first64 >= p.n) return;
    const uint32_t e0 = (uint32_t)first64 + k * VEC;
    const bool two_arrays = TWO && use_scalar == 0;
    if (first64 + 32 * UNR <= p.n) {
        A xv[UNR][VEC];
        B yv[UNR][VEC];
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            const uint32_t e = e0 + 32 * u;
            const uint32_t q = div31(e, p.div);
            const uint32_t r = e - q * p.period;
            const bool inside = r + VEC <= p.period;
            ew_addressed_fetch<A, VEC>(p, 0, q, r, (uint32_t)VEC, inside, xv[u]);
            if (two_arrays) {
                ew_addressed_fetch<B, VEC>(p, 1, q, r, (uint32_t)VEC, inside, yv[u]);
            } else {
#pragma unroll
                for (int j = 0; j < VEC; ++j) yv[u][j] = B();
            }
        }
        uint32_t words[UNR];
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            uint32_t bits = 0;
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                A x = xv[u][j];
                B y = yv[u][j];
                if (TWO) {
                    if (use_scalar == 1) y = (B)sv;
                    else if (use_scalar == 2) { y = (B)x; x = (A)sv; }
                }
                uint32_t z = 0;
                op(x, y, z);
                bits |= (z ? 1u : 0u) << j;
            }
            words[u] = ew_gather_word<VEC>(bits);
        }
        if (k == 0) *reinterpret_cast<u32x4*>(pz + (size_t)group * UNR) = u32x4{words[0], words[1], words[2], words[3]};
        return;
    }
    // the ragged end: at most 32 * UNR - 1 elements in the whole launch
    for (int u = 0; u < UNR; ++u) {
        for (int j = 0; j < VEC; ++j) {
            const uint64_t e = (uint64_t)e0 + 32 * u + j;
            if (e >= p.n) continue;
            const uint32_t q = div31((uint32_t)e, p.div);
            const uint32_t r = (uint32_t)e - q * p.period;
            A x = *reinterpret_cast<const A*>(p.in[0] + ew_addressed_row(p, 0, q) + (int64_t)r * p.s_inner[0]);
            B y = B();
            if (two_arrays) y = *reinterpret_cast<const B*>(p.in[1] + ew_addressed_row(p, 1, q) + (int64_t)r * p.s_inner[1]);
            if (TWO) {
                if (use_scalar == 1) y = (B)sv;
                else if (use_scalar == 2) { y = (B)x; x = (A)sv; }
            }
            uint32_t z = 0;
            op(x, y, z);
            const uint32_t bit = 1u << (e & 31);
            if (z) atomicOr(&pz[e >> 5], bit);
            else atomicAnd(&pz[e >> 5], ~bit);
        }
    }
}

// ---------------------------------------------------------------------------
// Two-dimensional kernel for typed results: rows x inner, every operand either
// walks the inner dimension contiguously or is constant along it (a column
// vector, or the scalar), and may repeat along rows (a row vector). 32-bit
// index arithmetic, one 128-bit access per lane, no ragged vectors: the launcher
// only picks it when inner is a whole number of vectors.
// Three dimensions (outer x mid x inner, an operand repeating along outer or mid:
// [B,T,C] with [T,1] or [B,1,C]) use the same tiles over outer * mid rows; a row
// number then splits once per lane and tile into its two parts.
// ---------------------------------------------------------------------------
struct EwR2Params {
    char* ptr[3];        // in1, in2, out
    int64_t rstep[3];    // byte step from one row to the next (0: the operand repeats)
    int64_t ostep[3];    // three dimensions: byte step along outer (rstep is then the step along mid)
    uint32_t mid;        // three dimensions: extent of mid; 0 for two dimensions
    int walk[3];         // 1: contiguous along inner, 0: constant along inner, 2 (inputs): contiguous, backwards in memory
    uint32_t rows;
    uint32_t inner_vecs; // inner / VEC
    uint32_t col_tiles;
    uint32_t n_tiles;
    int tx_bits;
    int use_scalar;
    int* flag;
};

// NTM: which accesses are non-temporal (bit 0 the first input, bit 1 the second, bit 2 the
// result). An operand that repeats from row to row is the one thing worth keeping in
// the caches, so it is read with plain loads while the full-size operands stream past.
template <class Op, int VEC, int NTM>
__global__ __launch_bounds__(kEwBlock) void ew_rows2_kernel(EwR2Params p, Op op, typename Op::S sv) {
    ew_op_prepare<Op>();
    typedef typename Op::A A;
    typedef typename Op::B B;
    typedef typename Op::R R;
    constexpr int NIN = Op::NIN;
    constexpr bool TWO = (NIN == 2);
    const unsigned TX = 1u << p.tx_bits;
    const unsigned tx = threadIdx.x & (TX - 1);
    const unsigned ty = threadIdx.x >> p.tx_bits;
    const unsigned TY = (unsigned)kEwBlock >> p.tx_bits;
    const bool two_arrays = TWO && p.use_scalar == 0;
    for (uint32_t tile = blockIdx.x; tile < p.n_tiles; tile += gridDim.x) {
        uint32_t rt = tile, ct = 0;
        if (p.col_tiles != 1) {
            rt = tile / p.col_tiles;
            ct = tile - rt * p.col_tiles;
        }
        const uint32_t row = rt * TY + ty;
        const uint32_t cv = ct * TX + tx;
        if (row >= p.rows || cv >= p.inner_vecs) continue;
        int64_t roff[3];
        if (p.mid == 0) {
#pragma unroll
            for (int k = 0; k < 3; ++k) roff[k] = (int64_t)row * p.rstep[k];
        } else {
            const uint32_t r0 = row / p.mid;
            const uint32_t r1 = row - r0 * p.mid;
#pragma unroll
            for (int k = 0; k < 3; ++k) roff[k] = (int64_t)r0 * p.ostep[k] + (int64_t)r1 * p.rstep[k];
        }
        A xv[VEC];
        B yv[VEC];
        R zv[VEC];
        if (NIN >= 1) {
            const char* a = p.ptr[0] + roff[0];
            if (p.walk[0] == 1) {
                raw_load<A, VEC, (NTM & 1) != 0>(a + (uint64_t)cv * (VEC * sizeof(A)), xv);
            } else if (p.walk[0] == 2) {
                A rev[VEC];
                raw_load<A, VEC, (NTM & 1) != 0>(a - ((int64_t)cv * VEC + (VEC - 1)) * (int64_t)sizeof(A), rev);
#pragma unroll
                for (int j = 0; j < VEC; ++j) xv[j] = rev[VEC - 1 - j];
            } else {
                const A v = *reinterpret_cast<const A*>(a);
#pragma unroll
                for (int j = 0; j < VEC; ++j) xv[j] = v;
            }
        }
        if (two_arrays) {
            const char* a = p.ptr[1] + roff[1];
            if (p.walk[1] == 1) {
                raw_load<B, VEC, (NTM & 2) != 0>(a + (uint64_t)cv * (VEC * sizeof(B)), yv);
            } else if (p.walk[1] == 2) {
                B rev[VEC];
                raw_load<B, VEC, (NTM & 2) != 0>(a - ((int64_t)cv * VEC + (VEC - 1)) * (int64_t)sizeof(B), rev);
#pragma unroll
                for (int j = 0; j < VEC; ++j) yv[j] = rev[VEC - 1 - j];
            } else {
                const B v = *reinterpret_cast<const B*>(a);
#pragma unroll
                for (int j = 0; j < VEC; ++j) yv[j] = v;
            }
        }
        uint32_t okmask = 0;
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            A x = (NIN >= 1) ? xv[j] : A();
            B y = B();
            if (TWO) {
                if (p.use_scalar == 0) y = yv[j];
                else if (p.use_scalar == 1) y = (B)sv;
                else { y = (B)x; x = (A)sv; }
            }
            R z = R();
            if (op(x, y, z)) okmask |= 1u << j;
            zv[j] = z;
        }
        char* o = p.ptr[2] + roff[2] + (uint64_t)cv * (VEC * sizeof(R));
        constexpr uint32_t full = (1u << VEC) - 1u;
        if (!Op::CHECKED || okmask == full) {
            raw_store<R, VEC, (NTM & 4) != 0>(o, zv);
        } else {
            if (p.flag) *p.flag = 1;
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                if ((okmask >> j) & 1u) reinterpret_cast<R*>(o)[j] = zv[j];
            }
        }
    }
}

// The two-dimensional case of the kernel above for large arrays, with less to work out per
// vector: the inputs that are arrays walk the inner dimension contiguously or (the second
// one) stay constant along it, a tile is 2 * TY rows by TX vectors and a lane takes the same
// vector of two rows TY apart, so its column offset, and an operand that repeats from row to
// row, are worked out and loaded once per pair. The tile's place comes from the block number
// by a multiply and a shift. Measured on DFloat [4096,4096] + [1,4096] (fresh operands):
// 42.1 us against 45.6 us for the general form, 43.3 us with one row per lane.
struct EwR2LeanParams {
    char* ptr[3];
    int64_t rstep[3];
    uint32_t rows, inner_vecs;
    Div31 col_div;       // tile -> (row tile, column tile)
    uint32_t col_tiles;
    int tx_bits;
    int mode;            // see ew_rows2_lean_body
    int* flag;
};

// MODE, where the second operand of a binary op comes from: 0 an array that walks the inner
// dimension and changes from row to row, 1 one that walks it and repeats, 2 one that is
// constant along it, 3 the scalar as second operand, 4 the scalar as first. (Unary: 0.)
// Decided once per block, so that the body holds no choice per element.
template <class Op, int VEC, int NTM, int MODE>
__device__ __forceinline__ void ew_rows2_lean_body(const EwR2LeanParams& p, Op op, typename Op::S sv, uint32_t row0, uint32_t TY, uint32_t cv) {
    typedef typename Op::A A;
    typedef typename Op::B B;
    typedef typename Op::R R;
    constexpr int NIN = Op::NIN;
    constexpr bool TWO = (NIN == 2);
    constexpr int U = 2;
    // an absent second row (the last tile of an odd number) is loaded as the last row and not stored
    uint32_t row[U];
    bool live[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint32_t r = row0 + u * TY;
        live[u] = r < p.rows;
        row[u] = live[u] ? r : p.rows - 1;
    }
    A xv[U][VEC];
    B yv[U][VEC];
    const uint64_t coff_a = (uint64_t)cv * (VEC * sizeof(A));
    const uint64_t coff_b = (uint64_t)cv * (VEC * sizeof(B));
    if (TWO && MODE == 1) raw_load<B, VEC, false>(p.ptr[1] + coff_b, yv[0]);
#pragma unroll
    for (int u = 0; u < U; ++u) {
        if (NIN >= 1) raw_load<A, VEC, (NTM & 1) != 0>(p.ptr[0] + (int64_t)row[u] * p.rstep[0] + coff_a, xv[u]);
        if (TWO && MODE == 0) raw_load<B, VEC, (NTM & 2) != 0>(p.ptr[1] + (int64_t)row[u] * p.rstep[1] + coff_b, yv[u]);
        if (TWO && MODE == 2) {
            const B v = *reinterpret_cast<const B*>(p.ptr[1] + (int64_t)row[u] * p.rstep[1]);
#pragma unroll
            for (int j = 0; j < VEC; ++j) yv[u][j] = v;
        }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        R zv[VEC];
        uint32_t okmask = 0;
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            A x = (NIN >= 1) ? xv[u][j] : A();
            B y = B();
            if (TWO) {
                if (MODE == 0 || MODE == 2) y = yv[u][j];
                else if (MODE == 1) y = yv[0][j];
                else if (MODE == 3) y = (B)sv;
                else { y = (B)x; x = (A)sv; }
            }
            R z = R();
            if (op(x, y, z)) okmask |= 1u << j;
            zv[j] = z;
        }
        if (!live[u]) continue;
        char* o = p.ptr[2] + (int64_t)row[u] * p.rstep[2] + (uint64_t)cv * (VEC * sizeof(R));
        constexpr uint32_t full = (1u << VEC) - 1u;
        if (!Op::CHECKED || okmask == full) {
            raw_store<R, VEC, (NTM & 4) != 0>(o, zv);
        } else {
            if (p.flag) *p.flag = 1;
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                if ((okmask >> j) & 1u) reinterpret_cast<R*>(o)[j] = zv[j];
            }
        }
    }
}

template <class Op, int VEC, int NTM>
__global__ __launch_bounds__(kEwBlock) void ew_rows2_lean_kernel(EwR2LeanParams p, Op op, typename Op::S sv) {
    ew_op_prepare<Op>();
    const unsigned TX = 1u << p.tx_bits;
    const unsigned tx = threadIdx.x & (TX - 1);
    const unsigned ty = threadIdx.x >> p.tx_bits;
    const unsigned TY = (unsigned)kEwBlock >> p.tx_bits;
    const uint32_t tile = blockIdx.x;
    const uint32_t rt = p.col_tiles == 1 ? tile : div31(tile, p.col_div);
    const uint32_t ct = tile - rt * p.col_tiles;
    const uint32_t cv = ct * TX + tx;
    const uint32_t row0 = rt * (TY * 2) + ty;
    if (cv >= p.inner_vecs || row0 >= p.rows) return;
    if constexpr (Op::NIN == 2) {
        switch (p.mode) {
            case 1: ew_rows2_lean_body<Op, VEC, NTM, 1>(p, op, sv, row0, TY, cv); break;
            case 2: ew_rows2_lean_body<Op, VEC, NTM, 2>(p, op, sv, row0, TY, cv); break;
            case 3: ew_rows2_lean_body<Op, VEC, NTM, 3>(p, op, sv, row0, TY, cv); break;
            case 4: ew_rows2_lean_body<Op, VEC, NTM, 4>(p, op, sv, row0, TY, cv); break;
            default: ew_rows2_lean_body<Op, VEC, NTM, 0>(p, op, sv, row0, TY, cv); break;
        }
    } else {
        ew_rows2_lean_body<Op, VEC, NTM, 0>(p, op, sv, row0, TY, cv);
    }
}

// ---------------------------------------------------------------------------
// Transposed-operand kernel. Dims: outer..., G (second last), F (last, the
// output's fast dim). An input whose step along G is smaller than along F is
// read with lanes along G into LDS and picked up transposed.
// ---------------------------------------------------------------------------
struct EwTParams {
    uint64_t nf, ng;          // extents of F and G
    uint64_t f_tiles, g_tiles, n_tiles;
    int nouter;
    int use_scalar;
    int tr[2];                // input k goes through LDS
    int order;                // how block index maps to tiles: 0 F fastest, 1 G fastest, 2 8x8 super-tiles, 3 F fastest along diagonals
    int* flag;
    uint64_t oshape[kMaxDim - 2];
    int64_t ostep[3][kMaxDim - 2];
    int64_t fstep[3], gstep[3];
    char* ptr[3];
};

// A barrier for blocks that only share LDS: it waits for this wave's LDS traffic
// and not, as __syncthreads() does, for its global loads and stores as well, so
// loads that were sent ahead stay in flight across it and stores need not land.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Tile number -> tile origin (f0, g0) and the operands' byte offsets of the outer dimensions.
template <int TF, int TG>
__device__ __forceinline__ void ew_tile_at(const EwTParams& p, uint64_t tile, uint64_t& f0, uint64_t& g0, int64_t (&off)[3]) {
    if (p.order == 1 && p.nouter == 0 && p.n_tiles <= 0xffffffffull) {
        // the common case in 32-bit arithmetic: a matrix, tiles along G first
        const uint32_t t32 = (uint32_t)tile, ngt = (uint32_t)p.g_tiles;
        const uint32_t ft32 = t32 / ngt;
        off[0] = off[1] = off[2] = 0;
        f0 = (uint64_t)ft32 * TF;
        g0 = (uint64_t)(t32 - ft32 * ngt) * TG;
        return;
    }
    if (p.order == 3 && p.nouter == 0 && p.n_tiles <= 0xffffffffull) {
        const uint32_t t32 = (uint32_t)tile, nft = (uint32_t)p.f_tiles, ngt = (uint32_t)p.g_tiles;
        const uint32_t q = t32 / nft, ft32 = t32 - q * nft;
        off[0] = off[1] = off[2] = 0;
        f0 = (uint64_t)ft32 * TF;
        g0 = (uint64_t)((q + ft32 % ngt) % ngt) * TG;
        return;
    }
    uint64_t t = tile;
    uint64_t ft, gt;
    if (p.order == 1) {
        gt = t % p.g_tiles; t /= p.g_tiles;
        ft = t % p.f_tiles; t /= p.f_tiles;
    } else if (p.order == 2) {
        // 8 x 8 super-tiles (both tile counts are multiples of 8)
        const uint64_t per_plane = p.f_tiles * p.g_tiles;
        const uint64_t q = t % per_plane; t /= per_plane;
        const uint64_t st = q >> 6, w = q & 63;
        const uint64_t sf = p.f_tiles >> 3;
        ft = (st % sf) * 8 + (w & 7);
        gt = (st / sf) * 8 + (w >> 3);
    } else if (p.order == 3) {
        // F fastest, and each step along F also moves one tile along G: blocks that run
        // together then differ in both directions and spread over the memory channels on
        // the read side as well as on the write side
        ft = t % p.f_tiles; t /= p.f_tiles;
        gt = (t + ft) % p.g_tiles; t /= p.g_tiles;
    } else {
        ft = t % p.f_tiles; t /= p.f_tiles;
        gt = t % p.g_tiles; t /= p.g_tiles;
    }
    off[0] = off[1] = off[2] = 0;
    for (int d = p.nouter - 1; d >= 0; --d) {
        const uint64_t n = p.oshape[d];
        const uint64_t i = (d == 0) ? t : (t % n);
        t = (d == 0) ? 0 : (t / n);
        off[0] += (int64_t)i * p.ostep[0][d];
        off[1] += (int64_t)i * p.ostep[1][d];
        off[2] += (int64_t)i * p.ostep[2][d];
    }
    f0 = ft * TF;
    g0 = gt * TG;
}

// The 128-bit form: every operand is contiguous along its own fast dimension, so both
// the reads along G and the writes along F move 16 bytes per lane (from any 4-byte
// boundary; the one vector on either side that lies partly inside the array goes
// element by element).
// PREFETCH: a block walks several tiles and keeps the transposed inputs of its
// next tile in flight, in registers, while it computes and stores the current
// one. That pays for an op with many instructions per element, whose blocks
// would otherwise have no loads outstanding while they compute; for a cheap op
// the registers it holds cost as much as it wins, and wider tiles do more.
// TRMODE says at compile time which inputs go through LDS (bit 0: the first, bit 1:
// the second; an input that is not an array is neither): behind a run-time switch
// the compiler has to assume a global load on the way to every op and waits for
// all memory traffic there, the loads sent ahead and the last stores included.
// NT: the transposed reads and the stores are non-temporal (operations too large for
// the caches; measured on an 8192 x 4096 SFloat transposed copy with every launch on
// fresh operands: 58 us with plain accesses, 50 us with non-temporal ones).
template <class Op, int TF, int TG, bool PREFETCH, int TRMODE, bool NT>
__global__ __launch_bounds__(kEwBlock) void ew_transpose_vec_kernel(EwTParams p, Op op, typename Op::S sv) {
    ew_op_prepare<Op>();
    typedef typename Op::A A;
    typedef typename Op::B B;
    typedef typename Op::R R;
    constexpr int NIN = Op::NIN;
    constexpr bool TWO = (NIN == 2);
    constexpr int V = 16 / (int)sizeof(A);
    constexpr unsigned GV = TG / V;          // 128-bit slots along G
    constexpr unsigned FP = kEwBlock / GV;   // F positions per pass of the read
    constexpr unsigned NP = TF / FP;
    constexpr unsigned FV = TF / V;          // 128-bit slots along F
    constexpr unsigned GP = kEwBlock / FV;   // G positions per pass of the write
    constexpr unsigned NQ = TG / GP;
    // the launcher sizes the LDS: tile_b only when the second input goes through it
    extern __shared__ __align__(16) unsigned char ew_transpose_lds[];
    A(*tile_a)[TF + 1] = reinterpret_cast<A(*)[TF + 1]>(ew_transpose_lds);
    B(*tile_b)[TF + 1] = reinterpret_cast<B(*)[TF + 1]>(ew_transpose_lds + sizeof(A) * TG * (TF + 1));

    constexpr bool tr_a = NIN >= 1 && (TRMODE & 1) != 0;
    constexpr bool tr_b = TWO && (TRMODE & 2) != 0;
    // EARLY: the operation is applied on the way INTO the tile (to the transposed input as it
    // arrives, vector by vector, while the later loads are still in flight) and the tile holds
    // results; the pick-up side then does nothing between its stores, which go out back to back.
    // Possible when the one array input is the transposed one (a unary op, or a binary op whose
    // other operand is the scalar: TRMODE bit 2) and no element can be rejected. Measured on exp
    // of the transposed 8192 x 4096 SFloat view, fresh operands: 48.2 -> 47.4 us.
    constexpr bool EARLY = tr_a && !Op::CHECKED && (NIN == 1 || (TWO && (TRMODE & 4) != 0));
    static_assert(!EARLY || sizeof(R) == sizeof(A), "the tile holds results");
    const bool two_arrays = TWO && (tr_b || p.use_scalar == 0);
    const unsigned gv = threadIdx.x % GV, lf0 = threadIdx.x / GV;  // this lane's place while reading
    const unsigned fv = threadIdx.x % FV, lg0 = threadIdx.x / FV;  // and while writing

    A va[NP][V];
    B vb[TWO ? NP : 1][V];
    uint64_t f0 = 0, g0 = 0;
    int64_t off[3] = {0, 0, 0};

    // Loads of a tile's edge are not skipped but pulled back inside the array: with no
    // branch between them the loads of a lane go out back to back. What the pulled-back
    // lanes put into LDS is never read. The one vector along G that is partly inside the
    // array (G need not be a whole number of vectors) is read element by element, in place.
    auto fetch = [&](uint64_t tf0, uint64_t tg0, const int64_t (&toff)[3]) {
        const uint64_t g_own = tg0 + (uint64_t)gv * V;
        const bool partial = g_own < p.ng && g_own + V > p.ng;
        uint64_t g = g_own;
        if (g > p.ng - V) g = p.ng - V;
        if (tr_a) {
            const char* src = p.ptr[0] + toff[0] + (int64_t)g * (int64_t)sizeof(A);
#pragma unroll
            for (unsigned k = 0; k < NP; ++k) {
                uint64_t f = tf0 + lf0 + k * FP;
                if (f > p.nf - 1) f = p.nf - 1;
                raw_load<A, V, NT>(src + (int64_t)f * p.fstep[0], va[k]);
            }
            if (partial) {
                const char* own = p.ptr[0] + toff[0] + (int64_t)g_own * (int64_t)sizeof(A);
#pragma unroll
                for (unsigned k = 0; k < NP; ++k) {
                    uint64_t f = tf0 + lf0 + k * FP;
                    if (f > p.nf - 1) f = p.nf - 1;
#pragma unroll
                    for (int q = 0; q < V; ++q)
                        if (g_own + q < p.ng) va[k][q] = reinterpret_cast<const A*>(own + (int64_t)f * p.fstep[0])[q];
                }
            }
        }
        if constexpr (TWO) {
            if (tr_b) {
                const char* src = p.ptr[1] + toff[1] + (int64_t)g * (int64_t)sizeof(B);
#pragma unroll
                for (unsigned k = 0; k < NP; ++k) {
                    uint64_t f = tf0 + lf0 + k * FP;
                    if (f > p.nf - 1) f = p.nf - 1;
                    raw_load<B, V, NT>(src + (int64_t)f * p.fstep[1], vb[k]);
                }
                if (partial) {
                    const char* own = p.ptr[1] + toff[1] + (int64_t)g_own * (int64_t)sizeof(B);
#pragma unroll
                    for (unsigned k = 0; k < NP; ++k) {
                        uint64_t f = tf0 + lf0 + k * FP;
                        if (f > p.nf - 1) f = p.nf - 1;
#pragma unroll
                        for (int q = 0; q < V; ++q)
                            if (g_own + q < p.ng) vb[k][q] = reinterpret_cast<const B*>(own + (int64_t)f * p.fstep[1])[q];
                    }
                }
            }
        }
    };

    if (PREFETCH && blockIdx.x < p.n_tiles) {
        ew_tile_at<TF, TG>(p, blockIdx.x, f0, g0, off);
        fetch(f0, g0, off);
    }
    for (uint64_t tile = blockIdx.x; tile < p.n_tiles; tile += gridDim.x) {
        if (!PREFETCH) {
            ew_tile_at<TF, TG>(p, tile, f0, g0, off);
            fetch(f0, g0, off);
        }
        // registers -> LDS, transposed
        if constexpr (EARLY) {
            R(*tile_r)[TF + 1] = reinterpret_cast<R(*)[TF + 1]>(ew_transpose_lds);
#pragma unroll
            for (unsigned k = 0; k < NP; ++k) {
#pragma unroll
                for (int q = 0; q < V; ++q) {
                    A xa = va[k][q];
                    B yb = B();
                    if (TWO) {
                        if (p.use_scalar == 1) yb = (B)sv;
                        else { yb = (B)xa; xa = (A)sv; }
                    }
                    R zz = R();
                    (void)op(xa, yb, zz);
                    tile_r[gv * V + q][lf0 + k * FP] = zz;
                }
            }
        } else if (tr_a) {
#pragma unroll
            for (unsigned k = 0; k < NP; ++k) {
#pragma unroll
                for (int q = 0; q < V; ++q) tile_a[gv * V + q][lf0 + k * FP] = va[k][q];
            }
        }
        if constexpr (TWO) {
            if (tr_b) {
#pragma unroll
                for (unsigned k = 0; k < NP; ++k) {
#pragma unroll
                    for (int q = 0; q < V; ++q) tile_b[gv * V + q][lf0 + k * FP] = vb[k][q];
                }
            }
        }
        lds_barrier();
        uint64_t nf0 = 0, ng0 = 0;
        int64_t noff[3] = {0, 0, 0};
        if (PREFETCH && tile + gridDim.x < p.n_tiles) {
            // the next tile's transposed inputs set out now
            ew_tile_at<TF, TG>(p, tile + gridDim.x, nf0, ng0, noff);
            fetch(nf0, ng0, noff);
        }
        // lanes along F: pick the tile up transposed, compute, store
        const uint64_t f = f0 + (uint64_t)fv * V;
        if (f < p.nf && f + V > p.nf) {
            // the one vector along F that is partly inside the array (F need not be a whole number
            // of vectors): its elements one by one, nothing read or written past the row
            for (unsigned k = 0; k < NQ; ++k) {
                const unsigned lg = lg0 + k * GP;
                const uint64_t g = g0 + lg;
                if (g >= p.ng) continue;
                for (int q = 0; q < V; ++q) {
                    if (f + q >= p.nf) break;
                    if constexpr (EARLY) {
                        R(*tile_r)[TF + 1] = reinterpret_cast<R(*)[TF + 1]>(ew_transpose_lds);
                        *reinterpret_cast<R*>(p.ptr[2] + off[2] + (int64_t)g * p.gstep[2] + (int64_t)(f + q) * (int64_t)sizeof(R)) = tile_r[lg][fv * V + q];
                        continue;
                    }
                    A xa = A();
                    B yb = B();
                    if (NIN >= 1) xa = tr_a ? tile_a[lg][fv * V + q]
                                            : *reinterpret_cast<const A*>(p.ptr[0] + off[0] + (int64_t)g * p.gstep[0] + (int64_t)(f + q) * p.fstep[0]);
                    if (TWO) {
                        if (p.use_scalar == 0) yb = tr_b ? tile_b[lg][fv * V + q]
                                                         : *reinterpret_cast<const B*>(p.ptr[1] + off[1] + (int64_t)g * p.gstep[1] + (int64_t)(f + q) * p.fstep[1]);
                        else if (p.use_scalar == 1) yb = (B)sv;
                        else { yb = (B)xa; xa = (A)sv; }
                    }
                    R zz = R();
                    if (op(xa, yb, zz)) *reinterpret_cast<R*>(p.ptr[2] + off[2] + (int64_t)g * p.gstep[2] + (int64_t)(f + q) * (int64_t)sizeof(R)) = zz;
                    else if (p.flag) *p.flag = 1;
                }
            }
        } else if (f < p.nf) {
            // an op with many instructions per element is not unrolled over the rows:
            // its V elements side by side already fill the registers eight waves can have
            constexpr int UNROLL_ROWS = (op_is_heavy<Op>::value && !EARLY) ? 1 : (int)NQ;
#pragma unroll UNROLL_ROWS
            for (unsigned k = 0; k < NQ; ++k) {
                const unsigned lg = lg0 + k * GP;
                const uint64_t g = g0 + lg;
                if (g >= p.ng) continue;
                if constexpr (EARLY) {
                    R(*tile_r)[TF + 1] = reinterpret_cast<R(*)[TF + 1]>(ew_transpose_lds);
                    R zr[V];
#pragma unroll
                    for (int q = 0; q < V; ++q) zr[q] = tile_r[lg][fv * V + q];
                    char* dstr = p.ptr[2] + off[2] + (int64_t)g * p.gstep[2] + (int64_t)f * (int64_t)sizeof(R);
                    if constexpr (NT && sizeof(R) * V == 16) raw_store_scattered_stream<R, V>(dstr, zr);
                    else raw_store<R, V, NT>(dstr, zr);
                    continue;
                }
                A x[V];
                B y[V];
                if (NIN >= 1) {
                    if (tr_a) {
#pragma unroll
                        for (int q = 0; q < V; ++q) x[q] = tile_a[lg][fv * V + q];
                    } else {
                        ew_load<A, V, false>(p.ptr[0] + off[0] + (int64_t)g * p.gstep[0], p.fstep[0], (int64_t)f, x);
                    }
                }
                if (two_arrays) {
                    if (tr_b) {
#pragma unroll
                        for (int q = 0; q < V; ++q) y[q] = tile_b[lg][fv * V + q];
                    } else {
                        ew_load<B, V, false>(p.ptr[1] + off[1] + (int64_t)g * p.gstep[1], p.fstep[1], (int64_t)f, y);
                    }
                }
                R z[V];
                bool ok = true;
#pragma unroll
                for (int q = 0; q < V; ++q) {
                    A xa = (NIN >= 1) ? x[q] : A();
                    B yb = B();
                    if (TWO) {
                        if (p.use_scalar == 0) yb = y[q];
                        else if (p.use_scalar == 1) yb = (B)sv;
                        else { yb = (B)xa; xa = (A)sv; }
                    }
                    z[q] = R();
                    ok = op(xa, yb, z[q]) && ok;
                }
                char* dst = p.ptr[2] + off[2] + (int64_t)g * p.gstep[2] + (int64_t)f * (int64_t)sizeof(R);
                if (!Op::CHECKED || ok) {
                    if constexpr (NT && sizeof(R) * V == 16) raw_store_scattered_stream<R, V>(dst, z);
                    else raw_store<R, V, NT>(dst, z);
                } else {
                    // some element was rejected: store the others one by one
                    if (p.flag) *p.flag = 1;
#pragma unroll
                    for (int q = 0; q < V; ++q) {
                        A xa = (NIN >= 1) ? x[q] : A();
                        B yb = B();
                        if (TWO) {
                            if (p.use_scalar == 0) yb = y[q];
                            else if (p.use_scalar == 1) yb = (B)sv;
                            else { yb = (B)xa; xa = (A)sv; }
                        }
                        R zz = R();
                        if (op(xa, yb, zz)) reinterpret_cast<R*>(dst)[q] = zz;
                    }
                }
            }
        }
        lds_barrier();
        if (PREFETCH) {
            f0 = nf0;
            g0 = ng0;
            off[0] = noff[0];
            off[1] = noff[1];
            off[2] = noff[2];
        }
    }
}

// The element-wise form, for operands that do not tolerate 128-bit accesses.
template <class Op, int TG>
__global__ __launch_bounds__(kEwBlock) void ew_transpose_kernel(EwTParams p, Op op, typename Op::S sv) {
    ew_op_prepare<Op>();
    typedef typename Op::A A;
    typedef typename Op::B B;
    typedef typename Op::R R;
    constexpr int NIN = Op::NIN;
    constexpr bool TWO = (NIN == 2);
    constexpr int TF = 64;
    __shared__ A tile_a[TG][TF + 1];
    __shared__ B tile_b[TWO ? TG : 1][TF + 1];

    const bool two_arrays = TWO && p.use_scalar == 0;
    for (uint64_t tile = blockIdx.x; tile < p.n_tiles; tile += gridDim.x) {
        uint64_t f0, g0;
        int64_t off[3];
        ew_tile_at<TF, TG>(p, tile, f0, g0, off);

        // phase 1: transposed inputs, lanes along G
        {
            const unsigned lg = threadIdx.x % TG;
            const unsigned lf0 = threadIdx.x / TG;
            constexpr unsigned FSTEP = kEwBlock / TG;
            const uint64_t g = g0 + lg;
            if (p.tr[0]) {
#pragma unroll 4
                for (unsigned lf = lf0; lf < TF; lf += FSTEP) {
                    const uint64_t f = f0 + lf;
                    if (g < p.ng && f < p.nf)
                        tile_a[lg][lf] = *reinterpret_cast<const A*>(p.ptr[0] + off[0] + (int64_t)g * p.gstep[0] + (int64_t)f * p.fstep[0]);
                }
            }
            if (two_arrays && p.tr[1]) {
#pragma unroll 4
                for (unsigned lf = lf0; lf < TF; lf += FSTEP) {
                    const uint64_t f = f0 + lf;
                    if (g < p.ng && f < p.nf)
                        tile_b[TWO ? lg : 0][lf] = *reinterpret_cast<const B*>(p.ptr[1] + off[1] + (int64_t)g * p.gstep[1] + (int64_t)f * p.fstep[1]);
                }
            }
        }
        __syncthreads();
        // phase 2: lanes along F
        {
            const unsigned lf = threadIdx.x % TF;
            const unsigned lg0 = threadIdx.x / TF;
            constexpr unsigned GSTEP = kEwBlock / TF;
            const uint64_t f = f0 + lf;
#pragma unroll 4
            for (unsigned lg = lg0; lg < TG; lg += GSTEP) {
                const uint64_t g = g0 + lg;
                if (g < p.ng && f < p.nf) {
                    A x = A();
                    B y = B();
                    if (NIN >= 1) {
                        x = p.tr[0] ? tile_a[lg][lf]
                                    : *reinterpret_cast<const A*>(p.ptr[0] + off[0] + (int64_t)g * p.gstep[0] + (int64_t)f * p.fstep[0]);
                    }
                    if (TWO) {
                        if (p.use_scalar == 0) {
                            y = p.tr[1] ? tile_b[TWO ? lg : 0][lf]
                                        : *reinterpret_cast<const B*>(p.ptr[1] + off[1] + (int64_t)g * p.gstep[1] + (int64_t)f * p.fstep[1]);
                        } else if (p.use_scalar == 1) {
                            y = (B)sv;
                        } else {
                            y = (B)x;
                            x = (A)sv;
                        }
                    }
                    R z = R();
                    if (op(x, y, z)) {
                        *reinterpret_cast<R*>(p.ptr[2] + off[2] + (int64_t)g * p.gstep[2] + (int64_t)f * p.fstep[2]) = z;
                    } else if (p.flag) {
                        *p.flag = 1;
                    }
                }
            }
        }
        __syncthreads();
    }
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------
static inline unsigned ew_grid_cap() {
    static unsigned cap = 0;
    if (cap == 0) {
        const char* e = std::getenv("CUMO_HIP_EW_GRID_CAP");
        cap = e ? (unsigned)std::strtoul(e, nullptr, 10) : 0;
        if (cap == 0) cap = (unsigned)kNumCU * 64;  // measured: more, shorter blocks stream better than a long grid-stride loop
    }
    return cap;
}

// Largest x extent of a grid.
static inline uint64_t ew_grid_max() { return 0x7fffffffull; }

// Blocks of a flat launch whose operator fills tables in LDS (CUMO_HIP_EW_TABLE_BLOCKS; 12 per compute unit)
static inline unsigned ew_table_op_blocks() {
    static unsigned blocks = 0;
    if (blocks == 0) {
        const char* e = std::getenv("CUMO_HIP_EW_TABLE_BLOCKS");
        const long v = e ? std::strtol(e, nullptr, 10) : 0;
        blocks = v > 0 ? (unsigned)v : (unsigned)kNumCU * 12;
    }
    return blocks;
}

// Non-temporal accesses once an operation touches more than the caches could keep for
// the next operation anyway. Measured with every launch on fresh operands (the state a
// long computation is in): a 1R+1W operation over 2 x 128 MiB runs at 72-73% of the HBM
// peak with plain accesses and 77-78% with non-temporal ones; no difference at 32 MiB.
// (Launching the same operation on the same buffers again and again favours plain
// accesses up to 256 MB, because the last-level cache then still holds the operands.)
// The decision is stream_past_caches(bytes), shared by every kernel family.

// CUMO_HIP_EW_LEAN_ROWS=0 (read once): large two-dimensional arrays take the general row kernel
static inline bool ew_lean_rows_enabled() {
    static const bool on = [] {
        const char* e = std::getenv("CUMO_HIP_EW_LEAN_ROWS");
        return !(e && e[0] == '0');
    }();
    return on;
}

// in1/in2 may be NULL (NIN < 2 or the scalar form). out_bit is non-NULL for a
// Bit result, in which case out is ignored.
// HEAVY_CALL (a compile-time choice, so that the kernels it rules out are never built): a function
// with many instructions per element -- capped grids, and no lean two-rows-per-lane form.
template <class Op, bool HEAVY_CALL = false>
static void ew_launch(Op op, const cumo_na_iarray_t* in1, const cumo_na_iarray_t* in2, const cumo_na_iarray_t* out,
                      const cumo_na_bit_iarray_t* out_bit, const cumo_na_indexer_t* indexer, typename Op::S sv, int use_scalar,
                      int* flag) {
    constexpr bool heavy = HEAVY_CALL;
    typedef typename Op::A A;
    typedef typename Op::B B;
    typedef typename Op::R R;
    // A Bit result from an input that walks another dimension fastest than the result does (a comparison of a
    // transposed view): the tile-transposing kernels write typed results only, and lanes along the result's bits would
    // read such an input one element per cache line. The input is first copied into the result's order (the typed
    // store, which transposes through LDS), then compared from there: [8192,4096] SFloat x.transpose > 0, 370 -> 75 us.
    if constexpr (Op::BIT_OUT && Op::NIN >= 1 && (sizeof(A) == 4 || sizeof(A) == 8)) {
        const cumo_na_iarray_t* ins[2] = {in1, (Op::NIN >= 2 && use_scalar == 0 && sizeof(B) == sizeof(A)) ? in2 : nullptr};
        const int nd = indexer->ndim;
        int F = -1;
        for (int d = 0; d < nd; ++d)
            if (indexer->shape[d] >= 16 && out_bit->step[d] == 1) F = d;
        bool stage[2] = {false, false};
        if (F >= 0 && indexer->total_size >= 65536 && nd <= CUMO_NA_MAX_DIMENSION) {
            for (int k = 0; k < 2; ++k) {
                if (!ins[k]) continue;
                const int64_t sf = (int64_t)ins[k]->step[F];
                if (sf == 0 || sf == (int64_t)sizeof(A) || sf == -(int64_t)sizeof(A)) continue;
                for (int d = 0; d < nd; ++d) {
                    const int64_t sd = (int64_t)ins[k]->step[d];
                    if (d != F && indexer->shape[d] >= 16 && (sd == (int64_t)sizeof(A) || sd == -(int64_t)sizeof(A))) stage[k] = true;
                }
            }
        }
        if (stage[0] || stage[1]) {
            cumo_na_iarray_t tmp[2];
            char* held[2] = {nullptr, nullptr};
            bool ok = true;
            for (int k = 0; k < 2 && ok; ++k) {
                if (!stage[k]) continue;
                held[k] = cumo_cuda_runtime_malloc(indexer->total_size * sizeof(A));
                if (!held[k]) { ok = false; break; }   // (the pool has reported it)
                tmp[k].ptr = held[k];
                ssize_t s = (ssize_t)sizeof(A);
                for (int d = nd - 1; d >= 0; --d) {
                    tmp[k].step[d] = s;
                    s *= (ssize_t)indexer->shape[d];
                }
                cumo_na_indexer_t ix = *indexer;
                if (sizeof(A) == 4) cumo_iter_int32_store_int32_kernel_launch(&tmp[k], const_cast<cumo_na_iarray_t*>(ins[k]), &ix);
                else cumo_iter_dfloat_store_dfloat_kernel_launch(&tmp[k], const_cast<cumo_na_iarray_t*>(ins[k]), &ix);
            }
            if (ok)
                ew_launch<Op, HEAVY_CALL>(op, stage[0] ? &tmp[0] : in1, stage[1] ? &tmp[1] : in2, out, out_bit, indexer, sv, use_scalar, flag);
            for (int k = 0; k < 2; ++k)
                if (held[k]) cumo_cuda_runtime_free(held[k]);
            return;
        }
    }
    EwOperand ops[3];
    int slot[3];
    int nops = 0;
    if (Op::NIN >= 1 && in1) { ops[nops] = EwOperand{in1->ptr, in1->step, (int)sizeof(A), 0}; slot[nops++] = 0; }
    if (Op::NIN >= 2 && in2 && use_scalar == 0) { ops[nops] = EwOperand{in2->ptr, in2->step, (int)sizeof(B), 0}; slot[nops++] = 1; }
    if (Op::BIT_OUT) {
        ops[nops] = EwOperand{(const char*)out_bit->ptr, out_bit->step, 0, out_bit->pos};
    } else {
        ops[nops] = EwOperand{out->ptr, out->step, (int)sizeof(R), 0};
    }
    slot[nops++] = 2;

    EwPlan plan;
    plan_elementwise(indexer->ndim, indexer->shape, nops, ops, &plan);
    if (plan.kind == EW_EMPTY) return;
    hipStream_t stream = current_stream();

    if (plan.kind == EW_TRANSPOSE) {
        EwTParams tp;
        std::memset(&tp, 0, sizeof(tp));
        const int n = plan.ndim;
        tp.nf = plan.shape[n - 1];
        tp.ng = plan.shape[n - 2];
        tp.nouter = n - 2;
        tp.use_scalar = use_scalar;
        tp.flag = flag;
        // bytes the operation moves (every operand at the full extent: a transposed operand is never a repeated one here)
        uint64_t tr_bytes = 0;
        for (int o = 0; o < nops; ++o) {
            uint64_t nb = slot[o] == 0 ? sizeof(A) : (slot[o] == 1 ? sizeof(B) : sizeof(R));
            for (int d = 0; d < n; ++d)
                if (plan.step[o][d] != 0) nb *= plan.shape[d];
            tr_bytes += nb;
        }
        const bool tr_nt = stream_past_caches(tr_bytes);
        {
            static int order = -2;
            if (order == -2) {
                const char* e = std::getenv("CUMO_HIP_TR_ORDER");
                order = e ? std::atoi(e) : -1;
            }
            // Consecutive blocks take tiles that are neighbours along the result's fast dimension when
            // the operation streams from and to memory (their stores then fill whole stretches of the
            // same result rows: 50 us against 60 us on the transposed 8192 x 4096 copy), and each step
            // that way also moves one tile along the inputs' fast dimension: the blocks that run together
            // would otherwise all read the same few columns of rows a power of two apart (exp of the
            // transposed 8192 x 4096 SFloat view: 56.9 -> 52.9 us; steps of 3 to 17 tiles: 54 to 55 us).
            // Operands that fit the caches prefer neighbours along the inputs' fast dimension.
            tp.order = order >= 0 ? order : (tr_nt ? 3 : 1);
        }
        constexpr int TG = (sizeof(A) >= 8 || sizeof(B) >= 8) ? 32 : 64;
        tp.f_tiles = (tp.nf + 63) / 64;
        tp.g_tiles = (tp.ng + TG - 1) / TG;
        uint64_t outer = 1;
        for (int d = 0; d < n - 2; ++d) { tp.oshape[d] = plan.shape[d]; outer *= plan.shape[d]; }
        tp.n_tiles = tp.f_tiles * tp.g_tiles * outer;
        if (tp.order == 2 && ((tp.f_tiles & 7) || (tp.g_tiles & 7))) tp.order = 0;
        for (int o = 0; o < nops; ++o) {
            const int s = slot[o];
            tp.ptr[s] = const_cast<char*>(ops[o].ptr);
            tp.fstep[s] = plan.step[o][n - 1];
            tp.gstep[s] = plan.step[o][n - 2];
            for (int d = 0; d < n - 2; ++d) tp.ostep[s][d] = plan.step[o][d];
            if (s < 2) {
                const uint64_t gs = tp.gstep[s] < 0 ? -tp.gstep[s] : tp.gstep[s];
                const uint64_t fs = tp.fstep[s] < 0 ? -tp.fstep[s] : tp.fstep[s];
                tp.tr[s] = (gs != 0 && fs != 0 && gs < fs) ? 1 : 0;
            }
        }
        uint64_t grid = tp.n_tiles;
        if (grid > 0x7fffffffull) grid = 0x7fffffffull;
        // 128-bit form: same element size everywhere, whole vectors in both tile
        // directions, every operand aligned along the dimension it is walked in
        constexpr int V = 16 / (int)sizeof(A);
        // (neither extent need be a whole number of vectors, and the operands need their element's alignment
        // only: a 128-bit access works on any 4-byte boundary, and the one vector that is partly inside the
        // array on either side goes element by element)
        bool vt = sizeof(A) == sizeof(R) && (Op::NIN < 2 || sizeof(B) == sizeof(A)) && (16 % sizeof(A)) == 0 && sizeof(A) >= 4 &&
                  tp.ng >= (uint64_t)V && tp.nf >= (uint64_t)V;
        for (int o = 0; o < nops && vt; ++o) {
            const int sl = slot[o];
            const int64_t es = (int64_t)sizeof(A);
            const bool through_lds = sl < 2 && tp.tr[sl];
            const int64_t along = through_lds ? tp.gstep[sl] : tp.fstep[sl];
            const int64_t across = through_lds ? tp.fstep[sl] : tp.gstep[sl];
            if (sl < 2 && !through_lds && along == 0) continue;  // broadcast along F: scalar loads
            vt = along == es && (across % es) == 0 && ((uintptr_t)tp.ptr[sl] % es) == 0;
            for (int d = 0; d < n - 2 && vt; ++d) vt = (tp.ostep[sl][d] % es) == 0;
        }
        if constexpr (sizeof(A) == sizeof(R) && (Op::NIN < 2 || sizeof(B) == sizeof(A)) && (16 % sizeof(A)) == 0 && sizeof(A) >= 4) {
            if (vt) {
                const uint64_t vgrid = 0x7fffffffull;
                const bool a_through_lds = Op::NIN >= 1 && tp.tr[0];
                const bool b_through_lds = Op::NIN >= 2 && use_scalar == 0 && tp.tr[1];
                // an op with many instructions per element: 256-byte tiles, eight blocks per compute
                // unit, each with its next tile in flight. Otherwise tiles of 512 bytes along the
                // transposed inputs' fast dimension, one per block (measured on a transposed
                // 8192 x 4096 SFloat copy that finds its operands in the caches: 39.4 us against 45.3 us
                // with 256 bytes).
                // Operations that stream past the caches take tiles of 128 x 256 bytes instead: the stores
                // then fill 512 bytes of a result row at a time (bare transposed copy of the 8192 x 4096
                // SFloat view on fresh operands: 49.1 -> 47.6 us).
                constexpr bool PF = op_is_heavy<Op>::value;
                constexpr int TGC = (PF ? 256 : 512) / (int)sizeof(A), TFC = 64;   // operands in the caches
                constexpr int TGS = 256 / (int)sizeof(A), TFS = PF ? 64 : 128;      // streaming
                const int TGV = tr_nt ? TGS : TGC, TFV = tr_nt ? TFS : TFC;
                tp.f_tiles = (tp.nf + TFV - 1) / TFV;
                tp.g_tiles = (tp.ng + TGV - 1) / TGV;
                if (tp.order == 2 && ((tp.f_tiles & 7) || (tp.g_tiles & 7))) tp.order = 0;
                tp.n_tiles = tp.f_tiles * tp.g_tiles * outer;
                grid = tp.n_tiles < vgrid ? tp.n_tiles : vgrid;
                if (PF) {
                    static uint64_t pgrid = 0;
                    if (pgrid == 0) {
                        const char* e = std::getenv("CUMO_HIP_TR_GRID");
                        pgrid = e ? std::strtoull(e, nullptr, 10) : 0;
                        if (pgrid == 0) pgrid = (uint64_t)kNumCU * 21;  // measured best on the transposed 8192 x 4096 SFloat exp (8192 tiles): 43 us, against 47.5 us with 8 and 49.5 us with a block per tile
                    }
                    if (grid > pgrid) grid = pgrid;
                }
                const size_t lds = sizeof(A) * TGV * (TFV + 1) + (b_through_lds ? sizeof(B) * TGV * (TFV + 1) : 0);
                const dim3 g((unsigned)grid), b(kEwBlock);
#define CUMO_TR_LAUNCH(MODE)                                                                                                       \
    do {                                                                                                                            \
        if (tr_nt) {                                                                                                                \
            auto kernel = ew_transpose_vec_kernel<Op, TFS, TGS, PF, MODE, true>;                                                    \
            if (lds > 65536) (void)hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);  \
            hipLaunchKernelGGL(kernel, g, b, lds, stream, tp, op, sv);                                                              \
        } else {                                                                                                                    \
            auto kernel = ew_transpose_vec_kernel<Op, TFC, TGC, PF, MODE, false>;                                                   \
            if (lds > 65536) (void)hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);  \
            hipLaunchKernelGGL(kernel, g, b, lds, stream, tp, op, sv);                                                              \
        }                                                                                                                           \
    } while (0)
                if constexpr (Op::NIN >= 2) {
                    if (a_through_lds && b_through_lds) CUMO_TR_LAUNCH(3);
                    else if (b_through_lds) CUMO_TR_LAUNCH(2);
                    else if (a_through_lds && use_scalar != 0) CUMO_TR_LAUNCH(5);   // array (transposed) op scalar
                    else CUMO_TR_LAUNCH(1);
                } else {
                    CUMO_TR_LAUNCH(1);
                }
#undef CUMO_TR_LAUNCH
                cumo_cuda_runtime_check_kernel_launch();
                return;
            }
        }
        hipLaunchKernelGGL((ew_transpose_kernel<Op, TG>), dim3((unsigned)grid), dim3(kEwBlock), 0, stream, tp, op, sv);
        cumo_cuda_runtime_check_kernel_launch();
        return;
    }

    EwKParams kp;
    std::memset(&kp, 0, sizeof(kp));
    const int n = plan.ndim;
    kp.inner = plan.shape[n - 1];
    kp.rows = plan.total / kp.inner;
    kp.nouter = n - 1;
    kp.use_scalar = use_scalar;
    kp.flag = flag;
    kp.small_rows = (kp.rows < 0xffffffffull && !force_wide_indices()) ? 1 : 0;
    for (int d = 0; d < n - 1; ++d) kp.oshape[d] = plan.shape[d];
    for (int o = 0; o < nops; ++o) {
        const int s = slot[o];
        kp.ptr[s] = const_cast<char*>(ops[o].ptr);
        kp.istep[s] = plan.step[o][n - 1];
        for (int d = 0; d < n - 1; ++d) kp.ostep[s][d] = plan.step[o][d];
    }
    if (Op::BIT_OUT) kp.out_bitpos = out_bit->pos;

    int vec = plan.vec;
    // the vector form of a Bit row needs the 32/vec lanes of a word inside one row
    if (Op::BIT_OUT && vec > 1 && kp.inner < 32) vec = 1;
    bool force_scalar = false;
    {
        static int force1 = -1;
        if (force1 < 0) force1 = std::getenv("CUMO_HIP_FORCE_VEC1") ? 1 : 0;
        if (force1) vec = 1;
        force_scalar = force1 != 0;
    }
    // the two lean kernels below also take inputs that only have their element's alignment
    // (a slice that starts at an odd column): a 128-bit global load works on any 4-byte boundary
    const int lean_vec = force_wide_indices() ? 1 : ((vec == 1 && plan.vec_loose > 1 && !force_scalar) ? plan.vec_loose : vec);
    const dim3 b(kEwBlock);

    // A Bit result over flat inputs, starting on a 128-bit unit: the lean Bit kernel
    // (measured on 2^25 SFloat > scalar: see the notes at the kernel).
    if constexpr (Op::BIT_OUT) {
        constexpr int VB = 16 / (int)sizeof(A);
        bool flat = n == 1 && vec == VB && (Op::NIN < 2 || sizeof(B) == sizeof(A)) && plan.step[nops - 1][0] == 1 &&
                    (out_bit->pos % 128) == 0 && ((uintptr_t)out_bit->ptr % 16) == 0;
        int one_element = -1;   // the slot of an input that is an array of a single element (x.eq(x.max)): read as the scalar
        for (int o = 0; o + 1 < nops && flat; ++o) {
            const int sl = slot[o];
            const int64_t es = sl == 0 ? (int64_t)sizeof(A) : (int64_t)sizeof(B);
            if (Op::NIN == 2 && std::is_same<A, B>::value && std::is_same<typename Op::S, A>::value && use_scalar == 0 &&
                plan.step[o][0] == 0 && one_element < 0 && ((uintptr_t)ops[o].ptr % sizeof(A)) == 0) {
                one_element = sl;
                continue;
            }
            flat = plan.step[o][0] == es;
        }
        const char* flat_px = kp.ptr[0];
        const char* flat_py = kp.ptr[1];
        int flat_scalar = use_scalar;
        if (flat && one_element >= 0) {
            flat_px = kp.ptr[1 - one_element];
            flat_py = kp.ptr[one_element];
            flat_scalar = (one_element == 1 ? 1 : 2) | 4;
        }
        if constexpr (VB == 4 || VB == 2) {
            const uint64_t groups = (kp.inner + 127) / 128;
            const uint64_t blocks = (groups * (32 / VB) + kEwBlock - 1) / kEwBlock;
            if (flat && blocks <= ew_grid_max()) {
                const bool nt = stream_past_caches(kp.inner * sizeof(A) * (uint64_t)(nops - 1));
                CUMO_BIT_DIGIT* dst = reinterpret_cast<CUMO_BIT_DIGIT*>(const_cast<char*>(ops[nops - 1].ptr)) + out_bit->pos / 32;
                const dim3 g((unsigned)blocks);
                if (nt) hipLaunchKernelGGL((ew_flat_bit_kernel<Op, VB, true>), g, b, 0, stream, flat_px, flat_py, dst, kp.inner, flat_scalar, op, sv);
                else hipLaunchKernelGGL((ew_flat_bit_kernel<Op, VB, false>), g, b, 0, stream, flat_px, flat_py, dst, kp.inner, flat_scalar, op, sv);
                cumo_cuda_runtime_check_kernel_launch();
                return;
            }
            // a contiguous matrix (op) a second two-dimensional operand, the bits one run as well
            if constexpr (Op::NIN == 2 && std::is_same<A, B>::value) {
                bool bits_one_run = (n == 2 || n == 3) && plan.step[2][n - 1] == 1 && plan.step[2][n - 2] == (int64_t)kp.inner;
                if (n == 3) bits_one_run = bits_one_run && plan.step[2][0] == (int64_t)kp.inner * (int64_t)plan.shape[1];
                if (bits_one_run && nops == 3 && use_scalar == 0 && !force_scalar && !force_wide_indices() && plan.total < 0x7fffffffull && kp.inner >= 64 &&
                    (out_bit->pos % 128) == 0 && ((uintptr_t)out_bit->ptr % 16) == 0) {
                    const int64_t es = (int64_t)sizeof(A);
                    auto one_run = [&](int sl) {
                        bool run = kp.istep[sl] == es && kp.ostep[sl][n - 2] == es * (int64_t)kp.inner && ((uintptr_t)kp.ptr[sl] % 16) == 0;
                        if (n == 3) run = run && kp.ostep[sl][0] == es * (int64_t)kp.inner * (int64_t)plan.shape[1];
                        return run;
                    };
                    const int full = one_run(0) ? 0 : (one_run(1) ? 1 : -1);
                    if (full >= 0) {
                        const int per = 1 - full;
                        EwPeriod pr;
                        pr.period = (uint32_t)kp.inner;
                        pr.div = div31_make(pr.period);
                        pr.s_outer = kp.ostep[per][n - 2];
                        pr.s_inner = kp.istep[per];
                        pr.first = per == 0 ? 1 : 0;
                        pr.mid = n == 3 ? (uint32_t)plan.shape[1] : 0u;
                        pr.div_mid = div31_make(n == 3 ? (uint32_t)plan.shape[1] : 1u);
                        pr.s_outermost = n == 3 ? kp.ostep[per][0] : 0;
                        const uint32_t total = (uint32_t)plan.total;
                        const uint64_t pgroups = ((uint64_t)total + 127) / 128;
                        const uint64_t pblocks = (pgroups * (32 / VB) + kEwBlock - 1) / kEwBlock;
                        if (pblocks <= ew_grid_max()) {
                            const bool nt = stream_past_caches((uint64_t)total * sizeof(A));
                            CUMO_BIT_DIGIT* dst = reinterpret_cast<CUMO_BIT_DIGIT*>(const_cast<char*>(ops[nops - 1].ptr)) + out_bit->pos / 32;
                            const dim3 g((unsigned)pblocks);
                            if (nt) hipLaunchKernelGGL((ew_flat_bit_period_kernel<Op, VB, true>), g, b, 0, stream, kp.ptr[full], kp.ptr[per], dst, total, pr, op);
                            else hipLaunchKernelGGL((ew_flat_bit_period_kernel<Op, VB, false>), g, b, 0, stream, kp.ptr[full], kp.ptr[per], dst, total, pr, op);
                            cumo_cuda_runtime_check_kernel_launch();
                            return;
                        }
                    }
                }
            }
            // every input addressed by row and column, the bits one run (comparisons of slices whose rows are not whole
            // vectors, with one another or with the scalar; one dimension is one row)
            if constexpr (Op::NIN == 1 || (Op::NIN == 2 && std::is_same<A, B>::value)) {
                const int ob = nops - 1;
                bool bits_one_run = n <= 3 && plan.step[ob][n - 1] == 1;
                if (n >= 2) bits_one_run = bits_one_run && plan.step[ob][n - 2] == (int64_t)kp.inner;
                if (n == 3) bits_one_run = bits_one_run && plan.step[ob][0] == (int64_t)kp.inner * (int64_t)plan.shape[1];
                if (bits_one_run && vec == 1 && !force_scalar && !force_wide_indices() && plan.total < 0x7fffffffull && plan.total >= 16384 &&
                    kp.inner >= 64 && (out_bit->pos % 128) == 0 && ((uintptr_t)out_bit->ptr % 16) == 0) {
                    const int64_t es = (int64_t)sizeof(A);
                    bool fits = true;
                    for (int o = 0; o + 1 < nops && fits; ++o) {
                        const int sl = slot[o];
                        fits = (kp.istep[sl] == es || kp.istep[sl] == 0) && ((uintptr_t)kp.ptr[sl] % (uintptr_t)es) == 0;
                    }
                    if (fits) {
                        EwAddressed pa;
                        std::memset(&pa, 0, sizeof(pa));
                        for (int o = 0; o + 1 < nops; ++o) {
                            const int sl = slot[o];
                            pa.in[sl] = kp.ptr[sl];
                            pa.s_outer[sl] = n >= 2 ? kp.ostep[sl][n - 2] : 0;
                            pa.s_inner[sl] = kp.istep[sl];
                            pa.s_outermost[sl] = n == 3 ? kp.ostep[sl][0] : 0;
                        }
                        pa.n = (uint32_t)plan.total;
                        pa.period = (uint32_t)kp.inner;
                        pa.div = div31_make(pa.period);
                        pa.mid = n == 3 ? (uint32_t)plan.shape[1] : 0u;
                        pa.div_mid = div31_make(n == 3 ? (uint32_t)plan.shape[1] : 1u);
                        const uint64_t pgroups = ((uint64_t)pa.n + 127) / 128;
                        const uint64_t pblocks = (pgroups * (32 / VB) + kEwBlock - 1) / kEwBlock;
                        if (pblocks <= ew_grid_max()) {
                            const bool nt = stream_past_caches((uint64_t)pa.n * sizeof(A) * (uint64_t)(nops - 1));
                            CUMO_BIT_DIGIT* dst = reinterpret_cast<CUMO_BIT_DIGIT*>(const_cast<char*>(ops[nops - 1].ptr)) + out_bit->pos / 32;
                            const dim3 g((unsigned)pblocks);
                            if (nt) hipLaunchKernelGGL((ew_flat_bit_addressed_kernel<Op, VB, true>), g, b, 0, stream, pa, dst, use_scalar, op, sv);
                            else hipLaunchKernelGGL((ew_flat_bit_addressed_kernel<Op, VB, false>), g, b, 0, stream, pa, dst, use_scalar, op, sv);
                            cumo_cuda_runtime_check_kernel_launch();
                            return;
                        }
                    }
                }
            }
        }
    }

    // Matrix with rows of an odd length (op) a second two-dimensional operand: flat over the matrix
    // and the result, the other operand addressed by row and column (see ew_flat_period_kernel).
    if constexpr (!Op::BIT_OUT && Op::NIN == 2 && std::is_same<A, B>::value && sizeof(A) == sizeof(R) && (sizeof(A) == 4 || sizeof(A) == 8) &&
                  !op_is_heavy<Op>::value && !op_has_rare<Op>::value && !heavy) {
        constexpr int V = 16 / (int)sizeof(A);
        if ((n == 2 || n == 3) && nops == 3 && use_scalar == 0 && !force_scalar && !force_wide_indices() && (kp.inner % V) != 0 && kp.inner >= 64 &&
            plan.total < 0x7fffffffull) {
            const int64_t es = (int64_t)sizeof(A);
            auto one_run = [&](int sl) {
                bool run = kp.istep[sl] == es && kp.ostep[sl][n - 2] == es * (int64_t)kp.inner && ((uintptr_t)kp.ptr[sl] % 16) == 0;
                if (n == 3) run = run && kp.ostep[sl][0] == es * (int64_t)kp.inner * (int64_t)plan.shape[1];
                return run;
            };
            int full = -1;
            if (one_run(2)) {
                if (one_run(0)) full = 0;
                else if (one_run(1)) full = 1;
            }
            if (full >= 0) {
                const int per = 1 - full;
                EwPeriod pr;
                pr.period = (uint32_t)kp.inner;
                pr.div = div31_make(pr.period);
                pr.s_outer = kp.ostep[per][n - 2];
                pr.s_inner = kp.istep[per];
                pr.first = per == 0 ? 1 : 0;
                pr.mid = n == 3 ? (uint32_t)plan.shape[1] : 0u;
                pr.div_mid = div31_make(n == 3 ? (uint32_t)plan.shape[1] : 1u);
                pr.s_outermost = n == 3 ? kp.ostep[per][0] : 0;
                const uint32_t total = (uint32_t)plan.total;
                const uint64_t blocks = ((uint64_t)total + (uint64_t)kEwBlock * V - 1) / ((uint64_t)kEwBlock * V);
                if (blocks <= ew_grid_max()) {
                    const bool nt = stream_past_caches(2 * (uint64_t)total * sizeof(A));
                    const dim3 g((unsigned)blocks);
                    if (nt) hipLaunchKernelGGL((ew_flat_period_kernel<Op, V, true>), g, b, 0, stream, kp.ptr[full], kp.ptr[per], kp.ptr[2], total, pr, flag, op);
                    else hipLaunchKernelGGL((ew_flat_period_kernel<Op, V, false>), g, b, 0, stream, kp.ptr[full], kp.ptr[per], kp.ptr[2], total, pr, flag, op);
                    cumo_cuda_runtime_check_kernel_launch();
                    return;
                }
            }
        }
    }

    // A result that is one run of rows that are not whole vectors, every input a two-dimensional view that runs along
    // its rows or is constant along them (see ew_flat_addressed_kernel): what would otherwise go element by element.
    // (a result of another width than the inputs, a cast, too: the lane's vector is the result's)
    if constexpr (!Op::BIT_OUT && (Op::NIN == 1 || (Op::NIN == 2 && std::is_same<A, B>::value)) && (sizeof(R) == 4 || sizeof(R) == 8) &&
                  (sizeof(A) == 4 || sizeof(A) == 8)) {
        constexpr int V = 16 / (int)sizeof(R);
        if ((n == 2 || n == 3) && lean_vec == 1 && !force_scalar && !force_wide_indices() && (kp.inner % V) != 0 && kp.inner >= 64 &&
            plan.total < 0x7fffffffull && plan.total >= 16384) {
            const int64_t es = (int64_t)sizeof(A), rs = (int64_t)sizeof(R);
            bool fits = kp.istep[2] == rs && kp.ostep[2][n - 2] == rs * (int64_t)kp.inner && ((uintptr_t)kp.ptr[2] % 16) == 0;
            if (n == 3) fits = fits && kp.ostep[2][0] == rs * (int64_t)kp.inner * (int64_t)plan.shape[1];
            for (int o = 0; o + 1 < nops && fits; ++o) {
                const int sl = slot[o];
                fits = (kp.istep[sl] == es || kp.istep[sl] == 0) && ((uintptr_t)kp.ptr[sl] % (uintptr_t)es) == 0;
            }
            if (fits) {
                EwAddressed pa;
                std::memset(&pa, 0, sizeof(pa));
                for (int o = 0; o + 1 < nops; ++o) {
                    const int sl = slot[o];
                    pa.in[sl] = kp.ptr[sl];
                    pa.s_outer[sl] = kp.ostep[sl][n - 2];
                    pa.s_inner[sl] = kp.istep[sl];
                    pa.s_outermost[sl] = n == 3 ? kp.ostep[sl][0] : 0;
                }
                pa.out = kp.ptr[2];
                pa.n = (uint32_t)plan.total;
                pa.period = (uint32_t)kp.inner;
                pa.div = div31_make(pa.period);
                pa.mid = n == 3 ? (uint32_t)plan.shape[1] : 0u;
                pa.div_mid = div31_make(n == 3 ? (uint32_t)plan.shape[1] : 1u);
                const uint64_t blocks = ((uint64_t)pa.n + (uint64_t)kEwBlock * V - 1) / ((uint64_t)kEwBlock * V);
                if (blocks <= ew_grid_max()) {
                    const bool nt = stream_past_caches((uint64_t)pa.n * ((uint64_t)(nops - 1) * sizeof(A) + sizeof(R)));
                    const dim3 g((unsigned)blocks);
                    if (nt) hipLaunchKernelGGL((ew_flat_addressed_kernel<Op, V, true>), g, b, 0, stream, pa, use_scalar, flag, op, sv);
                    else hipLaunchKernelGGL((ew_flat_addressed_kernel<Op, V, false>), g, b, 0, stream, pa, use_scalar, flag, op, sv);
                    cumo_cuda_runtime_check_kernel_launch();
                    return;
                }
            }
        }
    }

    // Typed results through 128-bit accesses have two lean kernels: one access per
    // lane, one 4 KiB tile per block, 32-bit index arithmetic. Measured on 1 GiB
    // arrays against the general kernel below: 83% of peak against 70% (1R+1W),
    // 82% against 61% (2R+1W), 80% against 74% (matrix minus column vector).
    if (!Op::BIT_OUT && lean_vec > 1) {
        const int vec = lean_vec;
        // bytes the operation touches: an operand that repeats along a dimension
        // counts once along it
        uint64_t bytes = 0;
        for (int o = 0; o < nops; ++o) {
            const int sl = slot[o];
            uint64_t nb = sl == 0 ? sizeof(A) : (sl == 1 ? sizeof(B) : sizeof(R));
            for (int d = 0; d < n; ++d)
                if (plan.step[o][d] != 0) nb *= plan.shape[d];
            bytes += nb;
        }
        const bool nt = stream_past_caches(bytes);

        // every operand one contiguous run -- or one of two inputs an array of a single element (x - x.mean,
        // x / x.sum): the kernel reads it from memory and goes on as the scalar form does
        bool flat = n == 1;
        int one_element = -1;   // the slot of such an input
        for (int o = 0; o < nops && flat; ++o) {
            const int sl = slot[o];
            const int64_t es = sl == 0 ? (int64_t)sizeof(A) : (sl == 1 ? (int64_t)sizeof(B) : (int64_t)sizeof(R));
            if (Op::NIN == 2 && std::is_same<A, B>::value && std::is_same<typename Op::S, A>::value && use_scalar == 0 && sl != 2 &&
                plan.step[o][0] == 0 && one_element < 0 && ((uintptr_t)ops[o].ptr % sizeof(A)) == 0) {
                one_element = sl;
                continue;
            }
            flat = plan.step[o][0] == es;
        }
        const char* flat_px = kp.ptr[0];
        const char* flat_py = kp.ptr[1];
        int flat_scalar = use_scalar;
        if (flat && one_element >= 0) {
            flat_px = kp.ptr[1 - one_element];   // the array
            flat_py = kp.ptr[one_element];       // the element that stands for the scalar
            flat_scalar = (one_element == 1 ? 1 : 2) | 4;
        }
        // A result wider than the input (SFloat or Int32 -> DFloat): two elements per lane, so that a lane
        // stores one 128-bit vector and a wave one contiguous KiB, rather than two vectors 32 bytes apart
        // (SFloat [8192,4096] -> DFloat: 89.7 -> 62.4 us).
        const int fvec = (sizeof(R) > sizeof(A) && vec == 4) ? 2 : vec;
        const uint64_t per_block = (uint64_t)kEwBlock * fvec * ew_flat_vectors_per_lane<Op>::value;
        const uint64_t blocks = (kp.inner + per_block - 1) / per_block;
        if (flat && blocks <= ew_grid_max()) {
            // (an operator that fills tables: at most a dozen blocks per compute unit, which then take a tile after the other)
            const uint64_t looping = (uint64_t)ew_table_op_blocks();
            const dim3 g((unsigned)((op_fills_tables<Op>::value && blocks > looping) ? looping : blocks));
            if (fvec == 4) {
                if (nt) hipLaunchKernelGGL((ew_flat_kernel<Op, 4, true>), g, b, 0, stream, flat_px, flat_py, kp.ptr[2], kp.inner, flat_scalar, flag, op, sv);
                else hipLaunchKernelGGL((ew_flat_kernel<Op, 4, false>), g, b, 0, stream, flat_px, flat_py, kp.ptr[2], kp.inner, flat_scalar, flag, op, sv);
            } else {
                if (nt) hipLaunchKernelGGL((ew_flat_kernel<Op, 2, true>), g, b, 0, stream, flat_px, flat_py, kp.ptr[2], kp.inner, flat_scalar, flag, op, sv);
                else hipLaunchKernelGGL((ew_flat_kernel<Op, 2, false>), g, b, 0, stream, flat_px, flat_py, kp.ptr[2], kp.inner, flat_scalar, flag, op, sv);
            }
            cumo_cuda_runtime_check_kernel_launch();
            return;
        }

        // rows x inner, every operand contiguous or constant along inner
        // (or outer x mid x inner, which the planner leaves apart only when an operand repeats along one of the two)
        bool r2 = (n == 2 || n == 3) && (kp.inner % (uint64_t)vec) == 0 && kp.rows < 0xffffffffull && kp.inner / vec < 0xffffffffull;
        EwR2Params rp;
        std::memset(&rp, 0, sizeof(rp));
        if (n == 3) rp.mid = (uint32_t)plan.shape[1];
        for (int o = 0; o < nops && r2; ++o) {
            const int sl = slot[o];
            const int64_t es = sl == 0 ? (int64_t)sizeof(A) : (sl == 1 ? (int64_t)sizeof(B) : (int64_t)sizeof(R));
            const int64_t is = plan.step[o][n - 1];
            if (is == es) rp.walk[sl] = 1;
            else if (is == 0 && sl != 2) rp.walk[sl] = 0;
            else if (is == -es && sl != 2 && es >= 4) rp.walk[sl] = 2;
            else r2 = false;
            rp.ptr[sl] = const_cast<char*>(ops[o].ptr);
            rp.rstep[sl] = plan.step[o][n - 2];
            if (n == 3) rp.ostep[sl] = plan.step[o][0];
        }
        if (r2) {
            const uint64_t inner_vecs = kp.inner / vec;
            int txb = 0;
            while (txb < 8 && (1ull << txb) < inner_vecs) ++txb;
            const uint64_t ty = (uint64_t)kEwBlock >> txb;
            const uint64_t ctiles = (inner_vecs + (1ull << txb) - 1) >> txb;
            const uint64_t ntiles = ctiles * ((kp.rows + ty - 1) / ty);
            if (ntiles < 0xffffffffull) {
                rp.rows = (uint32_t)kp.rows;
                rp.inner_vecs = (uint32_t)inner_vecs;
                rp.col_tiles = (uint32_t)ctiles;
                rp.n_tiles = (uint32_t)ntiles;
                rp.tx_bits = txb;
                rp.use_scalar = use_scalar;
                rp.flag = flag;
                // non-temporal for what streams past once; an operand that repeats along the rows stays cached
                int ntm = 0;
                if (nt) {
                    ntm = 4;
                    if (Op::NIN >= 1 && rp.walk[0] && rp.rstep[0] != 0 && (n == 2 || rp.ostep[0] != 0)) ntm |= 1;
                    if (Op::NIN >= 2 && use_scalar == 0 && rp.walk[1] && rp.rstep[1] != 0 && (n == 2 || rp.ostep[1] != 0)) ntm |= 2;
                }
#define CUMO_R2_BY_MASK(V)                                            \
    do {                                                              \
        bool done = false;                                            \
        if constexpr (Op::NIN >= 2) {                                 \
            if (ntm == 7) { CUMO_R2_LAUNCH(V, 7); done = true; }      \
            else if (ntm == 6) { CUMO_R2_LAUNCH(V, 6); done = true; } \
        }                                                             \
        if (!done) {                                                  \
            if (ntm == 5) CUMO_R2_LAUNCH(V, 5);                       \
            else if (ntm == 4) CUMO_R2_LAUNCH(V, 4);                  \
            else CUMO_R2_LAUNCH(V, 0);                                \
        }                                                             \
    } while (0);
                // large two-dimensional arrays of a cheap function: the lean form, two rows per lane
                const uint64_t lean_tiles = ctiles * ((kp.rows + 2 * ty - 1) / (2 * ty));
                if constexpr (!heavy) if (n == 2 && nt && Op::NIN >= 1 && rp.walk[0] == 1 && rp.walk[1] != 2 && lean_tiles <= ew_grid_max() && ew_lean_rows_enabled()) {
                    EwR2LeanParams lp;
                    std::memset(&lp, 0, sizeof(lp));
                    for (int k = 0; k < 3; ++k) { lp.ptr[k] = rp.ptr[k]; lp.rstep[k] = rp.rstep[k]; }
                    lp.rows = rp.rows;
                    lp.inner_vecs = rp.inner_vecs;
                    lp.col_tiles = rp.col_tiles;
                    lp.col_div = div31_make(rp.col_tiles);
                    lp.tx_bits = txb;
                    lp.mode = use_scalar == 1 ? 3 : (use_scalar == 2 ? 4 : (!rp.walk[1] ? 2 : (rp.rstep[1] == 0 ? 1 : 0)));
                    lp.flag = flag;
                    const dim3 g((unsigned)lean_tiles);
#define CUMO_R2_LAUNCH(V, M) hipLaunchKernelGGL((ew_rows2_lean_kernel<Op, V, M>), g, b, 0, stream, lp, op, sv)
                    if (vec == 4) {
                        CUMO_R2_BY_MASK(4)
                    } else {
                        CUMO_R2_BY_MASK(2)
                    }
#undef CUMO_R2_LAUNCH
                    cumo_cuda_runtime_check_kernel_launch();
                    return;
                }
                // a function that costs many instructions per element keeps a capped
                // grid, so that a block's set-up is paid once for many tiles
                uint64_t grid = ntiles;
                if (grid > ew_grid_max()) grid = ew_grid_max();
                if (heavy && grid > ew_grid_cap()) grid = ew_grid_cap();
                const dim3 g((unsigned)grid);
#define CUMO_R2_LAUNCH(V, M) hipLaunchKernelGGL((ew_rows2_kernel<Op, V, M>), g, b, 0, stream, rp, op, sv)
                if (vec == 4) {
                    CUMO_R2_BY_MASK(4)
                } else {
                    CUMO_R2_BY_MASK(2)
                }
#undef CUMO_R2_BY_MASK
#undef CUMO_R2_LAUNCH
                cumo_cuda_runtime_check_kernel_launch();
                return;
            }
        }
    }

    // everything else: more dimensions, ragged or strided rows, Bit results
    const bool shift = Op::BIT_OUT && vec == 1;
    const uint64_t span = kp.inner + (shift ? 31 : 0);
    uint64_t lanes_needed = (span + vec - 1) / vec;
    int tx_bits = 0;
    while (tx_bits < 8 && (1ull << tx_bits) < lanes_needed) ++tx_bits;
    if (kp.rows == 1) tx_bits = 8;
    kp.tx_bits = tx_bits;
    const uint64_t tile_cols = (1ull << tx_bits) * vec * kEwUnroll;
    const uint64_t TY = (uint64_t)kEwBlock >> tx_bits;
    kp.col_tiles = (span + tile_cols - 1) / tile_cols;
    const uint64_t row_tiles = (kp.rows + TY - 1) / TY;
    kp.n_tiles = kp.col_tiles * row_tiles;
    kp.small_tiles = (kp.n_tiles < 0xffffffffull && !force_wide_indices()) ? 1 : 0;
    uint64_t grid = kp.n_tiles;
    if (grid > ew_grid_cap()) grid = ew_grid_cap();
    const dim3 g((unsigned)grid);
    switch (vec) {
    case 4:
        hipLaunchKernelGGL((ew_rows_kernel<Op, 4>), g, b, 0, stream, kp, op, sv);
        break;
    case 2:
        hipLaunchKernelGGL((ew_rows_kernel<Op, 2>), g, b, 0, stream, kp, op, sv);
        break;
    default:
        hipLaunchKernelGGL((ew_rows_kernel<Op, 1>), g, b, 0, stream, kp, op, sv);
        break;
    }
    cumo_cuda_runtime_check_kernel_launch();
}

}  // namespace cumo_hip

#endif
