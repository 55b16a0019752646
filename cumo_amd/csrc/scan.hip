// cumsum / cumprod: inclusive scans along one run of a view.
//
// Replaces narray/gen/tmpl/cum_kernel.cu of the reference, which hands each run
// to thrust::inclusive_scan (one call per run, walked on the host:
// narray/gen/tmpl/cum.c:12-46). The operators are the reference's
// (types/real_accum_kernel.h:12-26, xint_macro_kernel.h:46-47); the nan forms
// treat NaN as "nothing yet", which makes them associative like the plain ones.
// Like a sum, a parallel float scan does not add strictly left to right.
//
// The forms, by layout:
//   scan_rows_kernel        one block per run, tile after tile with the running value
//                           carried along: many runs (an axis of a matrix), or short ones;
//   scan_rows_whole_kernel  the same for contiguous runs of whole 256-vector chunks, held
//                           in registers wave by wave;
//   scan_chain_kernel       one long contiguous run in one pass: tiles hand their totals on
//                           through words in memory (read once, written once);
//   three launches          one long run that is strided or unaligned: per-tile totals, a
//                           scan of the totals, then every tile scans itself from its
//                           offset (reads the input twice);
//   scan_cols_chain_kernel  long runs that lie across memory (down the rows of a matrix) in
//                           one pass, tiles of 256 rows handing on their column totals;
//   scan_cols_kernel        other runs across memory, in segments and two passes.
// Inside a tile each lane owns 8 consecutive elements: it scans them in registers,
// the lane totals are scanned across the wave with shuffles and the four wave
// totals through LDS. Everything is in a fixed order, so results do not change
// from launch to launch.
#include "common.h"
#include "wait_ctl.h"

#include <cstdlib>
#include <cstring>
#include <mutex>

namespace cumo_hip {
namespace {

constexpr int kScanBlock = 256;
constexpr int kScanPer = 8;                         // elements per lane
constexpr int kScanTile = kScanBlock * kScanPer;    // 2048

template <class T> __device__ __forceinline__ bool scan_is_nan(T x) { return x != x; }
template <> __device__ __forceinline__ bool scan_is_nan<int32_t>(int32_t) { return false; }

template <class T> struct scan_is_int { static constexpr bool value = false; };
template <> struct scan_is_int<int32_t> { static constexpr bool value = true; };

// OP: 0 sum, 1 prod. NANF: NaN is skipped.
template <class T, int OP, bool NANF>
struct ScanOp {
    __device__ __forceinline__ static T apply(T a, T b) {
        if (NANF) {
            if (scan_is_nan(a)) return b;
            if (scan_is_nan(b)) return a;
        }
        if constexpr (scan_is_int<T>::value) {
            // Int32: wrapping arithmetic done in unsigned
            return OP == 0 ? (T)((uint32_t)a + (uint32_t)b) : (T)((uint32_t)a * (uint32_t)b);
        } else {
            return OP == 0 ? a + b : a * b;
        }
    }
};

template <class T>
__device__ __forceinline__ T scan_shfl_up(T v, unsigned d) {
    if constexpr (sizeof(T) == 8) {
        union { T t; uint32_t w[2]; } a, b;
        a.t = v;
        b.w[0] = __shfl_up(a.w[0], d);
        b.w[1] = __shfl_up(a.w[1], d);
        return b.t;
    } else {
        union { T t; uint32_t w; } a, b;
        a.t = v;
        b.w = __shfl_up(a.w, d);
        return b.t;
    }
}

// Inclusive scan of one tile held as v[kScanPer] per lane (element k of lane t is
// tile position t * kScanPer + k; cnt = how many positions of the tile exist).
// `carry` is the running value before the tile and has_carry says whether there is
// one. Returns the running value after the tile in every lane (has_carry becomes true
// when the tile is not empty).
template <class T, class Op, int NWAVES = kScanBlock / 64>
__device__ __forceinline__ void scan_tile(T (&v)[kScanPer], int cnt, T& carry, bool& has_carry) {
    __shared__ T wave_tot[NWAVES];
    __shared__ int wave_has[NWAVES];
    const int t = threadIdx.x;
    const int base = t * kScanPer;
    int mine = cnt - base;  // how many of this lane's elements exist
    mine = mine < 0 ? 0 : (mine > kScanPer ? kScanPer : mine);
    // lane-local inclusive scan
#pragma unroll
    for (int k = 1; k < kScanPer; ++k)
        if (k < mine) v[k] = Op::apply(v[k - 1], v[k]);
    T tot = mine > 0 ? v[mine - 1] : T();
    bool has = mine > 0;
    // inclusive scan of the lane totals across the wave
    const int lane = t & 63;
#pragma unroll
    for (unsigned d = 1; d < 64; d <<= 1) {
        const T o = scan_shfl_up(tot, d);
        const int oh = __shfl_up((int)has, d);
        if (lane >= (int)d && oh) {
            tot = has ? Op::apply(o, tot) : o;
            has = true;
        }
    }
    const int w = t >> 6;
    if (lane == 63) {
        wave_tot[w] = tot;
        wave_has[w] = has ? 1 : 0;
    }
    __syncthreads();
    // what precedes this lane: the carry, the earlier waves, the earlier lanes of its wave
    T pre = carry;
    bool pre_has = has_carry;
    for (int j = 0; j < w; ++j) {
        if (wave_has[j]) {
            pre = pre_has ? Op::apply(pre, wave_tot[j]) : wave_tot[j];
            pre_has = true;
        }
    }
    T run = carry;          // the running value after the whole tile, for every lane
    bool run_has = has_carry;
#pragma unroll
    for (int j = 0; j < NWAVES; ++j) {
        if (wave_has[j]) {
            run = run_has ? Op::apply(run, wave_tot[j]) : wave_tot[j];
            run_has = true;
        }
    }
    const T lane_excl = scan_shfl_up(tot, 1);
    const int lane_excl_has = __shfl_up((int)has, 1);
    if (lane > 0 && lane_excl_has) {
        pre = pre_has ? Op::apply(pre, lane_excl) : lane_excl;
        pre_has = true;
    }
    if (pre_has) {
#pragma unroll
        for (int k = 0; k < kScanPer; ++k)
            if (k < mine) v[k] = Op::apply(pre, v[k]);
    }
    __syncthreads();  // wave_tot is written again by the next tile
    carry = run;
    has_carry = run_has;
}

template <class T, bool NT = false>
__device__ __forceinline__ void scan_load(const char* p, int64_t s, uint64_t first, int cnt, T (&v)[kScanPer]) {
    const int base = threadIdx.x * kScanPer;
    if (s == (int64_t)sizeof(T) && base + kScanPer <= cnt && ((reinterpret_cast<uintptr_t>(p) + (first + base) * sizeof(T)) & 15) == 0) {
        typedef uint32_t u4 __attribute__((ext_vector_type(4)));
        constexpr int NV = (int)(kScanPer * sizeof(T) / 16);
        union { T t[kScanPer]; u4 q[NV]; } u;
        const u4* src = reinterpret_cast<const u4*>(p + (first + base) * sizeof(T));
#pragma unroll
        for (int i = 0; i < NV; ++i) u.q[i] = NT ? __builtin_nontemporal_load(src + i) : src[i];
#pragma unroll
        for (int k = 0; k < kScanPer; ++k) v[k] = u.t[k];
        return;
    }
#pragma unroll
    for (int k = 0; k < kScanPer; ++k)
        if (base + k < cnt) v[k] = *reinterpret_cast<const T*>(p + (int64_t)(first + base + k) * s);
}

template <class T, bool NT = false>
__device__ __forceinline__ void scan_store(char* p, int64_t s, uint64_t first, int cnt, const T (&v)[kScanPer]) {
    const int base = threadIdx.x * kScanPer;
    if (s == (int64_t)sizeof(T) && base + kScanPer <= cnt && ((reinterpret_cast<uintptr_t>(p) + (first + base) * sizeof(T)) & 15) == 0) {
        typedef uint32_t u4 __attribute__((ext_vector_type(4)));
        constexpr int NV = (int)(kScanPer * sizeof(T) / 16);
        union { T t[kScanPer]; u4 q[NV]; } u;
#pragma unroll
        for (int k = 0; k < kScanPer; ++k) u.t[k] = v[k];
        u4* dst = reinterpret_cast<u4*>(p + (first + base) * sizeof(T));
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            if (NT) __builtin_nontemporal_store(u.q[i], dst + i);
            else dst[i] = u.q[i];
        }
        return;
    }
#pragma unroll
    for (int k = 0; k < kScanPer; ++k)
        if (base + k < cnt) *reinterpret_cast<T*>(p + (int64_t)(first + base + k) * s) = v[k];
}

struct ScanRowsParams {
    int nouter;
    uint64_t rows, n;
    uint64_t oshape[CUMO_NA_MAX_DIMENSION];
    int64_t ostep_in[CUMO_NA_MAX_DIMENSION], ostep_out[CUMO_NA_MAX_DIMENSION];
    int64_t s_in, s_out;
    const char* in;
    char* out;
};

template <class T, class Op>
__global__ __launch_bounds__(kScanBlock) void scan_rows_kernel(ScanRowsParams p) {
    for (uint64_t row = blockIdx.x; row < p.rows; row += gridDim.x) {
        int64_t oi = 0, oo = 0;
        uint64_t r = row;
        for (int d = p.nouter - 1; d >= 0; --d) {
            const uint64_t m = p.oshape[d];
            const uint64_t q = r / m;
            const int64_t k = (int64_t)(r - q * m);
            r = q;
            oi += k * p.ostep_in[d];
            oo += k * p.ostep_out[d];
        }
        T carry = T();
        bool has_carry = false;
        for (uint64_t first = 0; first < p.n; first += kScanTile) {
            const uint64_t left = p.n - first;
            const int cnt = left < (uint64_t)kScanTile ? (int)left : kScanTile;
            T v[kScanPer];
            scan_load<T>(p.in + oi, p.s_in, first, cnt, v);
            scan_tile<T, Op>(v, cnt, carry, has_carry);
            scan_store<T>(p.out + oo, p.s_out, first, cnt, v);
        }
    }
}

template <class T>
__device__ __forceinline__ T scan_shfl_xor(T v, unsigned m) {
    if constexpr (sizeof(T) == 8) {
        union { T t; uint32_t w[2]; } a, b;
        a.t = v;
        b.w[0] = __shfl_xor(a.w[0], m);
        b.w[1] = __shfl_xor(a.w[1], m);
        return b.t;
    } else {
        union { T t; uint32_t w; } a, b;
        a.t = v;
        b.w = __shfl_xor(a.w, m);
        return b.t;
    }
}

// phase 1 of the three-launch form: the total of each tile, by a plain fold (the
// operators are associative and commutative: lane-local fold, wave butterfly, four LDS
// slots), which is lighter than the scan of the tile. A tile of nothing but NaN under a
// nan operator has the total NaN, which the operator reads as "nothing". The last tile
// may be partial; nothing comes after it, so its total is never used and none is formed.
template <class T, class Op>
__global__ __launch_bounds__(kScanBlock) void scan_tile_totals_kernel(const char* in, int64_t s_in, uint64_t n, T* totals) {
    __shared__ T wave_tot[kScanBlock / 64];
    const uint64_t first = (uint64_t)blockIdx.x * kScanTile;
    const uint64_t left = n - first;
    if (left < (uint64_t)kScanTile) {
        if (threadIdx.x == 0) totals[blockIdx.x] = T();
        return;
    }
    T v[kScanPer];
    scan_load<T>(in, s_in, first, kScanTile, v);
    T t = v[0];
#pragma unroll
    for (int k = 1; k < kScanPer; ++k) t = Op::apply(t, v[k]);
#pragma unroll
    for (unsigned m = 32; m > 0; m >>= 1) t = Op::apply(t, scan_shfl_xor(t, m));
    if ((threadIdx.x & 63) == 0) wave_tot[threadIdx.x >> 6] = t;
    __syncthreads();
    if (threadIdx.x == 0) {
        T tot = wave_tot[0];
#pragma unroll
        for (int w = 1; w < kScanBlock / 64; ++w) tot = Op::apply(tot, wave_tot[w]);
        totals[blockIdx.x] = tot;
    }
}

// phase 3: every block scans its tiles, starting from the scanned total of the blocks before it
template <class T, class Op>
__global__ __launch_bounds__(kScanBlock) void scan_apply_kernel(const char* in, int64_t s_in, char* out, int64_t s_out, uint64_t n, uint64_t per,
                                                                const T* scanned_totals) {
    bool hc = blockIdx.x > 0;
    T carry = hc ? scanned_totals[blockIdx.x - 1] : T();
    const uint64_t begin = (uint64_t)blockIdx.x * per * kScanTile;
    for (uint64_t k = 0; k < per; ++k) {
        const uint64_t first = begin + k * kScanTile;
        if (first >= n) break;
        const uint64_t left = n - first;
        const int cnt = left < (uint64_t)kScanTile ? (int)left : kScanTile;
        T v[kScanPer];
        scan_load<T>(in, s_in, first, cnt, v);
        scan_tile<T, Op>(v, cnt, carry, hc);
        scan_store<T>(out, s_out, first, cnt, v);
    }
}

// ---- one long run in one pass ----------------------------------------------------
// Every block takes the next tile from a ticket (so a tile only ever waits for tiles whose
// blocks are already running), scans it in registers, publishes the tile's total and then
// needs the total of everything before it. That comes in a fixed shape, so that results
// do not change from launch to launch: tiles form groups of 64 and groups form supergroups
// of 64; the last tile of a group also publishes the group's total and the last tile of a
// supergroup the supergroup's. A tile folds, each with one wave-wide butterfly, the totals
// of the earlier tiles of its group, of the earlier groups of its supergroup and of the
// earlier supergroups. Reads the input once and writes the output once.
// A published value travels as 64-bit words {the launch's number, 32 bits of the value},
// stored and loaded with agent-scope atomics: a word is there when its upper half is the
// launch's number, no fence needed. The words live in a region that the stream keeps from
// launch to launch (chain_words_acquire below), so nothing is cleared: what an earlier launch
// left carries another number, and the ticket word just counts on (a launch takes exactly one
// ticket per block; the host knows where it stood). A wait gives up after kChainSpinLimit polls
// (it cannot be reached while every tile before this one has a running block); it then counts
// that and raises the host's give-up word (wait_ctl.h), so the next point where the host waits
// for the device reports the launch as failed.
// The ticket is a relaxed add on purpose: it hands out tile numbers and publishes nothing; what
// a tile publishes travels whole in its tagged words.
constexpr uint32_t kChainSpinLimit = 1u << 22;
constexpr uint64_t kChainMaxTiles = 64ull * 64ull * 64ull;

template <class T>
struct ScanChain {
    static constexpr int W = (int)(sizeof(T) / 4);
    static constexpr int SUB = 64 / (int)sizeof(T) / 2;        // sub-tiles of the block-wide scan per tile: 64 KiB of elements
    static constexpr int TILE = kScanTile * SUB;
    WaitCtl* wait;     // where a look-back that gives up reports it
    uint32_t* ticket;
    uint64_t* tile;    // [n_tiles * W]
    uint64_t* group;   // [n_groups * W]
    uint64_t* super;   // [n_supers * W]
    uint32_t flag;         // the upper half of a word of this launch
    uint32_t ticket_base;  // what the ticket word held before this launch
};

template <class T>
__device__ __forceinline__ void chain_publish(uint64_t* slot, T value, uint32_t flag) {
    constexpr int W = ScanChain<T>::W;
    union { T t; uint32_t w[W]; } u;
    u.t = value;
#pragma unroll
    for (int i = 0; i < W; ++i)
        __hip_atomic_store(slot + i, ((uint64_t)flag << 32) | u.w[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// one look at a published value: true when all of it is there
template <class T>
__device__ __forceinline__ bool chain_peek(const uint64_t* slot, T& value, uint32_t flag) {
    constexpr int W = ScanChain<T>::W;
    union { T t; uint32_t w[W]; } u;
    uint64_t x[W];
#pragma unroll
    for (int i = 0; i < W; ++i) x[i] = __hip_atomic_load(slot + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    bool all = true;
#pragma unroll
    for (int i = 0; i < W; ++i) {
        all = all && (uint32_t)(x[i] >> 32) == flag;
        u.w[i] = (uint32_t)x[i];
    }
    value = u.t;
    return all;
}

// (x, has) of the 64 lanes folded in a fixed shape; every lane ends with the result
template <class T, class Op>
__device__ __forceinline__ void chain_wave_fold(T& x, bool& has) {
    const unsigned lane = threadIdx.x & 63u;
#pragma unroll
    for (unsigned m = 1; m < 64; m <<= 1) {
        const T o = scan_shfl_xor(x, m);
        const bool oh = __shfl_xor((int)has, (int)m) != 0;
        if (oh) {
            if (!has) x = o;
            else x = (lane & m) ? Op::apply(o, x) : Op::apply(x, o);
            has = true;
        }
    }
}

template <class T, class Op>
__device__ __forceinline__ void chain_join(T& a, bool& a_has, T b, bool b_has) {  // a = a (+) b, a the earlier
    if (b_has) {
        a = a_has ? Op::apply(a, b) : b;
        a_has = true;
    }
}

template <class T>
__device__ __forceinline__ T scan_shfl_idx(T v, int src) {
    if constexpr (sizeof(T) == 8) {
        union { T t; uint32_t w[2]; } a, b;
        a.t = v;
        b.w[0] = __shfl(a.w[0], src);
        b.w[1] = __shfl(a.w[1], src);
        return b.t;
    } else {
        union { T t; uint32_t w; } a, b;
        a.t = v;
        b.w = __shfl(a.w, src);
        return b.t;
    }
}

// What a tile needs from the tiles before it, through the published totals (wave 0 of the
// block; every lane returns the same). Lane l wants the l-th earlier tile of this group, the
// l-th earlier group of this supergroup and the l-th supergroup. Whatever this tile waits
// for, the tile just before it publishes last, so one lane first polls that one word, with
// pauses (64 lanes of every running block polling would flood the memory system); then every
// lane looks at its own words, all in flight together, until they are there.
template <class T, class Op>
__device__ __forceinline__ void chain_look_back(const ScanChain<T>& c, uint32_t t, T total, bool total_has, T& prefix, bool& prefix_has) {
    constexpr int W = ScanChain<T>::W;
    const unsigned lane = threadIdx.x & 63u;
    const uint32_t pos = t & 63u, g = t >> 6, gpos = g & 63u, sg = g >> 6;
    if (lane == 0) chain_publish<T>(c.tile + (size_t)t * W, total, c.flag);
    T x = T(), y = T(), z = T();
    const bool has_x = lane < pos, has_y = lane < gpos, has_z = lane < sg;
    bool need_x = has_x, need_y = has_y, need_z = has_z;
    const uint64_t* px = c.tile + (size_t)(g * 64u + lane) * W;
    const uint64_t* py = c.group + (size_t)(sg * 64u + lane) * W;
    const uint64_t* pz = c.super + (size_t)lane * W;
    uint32_t polls = 0;
    const uint32_t spin_limit = wait_limit(c.wait, kChainSpinLimit);
    if (t > 0) {
        // the last word that the tile before this one publishes
        const uint64_t* latest = pos > 0 ? c.tile + (size_t)(t - 1) * W + (W - 1)
                                         : (gpos > 0 ? c.group + (size_t)(g - 1) * W + (W - 1) : c.super + (size_t)(sg - 1) * W + (W - 1));
        if (lane == 0) {
            // (running out of looks here is not yet a failure: the loop below looks again and reports)
            while ((uint32_t)(__hip_atomic_load(latest, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >> 32) != c.flag) {
                if (++polls > spin_limit) break;
                __builtin_amdgcn_s_sleep(16);
            }
        }
    }
    // A tile that closes its group publishes the group's total as soon as the group's tiles
    // are in, before it has everything it needs itself (and likewise the supergroup's):
    // otherwise every group would wait for the group before it, one memory round trip each.
    const bool closes_group = pos == 63u, closes_super = closes_group && gpos == 63u;
    bool group_out = !closes_group, super_out = !closes_super;
    bool xh = has_x, yh = has_y, zh = has_z;
    bool x_folded = false, y_folded = false;
    T gt = T();
    bool gt_has = false;
    for (;;) {
        if (need_x) need_x = !chain_peek<T>(px, x, c.flag);
        if (need_y) need_y = !chain_peek<T>(py, y, c.flag);
        if (need_z) need_z = !chain_peek<T>(pz, z, c.flag);
        if (!x_folded && __ballot(need_x) == 0) {
            chain_wave_fold<T, Op>(x, xh);
            x_folded = true;
            if (!group_out) {
                gt = x;
                gt_has = xh;
                chain_join<T, Op>(gt, gt_has, total, total_has);
                if (lane == 0) chain_publish<T>(c.group + (size_t)g * W, gt, c.flag);
                group_out = true;
            }
        }
        if (!y_folded && x_folded && __ballot(need_y) == 0) {
            chain_wave_fold<T, Op>(y, yh);
            y_folded = true;
            if (!super_out) {
                T st = y;
                bool st_has = yh;
                chain_join<T, Op>(st, st_has, gt, gt_has);
                if (lane == 0) chain_publish<T>(c.super + (size_t)sg * W, st, c.flag);
                super_out = true;
            }
        }
        if (__ballot(need_x || need_y || need_z) == 0) break;
        if (++polls > spin_limit) {
            if (lane == 0) wait_gave_up(c.wait, WAIT_SCAN);
            break;
        }
        __builtin_amdgcn_s_sleep(16);
    }
    if (!x_folded) chain_wave_fold<T, Op>(x, xh);  // (only after giving up)
    if (!y_folded) chain_wave_fold<T, Op>(y, yh);
    chain_wave_fold<T, Op>(z, zh);
    chain_join<T, Op>(z, zh, y, yh);
    chain_join<T, Op>(z, zh, x, xh);
    prefix = z;
    prefix_has = zh;
}

// Both sides are contiguous and 16-byte aligned. A whole tile goes wave by wave: a wave owns a
// quarter of the tile as R rows of 64 vectors, lane l holding vector l of every row (each load
// and store covers 1 KiB without gaps); the rows are scanned side by side with shuffles, the
// four waves meet once, in LDS, and what is left to add after the look-back is one value per
// wave, so only the tile's elements stay in registers while the block waits. The ragged last
// tile of a run goes sub-tile by sub-tile through the block-wide scan, reading its input twice.
// Measured on 2^26 SFloat (fresh operands): 116 us with 64 KiB tiles, against 139 us with
// 32 KiB tiles (twice the tickets and look-backs, each a trip through memory with nothing else
// for the block to do), 155 us for the three launches, and 92 us for the same kernel with
// neither ticket nor look-back. Blocks that keep a second tile's loads in flight while they
// wait were slower still (170 us): the registers that takes cost more blocks than it wins.
template <class T>
struct ChainVec {
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    static constexpr int V = 16 / (int)sizeof(T);
    union { u4 q; T e[V]; };
};

struct ChainShared {
    uint32_t tile;
    int prefix_has;
};

// RAGGED: only the first nelem elements from `first` on exist; the others read as zeros (they lie
// after everything that exists, so what they add to never reaches an element that is stored).
// The one vector that is partly there goes element by element: nothing is read past the run.
template <class T, bool NT, int R, bool RAGGED = false>
__device__ __forceinline__ void chain_issue_loads(const char* in, uint64_t first, ChainVec<T> (&v)[R], uint32_t nelem = 0) {
    typedef typename ChainVec<T>::u4 u4;
    constexpr int V = ChainVec<T>::V;
    const unsigned lane = threadIdx.x & 63u;
    const int w = threadIdx.x >> 6;
    const u4* src = reinterpret_cast<const u4*>(in + (first + (uint64_t)w * (R * 64 * V)) * sizeof(T)) + lane;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (RAGGED) {
            const u4 zero = {0u, 0u, 0u, 0u};
            v[r].q = zero;
            const uint32_t e0 = ((uint32_t)(w * R * 64 + r * 64) + lane) * V;
            if (e0 + V <= nelem) {
                v[r].q = NT ? __builtin_nontemporal_load(src + r * 64) : src[r * 64];
            } else if (e0 < nelem) {
                const T* s1 = reinterpret_cast<const T*>(src + r * 64);
#pragma unroll
                for (int e = 0; e < V; ++e)
                    if (e0 + e < nelem) v[r].e[e] = s1[e];
            }
        } else {
            v[r].q = NT ? __builtin_nontemporal_load(src + r * 64) : src[r * 64];
        }
    }
}

// The tile in v (already loaded) scanned by itself: afterwards every element holds the running
// value from the start of its wave's quarter, `total` is the tile's total and `wave_pre` the
// total of the waves before this one (for wave 0: nothing). One barrier, met by every thread.
template <class T, class Op, int R, int NW = kScanBlock / 64>
__device__ __forceinline__ void chain_scan_tile(ChainVec<T> (&v)[R], T* s_wave_tot, T& total, T& wave_pre) {
    constexpr int V = ChainVec<T>::V;
    const unsigned lane = threadIdx.x & 63u;
    const int w = threadIdx.x >> 6;
    T inc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
#pragma unroll
        for (int e = 1; e < V; ++e) v[r].e[e] = Op::apply(v[r].e[e - 1], v[r].e[e]);
        inc[r] = v[r].e[V - 1];
    }
    // the lane totals of each row, scanned across the wave (the rows are independent)
#pragma unroll
    for (unsigned d = 1; d < 64; d <<= 1) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const T o = scan_shfl_up(inc[r], d);
            if (lane >= d) inc[r] = Op::apply(o, inc[r]);
        }
    }
    // every element takes on what precedes its vector inside the wave's quarter
    T run = T();  // the rows so far
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const T ex = scan_shfl_up(inc[r], 1);       // the lanes before, in this row
        const T row = scan_shfl_idx(inc[r], 63);    // the whole row
        T before = ex;
        if (r > 0) before = lane > 0 ? Op::apply(run, ex) : run;
        if (r > 0 || lane > 0) {
#pragma unroll
            for (int e = 0; e < V; ++e) v[r].e[e] = Op::apply(before, v[r].e[e]);
        }
        run = r == 0 ? row : Op::apply(run, row);
    }
    if (lane == 0) s_wave_tot[w] = run;
    __syncthreads();
    total = s_wave_tot[0];
    wave_pre = T();
#pragma unroll
    for (int j = 1; j < NW; ++j) {
        if (j == w) wave_pre = total;
        total = Op::apply(total, s_wave_tot[j]);
    }
}

// adds what precedes the tile (if anything) and the earlier waves' total, and stores
template <class T, class Op, bool NT, int R, bool RAGGED = false>
__device__ __forceinline__ void chain_store_tile(char* out, uint64_t first, ChainVec<T> (&v)[R], T head, bool head_has, T wave_pre, uint32_t nelem = 0) {
    typedef typename ChainVec<T>::u4 u4;
    constexpr int V = ChainVec<T>::V;
    const unsigned lane = threadIdx.x & 63u;
    const int w = threadIdx.x >> 6;
    if (w > 0) {
        head = head_has ? Op::apply(head, wave_pre) : wave_pre;
        head_has = true;
    }
    u4* dst = reinterpret_cast<u4*>(out + (first + (uint64_t)w * (R * 64 * V)) * sizeof(T)) + lane;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (head_has) {
#pragma unroll
            for (int e = 0; e < V; ++e) v[r].e[e] = Op::apply(head, v[r].e[e]);
        }
        if (RAGGED) {
            const uint32_t e0 = ((uint32_t)(w * R * 64 + r * 64) + lane) * V;
            if (e0 >= nelem) continue;
            if (e0 + V > nelem) {
                T* d1 = reinterpret_cast<T*>(dst + r * 64);
#pragma unroll
                for (int e = 0; e < V; ++e)
                    if (e0 + e < nelem) d1[e] = v[r].e[e];
                continue;
            }
        }
        if (NT) __builtin_nontemporal_store(v[r].q, dst + r * 64);
        else dst[r * 64] = v[r].q;
    }
}

// scans the tile in v (already loaded), looks back, stores; the barriers inside are met by every thread
template <class T, class Op, bool NT, int R, int NW>
__device__ __forceinline__ void chain_finish_tile(char* out, uint64_t first, uint32_t t, ChainVec<T> (&v)[R], const ScanChain<T>& c,
                                                  T* s_wave_tot, T* s_prefix, ChainShared* sh) {
    T total, wave_pre;
    chain_scan_tile<T, Op, R, NW>(v, s_wave_tot, total, wave_pre);
    if (threadIdx.x < 64) {
        T pre;
        bool pre_has;
        chain_look_back<T, Op>(c, t, total, true, pre, pre_has);
        if (threadIdx.x == 0) {
            *s_prefix = pre;
            sh->prefix_has = pre_has ? 1 : 0;
        }
    }
    __syncthreads();
    chain_store_tile<T, Op, NT, R>(out, first, v, *s_prefix, sh->prefix_has != 0, wave_pre);
}

// Many runs, each contiguous on both sides (64 vectors at least, aligned as their elements are):
// one block per run, chunk after chunk of R * 256 vectors in the same wave-by-wave form,
// the running value handed on in a register; the last chunk may be partly there.
template <class T, class Op, bool NT, int R>
__global__ __launch_bounds__(kScanBlock) void scan_rows_whole_kernel(ScanRowsParams p) {
    constexpr int V = ChainVec<T>::V;
    constexpr uint64_t CHUNK = (uint64_t)R * kScanBlock * V;
    __shared__ T s_wave_tot[kScanBlock / 64];
    for (uint64_t row = blockIdx.x; row < p.rows; row += gridDim.x) {
        int64_t oi = 0, oo = 0;
        uint64_t q = row;
        for (int d = p.nouter - 1; d >= 0; --d) {
            const uint64_t m = p.oshape[d];
            const uint64_t qq = q / m;
            const int64_t k = (int64_t)(q - qq * m);
            q = qq;
            oi += k * p.ostep_in[d];
            oo += k * p.ostep_out[d];
        }
        T carry = T();
        bool has_carry = false;
        for (uint64_t first = 0; first < p.n; first += CHUNK) {
            ChainVec<T> v[R];
            T total, wave_pre;
            if (p.n - first >= CHUNK) {
                chain_issue_loads<T, NT, R>(p.in + oi, first, v);
                chain_scan_tile<T, Op, R>(v, s_wave_tot, total, wave_pre);
                chain_store_tile<T, Op, NT, R>(p.out + oo, first, v, carry, has_carry, wave_pre);
            } else {
                // the run's last chunk, partly there
                const uint32_t nelem = (uint32_t)(p.n - first);
                chain_issue_loads<T, NT, R, true>(p.in + oi, first, v, nelem);
                chain_scan_tile<T, Op, R>(v, s_wave_tot, total, wave_pre);
                chain_store_tile<T, Op, NT, R, true>(p.out + oo, first, v, carry, has_carry, wave_pre, nelem);
            }
            carry = has_carry ? Op::apply(carry, total) : total;
            has_carry = true;
            __syncthreads();  // s_wave_tot is written again by the next chunk
        }
    }
}

template <class T, class Op, bool NT, int NW>
__global__ __launch_bounds__(NW * 64, sizeof(T) == 8 ? 3 : 4) void scan_chain_kernel(const char* in, char* out, uint64_t n, ScanChain<T> c) {
    constexpr int V = ChainVec<T>::V;
    constexpr int R = ScanChain<T>::TILE / (kScanBlock * V);   // rows of 64 vectors per wave
    constexpr int TILE = NW * R * 64 * V;
    constexpr int PIECE = NW * 64 * kScanPer;                  // what the block-wide scan takes at a time
    __shared__ ChainShared sh;
    __shared__ T s_prefix;
    __shared__ T s_wave_tot[NW];
    if (threadIdx.x == 0) sh.tile = __hip_atomic_fetch_add(c.ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - c.ticket_base;
    __syncthreads();
    const uint32_t t = sh.tile;
    const uint64_t first = (uint64_t)t * TILE;
    if (first >= n) return;  // (the grid is exactly the tiles; a stray ticket does nothing)
    if (n - first >= (uint64_t)TILE) {
        ChainVec<T> v[R];
        chain_issue_loads<T, NT, R>(in, first, v);
        chain_finish_tile<T, Op, NT, R, NW>(out, first, t, v, c, s_wave_tot, &s_prefix, &sh);
        return;
    }
    // the ragged last tile: its total first, then the scan from what the look-back gives
    T total = T();
    bool total_has = false;
#pragma clang loop unroll(disable)
    for (uint64_t f = first; f < n; f += PIECE) {
        const uint64_t left = n - f;
        const int cnt = left < (uint64_t)PIECE ? (int)left : PIECE;
        T v[kScanPer];
        scan_load<T>(in, (int64_t)sizeof(T), f, cnt, v);
        scan_tile<T, Op, NW>(v, cnt, total, total_has);
    }
    if (threadIdx.x < 64) {
        T pre;
        bool pre_has;
        chain_look_back<T, Op>(c, t, total, total_has, pre, pre_has);
        if (threadIdx.x == 0) {
            s_prefix = pre;
            sh.prefix_has = pre_has ? 1 : 0;
        }
    }
    __syncthreads();
    T carry = s_prefix;
    bool has_carry = sh.prefix_has != 0;
#pragma clang loop unroll(disable)
    for (uint64_t f = first; f < n; f += PIECE) {
        const uint64_t left = n - f;
        const int cnt = left < (uint64_t)PIECE ? (int)left : PIECE;
        T v[kScanPer];
        scan_load<T>(in, (int64_t)sizeof(T), f, cnt, v);
        scan_tile<T, Op, NW>(v, cnt, carry, has_carry);
        scan_store<T>(out, (int64_t)sizeof(T), f, cnt, v);
    }
}

__global__ __launch_bounds__(256) void scan_chain_clear_kernel(uint64_t* words, uint64_t n) {
    for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256) words[i] = 0;
}

// The words of one launch: the ticket word first, the published totals from word kChainHead on.
// A stream that is not being captured keeps a region of its own (per device and stream slot,
// allocated from the driver at first use, grown when a launch needs more, never cleared after
// that): launches on it are numbered, and a launch's words carry its number. Under capture (a
// replay would repeat the number), without a slot, or beyond kChainKeptWords the words come from
// the pool and a small kernel clears them first; the number is 1 then.
constexpr uint64_t kChainHead = 32;
constexpr uint64_t kChainKeptWords = 8ull << 20;  // 64 MiB
constexpr int kChainDevices = 16;
struct ChainRegion {
    uint64_t* ptr;
    uint64_t cap;
    uint32_t launch, ticket;
};
ChainRegion g_chain_region[kChainDevices][kStreamSlots];
std::mutex g_chain_lock;

struct ChainWords {
    uint64_t* ws;
    uint32_t flag, ticket_base;
    bool pooled;
};

// CUMO_HIP_SCAN_KEEP_WORDS=0 (read once): always the pool and the clearing kernel
static bool chain_keep_enabled() {
    static const bool on = [] {
        const char* e = std::getenv("CUMO_HIP_SCAN_KEEP_WORDS");
        return !(e && e[0] == '0');
    }();
    return on;
}

// words counts the head; tickets = blocks of the launch. False: no memory (the error is set).
static bool chain_words_acquire(hipStream_t stream, uint64_t words, uint32_t tickets, ChainWords* w) {
    w->flag = 1;
    w->ticket_base = 0;
    w->pooled = true;
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capturing) != hipSuccess) {
        (void)hipGetLastError();
        capturing = hipStreamCaptureStatusActive;
    }
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        dev = -1;
    }
    const int slot = stream_slot(stream);
    if (chain_keep_enabled() && capturing == hipStreamCaptureStatusNone && slot >= 0 && dev >= 0 && dev < kChainDevices && words <= kChainKeptWords) {
        // held until chain_words_release, that is across the launch itself: launches that share a
        // stream must reach it in the order of their numbers and tickets
        g_chain_lock.lock();
        ChainRegion& r = g_chain_region[dev][slot];
        bool ok = true;
        if (r.cap < words) {
            if (r.ptr) {
                // only this stream's launches use the region
                ok = hipStreamSynchronize(stream) == hipSuccess && hipFree(r.ptr) == hipSuccess;
                r.ptr = nullptr;
                r.cap = 0;
            }
            uint64_t cap = 1ull << 16;
            while (cap < words) cap <<= 1;
            void* p = nullptr;
            if (ok && hipMalloc(&p, cap * sizeof(uint64_t)) == hipSuccess) {
                if (hipMemsetAsync(p, 0, cap * sizeof(uint64_t), stream) == hipSuccess) {
                    r.ptr = static_cast<uint64_t*>(p);
                    r.cap = cap;
                    r.launch = 0;
                    r.ticket = 0;
                } else {
                    (void)hipFree(p);
                    ok = false;
                }
            } else {
                ok = false;
            }
            if (!ok) (void)hipGetLastError();
        }
        if (ok && r.launch == 0xffffffffu) {
            // every number has been used once: start over from cleared words
            ok = hipMemsetAsync(r.ptr, 0, r.cap * sizeof(uint64_t), stream) == hipSuccess;
            r.launch = 0;
            r.ticket = 0;
            if (!ok) (void)hipGetLastError();
        }
        if (ok) {
            r.launch += 1;
            w->ws = r.ptr;
            w->flag = r.launch;
            w->ticket_base = r.ticket;
            r.ticket += tickets;
            w->pooled = false;
            return true;
        }
        g_chain_lock.unlock();
    }
    w->ws = reinterpret_cast<uint64_t*>(cumo_cuda_runtime_malloc(words * sizeof(uint64_t)));
    if (!w->ws) return false;
    uint64_t clear_grid = (words + 255) / 256;
    if (clear_grid > 2048) clear_grid = 2048;
    hipLaunchKernelGGL(scan_chain_clear_kernel, dim3((unsigned)clear_grid), dim3(256), 0, stream, w->ws, words);
    return true;
}

// after the launch that uses the words has been issued
static void chain_words_release(const ChainWords& w) {
    // stream-ordered reuse: whoever gets the block next can only touch it from later work on this stream
    if (w.pooled) cumo_cuda_runtime_free(reinterpret_cast<char*>(w.ws));
    else g_chain_lock.unlock();
}

// returns hipSuccess, or an error; -1 when the run does not suit this form
template <class T, class Op>
int scan_chain_launch(const char* p1, char* p2, ssize_t s1, ssize_t s2, uint64_t n, hipStream_t stream) {
    constexpr int W = ScanChain<T>::W;
    // Blocks of eight waves and 128 KiB tiles for four-byte elements wherever that leaves 64 tiles (half the
    // tickets and look-backs per byte: 2^26 SFloat 115 -> 111 us, 2^24 39 -> 33 us), else blocks of four waves
    // and 64 KiB tiles; eight-byte elements always those (their kernel needs 168 registers, and one block of
    // eight waves would have a compute unit to itself: 2^26 DFloat 224 us against 260 us).
    // CUMO_HIP_SCAN_CHAIN_WAVES=4 or 8, read once, fixes the choice.
    static const int forced_waves = [] {
        const char* e = std::getenv("CUMO_HIP_SCAN_CHAIN_WAVES");
        return e ? std::atoi(e) : 0;
    }();
    const uint64_t wide_tile = 2ull * ScanChain<T>::TILE;
    const bool wide = forced_waves == 8 || (forced_waves != 4 && sizeof(T) == 4 && (n + wide_tile - 1) / wide_tile >= 64);
    const uint64_t tile = wide ? wide_tile : (uint64_t)ScanChain<T>::TILE;
    const uint64_t n_tiles = (n + tile - 1) / tile;
    if (n_tiles < 64 || n_tiles > kChainMaxTiles) return -1;
    if (s1 != (ssize_t)sizeof(T) || s2 != (ssize_t)sizeof(T) || (((uintptr_t)p1 | (uintptr_t)p2) & 15) != 0) return -1;
    const uint64_t n_groups = (n_tiles + 63) / 64, n_supers = (n_groups + 63) / 64;
    const uint64_t words = kChainHead + (n_tiles + n_groups + n_supers) * W;
    WaitCtl* wait = wait_ctl();
    if (wait == nullptr) return -1;  // nowhere to report a wait that gives up: the form without waits
    ChainWords cw;
    if (!chain_words_acquire(stream, words, (uint32_t)n_tiles, &cw)) return (int)hipErrorOutOfMemory;
    ScanChain<T> c;
    c.wait = wait;
    c.ticket = reinterpret_cast<uint32_t*>(cw.ws);
    c.tile = cw.ws + kChainHead;
    c.group = c.tile + n_tiles * W;
    c.super = c.group + n_groups * W;
    c.flag = cw.flag;
    c.ticket_base = cw.ticket_base;
    const bool nt = stream_past_caches(2 * n * sizeof(T));
    const uint64_t grid = n_tiles;
    if (wide) {
        if (nt) hipLaunchKernelGGL((scan_chain_kernel<T, Op, true, 8>), dim3((unsigned)grid), dim3(8 * 64), 0, stream, p1, p2, n, c);
        else hipLaunchKernelGGL((scan_chain_kernel<T, Op, false, 8>), dim3((unsigned)grid), dim3(8 * 64), 0, stream, p1, p2, n, c);
    } else {
        if (nt) hipLaunchKernelGGL((scan_chain_kernel<T, Op, true, 4>), dim3((unsigned)grid), dim3(kScanBlock), 0, stream, p1, p2, n, c);
        else hipLaunchKernelGGL((scan_chain_kernel<T, Op, false, 4>), dim3((unsigned)grid), dim3(kScanBlock), 0, stream, p1, p2, n, c);
    }
    const int st = (int)hipGetLastError();
    chain_words_release(cw);
    return st;
}

// ---- runs that lie across memory (the scan goes down the rows of a matrix) ------
// Lanes sit along the dimension that is contiguous in memory and each lane walks
// its VEC columns down the run, so every load is coalesced across the wave. A run
// is cut into segments to fill the device: phase 0 leaves each segment's total per
// column and phase 2 scans each segment from what the segments before it add up to:
// with up to 32 segments it folds their totals itself, with more the totals are first
// turned into running totals by a column scan of their own (they form a small matrix).
// With enough columns there is one segment and only phase 2 runs (one read, one write).
struct ScanColsParams {
    int nouter;               // dimensions outside the run and the column dimension
    uint64_t planes, cols, n; // planes = product of those dimensions
    uint64_t oshape[CUMO_NA_MAX_DIMENSION];
    int64_t ostep_in[CUMO_NA_MAX_DIMENSION], ostep_out[CUMO_NA_MAX_DIMENSION];
    int64_t s_in, s_out;      // byte step along the run
    uint64_t seg_len, n_seg;
    int tx_bits;              // 2^tx_bits lanes along the columns, the rest of the block along segments
    const char* in;
    char* out;
};

template <class T, int VEC, bool NT = false>
__device__ __forceinline__ void scan_cols_load(const char* p, T (&v)[VEC]) {
    if constexpr (VEC * sizeof(T) == 16) {
        typedef uint32_t u4 __attribute__((ext_vector_type(4)));
        union { u4 q; T t[VEC]; } u;
        u.q = NT ? __builtin_nontemporal_load(reinterpret_cast<const u4*>(p)) : *reinterpret_cast<const u4*>(p);
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = u.t[j];
    } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = reinterpret_cast<const T*>(p)[j];
    }
}
template <class T, int VEC, bool NT = false>
__device__ __forceinline__ void scan_cols_store(char* p, const T (&v)[VEC]) {
    if constexpr (VEC * sizeof(T) == 16) {
        typedef uint32_t u4 __attribute__((ext_vector_type(4)));
        union { u4 q; T t[VEC]; } u;
#pragma unroll
        for (int j = 0; j < VEC; ++j) u.t[j] = v[j];
        if (NT) __builtin_nontemporal_store(u.q, reinterpret_cast<u4*>(p));
        else *reinterpret_cast<u4*>(p) = u.q;
    } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) reinterpret_cast<T*>(p)[j] = v[j];
    }
}

// PHASE 0: totals[(plane * n_seg + seg) * cols + col] = total of the segment.
// PHASE 2: scan the segment, starting from what the segments before it add up to:
//   LOOKBACK false  totals holds running totals already: one load of totals[.. seg - 1 ..]
//   LOOKBACK true   totals holds each segment's own total: they are folded here, in
//                   segment order (few segments: cheaper than a launch that does it)
template <class T, class Op, int VEC, int PHASE, bool LOOKBACK, bool NT>
__global__ __launch_bounds__(kScanBlock) void scan_cols_kernel(ScanColsParams p, T* totals) {
    constexpr int UNR = 4;  // four rows in flight per lane (more open more rows at once in memory and measured slower)
    const unsigned TX = 1u << p.tx_bits, TY = (unsigned)kScanBlock >> p.tx_bits;
    const unsigned tx = threadIdx.x & (TX - 1), ty = threadIdx.x >> p.tx_bits;
    const uint64_t col_groups = p.cols / VEC;
    const uint64_t strips = (col_groups + TX - 1) / TX;
    const uint64_t seg_blocks = (p.n_seg + TY - 1) / TY;
    const uint64_t n_blocks = strips * seg_blocks * p.planes;
    for (uint64_t b = blockIdx.x; b < n_blocks; b += gridDim.x) {
        const uint64_t strip = b % strips;
        const uint64_t sb = (b / strips) % seg_blocks;
        const uint64_t plane = b / (strips * seg_blocks);
        const uint64_t cg = strip * TX + tx;
        const uint64_t seg = sb * TY + ty;
        if (cg >= col_groups || seg >= p.n_seg) continue;
        int64_t oi = 0, oo = 0;
        uint64_t r = plane;
        for (int d = p.nouter - 1; d >= 0; --d) {
            const uint64_t m = p.oshape[d];
            const uint64_t q = r / m;
            const int64_t k = (int64_t)(r - q * m);
            r = q;
            oi += k * p.ostep_in[d];
            oo += k * p.ostep_out[d];
        }
        const uint64_t col = cg * VEC;
        const uint64_t begin = seg * p.seg_len;
        uint64_t end = begin + p.seg_len;
        if (end > p.n) end = p.n;
        const char* src = p.in + oi + (int64_t)col * (int64_t)sizeof(T);
        char* dst = p.out + oo + (int64_t)col * (int64_t)sizeof(T);
        T acc[VEC];
        bool has = false;
        if (PHASE == 2 && seg > 0) {
            if (LOOKBACK) {
                const T* t = totals + plane * p.n_seg * p.cols + col;
                scan_cols_load<T, VEC>(reinterpret_cast<const char*>(t), acc);
#pragma unroll 4
                for (uint64_t q = 1; q < seg; ++q) {
                    T v[VEC];
                    scan_cols_load<T, VEC>(reinterpret_cast<const char*>(t + q * p.cols), v);
#pragma unroll
                    for (int j = 0; j < VEC; ++j) acc[j] = Op::apply(acc[j], v[j]);
                }
            } else {
                scan_cols_load<T, VEC>(reinterpret_cast<const char*>(totals + (plane * p.n_seg + seg - 1) * p.cols + col), acc);
            }
            has = true;
        }
        uint64_t i = begin;
        for (; i + UNR <= end; i += UNR) {
            T v[UNR][VEC];
#pragma unroll
            for (int u = 0; u < UNR; ++u) scan_cols_load<T, VEC, NT>(src + (int64_t)(i + u) * p.s_in, v[u]);
            __builtin_amdgcn_sched_barrier(0);  // the step's loads go out before anything is folded
#pragma unroll
            for (int u = 0; u < UNR; ++u) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) acc[j] = has ? Op::apply(acc[j], v[u][j]) : v[u][j];
                has = true;
                if (PHASE == 2) scan_cols_store<T, VEC, NT>(dst + (int64_t)(i + u) * p.s_out, acc);
            }
        }
        for (; i < end; ++i) {
            T v[VEC];
            scan_cols_load<T, VEC, NT>(src + (int64_t)i * p.s_in, v);
#pragma unroll
            for (int j = 0; j < VEC; ++j) acc[j] = has ? Op::apply(acc[j], v[j]) : v[j];
            has = true;
            if (PHASE == 2) scan_cols_store<T, VEC, NT>(dst + (int64_t)i * p.s_out, acc);
        }
        if (PHASE == 0) scan_cols_store<T, VEC>(reinterpret_cast<char*>(totals + (plane * p.n_seg + seg) * p.cols + col), acc);
    }
}

constexpr uint64_t kScanLookbackSegs = 32;

// Two passes over the data with the segment totals between them. With few segments
// the second pass folds the totals of the segments before its own by itself (two
// launches); with many, the totals, a [segments x columns] matrix per plane, are
// scanned in place by this same routine first (a column scan of a much smaller array).
template <class T, class Op, int VEC>
void scan_cols_launch_vec(ScanColsParams& p, hipStream_t stream) {
    const uint64_t col_groups = p.cols / VEC;
    int txb = 0;
    while (txb < 8 && (1ull << txb) < col_groups) ++txb;
    p.tx_bits = txb;
    const uint64_t TX = 1ull << txb, TY = (uint64_t)kScanBlock >> txb;
    // segments: enough threads for eight blocks on every compute unit, at least 16 rows each;
    // no more than the second pass folds by itself when those already give every compute unit four
    // blocks (with one block each, SFloat [8192,8192] ran its first pass at half the bandwidth)
    const uint64_t want_threads = 256ull * 8 * kScanBlock;
    const uint64_t lanes_per_seg = col_groups * p.planes;
    uint64_t n_seg = (want_threads + lanes_per_seg - 1) / lanes_per_seg;
    const uint64_t max_seg = (p.n + 15) / 16;
    if (n_seg > kScanLookbackSegs && lanes_per_seg * kScanLookbackSegs >= 1024ull * kScanBlock) n_seg = kScanLookbackSegs;
    if (n_seg > max_seg) n_seg = max_seg;
    if (n_seg > 1024) n_seg = 1024;
    if (n_seg < 1) n_seg = 1;
    p.seg_len = (p.n + n_seg - 1) / n_seg;
    p.n_seg = (p.n + p.seg_len - 1) / p.seg_len;
    const uint64_t strips = (col_groups + TX - 1) / TX;
    uint64_t grid = strips * ((p.n_seg + TY - 1) / TY) * p.planes;
    if (grid > 0x7fffffffull) grid = 0x7fffffffull;
    const dim3 g((unsigned)grid), b(kScanBlock);
    const bool nt = stream_past_caches(2 * p.planes * p.n * p.cols * sizeof(T));
#define CUMO_SCAN_COLS(PHASE_, LB_, TOTALS_)                                                                                  \
    do {                                                                                                                      \
        if (nt) hipLaunchKernelGGL((scan_cols_kernel<T, Op, VEC, PHASE_, LB_, true>), g, b, 0, stream, p, TOTALS_);           \
        else hipLaunchKernelGGL((scan_cols_kernel<T, Op, VEC, PHASE_, LB_, false>), g, b, 0, stream, p, TOTALS_);             \
    } while (0)
    if (p.n_seg == 1) {
        CUMO_SCAN_COLS(2, false, (T*)nullptr);
        return;
    }
    T* totals = reinterpret_cast<T*>(cumo_cuda_runtime_malloc(sizeof(T) * p.planes * p.n_seg * p.cols));
    if (!totals) return;
    CUMO_SCAN_COLS(0, false, totals);
    if (p.n_seg <= kScanLookbackSegs) {
        CUMO_SCAN_COLS(2, true, totals);
    } else {
        ScanColsParams q;
        std::memset(&q, 0, sizeof(q));
        q.nouter = 1;
        q.planes = p.planes;
        q.oshape[0] = p.planes;
        q.ostep_in[0] = q.ostep_out[0] = (int64_t)(p.n_seg * p.cols * sizeof(T));
        q.cols = p.cols;
        q.n = p.n_seg;
        q.s_in = q.s_out = (int64_t)(p.cols * sizeof(T));
        q.in = reinterpret_cast<const char*>(totals);
        q.out = reinterpret_cast<char*>(totals);
        scan_cols_launch_vec<T, Op, VEC>(q, stream);  // at most 1024 rows: the next level has at most 64 segments
        CUMO_SCAN_COLS(2, false, totals);
    }
#undef CUMO_SCAN_COLS
    // stream-ordered reuse: whoever gets the block next can only touch it from later work on this stream
    cumo_cuda_runtime_free(reinterpret_cast<char*>(totals));
}

// ---- long runs across memory in one pass ---------------------------------------
// The matrix is cut into tiles of NW * 16 rows by 64 vectors (1 KiB of a row): wave w of
// a block holds 16 rows of the tile, lane l their vector l, all in registers. A tile adds
// up its columns (in the lane, then across the waves through LDS), publishes the column
// totals, gathers what the tiles above it published, and scans its rows from there: the
// data is read once and written once. The published words are {the launch's number, 32 bits of
// the value}, in the region the stream keeps (see above). Tiles take their places by ticket, level by level
// (all strips of one band of rows, then the next band), so whatever a tile waits for
// belongs to a block that is already running, and no tile waits before it has published
// its own totals. What a tile gathers has a fixed shape, so results do not change from
// launch to launch: tiles come in groups of 8 and groups in supergroups of 8; a tile folds
// the supergroups before its own, then the groups before its own, then the tiles before it
// in its group, each in order. The tile that closes a group publishes the group's total,
// the one that closes a supergroup the supergroup's.
constexpr int kColsChainRows = 16;
constexpr uint32_t kColsChainFan = 8;

template <class T>
struct ScanColsChain {
    static constexpr int W = (int)(sizeof(T) / 4);
    WaitCtl* wait;     // where a look-back that gives up reports it
    uint32_t* ticket;
    uint64_t* tile;    // [strip][level][column][W]
    uint64_t* group;   // [strip][group][column][W]
    uint64_t* super;   // [strip][supergroup][column][W]
    uint32_t depth, n_groups, n_supers;  // per strip
    uint32_t strips;                     // per plane
    uint32_t all_strips;                 // planes * strips
    uint32_t flag;                       // the upper half of a word of this launch
    uint32_t ticket_base;                // what the ticket word held before this launch
};

// Up to seven published values, `stride` words apart, the earliest first: all are asked for at
// once (eight-byte types: four, then three; seven would not fit the registers beside the tile),
// asked for again until they are there, then folded in order. False when count is 0.
template <class T, class Op>
__device__ __forceinline__ bool cols_chain_gather(const uint64_t* base, size_t stride, uint32_t count, uint32_t flag, WaitCtl* ctl, T& out) {
    constexpr int W = ScanColsChain<T>::W;
    constexpr uint32_t N = kColsChainFan - 1, C = sizeof(T) == 8 ? 4 : N;
    uint32_t polls = 0;
    const uint32_t spin_limit = wait_limit(ctl, kChainSpinLimit);
    bool has = false;
#pragma unroll
    for (uint32_t c0 = 0; c0 < N; c0 += C) {
        uint64_t x[C][W];
#pragma unroll
        for (uint32_t i = 0; i < C; ++i)
#pragma unroll
            for (int h = 0; h < W; ++h)
                x[i][h] = c0 + i < count ? __hip_atomic_load(base + (c0 + i) * stride + h, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : ((uint64_t)flag << 32);
        for (;;) {
            bool all = true;
#pragma unroll
            for (uint32_t i = 0; i < C; ++i)
#pragma unroll
                for (int h = 0; h < W; ++h) all = all && (uint32_t)(x[i][h] >> 32) == flag;
            if (all) break;
            if (++polls > spin_limit) {
                wait_gave_up(ctl, WAIT_SCAN);
                break;
            }
            __builtin_amdgcn_s_sleep(8);
#pragma unroll
            for (uint32_t i = 0; i < C; ++i)
#pragma unroll
                for (int h = 0; h < W; ++h)
                    if ((uint32_t)(x[i][h] >> 32) != flag) x[i][h] = __hip_atomic_load(base + (c0 + i) * stride + h, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (uint32_t i = 0; i < C; ++i) {
            if (c0 + i < count) {
                union { T t; uint32_t w[W]; } u;
#pragma unroll
                for (int h = 0; h < W; ++h) u.w[h] = (uint32_t)x[i][h];
                out = has ? Op::apply(out, u.t) : u.t;
                has = true;
            }
        }
    }
    return has;
}

template <class T, class Op, bool NT, int NW>
__global__ __launch_bounds__(NW * 64) void scan_cols_chain_kernel(ScanColsParams p, ScanColsChain<T> c) {
    constexpr int V = 16 / (int)sizeof(T), R = kColsChainRows, SW = 64 * V, W = ScanColsChain<T>::W;
    __shared__ T part[NW][SW];
    __shared__ T s_groups[SW], s_supers[SW];
    __shared__ uint32_t s_ticket;
    static_assert(NW * 64 >= 3 * SW, "three roles of SW threads each");
    const unsigned w = threadIdx.x >> 6, l = threadIdx.x & 63u;
    if (threadIdx.x == 0) s_ticket = __hip_atomic_fetch_add(c.ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - c.ticket_base;
    __syncthreads();
    const uint32_t id = s_ticket;
    const uint32_t k = id / c.all_strips, ps = id - k * c.all_strips;
    const uint32_t plane = ps / c.strips, strip = ps - plane * c.strips;
    int64_t oi = 0, oo = 0;
    if (p.nouter > 0) {
        uint64_t r = plane;
#pragma unroll 1
        for (int d = p.nouter - 1; d >= 0; --d) {
            const uint64_t m = p.oshape[d];
            const uint64_t q = r / m;
            const int64_t i = (int64_t)(r - q * m);
            r = q;
            oi += i * p.ostep_in[d];
            oo += i * p.ostep_out[d];
        }
    }
    const int64_t row0 = (int64_t)k * (NW * R) + (int64_t)w * R;
    const int64_t colb = ((int64_t)strip * SW + (int64_t)l * V) * (int64_t)sizeof(T);
    const char* src = p.in + oi + row0 * p.s_in + colb;
    char* dst = p.out + oo + row0 * p.s_out + colb;
    // A tile at the lower edge has fewer rows and one at the right edge fewer columns: this wave's first
    // `rows` rows exist, and of this lane's columns the first ncol. What such a tile reads as missing is zeros;
    // the totals they enter are only ever used by rows or columns that do not exist either.
    const int64_t rows_left = (int64_t)p.n - row0;
    const int rows = rows_left >= R ? R : (rows_left > 0 ? (int)rows_left : 0);
    const int64_t cols_left = (int64_t)p.cols - (int64_t)((uint64_t)strip * SW + (uint64_t)l * V);
    const int ncol = cols_left >= V ? V : (cols_left > 0 ? (int)cols_left : 0);  // this lane's columns that exist
    const bool all_there = rows == R && __builtin_amdgcn_ballot_w64(ncol != V) == 0;
    T raw[R][V];
    if (all_there) {
#pragma unroll
        for (int r = 0; r < R; ++r) scan_cols_load<T, V, NT>(src + (int64_t)r * p.s_in, raw[r]);
    } else {
#pragma unroll
        for (int r = 0; r < R; ++r) {
#pragma unroll
            for (int j = 0; j < V; ++j) raw[r][j] = T();
            if (r < rows) {
                if (ncol == V) {
                    scan_cols_load<T, V, NT>(src + (int64_t)r * p.s_in, raw[r]);
                } else {
                    // the row's last vector, partly there: element by element, nothing read past the row
#pragma unroll
                    for (int j = 0; j < V; ++j)
                        if (j < ncol) raw[r][j] = reinterpret_cast<const T*>(src + (int64_t)r * p.s_in)[j];
                }
            }
        }
    }
    {
        T tot[V];
#pragma unroll
        for (int j = 0; j < V; ++j) tot[j] = raw[0][j];
#pragma unroll
        for (int r = 1; r < R; ++r)
#pragma unroll
            for (int j = 0; j < V; ++j) tot[j] = Op::apply(tot[j], raw[r][j]);
#pragma unroll
        for (int j = 0; j < V; ++j) part[w][l * V + j] = tot[j];
    }
    __syncthreads();
    // Threads 0 .. SW-1 see to the tile's own totals and to the tiles before it in its group,
    // the next SW threads to the groups before its group, the SW after those to the supergroups:
    // the three waits run side by side in different waves, each with seven loads in flight.
    const unsigned col = threadIdx.x % SW, role = threadIdx.x / SW;
    const uint32_t pos = k % kColsChainFan, g = k / kColsChainFan, gpos = g % kColsChainFan, sg = g / kColsChainFan;
    const size_t cw = (size_t)SW * W;  // words from one tile's (group's) totals to the next one's
    T gt = T();
    if (role == 0) {
        // part[ww][col] becomes what the waves above ww add up to; gt, the tile's total
        gt = part[0][col];
#pragma unroll
        for (int ww = 1; ww < NW; ++ww) {
            const T e = gt;
            gt = Op::apply(gt, part[ww][col]);
            part[ww][col] = e;
        }
        chain_publish<T>(c.tile + (((size_t)ps * c.depth + k) * SW + col) * W, gt, c.flag);
    }
    const uint64_t* from = c.tile + (((size_t)ps * c.depth + (size_t)g * kColsChainFan) * SW + col) * W;
    uint32_t count = pos;
    if (role == 1) {
        from = c.group + (((size_t)ps * c.n_groups + (size_t)sg * kColsChainFan) * SW + col) * W;
        count = gpos;
    } else if (role == 2) {
        from = c.super + ((size_t)ps * c.n_supers * SW + col) * W;
        count = sg;
    } else if (role > 2) {
        count = 0;
    }
    T xs = T();
    const bool xh = cols_chain_gather<T, Op>(from, cw, count, c.flag, c.wait, xs);
    if (role == 0) {
        if (xh) gt = Op::apply(xs, gt);  // the group's total so far
        if (pos == kColsChainFan - 1) chain_publish<T>(c.group + (((size_t)ps * c.n_groups + g) * SW + col) * W, gt, c.flag);
    } else if (role == 1) {
        s_groups[col] = xs;
    } else if (role == 2) {
        s_supers[col] = xs;
    }
    __syncthreads();
    if (role == 0 && k > 0) {
        const bool yh = gpos > 0;
        T ys = T();
        if (yh) ys = s_groups[col];
        if (pos == kColsChainFan - 1 && gpos == kColsChainFan - 1) {
            const T st = yh ? Op::apply(ys, gt) : gt;
            chain_publish<T>(c.super + (((size_t)ps * c.n_supers + sg) * SW + col) * W, st, c.flag);
        }
        bool ph = sg > 0;
        T pre = T();
        if (ph) pre = s_supers[col];
        if (yh) { pre = ph ? Op::apply(pre, ys) : ys; ph = true; }
        if (xh) { pre = ph ? Op::apply(pre, xs) : xs; ph = true; }
        // k > 0: something lies above, so ph holds
        part[0][col] = pre;
#pragma unroll
        for (int ww = 1; ww < NW; ++ww) part[ww][col] = Op::apply(pre, part[ww][col]);
    }
    __syncthreads();
    // The topmost wave of the topmost tile has nothing above it; it goes the same way as the others
    // from a first row the compiler cannot see through (it would otherwise find this wave's running
    // values equal to the column totals' and keep all sixteen of them in registers from there to here,
    // beside the tile: there is no room for both).
    T acc[V];
    const bool topmost = k == 0 && w == 0;
#pragma unroll
    for (int j = 0; j < V; ++j) {
        const T above = topmost ? raw[0][j] : part[w][l * V + j];
        acc[j] = topmost ? above : Op::apply(above, raw[0][j]);
        if constexpr (sizeof(T) == 8) {
            union { T t; uint64_t u; } o;
            o.t = acc[j];
            asm volatile("" : "+v"(o.u));
            acc[j] = o.t;
        } else {
            union { T t; uint32_t u; } o;
            o.t = acc[j];
            asm volatile("" : "+v"(o.u));
            acc[j] = o.t;
        }
    }
    if (all_there) {
        scan_cols_store<T, V, NT>(dst, acc);
#pragma unroll
        for (int r = 1; r < R; ++r) {
#pragma unroll
            for (int j = 0; j < V; ++j) acc[j] = Op::apply(acc[j], raw[r][j]);
            scan_cols_store<T, V, NT>(dst + (int64_t)r * p.s_out, acc);
        }
    } else if (ncol > 0) {
        auto put = [&](int r) {
            if (ncol == V) {
                scan_cols_store<T, V, NT>(dst + (int64_t)r * p.s_out, acc);
            } else {
#pragma unroll
                for (int j = 0; j < V; ++j)
                    if (j < ncol) reinterpret_cast<T*>(dst + (int64_t)r * p.s_out)[j] = acc[j];
            }
        };
        if (rows > 0) put(0);
#pragma unroll
        for (int r = 1; r < R; ++r) {
#pragma unroll
            for (int j = 0; j < V; ++j) acc[j] = Op::apply(acc[j], raw[r][j]);
            if (r < rows) put(r);
        }
    }
}

static bool scan_cols_chain_enabled() {
    static const bool on = [] {
        const char* e = std::getenv("CUMO_HIP_SCAN_COLS_CHAIN");
        return !(e && e[0] == '0');
    }();
    return on;
}

// true when the launch was made (or failed: the error is left for the caller's check)
template <class T, class Op>
bool scan_cols_chain_launch(ScanColsParams& p, hipStream_t stream) {
    constexpr int V = 16 / (int)sizeof(T), W = ScanColsChain<T>::W, NW = 16;
    constexpr uint64_t SW = 64 * V, TR = (uint64_t)NW * kColsChainRows;
    if (!scan_cols_chain_enabled()) return false;
    if (p.cols < SW) return false;  // (a strip of 64 vectors is the unit: narrower arrays would leave most lanes idle)
    const uint64_t depth = (p.n + TR - 1) / TR, strips = (p.cols + SW - 1) / SW;
    constexpr uint64_t F = kColsChainFan;
    if (depth < 2 || depth > F * F * F) return false;
    const uint64_t all_strips = strips * p.planes;
    const uint64_t n_tiles = all_strips * depth;
    // (worth it from few tiles on: SFloat [512, 4096], 32 tiles, 9.5 us against 11.7 us for the launches of
    // the two-pass form; [4096, 4096], 256 tiles, 27 us against 51 us)
    if (n_tiles < 16 || n_tiles > 0x7fffffffull) return false;
    const uint64_t n_groups = (depth + F - 1) / F, n_supers = (n_groups + F - 1) / F;
    const uint64_t words = kChainHead + all_strips * (depth + n_groups + n_supers) * SW * W;
    WaitCtl* wait = wait_ctl();
    if (wait == nullptr) return false;  // nowhere to report a wait that gives up: the form without waits
    ChainWords cw;
    if (!chain_words_acquire(stream, words, (uint32_t)n_tiles, &cw)) return true;
    ScanColsChain<T> c;
    c.wait = wait;
    c.ticket = reinterpret_cast<uint32_t*>(cw.ws);
    c.tile = cw.ws + kChainHead;
    c.flag = cw.flag;
    c.ticket_base = cw.ticket_base;
    c.group = c.tile + all_strips * depth * SW * W;
    c.super = c.group + all_strips * n_groups * SW * W;
    c.depth = (uint32_t)depth;
    c.n_groups = (uint32_t)n_groups;
    c.n_supers = (uint32_t)n_supers;
    c.strips = (uint32_t)strips;
    c.all_strips = (uint32_t)all_strips;
    const bool nt = stream_past_caches(2 * p.planes * p.n * p.cols * sizeof(T));
    const dim3 g((unsigned)n_tiles), b(NW * 64);
    if (nt) hipLaunchKernelGGL((scan_cols_chain_kernel<T, Op, true, NW>), g, b, 0, stream, p, c);
    else hipLaunchKernelGGL((scan_cols_chain_kernel<T, Op, false, NW>), g, b, 0, stream, p, c);
    chain_words_release(cw);
    return true;
}

template <class T, class Op>
void scan_cols_launch(ScanColsParams& p, hipStream_t stream) {
    constexpr int V = 16 / (int)sizeof(T);
    bool vec = (p.cols % V) == 0 && ((uintptr_t)p.in % 16) == 0 && ((uintptr_t)p.out % 16) == 0 && (p.s_in % 16) == 0 && (p.s_out % 16) == 0;
    for (int d = 0; d < p.nouter && vec; ++d) vec = (p.ostep_in[d] % 16) == 0 && (p.ostep_out[d] % 16) == 0;
    // the one-pass form needs the elements' alignment only (128-bit accesses work on any 4-byte boundary)
    // and takes a last vector of a row that is partly there
    bool elem = ((uintptr_t)p.in % sizeof(T)) == 0 && ((uintptr_t)p.out % sizeof(T)) == 0 && (p.s_in % (int64_t)sizeof(T)) == 0 &&
                (p.s_out % (int64_t)sizeof(T)) == 0;
    for (int d = 0; d < p.nouter && elem; ++d) elem = (p.ostep_in[d] % (int64_t)sizeof(T)) == 0 && (p.ostep_out[d] % (int64_t)sizeof(T)) == 0;
    if (elem && scan_cols_chain_launch<T, Op>(p, stream)) return;
    if (vec) scan_cols_launch_vec<T, Op, V>(p, stream);
    else scan_cols_launch_vec<T, Op, 1>(p, stream);
}

template <class T>
void scan_cols_dispatch(int prod, int nan, ScanColsParams& p, hipStream_t stream) {
    if (prod) {
        if (nan) scan_cols_launch<T, ScanOp<T, 1, true> >(p, stream);
        else scan_cols_launch<T, ScanOp<T, 1, false> >(p, stream);
    } else {
        if (nan) scan_cols_launch<T, ScanOp<T, 0, true> >(p, stream);
        else scan_cols_launch<T, ScanOp<T, 0, false> >(p, stream);
    }
}

template <class T, class Op>
void scan_rows_launch(const ScanRowsParams& p, hipStream_t stream) {
    if (p.rows == 0 || p.n == 0) return;
    uint64_t grid = p.rows;
    if (grid > 65536) grid = 65536;
    constexpr uint64_t V = 16 / sizeof(T);
    // (runs need their element's alignment only: 128-bit accesses work on any 4-byte boundary)
    bool whole = p.s_in == (int64_t)sizeof(T) && p.s_out == (int64_t)sizeof(T) && p.n >= 64 * V &&
                 (((uintptr_t)p.in | (uintptr_t)p.out) % sizeof(T)) == 0;
    for (int d = 0; d < p.nouter && whole; ++d) whole = (p.ostep_in[d] % (int64_t)sizeof(T)) == 0 && (p.ostep_out[d] % (int64_t)sizeof(T)) == 0;
    if (whole) {
        const uint64_t vec_rows = (p.n + kScanBlock * V - 1) / (kScanBlock * V);  // rows of 256 vectors in a run, the last one maybe partly there
        const bool nt = stream_past_caches(2 * p.rows * p.n * sizeof(T));
        const dim3 g((unsigned)grid), b(kScanBlock);
#define CUMO_SCAN_WHOLE(R_) do { if (nt) hipLaunchKernelGGL((scan_rows_whole_kernel<T, Op, true, R_>), g, b, 0, stream, p); \
                                 else hipLaunchKernelGGL((scan_rows_whole_kernel<T, Op, false, R_>), g, b, 0, stream, p); } while (0)
        // chunks of 8, 4, 2 or 1 such rows: the largest that the run fills at least once, or that holds all of it
        if (vec_rows > 4) CUMO_SCAN_WHOLE(8);
        else if (vec_rows > 2) CUMO_SCAN_WHOLE(4);
        else if (vec_rows > 1) CUMO_SCAN_WHOLE(2);
        else CUMO_SCAN_WHOLE(1);
#undef CUMO_SCAN_WHOLE
        return;
    }
    hipLaunchKernelGGL((scan_rows_kernel<T, Op>), dim3((unsigned)grid), dim3(kScanBlock), 0, stream, p);
}

// CUMO_HIP_SCAN_CHAIN=0 (read once): long runs take the three launches instead of the one pass
static bool scan_chain_enabled() {
    static const bool on = [] {
        const char* e = std::getenv("CUMO_HIP_SCAN_CHAIN");
        return !(e && e[0] == '0');
    }();
    return on;
}

// One run of n elements. Short runs take one block; from 64 tiles of 64 KiB on, contiguous and aligned, the one pass;
// the three launches are what is left (runs beyond 2^30 elements, or the knob above).
template <class T, class Op>
int scan_run_launch(const char* p1, char* p2, ssize_t s1, ssize_t s2, uint64_t n) {
    if (n == 0) return 0;
    hipStream_t stream = current_stream();
    const uint64_t n_tiles = (n + kScanTile - 1) / kScanTile;
    if (n_tiles <= 8) {
        ScanRowsParams p;
        std::memset(&p, 0, sizeof(p));
        p.rows = 1;
        p.n = n;
        p.s_in = s1;
        p.s_out = s2;
        p.in = p1;
        p.out = p2;
        scan_rows_launch<T, Op>(p, stream);
        return (int)hipGetLastError();
    }
    if (scan_chain_enabled()) {
        const int st = scan_chain_launch<T, Op>(p1, p2, s1, s2, n, stream);
        if (st >= 0) return st;
    }
    // One tile per block keeps the most loads in flight (a block that walks a stretch of
    // tiles waits at two barriers per tile: measured 15 % slower). The totals are scanned
    // in place by this same routine, so a long run never leaves many tiles to one block.
    const uint64_t per = 1;
    const uint64_t n_blocks = n_tiles;
    if (n_blocks > 0x7fffffffull) return (int)hipErrorInvalidValue;
    T* totals = reinterpret_cast<T*>(cumo_cuda_runtime_malloc(sizeof(T) * n_blocks));
    if (!totals) return (int)hipErrorOutOfMemory;
    hipLaunchKernelGGL((scan_tile_totals_kernel<T, Op>), dim3((unsigned)n_blocks), dim3(kScanBlock), 0, stream, p1, (int64_t)s1, n, totals);
    const int inner = scan_run_launch<T, Op>(reinterpret_cast<const char*>(totals), reinterpret_cast<char*>(totals), (ssize_t)sizeof(T),
                                             (ssize_t)sizeof(T), n_blocks);
    if (inner) {
        cumo_cuda_runtime_free(reinterpret_cast<char*>(totals));
        return inner;
    }
    hipLaunchKernelGGL((scan_apply_kernel<T, Op>), dim3((unsigned)n_blocks), dim3(kScanBlock), 0, stream, p1, (int64_t)s1, p2, (int64_t)s2, n, per,
                       (const T*)totals);
    const int st = (int)hipGetLastError();
    // stream-ordered reuse: whoever gets the block next can only touch it from later work on this stream
    cumo_cuda_runtime_free(reinterpret_cast<char*>(totals));
    return st;
}

template <class T>
void scan_rows_dispatch(int prod, int nan, const ScanRowsParams& p, hipStream_t stream) {
    if (prod) {
        if (nan) scan_rows_launch<T, ScanOp<T, 1, true> >(p, stream);
        else scan_rows_launch<T, ScanOp<T, 1, false> >(p, stream);
    } else {
        if (nan) scan_rows_launch<T, ScanOp<T, 0, true> >(p, stream);
        else scan_rows_launch<T, ScanOp<T, 0, false> >(p, stream);
    }
}

}  // namespace

// The kept regions go back to the driver when their stream is retired and when the caller asks
// the pool to give back what it holds (they are not the pool's blocks -- they must outlive a
// launch without being handed to anybody else -- but they are memory the library holds:
// up to kChainKeptWords * 8 bytes per stream that has run a one-pass scan).
// The stream of the slot must have finished its work.
void scan_chain_words_drop_slot(int slot) {
    if (slot < 0 || slot >= kStreamSlots) return;
    std::lock_guard<std::mutex> hold(g_chain_lock);
    for (int dev = 0; dev < kChainDevices; ++dev) {
        ChainRegion& r = g_chain_region[dev][slot];
        if (!r.ptr) continue;
        if (hipFree(r.ptr) != hipSuccess) (void)hipGetLastError();
        r = ChainRegion{nullptr, 0, 0, 0};
    }
}

// every region, after waiting for the device (a launch that still uses one may be queued)
void scan_chain_words_drop_all() {
    std::lock_guard<std::mutex> hold(g_chain_lock);
    bool any = false;
    for (int dev = 0; dev < kChainDevices && !any; ++dev)
        for (int slot = 0; slot < kStreamSlots && !any; ++slot) any = g_chain_region[dev][slot].ptr != nullptr;
    if (!any) return;
    if (hipDeviceSynchronize() != hipSuccess) {
        (void)hipGetLastError();
        return;
    }
    for (int dev = 0; dev < kChainDevices; ++dev)
        for (int slot = 0; slot < kStreamSlots; ++slot) {
            ChainRegion& r = g_chain_region[dev][slot];
            if (!r.ptr) continue;
            if (hipFree(r.ptr) != hipSuccess) (void)hipGetLastError();
            r = ChainRegion{nullptr, 0, 0, 0};
        }
}

size_t scan_chain_words_held_bytes() {
    std::lock_guard<std::mutex> hold(g_chain_lock);
    size_t total = 0;
    for (int dev = 0; dev < kChainDevices; ++dev)
        for (int slot = 0; slot < kStreamSlots; ++slot) total += (size_t)g_chain_region[dev][slot].cap * sizeof(uint64_t);
    return total;
}

}  // namespace cumo_hip

using namespace cumo_hip;

extern "C" {

#define CUMO_DEF_CUM(t, c, name, OP, NANF)                                                                        \
    int cumo_##t##_##name##_kernel_launch(char* p1, char* p2, ssize_t s1, ssize_t s2, uint64_t n) {               \
        return scan_run_launch<c, ScanOp<c, OP, NANF> >(p1, p2, s1, s2, n);                                       \
    }
CUMO_DEF_CUM(sfloat, float, cumsum, 0, false)
CUMO_DEF_CUM(sfloat, float, cumsum_nan, 0, true)
CUMO_DEF_CUM(sfloat, float, cumprod, 1, false)
CUMO_DEF_CUM(sfloat, float, cumprod_nan, 1, true)
CUMO_DEF_CUM(dfloat, double, cumsum, 0, false)
CUMO_DEF_CUM(dfloat, double, cumsum_nan, 0, true)
CUMO_DEF_CUM(dfloat, double, cumprod, 1, false)
CUMO_DEF_CUM(dfloat, double, cumprod_nan, 1, true)
CUMO_DEF_CUM(int32, int32_t, cumsum, 0, false)
CUMO_DEF_CUM(int32, int32_t, cumprod, 1, false)

void cumo_hip_scan_rows_kernel_launch(int type, int prod, int nan, const cumo_hip_scan_rows_t* d) {
    if (!d || d->rows == 0 || d->n == 0) return;
    ScanRowsParams p;
    std::memset(&p, 0, sizeof(p));
    p.nouter = d->nouter;
    p.rows = d->rows;
    p.n = d->n;
    for (int k = 0; k < d->nouter && k < CUMO_NA_MAX_DIMENSION; ++k) {
        p.oshape[k] = d->oshape[k];
        p.ostep_in[k] = d->ostep_in[k];
        p.ostep_out[k] = d->ostep_out[k];
    }
    p.s_in = d->s_in;
    p.s_out = d->s_out;
    p.in = d->in;
    p.out = d->out;
    hipStream_t stream = current_stream();
    switch (type) {
        case 0: scan_rows_dispatch<float>(prod, nan, p, stream); break;
        case 1: scan_rows_dispatch<double>(prod, nan, p, stream); break;
        case 2: scan_rows_dispatch<int32_t>(prod, 0, p, stream); break;
        default: report_error(CUMO_HIP_ERROR_TYPE, 0, "scan: element type is not SFloat, DFloat or Int32"); return;
    }
    cumo_cuda_runtime_check_kernel_launch();
}

void cumo_hip_scan_cols_kernel_launch(int type, int prod, int nan, const cumo_hip_scan_rows_t* d, uint64_t cols) {
    if (!d || d->rows == 0 || d->n == 0 || cols == 0) return;
    ScanColsParams p;
    std::memset(&p, 0, sizeof(p));
    p.nouter = d->nouter;
    p.planes = d->rows;
    p.cols = cols;
    p.n = d->n;
    for (int k = 0; k < d->nouter && k < CUMO_NA_MAX_DIMENSION; ++k) {
        p.oshape[k] = d->oshape[k];
        p.ostep_in[k] = d->ostep_in[k];
        p.ostep_out[k] = d->ostep_out[k];
    }
    p.s_in = d->s_in;
    p.s_out = d->s_out;
    p.in = d->in;
    p.out = d->out;
    hipStream_t stream = current_stream();
    switch (type) {
        case 0: scan_cols_dispatch<float>(prod, nan, p, stream); break;
        case 1: scan_cols_dispatch<double>(prod, nan, p, stream); break;
        case 2: scan_cols_dispatch<int32_t>(prod, 0, p, stream); break;
        default: report_error(CUMO_HIP_ERROR_TYPE, 0, "scan: element type is not SFloat, DFloat or Int32"); return;
    }
    cumo_cuda_runtime_check_kernel_launch();
}

}  // extern "C"
