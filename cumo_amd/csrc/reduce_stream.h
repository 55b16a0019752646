// Lean reduction kernels for the layouts that carry nearly all the bytes: the
// reduce axis is ONE run of elements (after merging), the outputs span at most two
// dimensions, every access is a whole 128-bit vector and all totals fit 32 bits.
// Included by reduce_kernels.h, which keeps the general kernels for everything else.
//
//  red_srow_kernel        the reduce axis runs along memory; 2^k lanes share an output.
//  red_srow_split_kernel  the same with the axis cut over several blocks per output, in
//                         ONE launch: every block leaves its accumulator in a scratch
//                         array and counts in on a ticket; the block that counts in last
//                         folds the accumulators of its output in index order. The order
//                         of the fold does not depend on which block that is, so results
//                         are the same bits on every run, as with a second launch.
//  red_scol_kernel        the outputs run along memory; a lane owns VEC neighbouring
//                         outputs and walks the axis; with LOCAL, 2^k lanes of a block
//                         share the axis and combine through LDS in axis order.
//
// What makes them lean: a 136-byte argument block instead of 620 bytes; every load of
// an unrolled step is unconditional (a position past the end is pulled back inside the
// run and its value not used), so the four 128-bit loads of a lane are in flight
// together; no per-element index decomposition at all; non-temporal loads for inputs
// that no cache level could hold anyway.
#ifndef CUMO_HIP_REDUCE_STREAM_H
#define CUMO_HIP_REDUCE_STREAM_H

namespace cumo_hip {

constexpr int kRsUnroll = 4;            // 128-bit loads a lane keeps in flight
constexpr int kRsGroup = 32;            // blocks that count in on one first-level ticket when an output has more than kRsOneLevel
constexpr int kRsOneLevel = 128;        // up to this many blocks per output count in on a single ticket
constexpr uint32_t kRsTicketWords = 16384;  // ticket words per stream slot

// An Impl whose accumulate_columns<U, VEC>(x[U][VEC], acc[VEC]) folds U positions of VEC neighbouring outputs at once,
// all of which have seen the same number of positions before
template <class I, class = void> struct folds_columns_together { static constexpr bool value = false; };
template <class I> struct folds_columns_together<I, decltype((void)I::COLUMNS_TOGETHER)> { static constexpr bool value = I::COLUMNS_TOGETHER; };

// An Impl whose accumulate_columns_by_position<U, VEC>(x[U][VEC], first position, acc[VEC]) folds U consecutive
// positions of VEC neighbouring outputs without a branch
template <class I, class = void> struct folds_columns_by_position { static constexpr bool value = false; };
template <class I> struct folds_columns_by_position<I, decltype((void)I::COLUMNS_BY_POSITION)> { static constexpr bool value = I::COLUMNS_BY_POSITION; };

struct RedSParams {
    const char* in;
    char* out;
    char* out2;
    uint64_t n;            // length of the reduce axis in elements (row form: of its whole vectors)
    uint32_t tail;         // row form: elements of the axis past its last whole vector (fewer than a vector)
    int64_t red_step;      // column form: byte step along the reduce axis
    int64_t in_step[2];    // input byte steps over the (at most two) output dimensions, outer first
    int64_t out_step[2];
    int64_t out2_step[2];
    uint32_t n_out;        // outputs
    uint32_t out_inner;    // extent of the inner output dimension (= n_out when there is one dimension)
    uint32_t n_split;      // split form: blocks per output
    uint64_t chunk;        // column form cut across blocks: positions of the axis a block takes 
    uint32_t group;        // split form: blocks that count in on one first-level ticket
    uint32_t tstride;      // split form: words between two tickets (tickets in one cache line serialise in one memory channel)
    uint32_t tpr_bits;     // row form: 2^tpr_bits lanes share an output
    uint32_t lsplit_bits;  // column form: 2^lsplit_bits lanes of a block share an output group
    int32_t index_mode;    // what accumulate() gets as idx: 1 = position along the axis, 2 = element offset from `in`
    char* partial;         // split form: n_out * n_split accumulators
    uint32_t* tickets;     // split form: n_out + n_out * ceil(n_split / group) words, zero between launches
    WaitCtl* wait;         // hand-over form: where a wait that gives up reports it
};

template <class In, int VEC, bool NT>
__device__ __forceinline__ void rs_load(const char* p, In (&x)[VEC]) {
    static_assert(sizeof(In) * VEC == 16, "whole 128-bit vectors");
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    union V {
        u4 q;
        In v[VEC];
        __device__ V() {}
    } t;
    if constexpr (NT) t.q = __builtin_nontemporal_load(reinterpret_cast<const u4*>(p));
    else t.q = *reinterpret_cast<const u4*>(p);
#pragma unroll
    for (int j = 0; j < VEC; ++j) x[j] = t.v[j];
}

__device__ __forceinline__ void rs_split_out(const RedSParams& p, uint32_t o, uint32_t& o0, uint32_t& o1) {
    if (p.out_inner == p.n_out) {
        o0 = 0;
        o1 = o;
    } else {
        o0 = o / p.out_inner;
        o1 = o - o0 * p.out_inner;
    }
}

// The 2^tpr_bits lanes of a group fold the tiles first, first + every, first + 2 * every, ...
// of the run [0, end) (base = its element 0); a tile is what the group loads in one step,
// kRsUnroll vectors per lane. end is a multiple of VEC. Every lane of the group runs the
// same number of steps. The run may go on for `tail` more elements, fewer than a vector: the
// group's first lane folds those one by one when the group has the run's first tile (first == 0).
template <class Impl, int VEC, bool NT>
__device__ __forceinline__ typename Impl::Acc rs_row_scan(const Impl& impl, const char* base, uint64_t first, uint64_t every, uint64_t end,
                                                          uint32_t tail, unsigned lane_r, unsigned tpr_bits, int64_t idx_base) {
    typedef typename Impl::In In;
    typename Impl::Acc acc = impl.identity();
    const uint64_t stride = (uint64_t)VEC << tpr_bits;
    const uint64_t per_step = stride * kRsUnroll;
    const uint64_t tiles = (end + per_step - 1) / per_step;
    if (first >= tiles) return acc;
    const uint64_t steps = (tiles - first + every - 1) / every;
    const uint64_t advance = per_step * every;
    const uint64_t last = end - VEC;
    uint64_t i0 = first * per_step + (uint64_t)lane_r * VEC;
    for (uint64_t s = 0; s < steps; ++s, i0 += advance) {
        In x[kRsUnroll][VEC];
#pragma unroll
        for (int u = 0; u < kRsUnroll; ++u) {
            const uint64_t i = i0 + (uint64_t)u * stride;
            const uint64_t ic = i < end ? i : last;
            rs_load<In, VEC, NT>(base + ic * sizeof(In), x[u]);
        }
        // every load of the step is issued before anything is folded (the scheduler would
        // otherwise start folding the first vector and hold the later loads back behind it)
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (has_group<Impl>::value) {
            if (i0 + (uint64_t)(kRsUnroll - 1) * stride < end) {
                int64_t idx[kRsUnroll];
#pragma unroll
                for (int u = 0; u < kRsUnroll; ++u) idx[u] = idx_base + (int64_t)(i0 + (uint64_t)u * stride);
                impl.template accumulate_group<kRsUnroll, VEC>(x, idx, acc);
                continue;
            }
        }
#pragma unroll
        for (int u = 0; u < kRsUnroll; ++u) {
            const uint64_t i = i0 + (uint64_t)u * stride;
            if (i < end) impl.template accumulate_n<VEC>(x[u], idx_base + (int64_t)i, acc);
        }
    }
    // (after the lane's other elements: a lane folds in the order of the axis, which an impl may rely on)
    if (tail != 0 && first == 0 && lane_r == 0) {
        const In* rest = reinterpret_cast<const In*>(base) + end;
        for (uint32_t e = 0; e < tail; ++e) impl.accumulate(rest[e], idx_base + (int64_t)(end + e), acc);
    }
    return acc;
}

// Lanes of one output combine; the group's first lane (thread 0 when a block shares the
// output) ends up with everything, later lanes folded into earlier ones in a fixed order.
template <class Impl>
__device__ __forceinline__ void rs_group_combine(const Impl& impl, typename Impl::Acc& acc, unsigned tpr_bits,
                                                 typename Impl::Acc* wave_slots) {
    typedef typename Impl::Acc Acc;
    const unsigned TPR = 1u << tpr_bits;
    const unsigned span = TPR < 64 ? TPR : 64;
    for (unsigned d = span >> 1; d > 0; d >>= 1) {
        const Acc other = shfl_down_any(acc, d);
        impl.combine(other, acc);
    }
    if (TPR > 64) {
        if ((threadIdx.x & 63) == 0) wave_slots[threadIdx.x >> 6] = acc;
        __syncthreads();
        if (threadIdx.x == 0) {
            for (unsigned w = 1; w < kRedBlock / 64; ++w) impl.combine(wave_slots[w], acc);
        }
        __syncthreads();
    }
}

// scan + combine (+ the exact second fold where the impl asks for one)
template <class Impl, int VEC, bool NT>
__device__ __forceinline__ typename Impl::Acc rs_row_reduce(const Impl& impl, const char* base, uint64_t first, uint64_t every, uint64_t end,
                                                            uint32_t tail, unsigned lane_r, unsigned tpr_bits, int64_t idx_base,
                                                            typename Impl::Acc* wave_slots, int* s_need) {
    typedef typename Impl::Acc Acc;
    Acc acc = rs_row_scan<Impl, VEC, NT>(impl, base, first, every, end, tail, lane_r, tpr_bits, idx_base);
    rs_group_combine(impl, acc, tpr_bits, wave_slots);
    if constexpr (has_exact<Impl>::value) {
        const unsigned TPR = 1u << tpr_bits;
        bool need;
        if (TPR > 64) {
            if (threadIdx.x == 0) *s_need = impl.needs_exact(acc) ? 1 : 0;
            __syncthreads();
            need = *s_need != 0;
            __syncthreads();
        } else {
            const int mine = impl.needs_exact(acc) ? 1 : 0;
            need = __shfl(mine, (int)((threadIdx.x & 63u) & ~(TPR - 1))) != 0;
        }
        if (need) {
            typedef typename Impl::Exact Exact;
            const Exact ex = impl.exact();
            // the exact accumulator is wider: its own LDS slots
            __shared__ typename Exact::Acc exact_slots[kRedBlock / 64];
            typename Exact::Acc e = rs_row_scan<Exact, VEC, false>(ex, base, first, every, end, tail, lane_r, tpr_bits, 0);
            rs_group_combine(ex, e, tpr_bits, exact_slots);
            acc = impl.from_exact(e);
        }
    }
    return acc;
}

template <class Impl, int VEC, bool NT>
__global__ __launch_bounds__(kRedBlock) void red_srow_kernel(RedSParams p, Impl impl) {
    typedef typename Impl::In In;
    typedef typename Impl::Acc Acc;
    __shared__ Acc wave_slots[kRedBlock / 64];
    __shared__ int s_need;
    const unsigned TPR = 1u << p.tpr_bits;
    const unsigned RPB = (unsigned)kRedBlock >> p.tpr_bits;
    const unsigned lane_r = threadIdx.x & (TPR - 1);
    const unsigned row_in_block = threadIdx.x >> p.tpr_bits;
    const uint32_t n_rb = (p.n_out + RPB - 1) / RPB;
    for (uint32_t rb = blockIdx.x; rb < n_rb; rb += gridDim.x) {
        const uint32_t row = rb * RPB + row_in_block;
        const bool ok = row < p.n_out;
        uint32_t o0, o1;
        rs_split_out(p, ok ? row : p.n_out - 1, o0, o1);
        const int64_t in_off = (int64_t)o0 * p.in_step[0] + (int64_t)o1 * p.in_step[1];
        const int64_t idx_base = p.index_mode == 2 ? in_off / (int64_t)sizeof(In) : 0;
        const Acc acc = rs_row_reduce<Impl, VEC, NT>(impl, p.in + in_off, 0, 1, p.n, p.tail, lane_r, p.tpr_bits, idx_base, wave_slots, &s_need);
        if (ok && lane_r == 0) {
            const int64_t a = (int64_t)o0 * p.out_step[0] + (int64_t)o1 * p.out_step[1];
            const int64_t b = (Impl::NOUT > 1) ? (int64_t)o0 * p.out2_step[0] + (int64_t)o1 * p.out2_step[1] : 0;
            impl.store(acc, p.out + a, (Impl::NOUT > 1) ? (p.out2 + b) : nullptr);
        }
    }
}

// accumulators cross between blocks as 32-bit words written through to memory
template <class Acc>
__device__ __forceinline__ void rs_publish(char* dst, const Acc& acc) {
    static_assert(sizeof(Acc) % 4 == 0, "accumulator must be a whole number of 32-bit words");
    constexpr int W = sizeof(Acc) / 4;
    union U {
        Acc a;
        uint32_t w[W];
        __device__ U() {}
    } u;
    u.a = acc;
#pragma unroll
    for (int i = 0; i < W; ++i)
        __hip_atomic_store(reinterpret_cast<uint32_t*>(dst) + i, u.w[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// read after the acquire fence of the block that counted in last: plain loads, all in flight together
template <class Acc>
__device__ __forceinline__ Acc rs_fetch(const char* src) {
    return *reinterpret_cast<const Acc*>(src);
}

// One block per (output, chunk of the axis). blockIdx.x = output * n_split + chunk.
template <class Impl, int VEC, bool NT>
__global__ __launch_bounds__(kRedBlock) void red_srow_split_kernel(RedSParams p, Impl impl) {
    typedef typename Impl::In In;
    typedef typename Impl::Acc Acc;
    __shared__ Acc wave_slots[kRedBlock / 64];
    __shared__ int s_need;
    __shared__ int s_last;
    const uint32_t vrow = blockIdx.x;
    const uint32_t i_out = vrow / p.n_split;
    const uint32_t i_split = vrow - i_out * p.n_split;
    uint32_t o0, o1;
    rs_split_out(p, i_out, o0, o1);
    const int64_t in_off = (int64_t)o0 * p.in_step[0] + (int64_t)o1 * p.in_step[1];
    const int64_t idx_base = p.index_mode == 2 ? in_off / (int64_t)sizeof(In) : 0;
    // the blocks of an output take its 16 KiB tiles in turn, so that together they read one window
    // of the run at a time (memory sees a few long streams instead of n_split short ones)
    Acc acc = rs_row_reduce<Impl, VEC, NT>(impl, p.in + in_off, i_split, p.n_split, p.n, p.tail, threadIdx.x, 8, idx_base, wave_slots, &s_need);

    if (threadIdx.x == 0) {
        // The accumulator is written through to memory and has arrived there before
        // this block counts in. Blocks count in on their group's ticket; the last of a
        // group counts in on the output's ticket; the last there finds every
        // accumulator of the output in memory. Tickets go back to zero on the way.
        // What orders the publication before the count:
        //  * the hardware: rs_publish stores with agent scope, which on this device writes through
        //    the compute die's second-level cache to the memory all dies share, and the wait below
        //    returns when those stores are acknowledged; the ticket add is issued after that;
        //  * the compiler: the fence. At workgroup scope it costs nothing beyond that same wait,
        //    but no memory operation may be moved across it.
        // A release on the ticket add itself (agent scope) would be the textbook form; on this
        // device it also writes back the whole second-level cache of the die, once per block:
        // measured on T.sum() of 2^25 SFloat with tickets, 25.2 -> 107 us. The emitted order
        // (store sc1 ... s_waitcnt vmcnt(0) ... atomic add) is pinned by tests/test_emitted_ordering.py.
        rs_publish<Acc>(p.partial + (size_t)vrow * sizeof(Acc), acc);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_waitcnt(0);  // vmcnt(0) expcnt(0) lgkmcnt(0): the stores are acknowledged
        const uint32_t groups = (p.n_split + p.group - 1) / p.group;
        const uint32_t g = i_split / p.group;
        const uint32_t g_size = (g + 1 == groups) ? p.n_split - g * p.group : p.group;
        uint32_t* t1 = p.tickets + (size_t)(p.n_out + i_out * groups + g) * p.tstride;
        uint32_t* t0 = p.tickets + (size_t)i_out * p.tstride;
        int last = 0;
        if (__hip_atomic_fetch_add(t1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == g_size - 1) {
            __hip_atomic_store(t1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (groups == 1) {
                last = 1;  // one group: its last block is the output's last
            } else if (__hip_atomic_fetch_add(t0, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == groups - 1) {
                __hip_atomic_store(t0, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                last = 1;
            }
        }
        s_last = last;
    }
    __syncthreads();
    if (!s_last) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");

    // fold the output's accumulators in index order: thread t takes chunks t, t + 256, ...
    const char* mine = p.partial + (size_t)i_out * p.n_split * sizeof(Acc);
    const int64_t o_a = (int64_t)o0 * p.out_step[0] + (int64_t)o1 * p.out_step[1];
    const int64_t o_b = (Impl::NOUT > 1) ? (int64_t)o0 * p.out2_step[0] + (int64_t)o1 * p.out2_step[1] : 0;
    if constexpr (has_exact<Impl>::value) {
        // the accumulators are values in axis order: the fast fold first, and only where
        // it cannot decide (which of two equal values came first) the exact rule over the same values
        typedef typename Impl::Exact Exact;
        Acc total = impl.identity();
        for (uint32_t k = threadIdx.x; k < p.n_split; k += kRedBlock) impl.combine(rs_fetch<Acc>(mine + (size_t)k * sizeof(Acc)), total);
        rs_group_combine(impl, total, 8, wave_slots);
        if (threadIdx.x == 0) s_need = impl.needs_exact(total) ? 1 : 0;
        __syncthreads();
        if (s_need) {
            const Exact ex = impl.exact();
            __shared__ typename Exact::Acc exact_slots[kRedBlock / 64];
            typename Exact::Acc e = ex.identity();
            for (uint32_t k = threadIdx.x; k < p.n_split; k += kRedBlock) ex.accumulate_acc(rs_fetch<Acc>(mine + (size_t)k * sizeof(Acc)), (int64_t)k, e);
            rs_group_combine(ex, e, 8, exact_slots);
            total = impl.from_exact(e);
        }
        if (threadIdx.x == 0) impl.store(total, p.out + o_a, (Impl::NOUT > 1) ? (p.out2 + o_b) : nullptr);
    } else {
        Acc total = impl.identity();
        for (uint32_t k = threadIdx.x; k < p.n_split; k += kRedBlock) impl.combine(rs_fetch<Acc>(mine + (size_t)k * sizeof(Acc)), total);
        rs_group_combine(impl, total, 8, wave_slots);
        if (threadIdx.x == 0) impl.store(total, p.out + o_a, (Impl::NOUT > 1) ? (p.out2 + o_b) : nullptr);
    }
}

// Second launch of the column form cut across blocks: folds partial[part][output] (rows of rs_parts_row
// accumulators) into the results. 2^p.lsplit_bits lanes share a group of VEC outputs, each with a run of its
// parts in axis order, up to eight of them in flight, and combine pairwise through LDS, earlier parts on the left.
__host__ __device__ __forceinline__ size_t rs_parts_row(uint32_t n_out, uint32_t out_inner, int vec) {
    const uint32_t gpo = (out_inner + vec - 1) / vec;
    return (size_t)gpo * vec * (n_out / out_inner);
}

template <class Impl, int VEC>
__global__ __launch_bounds__(kRedBlock) void red_fold_parts_kernel(RedSParams p, Impl impl) {
    typedef typename Impl::Acc Acc;
    constexpr int B = 8;
    __shared__ Acc slots[kRedBlock][VEC];
    const unsigned pbits = p.lsplit_bits;
    const unsigned PG = 1u << pbits, OV = (unsigned)kRedBlock >> pbits;
    const unsigned ov = threadIdx.x & (OV - 1), pg = threadIdx.x >> (8u - pbits);
    const size_t row = rs_parts_row(p.n_out, p.out_inner, VEC);
    const uint32_t o = (blockIdx.x * OV + ov) * VEC;   // the group's first output (groups are whole here: 1-D outputs, or out_inner a multiple of VEC)
    const bool ok = o < p.n_out;
    const uint32_t per = (p.n_split + PG - 1) / PG;
    const uint32_t k0 = pg * per < p.n_split ? pg * per : p.n_split;
    const uint32_t k1 = k0 + per < p.n_split ? k0 + per : p.n_split;
    const Acc* base = reinterpret_cast<const Acc*>(p.partial) + (ok ? o : 0);
    Acc total[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) total[j] = impl.identity();
    for (uint32_t k = k0; k < k1; k += B) {
        Acc v[B][VEC];
#pragma unroll
        for (int b = 0; b < B; ++b) {
            const uint32_t kk = k + b < k1 ? k + b : k1 - 1;
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[b][j] = base[(size_t)kk * row + j];
        }
#pragma unroll
        for (int b = 0; b < B; ++b)
            if (k + b < k1) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) impl.combine(v[b][j], total[j]);
            }
    }
    for (unsigned stride = 1; stride < PG; stride <<= 1) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) slots[threadIdx.x][j] = total[j];
        __syncthreads();
        if ((pg & (2 * stride - 1)) == 0 && pg + stride < PG) {
#pragma unroll
            for (int j = 0; j < VEC; ++j) impl.combine(slots[(pg + stride) * OV + ov][j], total[j]);
        }
        __syncthreads();
    }
    if (pg != 0 || !ok) return;
    if constexpr (has_exact<Impl>::value) {
        // the parts are plain values in axis order: where the fast fold cannot tell which of two equal
        // values came first, the exact rule over the same values
        typedef typename Impl::Exact Exact;
        const Exact ex = impl.exact();
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            if (impl.needs_exact(total[j])) {
                typename Exact::Acc e = ex.identity();
                for (uint32_t k = 0; k < p.n_split; ++k) ex.accumulate_acc(base[(size_t)k * row + j], (int64_t)k, e);
                total[j] = impl.from_exact(e);
            }
        }
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
        const uint32_t oj = o + j;
        if (oj >= p.n_out) break;
        const uint32_t q0 = p.out_inner == p.n_out ? 0u : oj / p.out_inner;
        const uint32_t q1 = oj - q0 * p.out_inner;
        const int64_t a = (int64_t)q0 * p.out_step[0] + (int64_t)q1 * p.out_step[1];
        const int64_t b2 = (Impl::NOUT > 1) ? (int64_t)q0 * p.out2_step[0] + (int64_t)q1 * p.out2_step[1] : 0;
        impl.store(total[j], p.out + a, (Impl::NOUT > 1) ? (p.out2 + b2) : nullptr);
    }
}

// The exact second fold by ONE wave over the tiles that a whole block (tpr_bits 8) folded: the
// tiles first, first + every, ... of kRedBlock * VEC * kRsUnroll elements each, every vector of
// them taken by one of the 64 lanes. For the streaming blocks of the kernel below, where only
// the first wave learns (by a shuffle, no barrier, no LDS) that the block's result needs it:
// it is rare (a minimum or maximum that is a zero), and asking the whole block cost every
// launch 0.7 us. Lane 0 returns the result.
template <class Impl, int VEC>
__device__ __attribute__((noinline)) typename Impl::Acc rs_exact_refold_wave(const Impl& impl, const char* base, uint64_t first, uint64_t every,
                                                                              uint64_t end, uint32_t tail) {
    typedef typename Impl::In In;
    typedef typename Impl::Exact Exact;
    const Exact ex = impl.exact();
    typename Exact::Acc e = ex.identity();
    const uint64_t per_tile = (uint64_t)kRedBlock * VEC * kRsUnroll;
    const uint64_t tiles = (end + per_tile - 1) / per_tile;
    const unsigned lane = threadIdx.x & 63u;
    for (uint64_t t = first; t < tiles; t += every) {
        const uint64_t t0 = t * per_tile;
        const uint64_t t1 = t0 + per_tile < end ? t0 + per_tile : end;
        for (uint64_t i = t0 + (uint64_t)lane * VEC; i < t1; i += 64u * VEC) {
            In x[VEC];
            rs_load<In, VEC, false>(base + i * sizeof(In), x);
            ex.template accumulate_n<VEC>(x, (int64_t)i, e);
        }
    }
    if (tail != 0 && first == 0 && lane == 0) {
        const In* rest = reinterpret_cast<const In*>(base) + end;
        for (uint32_t k = 0; k < tail; ++k) ex.accumulate(rest[k], (int64_t)(end + k), e);
    }
    for (unsigned d = 32; d > 0; d >>= 1) {
        const typename Exact::Acc other = shfl_down_any(e, d);
        ex.combine(other, e);
    }
    return impl.from_exact(e);
}

// Few outputs, the axis of each cut over n_split blocks, one launch, no tickets: the first n_out
// blocks read nothing of the input; each waits for the accumulators of its output's other blocks,
// which arrive as 64-bit words {launch number, 32 bits of the accumulator} written with agent-scope
// atomic stores, and folds them in index order as the split form above does. The chain after
// the last block has finished its part is then one store becoming visible and one look at it,
// instead of store, acknowledgement, two tickets in turn, fence and loads (C3 T.sum() on fresh
// operands: 25.0 -> 22.4 us; a sum of 4 MiB: 5.9 -> 4.0 us). A streaming block never waits for
// anything, so the waiting blocks (which the dispatcher starts first) cannot hold the others up;
// a wait gives up after kRsPollLimit looks, counts that and raises the host's give-up word (wait_ctl.h).
constexpr uint32_t kRsHandoverWords = 8192;
constexpr uint32_t kRsPollLimit = 1u << 24;

template <class Acc>
__device__ __forceinline__ Acc rs_await(const uint64_t* slot, uint32_t launch, WaitCtl* ctl) {
    constexpr int W = sizeof(Acc) / 4;
    union U {
        Acc a;
        uint32_t w[W];
        __device__ U() {}
    } u;
    uint64_t x[W];
#pragma unroll
    for (int i = 0; i < W; ++i) x[i] = __hip_atomic_load(slot + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    uint32_t looks = 0;
    const uint32_t limit = wait_limit(ctl, kRsPollLimit);
    for (;;) {
        bool all = true;
#pragma unroll
        for (int i = 0; i < W; ++i) all = all && (uint32_t)(x[i] >> 32) == launch;
        if (all) break;
        if (++looks > limit) {
            wait_gave_up(ctl, WAIT_REDUCE);
            break;
        }
        __builtin_amdgcn_s_sleep(4);
#pragma unroll
        for (int i = 0; i < W; ++i)
            if ((uint32_t)(x[i] >> 32) != launch) x[i] = __hip_atomic_load(slot + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
#pragma unroll
    for (int i = 0; i < W; ++i) u.w[i] = (uint32_t)x[i];
    return u.a;
}

template <class Impl, int VEC, bool NT>
__global__ __launch_bounds__(kRedBlock) void red_srow_poll_kernel(RedSParams p, Impl impl, uint64_t* words, uint32_t launch) {
    typedef typename Impl::In In;
    typedef typename Impl::Acc Acc;
    constexpr int W = sizeof(Acc) / 4;
    static_assert(sizeof(Acc) % 4 == 0, "accumulator must be a whole number of 32-bit words");
    __shared__ Acc wave_slots[kRedBlock / 64];
    __shared__ int s_need;
    if (blockIdx.x >= p.n_out) {
        const uint32_t vrow = blockIdx.x - p.n_out;
        const uint32_t i_out = vrow / p.n_split;
        const uint32_t i_split = vrow - i_out * p.n_split;
        uint32_t o0, o1;
        rs_split_out(p, i_out, o0, o1);
        const int64_t in_off = (int64_t)o0 * p.in_step[0] + (int64_t)o1 * p.in_step[1];
        const int64_t idx_base = p.index_mode == 2 ? in_off / (int64_t)sizeof(In) : 0;
        Acc acc = rs_row_scan<Impl, VEC, NT>(impl, p.in + in_off, i_split, p.n_split, p.n, p.tail, threadIdx.x, 8, idx_base);
        rs_group_combine(impl, acc, 8, wave_slots);
        if constexpr (has_exact<Impl>::value) {
            // thread 0 holds the block's result; its wave alone repeats the fold where that is needed
            if (threadIdx.x >= 64) return;
            const int mine = impl.needs_exact(acc) ? 1 : 0;
            if (__shfl(mine, 0) != 0) acc = rs_exact_refold_wave<Impl, VEC>(impl, p.in + in_off, i_split, p.n_split, p.n, p.tail);
        }
        if (threadIdx.x == 0) {
            union U {
                Acc a;
                uint32_t w[W];
                __device__ U() {}
            } u;
            u.a = acc;
#pragma unroll
            for (int i = 0; i < W; ++i)
                __hip_atomic_store(words + (size_t)vrow * W + i, ((uint64_t)launch << 32) | u.w[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        return;
    }
    // fold the output's accumulators in index order: thread t takes chunks t, t + 256, ...
    const uint32_t i_out = blockIdx.x;
    uint32_t o0, o1;
    rs_split_out(p, i_out, o0, o1);
    const uint64_t* mine = words + (size_t)i_out * p.n_split * W;
    const int64_t o_a = (int64_t)o0 * p.out_step[0] + (int64_t)o1 * p.out_step[1];
    const int64_t o_b = (Impl::NOUT > 1) ? (int64_t)o0 * p.out2_step[0] + (int64_t)o1 * p.out2_step[1] : 0;
    if constexpr (has_exact<Impl>::value) {
        typedef typename Impl::Exact Exact;
        Acc total = impl.identity();
        for (uint32_t k = threadIdx.x; k < p.n_split; k += kRedBlock) impl.combine(rs_await<Acc>(mine + (size_t)k * W, launch, p.wait), total);
        rs_group_combine(impl, total, 8, wave_slots);
        if (threadIdx.x == 0) s_need = impl.needs_exact(total) ? 1 : 0;
        __syncthreads();
        if (s_need) {
            const Exact ex = impl.exact();
            __shared__ typename Exact::Acc exact_slots[kRedBlock / 64];
            typename Exact::Acc e = ex.identity();
            for (uint32_t k = threadIdx.x; k < p.n_split; k += kRedBlock) ex.accumulate_acc(rs_await<Acc>(mine + (size_t)k * W, launch, p.wait), (int64_t)k, e);
            rs_group_combine(ex, e, 8, exact_slots);
            total = impl.from_exact(e);
        }
        if (threadIdx.x == 0) impl.store(total, p.out + o_a, (Impl::NOUT > 1) ? (p.out2 + o_b) : nullptr);
    } else {
        Acc total = impl.identity();
        for (uint32_t k = threadIdx.x; k < p.n_split; k += kRedBlock) impl.combine(rs_await<Acc>(mine + (size_t)k * W, launch, p.wait), total);
        rs_group_combine(impl, total, 8, wave_slots);
        if (threadIdx.x == 0) impl.store(total, p.out + o_a, (Impl::NOUT > 1) ? (p.out2 + o_b) : nullptr);
    }
}

// Column form. out_inner is a multiple of VEC, or the outputs span one dimension (n_out >= VEC).
// U: positions of the axis a lane has in flight (more when the outputs alone give too few lanes
// to keep the memory system busy: a block still reads 4 KiB runs of every row it touches).
// PARTIAL: the axis is also cut across blocks, p.n_split ways (blockIdx.y says which part this
// block has); a block leaves its accumulators in p.partial[part][output] and a second launch
// (red_fold_parts_kernel) folds them. Blocks stay 128 or 256 vectors wide that way however few the outputs are.
template <class Impl, int VEC, bool NT, bool LOCAL, int U, bool PARTIAL = false>
__global__ __launch_bounds__(kRedBlock) void red_scol_kernel(RedSParams p, Impl impl) {
    typedef typename Impl::In In;
    typedef typename Impl::Acc Acc;
    __shared__ Acc part[LOCAL ? kRedBlock : 1][VEC];
    const unsigned lbits = LOCAL ? p.lsplit_bits : 0u;
    const unsigned SB = 1u << lbits;
    const unsigned cbits = 8u - lbits;
    const unsigned CPB = 1u << cbits;
    const unsigned c = threadIdx.x & (CPB - 1);
    const unsigned s = threadIdx.x >> cbits;
    // (the inner output dimension need not be a whole number of vectors: its last group is pulled
    // back to its last VEC outputs and stores only those the group before it does not)
    const uint32_t gpo = (p.out_inner + VEC - 1) / VEC;            // groups per position of the outer output dimension
    const uint32_t groups = (p.n_out / p.out_inner) * gpo;
    const uint32_t n_cb = (groups + CPB - 1) / CPB;
    // this block's stretch of the axis, then this lane's part of it
    uint64_t b0 = 0, b1 = p.n;
    if (PARTIAL) {
        const uint64_t bchunk = p.chunk;
        b0 = (uint64_t)blockIdx.y * bchunk;
        if (b0 > p.n) b0 = p.n;
        b1 = b0 + bchunk;
        if (b1 > p.n) b1 = p.n;
    }
    const uint64_t lchunk = (b1 - b0 + SB - 1) / SB;
    uint64_t begin = b0 + (uint64_t)s * lchunk;
    if (begin > b1) begin = b1;
    uint64_t end = begin + lchunk;
    if (end > b1) end = b1;

    for (uint32_t cb = blockIdx.x; cb < n_cb; cb += gridDim.x) {
        const uint32_t g = cb * CPB + c;
        const bool ok = g < groups;
        const uint32_t gg = ok ? g : groups - 1;
        const uint32_t o0 = p.out_inner == p.n_out ? 0u : gg / gpo;
        const uint32_t own1 = (gg - o0 * gpo) * VEC;
        const uint32_t o1 = own1 + VEC <= p.out_inner ? own1 : p.out_inner - VEC;  // where the group's vector starts
        const uint32_t own0 = o0 * p.out_inner + own1;                // the group's first output
        const uint32_t i_out0 = o0 * p.out_inner + o1;
        const int64_t in_off = (int64_t)o0 * p.in_step[0] + (int64_t)o1 * p.in_step[1];
        const char* base = p.in + in_off;
        Acc acc[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[j] = impl.identity();
        for (uint64_t i0 = begin; i0 < end; i0 += U) {
            In x[U][VEC];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const uint64_t i = i0 + u;
                const uint64_t ic = i < end ? i : end - 1;
                rs_load<In, VEC, NT>(base + (int64_t)ic * p.red_step, x[u]);
            }
            __builtin_amdgcn_sched_barrier(0);  // all loads of the step issued before the first fold
            if (i0 + U <= end && p.index_mode != 2) {
                // a whole block of consecutive positions along the axis for each output
                if constexpr (folds_columns_together<Impl>::value) {
                    // (the lane's outputs have had the same positions so far: what depends on the count alone is worked out once)
                    impl.template accumulate_columns<U, VEC>(x, acc);
                } else if constexpr (folds_columns_by_position<Impl>::value) {
                    impl.template accumulate_columns_by_position<U, VEC>(x, (int64_t)i0, acc);
                } else {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) {
                        In t[U];
#pragma unroll
                        for (int u = 0; u < U; ++u) t[u] = x[u][j];
                        impl.template accumulate_n<U>(t, (int64_t)i0, acc[j]);
                    }
                }
            } else {
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const uint64_t i = i0 + u;
                    if (i < end) {
#pragma unroll
                        for (int j = 0; j < VEC; ++j) {
                            int64_t idx = 0;
                            if (Impl::USES_INDEX)
                                idx = (p.index_mode == 2) ? ((in_off + (int64_t)i * p.red_step) / (int64_t)sizeof(In) + j) : (int64_t)i;
                            impl.accumulate(x[u][j], idx, acc[j]);
                        }
                    }
                }
            }
        }
        if constexpr (has_exact<Impl>::value) {
            // this lane walked its part of the axis in order, but its fast fold may have lost
            // which of two equal elements came first: walk that output again, exactly
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                if (impl.needs_exact(acc[j])) {
                    typedef typename Impl::Exact Exact;
                    const Exact ex = impl.exact();
                    typename Exact::Acc e = ex.identity();
                    for (uint64_t i = begin; i < end; ++i)
                        ex.accumulate(*reinterpret_cast<const In*>(base + (int64_t)i * p.red_step + (int64_t)j * (int64_t)sizeof(In)), (int64_t)i, e);
                    acc[j] = impl.from_exact(e);
                }
            }
        }
        if constexpr (LOCAL) {
            // The SB parts of an output group meet pairwise through LDS, neighbours first and the earlier part
            // on the left: log2 SB rounds in which every left-hand lane works, where one lane folding all the
            // parts one after the other waited for SB reads of LDS in a row while the rest of the block idled
            // (blocks start and end together here, so nothing else covers that time).
            Acc own[has_exact<Impl>::value ? VEC : 1];
            if constexpr (has_exact<Impl>::value) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) own[j] = acc[j];
            }
#pragma unroll
            for (int j = 0; j < VEC; ++j) part[threadIdx.x][j] = acc[j];
            __syncthreads();
            for (unsigned d = 1; d < SB; d <<= 1) {
                if ((s & (2u * d - 1u)) == 0) {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) impl.combine(part[(s + d) * CPB + c][j], acc[j]);
                    if (2u * d < SB) {
#pragma unroll
                        for (int j = 0; j < VEC; ++j) part[threadIdx.x][j] = acc[j];
                    }
                }
                __syncthreads();
            }
            if constexpr (has_exact<Impl>::value) {
                // folded by value; an output that may have lost which of two equal parts came first is folded
                // again from the lanes' own parts, plain values in axis order, with the exact rule
                bool again = false;
                if (s == 0) {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) again = again || impl.needs_exact(acc[j]);
                }
                if (__syncthreads_or(again ? 1 : 0)) {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) part[threadIdx.x][j] = own[j];
                    __syncthreads();
                    if (s == 0) {
#pragma unroll
                        for (int j = 0; j < VEC; ++j) {
                            if (!impl.needs_exact(acc[j])) continue;
                            typedef typename Impl::Exact Exact;
                            const Exact ex = impl.exact();
                            typename Exact::Acc e = ex.identity();
                            for (unsigned k = 0; k < SB; ++k) ex.accumulate_acc(part[k * CPB + c][j], (int64_t)k, e);
                            acc[j] = impl.from_exact(e);
                        }
                    }
                    __syncthreads();
                }
            }
        }
        if (PARTIAL) {
            // partial[part][output], a part's outputs padded to whole groups: the lanes of a block write one run
            if (ok && s == 0) {
                Acc* mine = reinterpret_cast<Acc*>(p.partial) + (size_t)blockIdx.y * ((size_t)gpo * VEC * (p.n_out / p.out_inner)) + i_out0;
                if (i_out0 == own0) {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) mine[j] = acc[j];
                } else {
#pragma unroll
                    for (int j = 0; j < VEC; ++j)
                        if (i_out0 + j >= own0) mine[j] = acc[j];
                }
            }
            continue;
        }
        if (ok && s == 0) {
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                if (i_out0 + j < own0) continue;  // (the pulled-back last group: the group before it has these)
                // the VEC outputs of a group are neighbours along the inner output dimension
                const int64_t a = (int64_t)o0 * p.out_step[0] + (int64_t)(o1 + j) * p.out_step[1];
                const int64_t b = (Impl::NOUT > 1) ? (int64_t)o0 * p.out2_step[0] + (int64_t)(o1 + j) * p.out2_step[1] : 0;
                impl.store(acc[j], p.out + a, (Impl::NOUT > 1) ? (p.out2 + b) : nullptr);
            }
        }
    }
}

}  // namespace cumo_hip

#endif
