// Reduction engine for gfx950.
//
// Replaces ext/cumo/include/cumo/reduce_kernel.h of the reference (address
// planner, reduction_kernel / _arg_ / _pair_ / _partial_kernel and the
// cumo_reduce* orchestration). The reference runs 512-thread blocks that
// combine through a nine-level shared-memory tree with a barrier per level.
// Here:
//
//  red_row_kernel  the reduce axis runs along memory. 2^k lanes (1..64, or a
//                  whole 256-thread block for long axes) share one output;
//                  each lane strides over the axis with 128-bit loads, lanes
//                  combine with wave64 shuffles (no LDS, no barrier, up to a
//                  wave), four waves combine through 4 LDS slots.
//  red_col_kernel  the output axis runs along memory. Each lane owns VEC
//                  neighbouring outputs and walks the reduce axis itself, so
//                  loads are 128-bit and coalesced across lanes and nothing
//                  is combined across lanes at all.
//  red_col_local_kernel  the same when the outputs are too few to fill the
//                  chip: 2..16 lanes of a block share the reduce axis of an
//                  output group and combine through LDS in axis order.
//
// Either kernel can run as the first pass of a split reduction: the reduce
// axis is cut into n_split chunks, accumulators go to
// partial[i_out * n_split + i_split], and a second red_row_kernel launch
// combines them in a fixed order. Both passes are deterministic (fixed
// shuffle order, no atomics), like the reference's.
//
// Impl contract (all __device__):
//   typedef In, Acc;  static constexpr bool USES_INDEX; static constexpr int NOUT (1 or 2)
//   Acc identity() const
//   void accumulate(In x, int64_t idx, Acc& acc) const     -- fold one input element
//   void accumulate_n<N>(const In (&x)[N], int64_t idx0, Acc& acc) const
//                                                          -- fold N elements at consecutive positions idx0..idx0+N-1,
//                                                             later than anything this accumulator has seen
//   void combine(const Acc& next, Acc& acc) const          -- merge two accumulators; must not depend on the order
//                                                             in which accumulators arrive
//   void store(const Acc& acc, char* out, char* out2) const
// Optional: GROUPED + accumulate_group<U,N> (several blocks offered at once);
// HAS_EXACT + Exact/exact()/needs_exact()/from_exact() (a cheap fold with an exact
// second fold of the same elements where the cheap one cannot decide).
#ifndef CUMO_HIP_REDUCE_KERNELS_H
#define CUMO_HIP_REDUCE_KERNELS_H

#include "common.h"
#include "plan.h"
#include "wait_ctl.h"

#include <cstdlib>
#include <cstring>

namespace cumo_hip {

constexpr int kRedBlock = 256;
constexpr int kRedUnroll = 4;

struct RedKParams {
    int out_ndim, red_ndim;
    int tpr_bits;        // row kernel: 2^tpr_bits lanes per output
    int index_mode;      // what accumulate() gets as idx: 1 = position along the flattened reduce axes, 2 = element offset from in
    int small;           // totals fit 32 bits
    int lsplit_bits;     // column kernel: 2^lsplit_bits lanes of a block share an output's reduce axis
    uint64_t out_total, red_total;
    uint64_t n_split, chunk;
    uint64_t out_shape[kMaxDim], red_shape[kMaxDim];
    int64_t in_out_step[kMaxDim], in_red_step[kMaxDim], out_step[kMaxDim], out2_step[kMaxDim];
    char* in;
    char* out;
    char* out2;
};

template <class T>
__device__ __forceinline__ T shfl_down_any(const T& v, unsigned delta) {
    static_assert(sizeof(T) % 4 == 0, "accumulator must be a whole number of 32-bit words");
    constexpr int W = sizeof(T) / 4;
    union U {
        T t;
        uint32_t w[W];
        __device__ U() {}
    } a, b;
    a.t = v;
#pragma unroll
    for (int i = 0; i < W; ++i) b.w[i] = __shfl_down(a.w[i], delta);
    return b.t;
}

// Impls whose fast fold leaves a question only an exact fold can answer declare
// HAS_EXACT = true, a type Exact (an Impl over the same In), exact(),
// needs_exact(acc) and from_exact(exact_acc).
template <class I, class = void> struct has_exact { static constexpr bool value = false; };
template <class I> struct has_exact<I, decltype((void)I::HAS_EXACT)> { static constexpr bool value = I::HAS_EXACT; };

// Impls that can take several blocks at once declare GROUPED and accumulate_group.
template <class I, class = void> struct has_group { static constexpr bool value = false; };
template <class I> struct has_group<I, decltype((void)I::GROUPED)> { static constexpr bool value = true; };

template <class T, int N>
struct alignas((sizeof(T) * N) > 16 ? 16 : (sizeof(T) * N)) RedVec {
    T v[N];
};

// offset of flat index i over dims [0, nd) with the given steps
__device__ __forceinline__ int64_t red_decompose(uint64_t i, int nd, const uint64_t* shape, const int64_t* step, int small) {
    int64_t off = 0;
    if (nd == 1) return (int64_t)i * step[0];
    if (small) {
        uint32_t r = (uint32_t)i;
        for (int d = nd - 1; d >= 1; --d) {
            const uint32_t n = (uint32_t)shape[d];
            const uint32_t q = r / n;
            off += (int64_t)(r - q * n) * step[d];
            r = q;
        }
        if (nd > 0) off += (int64_t)r * step[0];
    } else {
        uint64_t r = i;
        for (int d = nd - 1; d >= 1; --d) {
            const uint64_t n = shape[d];
            const uint64_t q = r / n;
            off += (int64_t)(r - q * n) * step[d];
            r = q;
        }
        if (nd > 0) off += (int64_t)r * step[0];
    }
    return off;
}

// One output's share of the reduce axis, [begin, end), folded by the 2^tpr_bits
// lanes that share the output. The result is complete in the group's first lane
// (thread 0 of the block when a whole block shares the output). Every lane of the
// wave must call it; lanes whose group has no output pass ok == false.
// NT: 128-bit loads are non-temporal (the launcher asks for it when the input is larger
// than the last-level cache: measured on 512 MiB, 74% -> 85% of peak; at 256 MiB and
// below the plain loads are ahead, because a re-read still finds the array cached).
template <class Impl, int VEC, bool NT = false>
__device__ __forceinline__ typename Impl::Acc red_row_scan(const RedKParams& p, const Impl& impl, bool ok, const char* base,
                                                           int64_t in_off, uint64_t begin, uint64_t end) {
    typedef typename Impl::In In;
    typedef typename Impl::Acc Acc;
    __shared__ Acc wave_acc[kRedBlock / 64];
    const unsigned TPR = 1u << p.tpr_bits;
    const unsigned lane_r = threadIdx.x & (TPR - 1);
    const int64_t rstep = p.in_red_step[p.red_ndim > 0 ? p.red_ndim - 1 : 0];
    const uint64_t stride = (uint64_t)TPR * VEC;

    Acc acc = impl.identity();
    if (ok) {
        for (uint64_t i0 = begin + (uint64_t)lane_r * VEC; i0 < end; i0 += stride * kRedUnroll) {
            In x[kRedUnroll][VEC];
            int64_t eoff[kRedUnroll];
#pragma unroll
            for (int u = 0; u < kRedUnroll; ++u) {
                const uint64_t i = i0 + (uint64_t)u * stride;
                if (i < end) {
                    const int64_t off = (p.red_ndim <= 1) ? (int64_t)i * rstep
                                                          : red_decompose(i, p.red_ndim, p.red_shape, p.in_red_step, p.small);
                    eoff[u] = in_off + off;
                    if constexpr (VEC > 1) {
                        RedVec<In, VEC> v;
                        if constexpr (NT && sizeof(RedVec<In, VEC>) == 16) {
                            typedef uint32_t ntu4 __attribute__((ext_vector_type(4)));
                            union NTV { ntu4 q; RedVec<In, VEC> r; __device__ NTV() {} } ntv;
                            ntv.q = __builtin_nontemporal_load(reinterpret_cast<const ntu4*>(base + off));
                            v = ntv.r;
                        } else {
                            v = *reinterpret_cast<const RedVec<In, VEC>*>(base + off);
                        }
#pragma unroll
                        for (int j = 0; j < VEC; ++j) x[u][j] = v.v[j];
                    } else {
                        x[u][0] = *reinterpret_cast<const In*>(base + off);
                    }
                }
            }
            if constexpr (has_group<Impl>::value) {
                if (i0 + (uint64_t)(kRedUnroll - 1) * stride < end) {
                    // every access of the unrolled step is inside the row: offer them together
                    int64_t idx[kRedUnroll];
#pragma unroll
                    for (int u = 0; u < kRedUnroll; ++u)
                        idx[u] = (p.index_mode == 2) ? (eoff[u] / (int64_t)sizeof(In)) : (int64_t)(i0 + (uint64_t)u * stride);
                    impl.template accumulate_group<kRedUnroll, VEC>(x, idx, acc);
                    continue;
                }
            }
#pragma unroll
            for (int u = 0; u < kRedUnroll; ++u) {
                const uint64_t i = i0 + (uint64_t)u * stride;
                if (i < end) {
                    // the VEC elements of one access are consecutive along the axis
                    int64_t idx = 0;
                    if (Impl::USES_INDEX) idx = (p.index_mode == 2) ? (eoff[u] / (int64_t)sizeof(In)) : (int64_t)i;
                    impl.template accumulate_n<VEC>(x[u], idx, acc);
                }
            }
        }
    }
    // lanes of one output combine; lane 0 of the group ends up with everything,
    // later lanes folded into earlier ones in a fixed order
    const unsigned wave_span = TPR < 64 ? TPR : 64;
    for (unsigned d = wave_span >> 1; d > 0; d >>= 1) {
        const Acc other = shfl_down_any(acc, d);
        impl.combine(other, acc);
    }
    if (TPR > 64) {
        const unsigned wave = threadIdx.x >> 6;
        if ((threadIdx.x & 63) == 0) wave_acc[wave] = acc;
        __syncthreads();
        if (threadIdx.x == 0) {
            for (unsigned w = 1; w < kRedBlock / 64; ++w) impl.combine(wave_acc[w], acc);
        }
        __syncthreads();
    }
    return acc;
}

template <class Impl, int VEC, bool PARTIAL, bool NT = false>
__global__ __launch_bounds__(kRedBlock) void red_row_kernel(RedKParams p, Impl impl, typename Impl::Acc* partial) {
    typedef typename Impl::Acc Acc;
    const unsigned TPR = 1u << p.tpr_bits;
    const unsigned RPB = kRedBlock >> p.tpr_bits;
    const unsigned lane_r = threadIdx.x & (TPR - 1);
    const unsigned row_in_block = threadIdx.x >> p.tpr_bits;
    const uint64_t n_rows = p.out_total * p.n_split;
    const uint64_t n_blocks = (n_rows + RPB - 1) / RPB;

    for (uint64_t rb = blockIdx.x; rb < n_blocks; rb += gridDim.x) {
        const uint64_t vrow = rb * RPB + row_in_block;
        const bool ok = vrow < n_rows;
        uint64_t i_out = 0, i_split = 0;
        if (ok) {
            if (p.n_split == 1) {
                i_out = vrow;
            } else {
                i_out = vrow / p.n_split;
                i_split = vrow - i_out * p.n_split;
            }
        }
        uint64_t begin = 0, end = 0;
        int64_t in_off = 0;
        if (ok) {
            begin = i_split * p.chunk;
            end = begin + p.chunk;
            if (end > p.red_total) end = p.red_total;
            in_off = red_decompose(i_out, p.out_ndim, p.out_shape, p.in_out_step, p.small);
        }
        const char* base = p.in + in_off;
        Acc acc = red_row_scan<Impl, VEC, NT>(p, impl, ok, base, in_off, begin, end);

        if constexpr (has_exact<Impl>::value) {
            // The fast fold cannot tell which of two equal-valued elements came first.
            // Where that matters for the answer (the impl says so), the lanes of the
            // output fold their share again with the exact rule. The verdict comes
            // from the group's first lane, so the whole group takes the same way.
            __shared__ int s_need;
            bool need;
            if (TPR > 64) {
                if (threadIdx.x == 0) s_need = impl.needs_exact(acc) ? 1 : 0;
                __syncthreads();
                need = s_need != 0;
                __syncthreads();
            } else {
                const int mine = impl.needs_exact(acc) ? 1 : 0;
                need = __shfl(mine, (int)((threadIdx.x & 63u) & ~(TPR - 1))) != 0;
            }
            if (need) {
                typedef typename Impl::Exact Exact;
                const Exact ex = impl.exact();
                const typename Exact::Acc eacc = red_row_scan<Exact, VEC>(p, ex, ok, base, in_off, begin, end);
                acc = impl.from_exact(eacc);
            }
        }
        if (ok && lane_r == 0) {
            if (PARTIAL) {
                partial[vrow] = acc;
            } else {
                const int64_t o1 = red_decompose(i_out, p.out_ndim, p.out_shape, p.out_step, p.small);
                const int64_t o2 = (Impl::NOUT > 1) ? red_decompose(i_out, p.out_ndim, p.out_shape, p.out2_step, p.small) : 0;
                impl.store(acc, p.out + o1, (Impl::NOUT > 1) ? (p.out2 + o2) : nullptr);
            }
        }
    }
}

// One lane's VEC neighbouring outputs folded over positions [begin, end) of the reduce axis
// (base: the first of the outputs at position 0; in_off: its byte offset from the array's start).
template <class Impl, int VEC, bool NT>
__device__ __forceinline__ void red_col_walk(const RedKParams& p, const Impl& impl, const char* base, int64_t in_off, uint64_t begin, uint64_t end,
                                             typename Impl::Acc (&acc)[VEC]) {
    typedef typename Impl::In In;
    const int64_t ostep_in = p.in_out_step[p.out_ndim - 1];
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] = impl.identity();

    for (uint64_t i0 = begin; i0 < end; i0 += kRedUnroll) {
        In x[kRedUnroll][VEC];
        int64_t roff[kRedUnroll];
#pragma unroll
        for (int u = 0; u < kRedUnroll; ++u) {
            const uint64_t i = i0 + u;
            if (i < end) {
                const int64_t off = red_decompose(i, p.red_ndim, p.red_shape, p.in_red_step, p.small);
                roff[u] = off;
                if constexpr (VEC > 1) {
                    RedVec<In, VEC> v;
                    if constexpr (NT && sizeof(RedVec<In, VEC>) == 16) {
                        typedef uint32_t ntu4 __attribute__((ext_vector_type(4)));
                        union NTV { ntu4 q; RedVec<In, VEC> r; __device__ NTV() {} } ntv;
                        ntv.q = __builtin_nontemporal_load(reinterpret_cast<const ntu4*>(base + off));
                        v = ntv.r;
                    } else {
                        v = *reinterpret_cast<const RedVec<In, VEC>*>(base + off);
                    }
#pragma unroll
                    for (int j = 0; j < VEC; ++j) x[u][j] = v.v[j];
                } else {
                    x[u][0] = *reinterpret_cast<const In*>(base + off);
                }
            }
        }
        if (i0 + kRedUnroll <= end && p.index_mode != 2) {
            // a whole block of consecutive positions along the axis for each output
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                In t[kRedUnroll];
#pragma unroll
                for (int u = 0; u < kRedUnroll; ++u) t[u] = x[u][j];
                impl.template accumulate_n<kRedUnroll>(t, (int64_t)i0, acc[j]);
            }
        } else {
#pragma unroll
            for (int u = 0; u < kRedUnroll; ++u) {
                const uint64_t i = i0 + u;
                if (i < end) {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) {
                        int64_t idx = 0;
                        if (Impl::USES_INDEX) {
                            idx = (p.index_mode == 2) ? ((in_off + roff[u] + (int64_t)j * ostep_in) / (int64_t)sizeof(In)) : (int64_t)i;
                        }
                        impl.accumulate(x[u][j], idx, acc[j]);
                    }
                }
            }
        }
    }
    if constexpr (has_exact<Impl>::value) {
        // this thread walked the axis in order, but its fast fold may still have lost
        // which of two equal elements came first: walk that output again, exactly
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            if (impl.needs_exact(acc[j])) {
                typedef typename Impl::Exact Exact;
                const Exact ex = impl.exact();
                typename Exact::Acc e = ex.identity();
                for (uint64_t i = begin; i < end; ++i) {
                    const int64_t off = red_decompose(i, p.red_ndim, p.red_shape, p.in_red_step, p.small);
                    ex.accumulate(*reinterpret_cast<const In*>(base + off + (int64_t)j * ostep_in), (int64_t)i, e);
                }
                acc[j] = impl.from_exact(e);
            }
        }
    }
}

template <class Impl, int VEC, bool PARTIAL, bool NT = false>
__global__ __launch_bounds__(kRedBlock) void red_col_kernel(RedKParams p, Impl impl, typename Impl::Acc* partial) {
    typedef typename Impl::Acc Acc;
    const uint64_t groups = p.out_total / VEC;  // planner guarantees divisibility of the innermost out dim
    const uint64_t n_items = groups * p.n_split;

    for (uint64_t g = (uint64_t)blockIdx.x * kRedBlock + threadIdx.x; g < n_items; g += (uint64_t)gridDim.x * kRedBlock) {
        uint64_t i_split = 0, cg = g;
        if (p.n_split > 1) {
            i_split = g / groups;
            cg = g - i_split * groups;
        }
        const uint64_t i_out0 = cg * VEC;
        const int64_t in_off = red_decompose(i_out0, p.out_ndim, p.out_shape, p.in_out_step, p.small);
        const char* base = p.in + in_off;
        const uint64_t begin = i_split * p.chunk;
        uint64_t end = begin + p.chunk;
        if (end > p.red_total) end = p.red_total;

        Acc acc[VEC];
        red_col_walk<Impl, VEC, NT>(p, impl, base, in_off, begin, end, acc);
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            const uint64_t i_out = i_out0 + j;
            if (PARTIAL) {
                partial[i_out * p.n_split + i_split] = acc[j];
            } else {
                const int64_t o1 = red_decompose(i_out, p.out_ndim, p.out_shape, p.out_step, p.small);
                const int64_t o2 = (Impl::NOUT > 1) ? red_decompose(i_out, p.out_ndim, p.out_shape, p.out2_step, p.small) : 0;
                impl.store(acc[j], p.out + o1, (Impl::NOUT > 1) ? (p.out2 + o2) : nullptr);
            }
        }
    }
}

// The same with the reduce axis also cut inside the block: 2^lsplit_bits lanes share each group of
// VEC outputs, each walks its part of the (launch-level) chunk, and the parts are combined through
// LDS in axis order by the first of them. More blocks for an array with few outputs across memory,
// without a second launch (or with a much smaller one when the launch-level split is still needed).
template <class Impl, int VEC, bool PARTIAL, bool NT = false>
__global__ __launch_bounds__(kRedBlock) void red_col_local_kernel(RedKParams p, Impl impl, typename Impl::Acc* partial) {
    typedef typename Impl::Acc Acc;
    __shared__ Acc part[kRedBlock][VEC];
    const unsigned SB = 1u << p.lsplit_bits;
    const unsigned cbits = 8u - (unsigned)p.lsplit_bits;  // kRedBlock = 2^8
    const unsigned CPB = 1u << cbits;
    const unsigned c = threadIdx.x & (CPB - 1);
    const unsigned s = threadIdx.x >> cbits;
    const uint64_t groups = p.out_total / VEC;
    const uint64_t n_items = groups * p.n_split;
    const uint64_t n_blocks = (n_items + CPB - 1) / CPB;

    for (uint64_t blk = blockIdx.x; blk < n_blocks; blk += gridDim.x) {
        const uint64_t g = blk * CPB + c;
        const bool ok = g < n_items;
        uint64_t i_split = 0, cg = 0;
        if (ok) {
            cg = g;
            if (p.n_split > 1) {
                i_split = g / groups;
                cg = g - i_split * groups;
            }
        }
        const uint64_t i_out0 = cg * VEC;
        Acc acc[VEC];
        if (ok) {
            const int64_t in_off = red_decompose(i_out0, p.out_ndim, p.out_shape, p.in_out_step, p.small);
            const uint64_t gbegin = i_split * p.chunk;
            uint64_t gend = gbegin + p.chunk;
            if (gend > p.red_total) gend = p.red_total;
            const uint64_t lchunk = (gend - gbegin + SB - 1) / SB;
            uint64_t begin = gbegin + (uint64_t)s * lchunk;
            if (begin > gend) begin = gend;
            uint64_t end = begin + lchunk;
            if (end > gend) end = gend;
            red_col_walk<Impl, VEC, NT>(p, impl, p.in + in_off, in_off, begin, end, acc);
        } else {
#pragma unroll
            for (int j = 0; j < VEC; ++j) acc[j] = impl.identity();
        }
        // the SB parts of a group meet pairwise through LDS, neighbours first, the earlier part on the left
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
            if (ok && s == 0) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) again = again || impl.needs_exact(acc[j]);
            }
            if (__syncthreads_or(again ? 1 : 0)) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) part[threadIdx.x][j] = own[j];
                __syncthreads();
                if (ok && s == 0) {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) {
                        if (!impl.needs_exact(acc[j])) continue;
                        typedef typename Impl::Exact Exact;
                        const Exact ex = impl.exact();
                        typename Exact::Acc e = ex.identity();
                        for (unsigned k = 0; k < SB; ++k) ex.accumulate(part[k * CPB + c][j], (int64_t)k, e);
                        acc[j] = impl.from_exact(e);
                    }
                }
            }
        }
        if (ok && s == 0) {
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const uint64_t i_out = i_out0 + j;
                if (PARTIAL) {
                    partial[i_out * p.n_split + i_split] = acc[j];
                } else {
                    const int64_t o1 = red_decompose(i_out, p.out_ndim, p.out_shape, p.out_step, p.small);
                    const int64_t o2 = (Impl::NOUT > 1) ? red_decompose(i_out, p.out_ndim, p.out_shape, p.out2_step, p.small) : 0;
                    impl.store(acc[j], p.out + o1, (Impl::NOUT > 1) ? (p.out2 + o2) : nullptr);
                }
            }
        }
        __syncthreads();
    }
}

// Second pass of a split reduction: the input is accumulators.
template <class Impl>
struct CombineImpl {
    typedef typename Impl::Acc In;
    typedef typename Impl::Acc Acc;
    static constexpr bool USES_INDEX = false;
    static constexpr int NOUT = Impl::NOUT;
    Impl impl;
    __device__ __forceinline__ Acc identity() const { return impl.identity(); }
    __device__ __forceinline__ void accumulate(const In& x, int64_t, Acc& acc) const { impl.combine(x, acc); }
    template <int N>
    __device__ __forceinline__ void accumulate_n(const In (&x)[N], int64_t, Acc& acc) const {
#pragma unroll
        for (int k = 0; k < N; ++k) impl.combine(x[k], acc);
    }
    __device__ __forceinline__ void combine(const Acc& next, Acc& acc) const { impl.combine(next, acc); }
    __device__ __forceinline__ void store(const Acc& acc, char* out, char* out2) const { impl.store(acc, out, out2); }
};

// Device memory a caller lends for the partial results of a split reduction.
struct RedScratch {
    char* ptr;
    size_t bytes;
    mutable size_t used;   // set by the launch: bytes of ptr that its kernels write and read (0: none)
};

static inline unsigned red_grid_cap() {
    static unsigned cap = 0;
    if (cap == 0) {
        const char* e = std::getenv("CUMO_HIP_RED_GRID_CAP");
        cap = e ? (unsigned)std::strtoul(e, nullptr, 10) : 0;
        if (cap == 0) cap = (unsigned)kNumCU * 32;
    }
    return cap;
}

static inline void red_fill_params(RedKParams* kp, const ReducePlan& plan, const cumo_na_reduction_arg_t* arg,
                                   const cumo_na_iarray_t* out2, int index_mode) {
    std::memset(kp, 0, sizeof(*kp));
    kp->out_ndim = plan.out_ndim;
    kp->red_ndim = plan.red_ndim;
    kp->index_mode = index_mode;
    kp->out_total = plan.out_total;
    kp->red_total = plan.red_total;
    kp->n_split = 1;
    kp->chunk = plan.red_total;
    for (int d = 0; d < kMaxDim; ++d) {
        kp->out_shape[d] = plan.out_shape[d];
        kp->red_shape[d] = plan.red_shape[d];
        kp->in_out_step[d] = plan.in_out_step[d];
        kp->in_red_step[d] = plan.in_red_step[d];
        kp->out_step[d] = plan.out_step[d];
        kp->out2_step[d] = plan.out2_step[d];
    }
    kp->in = arg->in.ptr;
    kp->out = arg->out.ptr;
    kp->out2 = out2 ? out2->ptr : nullptr;
    kp->small = (arg->in_indexer.total_size < 0xffffffffull && !force_wide_indices()) ? 1 : 0;
}

// Inputs beyond this size are read with non-temporal loads: no cache level can hold them
// until they are needed again, and keeping them out leaves the caches to what can be
// (measured with every launch on fresh data: 128 MiB of SFloat summed at 76% of the HBM
// peak with plain loads, 82% with non-temporal ones; no difference at 32 MiB).
static inline bool red_use_nt(uint64_t bytes) { return stream_past_caches(bytes); }

template <class Impl, bool PARTIAL, bool SCALAR_ONLY = false>
static void red_launch_row(const RedKParams& kp, int vec, Impl impl, typename Impl::Acc* partial, hipStream_t stream) {
    constexpr int kMaxVec = SCALAR_ONLY ? 1 : (int)(16 / sizeof(typename Impl::In));
    const uint64_t n_rows = kp.out_total * kp.n_split;
    const uint64_t rpb = (uint64_t)kRedBlock >> kp.tpr_bits;
    uint64_t grid = (n_rows + rpb - 1) / rpb;
    if (grid > red_grid_cap()) grid = red_grid_cap();
    if (grid == 0) return;
    const dim3 g((unsigned)grid), b(kRedBlock);
    if constexpr (kMaxVec >= 2 && !SCALAR_ONLY) {
        // the widest access of an input too large for the last-level cache: non-temporal
        if (vec == kMaxVec && red_use_nt(kp.out_total * kp.red_total * sizeof(typename Impl::In))) {
            hipLaunchKernelGGL((red_row_kernel<Impl, kMaxVec, PARTIAL, true>), g, b, 0, stream, kp, impl, partial);
            return;
        }
    }
    if constexpr (kMaxVec >= 4) {
        if (vec == 4) { hipLaunchKernelGGL((red_row_kernel<Impl, 4, PARTIAL>), g, b, 0, stream, kp, impl, partial); return; }
    }
    if constexpr (kMaxVec >= 2) {
        if (vec == 2) { hipLaunchKernelGGL((red_row_kernel<Impl, 2, PARTIAL>), g, b, 0, stream, kp, impl, partial); return; }
    }
    hipLaunchKernelGGL((red_row_kernel<Impl, 1, PARTIAL>), g, b, 0, stream, kp, impl, partial);
}

template <class Impl, bool PARTIAL>
static void red_launch_col(const RedKParams& kp, int vec, Impl impl, typename Impl::Acc* partial, hipStream_t stream) {
    constexpr int kMaxVec = (int)(16 / sizeof(typename Impl::In));
    const uint64_t items = (kp.out_total / vec) * kp.n_split;
    const uint64_t per_block = (uint64_t)kRedBlock >> kp.lsplit_bits;
    uint64_t grid = (items + per_block - 1) / per_block;
    if (grid > red_grid_cap()) grid = red_grid_cap();
    if (grid == 0) return;
    const dim3 g((unsigned)grid), b(kRedBlock);
    if (kp.lsplit_bits > 0) {
        // lanes of a block share the reduce axis of an output (few outputs across memory)
        if constexpr (kMaxVec >= 4) {
            if (vec == 4) { hipLaunchKernelGGL((red_col_local_kernel<Impl, 4, PARTIAL>), g, b, 0, stream, kp, impl, partial); return; }
        }
        if constexpr (kMaxVec >= 2) {
            if (vec == 2) { hipLaunchKernelGGL((red_col_local_kernel<Impl, 2, PARTIAL>), g, b, 0, stream, kp, impl, partial); return; }
        }
        hipLaunchKernelGGL((red_col_local_kernel<Impl, 1, PARTIAL>), g, b, 0, stream, kp, impl, partial);
        return;
    }
    if constexpr (kMaxVec >= 2) {
        if (vec == kMaxVec && red_use_nt(kp.out_total * kp.red_total * sizeof(typename Impl::In))) {
            hipLaunchKernelGGL((red_col_kernel<Impl, kMaxVec, PARTIAL, true>), g, b, 0, stream, kp, impl, partial);
            return;
        }
    }
    if constexpr (kMaxVec >= 4) {
        if (vec == 4) { hipLaunchKernelGGL((red_col_kernel<Impl, 4, PARTIAL>), g, b, 0, stream, kp, impl, partial); return; }
    }
    if constexpr (kMaxVec >= 2) {
        if (vec == 2) { hipLaunchKernelGGL((red_col_kernel<Impl, 2, PARTIAL>), g, b, 0, stream, kp, impl, partial); return; }
    }
    hipLaunchKernelGGL((red_col_kernel<Impl, 1, PARTIAL>), g, b, 0, stream, kp, impl, partial);
}

}  // namespace cumo_hip

#include "reduce_stream.h"

namespace cumo_hip {

static inline bool red_stream_enabled() {
    static int on = -1;
    if (on < 0) {
        const char* e = std::getenv("CUMO_HIP_RED_STREAM");
        on = (e && std::atoi(e) == 0) ? 0 : 1;
    }
    return on != 0;
}

// CUMO_HIP_RED_POLL=0 (read once): full reductions take the ticket form
static bool red_poll_enabled() {
    static const bool on = [] {
        const char* e = std::getenv("CUMO_HIP_RED_POLL");
        return !(e && e[0] == '0');
    }();
    return on;
}

// Second pass of a reduction whose axis was cut across blocks: folds partial[out_total][n_split]
// (accumulators in axis order) into the results. kp: the first pass's parameters.
template <class Impl>
static void red_fold_partials(const ReducePlan& plan, const RedKParams& kp, typename Impl::Acc* partial, Impl impl, hipStream_t stream) {
    typedef typename Impl::In In;
    typedef typename Impl::Acc Acc;
    const uint64_t n_partial = plan.out_total * kp.n_split;
    RedKParams k2 = kp;
    k2.lsplit_bits = 0;
    k2.in = reinterpret_cast<char*>(partial);
    k2.red_ndim = 1;
    k2.red_shape[0] = kp.n_split;
    k2.in_red_step[0] = (int64_t)sizeof(Acc);
    k2.red_total = kp.n_split;
    k2.n_split = 1;
    k2.chunk = kp.n_split;
    int64_t s = (int64_t)sizeof(Acc) * (int64_t)kp.n_split;
    for (int d = plan.out_ndim - 1; d >= 0; --d) {
        k2.in_out_step[d] = s;
        s *= (int64_t)plan.out_shape[d];
    }
    k2.small = (n_partial < 0xffffffffull && plan.out_total < 0xffffffffull && !force_wide_indices()) ? 1 : 0;
    int tpr = 1;
    while (tpr < 64 && (uint64_t)tpr * 4 < kp.n_split) tpr <<= 1;
    if (kp.n_split > 1024) tpr = 256;
    k2.tpr_bits = 0;
    while ((1 << k2.tpr_bits) < tpr) ++k2.tpr_bits;
    if constexpr (has_exact<Impl>::value) {
        // the partials are plain values in axis order: fold them with the exact rule
        static_assert(sizeof(Acc) == sizeof(In), "an impl with an exact fallback keeps a plain value");
        k2.index_mode = 1;
        red_launch_row<typename Impl::Exact, false, true>(k2, 1, impl.exact(), nullptr, stream);
    } else {
        CombineImpl<Impl> cimpl;
        cimpl.impl = impl;
        red_launch_row<CombineImpl<Impl>, false, true>(k2, 1, cimpl, nullptr, stream);
    }
    cumo_cuda_runtime_check_kernel_launch();
}

// The lean kernels of reduce_stream.h for the layouts they take. Returns 1 when the
// reduction has been launched, 0 when the general kernels must take it, -1 when the
// caller's fixed scratch is too small (nothing launched).
template <class Impl>
static int red_stream_launch(const ReducePlan& plan, const cumo_na_reduction_arg_t* arg, const cumo_na_iarray_t* out2, Impl impl,
                             int index_mode, const RedScratch* fixed, hipStream_t stream) {
    typedef typename Impl::In In;
    typedef typename Impl::Acc Acc;
    constexpr int V = (int)(16 / sizeof(In));
    if (!red_stream_enabled() || force_wide_indices()) return 0;
    if (plan.vec != V || plan.red_ndim != 1 || plan.red_total == 0 || plan.out_ndim > 2) return 0;
    if (plan.out_total >= 0x7fffffffull) return 0;
    if (plan.kind != RED_ROW && plan.kind != RED_COL) return 0;
    {
        static int force1 = -1;
        if (force1 < 0) force1 = std::getenv("CUMO_HIP_FORCE_VEC1") ? 1 : 0;
        if (force1) return 0;
    }
    RedSParams p;
    std::memset(&p, 0, sizeof(p));
    p.in = arg->in.ptr;
    p.out = arg->out.ptr;
    p.out2 = out2 ? out2->ptr : nullptr;
    p.n = plan.red_total;
    p.red_step = plan.in_red_step[0];
    p.n_out = (uint32_t)plan.out_total;
    p.n_split = 1;
    p.index_mode = index_mode;
    if (plan.out_ndim == 2) {
        p.out_inner = (uint32_t)plan.out_shape[1];
        for (int d = 0; d < 2; ++d) {
            p.in_step[d] = plan.in_out_step[d];
            p.out_step[d] = plan.out_step[d];
            p.out2_step[d] = plan.out2_step[d];
        }
    } else {
        p.out_inner = p.n_out;
        if (plan.out_ndim == 1) {
            p.in_step[1] = plan.in_out_step[0];
            p.out_step[1] = plan.out_step[0];
            p.out2_step[1] = plan.out2_step[0];
        }
    }
    const bool nt = red_use_nt(plan.out_total * plan.red_total * sizeof(In));
    const dim3 b(kRedBlock);

    if (plan.kind == RED_COL) {
        if (plan.in_out_step[plan.out_ndim - 1] != (int64_t)sizeof(In)) return 0;
        p.lsplit_bits = (uint32_t)plan.local_split_bits;
        const uint64_t per_block = (uint64_t)kRedBlock >> p.lsplit_bits;
        const uint64_t groups = (uint64_t)(p.n_out / p.out_inner) * (((uint64_t)p.out_inner + V - 1) / V);
        uint64_t grid = (groups + per_block - 1) / per_block;
        if (plan.n_split > 1) {
            // The axis is cut across blocks as well: accumulators to scratch, a second launch folds them.
            if (grid > 65535) return 0;
            const uint64_t bchunk = (plan.red_total + (uint64_t)plan.n_split - 1) / (uint64_t)plan.n_split;
            const uint64_t n_split = (plan.red_total + bchunk - 1) / bchunk;  // no part is empty
            if (n_split < 2 || n_split > 65535) return 0;
            p.n_split = (uint32_t)n_split;
            p.chunk = bchunk;
            const size_t parts_row = rs_parts_row(p.n_out, p.out_inner, V);
            const uint64_t scratch_bytes = sizeof(Acc) * parts_row * n_split;
            if (fixed) {
                if (scratch_bytes > fixed->bytes) return -1;
                p.partial = fixed->ptr;
                fixed->used = scratch_bytes;
            } else {
                p.partial = cumo_cuda_runtime_malloc(scratch_bytes);
                if (!p.partial) return 1;  // the pool has reported it
            }
            const dim3 g2((unsigned)grid, (unsigned)n_split);
            if (nt) hipLaunchKernelGGL((red_scol_kernel<Impl, V, true, true, 4, true>), g2, b, 0, stream, p, impl);
            else hipLaunchKernelGGL((red_scol_kernel<Impl, V, false, true, 4, true>), g2, b, 0, stream, p, impl);
            cumo_cuda_runtime_check_kernel_launch();
            // the fold: as many lanes to a group of outputs as give each at most eight parts (a group's 16 bytes of every
            // part next to its neighbours': at least four groups side by side)
            RedSParams pf = p;
            pf.lsplit_bits = 0;
            while (pf.lsplit_bits < 6 && (8ull << pf.lsplit_bits) < n_split) ++pf.lsplit_bits;
            const uint64_t fold_groups = (uint64_t)kRedBlock >> pf.lsplit_bits;
            const dim3 gf((unsigned)((parts_row / V + fold_groups - 1) / fold_groups));
            hipLaunchKernelGGL((red_fold_parts_kernel<Impl, V>), gf, b, 0, stream, pf, impl);
            cumo_cuda_runtime_check_kernel_launch();
            if (!fixed) cumo_cuda_runtime_free(p.partial);
            return 1;
        }
        if (grid > red_grid_cap()) grid = red_grid_cap();
        const dim3 g((unsigned)grid);
        // four positions of the axis in flight per lane: more of them (or narrower blocks) read
        // more rows at a time and measured slower
        if (p.lsplit_bits > 0) {
            if (nt) hipLaunchKernelGGL((red_scol_kernel<Impl, V, true, true, 4>), g, b, 0, stream, p, impl);
            else hipLaunchKernelGGL((red_scol_kernel<Impl, V, false, true, 4>), g, b, 0, stream, p, impl);
        } else {
            if (nt) hipLaunchKernelGGL((red_scol_kernel<Impl, V, true, false, 4>), g, b, 0, stream, p, impl);
            else hipLaunchKernelGGL((red_scol_kernel<Impl, V, false, false, 4>), g, b, 0, stream, p, impl);
        }
        cumo_cuda_runtime_check_kernel_launch();
        return 1;
    }

    if (plan.in_red_step[0] != (int64_t)sizeof(In)) return 0;
    p.tail = (uint32_t)plan.red_tail;
    p.n = plan.red_total - p.tail;
    p.tpr_bits = 0;
    while ((1 << p.tpr_bits) < plan.threads_per_row) ++p.tpr_bits;
    {
        static int force_bits = -2;
        if (force_bits == -2) {
            const char* e = std::getenv("CUMO_HIP_RED_TPR_BITS");
            force_bits = e ? std::atoi(e) : -1;
        }
        if (force_bits >= 0 && force_bits <= 8 && plan.n_split <= 1) p.tpr_bits = (uint32_t)force_bits;
    }
    if (plan.n_split <= 1) {
        const uint64_t rpb = (uint64_t)kRedBlock >> p.tpr_bits;
        uint64_t grid = (plan.out_total + rpb - 1) / rpb;
        if (grid > red_grid_cap()) grid = red_grid_cap();
        const dim3 g((unsigned)grid);
        if (nt) hipLaunchKernelGGL((red_srow_kernel<Impl, V, true>), g, b, 0, stream, p, impl);
        else hipLaunchKernelGGL((red_srow_kernel<Impl, V, false>), g, b, 0, stream, p, impl);
        cumo_cuda_runtime_check_kernel_launch();
        return 1;
    }

    // the axis cut over several blocks per output, one launch
    // no more blocks than the axis has tiles (what a block loads in one step)
    const uint64_t tile = (uint64_t)kRedBlock * V * kRsUnroll;
    const uint64_t tiles = (plan.red_total + tile - 1) / tile;
    p.n_split = (uint32_t)((uint64_t)plan.n_split < tiles ? (uint64_t)plan.n_split : tiles);
    if (p.n_split <= 1) return 0;
    // few outputs: the form without tickets, when the accumulators fit the hand-over words. Not while
    // the stream is being captured: a replayed launch would carry the same launch number again and
    // find the last replay's words (the ticket form leaves its words at zero and replays safely).
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capturing) != hipSuccess) {
        (void)hipGetLastError();
        capturing = hipStreamCaptureStatusActive;
    }
    // The waiting blocks (one per output, started first) may take at most half of what the device
    // certainly keeps resident beside them (two blocks of this size per compute unit): the blocks
    // they wait for then always find room. With fewer compute units than this build was tuned for
    // (a partitioned device) fewer outputs qualify.
    const uint64_t poll_outputs_max = (uint64_t)device_compute_units() < 256 ? (uint64_t)device_compute_units() : 256;
    if (!fixed && red_poll_enabled() && capturing == hipStreamCaptureStatusNone && plan.out_total <= poll_outputs_max &&
        plan.out_total * (uint64_t)p.n_split * (sizeof(Acc) / 4) <= kRsHandoverWords) {
        uint32_t launch = 0;
        uint64_t* words = red_handover_words(stream_slot(stream), &launch);
        p.wait = words != nullptr ? wait_ctl() : nullptr;
        if (words != nullptr && p.wait != nullptr) {
            const dim3 g((unsigned)(plan.out_total * p.n_split + plan.out_total));
            if (nt) hipLaunchKernelGGL((red_srow_poll_kernel<Impl, V, true>), g, b, 0, stream, p, impl, words, launch);
            else hipLaunchKernelGGL((red_srow_poll_kernel<Impl, V, false>), g, b, 0, stream, p, impl, words, launch);
            cumo_cuda_runtime_check_kernel_launch();
            return 1;
        }
    }
    p.group = p.n_split <= (uint32_t)kRsOneLevel ? p.n_split : (uint32_t)kRsGroup;
    const uint64_t groups = (p.n_split + p.group - 1) / p.group;
    {
        static uint32_t stride = 0;
        if (stride == 0) {
            const char* e = std::getenv("CUMO_HIP_RED_TICKET_STRIDE");
            stride = e ? (uint32_t)std::strtoul(e, nullptr, 10) : 0;
            if (stride == 0) stride = 64;
        }
        p.tstride = stride;
        while (p.tstride > 1 && plan.out_total * (1 + groups) * p.tstride > kRsTicketWords) p.tstride >>= 1;
    }
    if (plan.out_total * (1 + groups) * p.tstride > kRsTicketWords) return 0;
    const uint64_t n_blocks = plan.out_total * p.n_split;
    if (n_blocks > 0x7fffffffull) return 0;
    p.tickets = red_ticket_words(stream_slot(stream));
    if (p.tickets == nullptr) return 0;
    const size_t scratch_bytes = sizeof(Acc) * (size_t)n_blocks;
    if (fixed) {
        if (scratch_bytes > fixed->bytes) return -1;
        p.partial = fixed->ptr;
        fixed->used = scratch_bytes;
    } else {
        p.partial = cumo_cuda_runtime_malloc(scratch_bytes);
        if (!p.partial) return 1;  // the pool has reported it
    }
    const dim3 g((unsigned)n_blocks);
    if (nt) hipLaunchKernelGGL((red_srow_split_kernel<Impl, V, true>), g, b, 0, stream, p, impl);
    else hipLaunchKernelGGL((red_srow_split_kernel<Impl, V, false>), g, b, 0, stream, p, impl);
    cumo_cuda_runtime_check_kernel_launch();
    // the next owner of the scratch can only touch it from work queued later on this stream
    if (!fixed) cumo_cuda_runtime_free(p.partial);
    return 1;
}

// index_mode: 1 for arg reductions, 2 for *_index reductions, ignored by impls
// that do not use the index. The scratch of a split reduction comes from the
// pool and goes back right after the second launch is queued: the next owner
// can only touch it from work queued later on the same stream
// (reference: include/cumo/reduce_kernel.h:493-496).
// With `fixed` the partial results of a split reduction go to the caller's device memory
// instead (fixed->ptr, fixed->bytes): nothing is allocated or released, and a reduction
// whose partial results do not fit is refused (returns false, nothing launched).
template <class I, class = void> struct reduces_own_results { static constexpr bool value = false; };
template <class I> struct reduces_own_results<I, decltype((void)I::OWN_RESULTS)> { static constexpr bool value = I::OWN_RESULTS; };

template <class Impl>
static bool reduce_launch(const cumo_na_reduction_arg_t* arg, const cumo_na_iarray_t* out2, Impl impl, int index_mode,
                          const RedScratch* fixed = nullptr) {
    typedef typename Impl::In In;
    typedef typename Impl::Acc Acc;
    if (arg->out_indexer.total_size == 0) return true;  // reference: reduce_kernel.h:444-446
    ReducePlan plan;
    // the lean row kernels fold what a run has past its last whole vector by themselves
    plan_reduce(arg, out2, (int)sizeof(In), (int)sizeof(Acc), &plan, true);
    if (plan.kind == RED_EMPTY) return true;
    hipStream_t stream = current_stream();
    // Lanes along a reduce axis that strides through memory while another dimension of the view runs along it (the
    // full reduction of a transposed view): every lane would fetch a cache line for one element. The view is copied
    // into its own order first (the typed store transposes through LDS) and reduced from the copy, positions and all:
    // [4096,8192] SFloat x.transpose.max 393 -> 70 us. Not for the forms that answer offsets into the original array.
    if constexpr (sizeof(In) == 4 || sizeof(In) == 8) {
        const int nd = arg->in_indexer.ndim, no = arg->out_indexer.ndim;
        if (plan.kind == RED_ROW && index_mode != 2 && fixed == nullptr && nd > no && nd <= CUMO_NA_MAX_DIMENSION &&
            arg->in_indexer.total_size >= 65536) {
            int L = -1;
            for (int d = no; d < nd; ++d)
                if (arg->in_indexer.shape[d] > 1) L = d;
            const int64_t es = (int64_t)sizeof(In);
            bool strided = L >= 0 && arg->in_indexer.shape[L] >= 16 && arg->in.step[L] != es && arg->in.step[L] != -es && arg->in.step[L] != 0;
            bool other_runs = false;
            for (int d = 0; d < nd && strided; ++d)
                if (d != L && arg->in_indexer.shape[d] >= 16 && (arg->in.step[d] == es || arg->in.step[d] == -es)) other_runs = true;
            if (strided && other_runs) {
                char* copy = cumo_cuda_runtime_malloc(arg->in_indexer.total_size * sizeof(In));
                if (!copy) return true;  // the pool has reported it
                cumo_na_reduction_arg_t staged = *arg;
                cumo_na_iarray_t dst;
                dst.ptr = copy;
                ssize_t s = (ssize_t)sizeof(In);
                for (int d = nd - 1; d >= 0; --d) {
                    dst.step[d] = s;
                    s *= (ssize_t)arg->in_indexer.shape[d];
                }
                cumo_na_indexer_t ix = arg->in_indexer;
                cumo_na_iarray_t src = arg->in;
                if (sizeof(In) == 4) cumo_iter_int32_store_int32_kernel_launch(&dst, &src, &ix);
                else cumo_iter_dfloat_store_dfloat_kernel_launch(&dst, &src, &ix);
                staged.in = dst;
                const bool done = reduce_launch(&staged, out2, impl, index_mode, fixed);
                cumo_cuda_runtime_free(copy);
                return done;
            }
        }
    }
    // One result over a view whose rows run along memory but do not follow one another (x[true, 1..-1].sum): the rows
    // first, each with the lanes of the row kernels, into a scratch vector, then the vector. Only where a result can
    // stand in for the elements it came from. SFloat [8192,4095] of [8192,4096]: sum 55 -> 27 us.
    if constexpr (reduces_own_results<Impl>::value) {
        const int64_t es = (int64_t)sizeof(In);
        const int nr = plan.red_ndim;
        if (fixed == nullptr && out2 == nullptr && plan.out_total == 1 && nr >= 2 && nr <= CUMO_NA_MAX_DIMENSION && plan.in_red_step[nr - 1] == es &&
            plan.red_shape[nr - 1] >= 64 && plan.red_total >= 65536) {
            const uint64_t inner = plan.red_shape[nr - 1], rows = plan.red_total / inner;
            char* partial = cumo_cuda_runtime_malloc(rows * sizeof(In));
            if (!partial) return true;  // the pool has reported it
            // the outer reduce dimensions are the first launch's output dimensions, their results one run
            cumo_na_reduction_arg_t a1;
            std::memset(&a1, 0, sizeof(a1));
            a1.in.ptr = arg->in.ptr;
            a1.out.ptr = partial;
            ssize_t run = (ssize_t)es;
            for (int d = nr - 2; d >= 0; --d) {
                a1.in.step[d] = (ssize_t)plan.in_red_step[d];
                a1.in_indexer.shape[d] = plan.red_shape[d];
                a1.out.step[d] = run;
                a1.out_indexer.shape[d] = plan.red_shape[d];
                run *= (ssize_t)plan.red_shape[d];
            }
            a1.in.step[nr - 1] = (ssize_t)es;
            a1.in_indexer.shape[nr - 1] = inner;
            a1.in_indexer.ndim = (unsigned char)nr;
            a1.in_indexer.total_size = rows * inner;
            a1.out_indexer.ndim = (unsigned char)(nr - 1);
            a1.out_indexer.total_size = rows;
            reduce_launch(&a1, nullptr, impl.before_the_last(), index_mode);
            cumo_na_reduction_arg_t a2;
            std::memset(&a2, 0, sizeof(a2));
            a2.in.ptr = partial;
            a2.in.step[0] = (ssize_t)es;
            a2.in_indexer.ndim = 1;
            a2.in_indexer.shape[0] = rows;
            a2.in_indexer.total_size = rows;
            a2.out.ptr = arg->out.ptr;
            a2.out_indexer.ndim = 0;
            a2.out_indexer.total_size = 1;
            const bool done = reduce_launch(&a2, nullptr, impl, index_mode);
            cumo_cuda_runtime_free(partial);
            return done;
        }
    }
    {
        const int taken = red_stream_launch(plan, arg, out2, impl, index_mode, fixed, stream);
        if (taken != 0) return taken > 0;
    }
    // the general kernels want whole vectors
    if (plan.red_tail != 0) plan_reduce(arg, out2, (int)sizeof(In), (int)sizeof(Acc), &plan, false);
    RedKParams kp;
    red_fill_params(&kp, plan, arg, out2, index_mode);
    kp.tpr_bits = 0;
    while ((1 << kp.tpr_bits) < plan.threads_per_row) ++kp.tpr_bits;
    kp.lsplit_bits = plan.kind == RED_COL ? plan.local_split_bits : 0;

    if (plan.n_split <= 1) {
        if (plan.kind == RED_COL) red_launch_col<Impl, false>(kp, plan.vec, impl, nullptr, stream);
        else red_launch_row<Impl, false>(kp, plan.vec, impl, nullptr, stream);
        cumo_cuda_runtime_check_kernel_launch();
        return true;
    }

    // first pass
    const uint64_t ns = (uint64_t)plan.n_split;
    uint64_t chunk = (plan.red_total + ns - 1) / ns;
    if (plan.kind == RED_ROW) {
        // whole vectors per lane: chunks start on a multiple of the vector width
        const uint64_t q = (uint64_t)plan.vec;
        chunk = ((chunk + q - 1) / q) * q;
    }
    kp.n_split = (plan.red_total + chunk - 1) / chunk;
    kp.chunk = chunk;
    const uint64_t n_partial = plan.out_total * kp.n_split;
    Acc* partial;
    if (fixed) {
        if (sizeof(Acc) * n_partial > fixed->bytes) return false;
        partial = reinterpret_cast<Acc*>(fixed->ptr);
        fixed->used = sizeof(Acc) * n_partial;
    } else {
        partial = reinterpret_cast<Acc*>(cumo_cuda_runtime_malloc(sizeof(Acc) * n_partial));
        if (!partial) return true;  // the pool has reported it
    }
    if (plan.kind == RED_COL) red_launch_col<Impl, true>(kp, plan.vec, impl, partial, stream);
    else red_launch_row<Impl, true>(kp, plan.vec, impl, partial, stream);
    cumo_cuda_runtime_check_kernel_launch();

    red_fold_partials<Impl>(plan, kp, partial, impl, stream);
    if (!fixed) cumo_cuda_runtime_free(reinterpret_cast<char*>(partial));
    return true;
}

// A form that only the lean kernels run (an accumulator their exact protocol knows and the general kernels' does
// not) where they take the reduction, the other form through everything else.
template <class Fast, class Slow>
static bool reduce_launch_lean_or(const cumo_na_reduction_arg_t* arg, const cumo_na_iarray_t* out2, Fast fast, Slow slow, int slow_index_mode) {
    if (arg->out_indexer.total_size == 0) return true;
    ReducePlan plan;
    plan_reduce(arg, out2, (int)sizeof(typename Fast::In), (int)sizeof(typename Fast::Acc), &plan, true);
    if (plan.kind == RED_EMPTY) return true;
    const int taken = red_stream_launch(plan, arg, out2, fast, 0, nullptr, current_stream());
    if (taken != 0) return taken > 0;
    return reduce_launch(arg, out2, slow, slow_index_mode);
}

}  // namespace cumo_hip

#endif