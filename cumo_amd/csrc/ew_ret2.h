// Elementwise operations with two results (frexp, modf, divmod; reference:
// narray/gen/tmpl/frexp_kernel.cu, unary_ret2_kernel.cu, binary2_kernel.cu). Rare enough
// to get the plain form: one element per thread, its position decomposed over the loop
// dimensions, every operand with its own steps.
//
// Op contract: static constexpr int NIN (1 or 2); typedef In, Out1, Out2;
// __device__ bool operator()(In x, In y, Out1& a, Out2& b) const -- false leaves the
// element unwritten and raises the flag (Int32 division by zero).
#ifndef CUMO_HIP_EW_RET2_H
#define CUMO_HIP_EW_RET2_H

#include "common.h"

namespace cumo_hip {

struct Ret2Params {
    int ndim;
    uint64_t total;
    uint64_t shape[CUMO_NA_MAX_DIMENSION];
    int64_t step[4][CUMO_NA_MAX_DIMENSION];  // inputs first, then the two results
    char* ptr[4];
    int* flag;
};

template <class Op>
__global__ __launch_bounds__(256) void ret2_kernel(Ret2Params p, Op op) {
    typedef typename Op::In In;
    constexpr int NA = Op::NIN + 2;
    for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < p.total; i += (uint64_t)gridDim.x * 256) {
        uint64_t r = i;
        int64_t off[NA];
#pragma unroll
        for (int a = 0; a < NA; ++a) off[a] = 0;
        for (int d = p.ndim - 1; d >= 0; --d) {
            const uint64_t n = p.shape[d];
            const uint64_t q = r / n;
            const int64_t k = (int64_t)(r - q * n);
            r = q;
#pragma unroll
            for (int a = 0; a < NA; ++a) off[a] += k * p.step[a][d];
        }
        const In x = *reinterpret_cast<const In*>(p.ptr[0] + off[0]);
        const In y = Op::NIN == 2 ? *reinterpret_cast<const In*>(p.ptr[1] + off[1]) : In();
        typename Op::Out1 a;
        typename Op::Out2 b;
        if (!op(x, y, a, b)) {
            if (p.flag) *p.flag = 1;
            continue;
        }
        *reinterpret_cast<typename Op::Out1*>(p.ptr[Op::NIN] + off[Op::NIN]) = a;
        *reinterpret_cast<typename Op::Out2*>(p.ptr[Op::NIN + 1] + off[Op::NIN + 1]) = b;
    }
}

// Every operand one contiguous run: a lane takes the elements of one 128-bit vector of the input type
// (vectors need the element's alignment only); an element that the op refuses is left unwritten, so a
// vector with one of those is stored element by element.
template <class X, int V, bool NT>
__device__ __forceinline__ void ret2_load(const X* p, X (&v)[V]) {
    typedef X XV __attribute__((ext_vector_type(V)));
    const XV t = NT ? __builtin_nontemporal_load(reinterpret_cast<const XV*>(p)) : *reinterpret_cast<const XV*>(p);
#pragma unroll
    for (int j = 0; j < V; ++j) v[j] = t[j];
}
template <class X, int V, bool NT>
__device__ __forceinline__ void ret2_store(X* p, const X (&v)[V]) {
    typedef X XV __attribute__((ext_vector_type(V)));
    XV t;
#pragma unroll
    for (int j = 0; j < V; ++j) t[j] = v[j];
    if (NT) __builtin_nontemporal_store(t, reinterpret_cast<XV*>(p));
    else *reinterpret_cast<XV*>(p) = t;
}

template <class Op, bool NT>
__global__ __launch_bounds__(256) void ret2_flat_kernel(const typename Op::In* px, const typename Op::In* py, typename Op::Out1* pa,
                                                        typename Op::Out2* pb, uint64_t n, int* flag, Op op) {
    typedef typename Op::In In;
    constexpr int V = 16 / sizeof(In);
    const uint64_t nv = (n + V - 1) / V;
    for (uint64_t v = (uint64_t)blockIdx.x * 256 + threadIdx.x; v < nv; v += (uint64_t)gridDim.x * 256) {
        const uint64_t e = v * V;
        const bool whole = e + V <= n;
        In x[V], y[V];
        if (whole) {
            ret2_load<In, V, NT>(px + e, x);
            if (Op::NIN == 2) ret2_load<In, V, NT>(py + e, y);
        } else {
#pragma unroll
            for (int j = 0; j < V; ++j) {
                x[j] = e + j < n ? px[e + j] : In();
                if (Op::NIN == 2) y[j] = e + j < n ? py[e + j] : In();
            }
        }
        typename Op::Out1 a[V];
        typename Op::Out2 b[V];
        bool ok[V], all = true;
#pragma unroll
        for (int j = 0; j < V; ++j) {
            ok[j] = op(x[j], Op::NIN == 2 ? y[j] : In(), a[j], b[j]);
            if (whole || e + j < n) all = all && ok[j];
        }
        if (whole && all) {
            ret2_store<typename Op::Out1, V, NT>(pa + e, a);
            ret2_store<typename Op::Out2, V, NT>(pb + e, b);
        } else {
#pragma unroll
            for (int j = 0; j < V; ++j) {
                if (e + j < n && ok[j]) {
                    pa[e + j] = a[j];
                    pb[e + j] = b[j];
                }
            }
            if (!all && flag) *flag = 1;
        }
    }
}

template <class X>
static bool ret2_one_run(const cumo_na_iarray_t* a, const cumo_na_indexer_t* indexer) {
    int64_t want = (int64_t)sizeof(X);
    for (int d = indexer->ndim - 1; d >= 0; --d) {
        if (indexer->shape[d] == 1) continue;
        if ((int64_t)a->step[d] != want) return false;
        want *= (int64_t)indexer->shape[d];
    }
    return ((uintptr_t)a->ptr % sizeof(X)) == 0;
}

// arr: the NIN inputs, then the two results
template <class Op>
static void ret2_launch(Op op, const cumo_na_iarray_t* const* arr, const cumo_na_indexer_t* indexer, int* flag) {
    if (indexer->total_size == 0) return;
    constexpr int NA = Op::NIN + 2;
    {
        typedef typename Op::In In;
        bool flat = !force_wide_indices() && indexer->total_size >= 1024 && ret2_one_run<In>(arr[0], indexer);
        if (Op::NIN == 2) flat = flat && ret2_one_run<In>(arr[1], indexer);
        flat = flat && ret2_one_run<typename Op::Out1>(arr[Op::NIN], indexer) && ret2_one_run<typename Op::Out2>(arr[Op::NIN + 1], indexer);
        if (flat) {
            constexpr uint64_t V = 16 / sizeof(In);
            const uint64_t n = indexer->total_size;
            uint64_t g = ((n + V - 1) / V + 255) / 256;
            if (g > 256u * 32u) g = 256u * 32u;
            const In* px = reinterpret_cast<const In*>(arr[0]->ptr);
            const In* py = Op::NIN == 2 ? reinterpret_cast<const In*>(arr[1]->ptr) : nullptr;
            typename Op::Out1* pa = reinterpret_cast<typename Op::Out1*>(arr[Op::NIN]->ptr);
            typename Op::Out2* pb = reinterpret_cast<typename Op::Out2*>(arr[Op::NIN + 1]->ptr);
            if (stream_past_caches(n * sizeof(In) * 2))
                hipLaunchKernelGGL((ret2_flat_kernel<Op, true>), dim3((unsigned)g), dim3(256), 0, current_stream(), px, py, pa, pb, n, flag, op);
            else
                hipLaunchKernelGGL((ret2_flat_kernel<Op, false>), dim3((unsigned)g), dim3(256), 0, current_stream(), px, py, pa, pb, n, flag, op);
            cumo_cuda_runtime_check_kernel_launch();
            return;
        }
    }
    Ret2Params p;
    p.ndim = indexer->ndim;
    p.total = indexer->total_size;
    for (int d = 0; d < CUMO_NA_MAX_DIMENSION; ++d) {
        p.shape[d] = d < indexer->ndim ? indexer->shape[d] : 1;
        for (int a = 0; a < 4; ++a) p.step[a][d] = (a < NA && d < indexer->ndim) ? arr[a]->step[d] : 0;
    }
    for (int a = 0; a < 4; ++a) p.ptr[a] = a < NA ? arr[a]->ptr : nullptr;
    p.flag = flag;
    uint64_t grid = (p.total + 255) / 256;
    if (grid > 65536) grid = 65536;
    hipLaunchKernelGGL((ret2_kernel<Op>), dim3((unsigned)grid), dim3(256), 0, current_stream(), p, op);
    cumo_cuda_runtime_check_kernel_launch();
}

// types/float_macro_kernel.h:123 (frexp), :51 (modf: y the fraction, z the integral part), :35 (divmod)
template <class T> struct OpFrexp {
    static constexpr int NIN = 1;
    typedef T In; typedef T Out1; typedef int32_t Out2;
    __device__ __forceinline__ bool operator()(T x, T, T& m, int32_t& e) const {
        int ex = 0;
        m = (T)frexp(x, &ex);
        e = (int32_t)ex;
        return true;
    }
};
template <class T> struct OpModf {
    static constexpr int NIN = 1;
    typedef T In; typedef T Out1; typedef T Out2;
    __device__ __forceinline__ bool operator()(T x, T, T& frac, T& whole) const {
        double d;
        frac = (T)modf((double)x, &d);
        whole = (T)d;
        return true;
    }
};
template <class T> struct OpDivmodF {
    static constexpr int NIN = 2;
    typedef T In; typedef T Out1; typedef T Out2;
    __device__ __forceinline__ bool operator()(T x, T y, T& a, T& b) const {
        a = x / y;
        b = (T)fmod((double)x, (double)y);
        return true;
    }
};
// types/xint_macro_kernel.h:19-20 with the zero check of binary2_kernel.cu:4-8; INT_MIN / -1 wraps
struct OpDivmodI {
    static constexpr int NIN = 2;
    typedef int32_t In; typedef int32_t Out1; typedef int32_t Out2;
    __device__ __forceinline__ bool operator()(int32_t x, int32_t y, int32_t& a, int32_t& b) const {
        if (y == 0) return false;
        if (y == -1) {
            a = (int32_t)(0u - (uint32_t)x);
            b = 0;
            return true;
        }
        a = x / y;
        b = x % y;
        return true;
    }
};

}  // namespace cumo_hip

#endif
