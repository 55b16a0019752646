// Row-wise composites that a Cumo program writes as a chain of array operations,
// done in one pass over each row:
//
//   softmax     m = x.max(axis:-1, keepdims:true); e = NMath.exp(x - m); e / e.sum(axis:-1, keepdims:true)
//   layernorm   (x - x.mean(axis:-1, keepdims:true)) / NMath.sqrt(x.var(axis:-1, keepdims:true) + eps)
//
// (the shapes of bench/transformer_bench.rb:110-124 of the reference). As separate
// launches the first moves 9 x the array (5 launches), the second 6.5 x (6
// launches); here a row is read once into registers, reduced across the lanes that
// share it with wave64 shuffles (and four LDS slots when a block shares it), and the
// result written once: 2 x the array. Every elementwise step is the same single
// IEEE operation the separate launches perform (float subtraction, the sqrt that is
// the double-precision function rounded once, float division); the SFloat softmax's
// exponential is the double-precision 2^(x log2 e) of the table-driven core rounded
// once, which differs from NMath.exp's float in the last place at about one argument
// in 10^4. Results differ from the chain through that and the order of the two row sums.
//
// The reference has no such entry point; the host layer (cumo_hip_na_softmax /
// cumo_hip_na_layernorm) uses these for contiguous rows of up to 16384 elements and
// composes the chain otherwise.
#include "common.h"
#include "ew_ops.h"

#include <cstring>

namespace cumo_hip {
namespace {

constexpr int kFrBlock = 256;

template <class T>
__device__ __forceinline__ T fr_shfl_xor(T v, int m) {
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

// Combines one value per lane over the TPR lanes that share a row; every lane gets
// the result. The order is fixed (butterfly within the wave, then the four waves in
// index order), so results do not vary from launch to launch.
template <class T, int TPR, class F>
__device__ __forceinline__ T fr_allreduce(T v, F f) {
    constexpr int SPAN = TPR < 64 ? TPR : 64;
#pragma unroll
    for (int m = SPAN >> 1; m > 0; m >>= 1) v = f(v, fr_shfl_xor(v, m));
    if constexpr (TPR > 64) {
        __shared__ T slot[kFrBlock / 64];
        __syncthreads();  // the slots may still be read from the previous use
        if ((threadIdx.x & 63) == 0) slot[threadIdx.x >> 6] = v;
        __syncthreads();
        v = slot[0];
#pragma unroll
        for (int w = 1; w < kFrBlock / 64; ++w) v = f(v, slot[w]);
    }
    return v;
}

template <class T> __device__ __forceinline__ T fr_exp(T x);
// SFloat: 2^(x log2 e) from the table-driven core of ew_ops.h (2^-39 relative before the rounding to float; the
// element operator's polynomial form is good to 2^-50, which a softmax, divided by a sum of 2^-24 terms, cannot
// show): eight double operations fewer an element in a kernel that the exponential's arithmetic bounds.
// A NaN passes through the arithmetic; the clamp keeps the exponent in the core's range.
template <> __device__ __forceinline__ float fr_exp<float>(float x) {
    float xc = (x < -105.0f) ? -105.0f : x;
    xc = (xc > 89.0f) ? 89.0f : xc;
    return (float)exp2_by_table(1.44269504088896338700e+00 * (double)xc, float_tables());
}
template <> __device__ __forceinline__ double fr_exp<double>(double x) { return exp(x); }
template <class T> __device__ __forceinline__ T fr_sqrt(T x) { return (T)sqrt((double)x); }

// max that answers NaN when any element is NaN, as the reduction does (all-NaN or
// any-NaN max is NaN on the device: narray_test.rb:2551-2560)
template <class T> __device__ __forceinline__ T fr_max_nan(T a, T b) { return (a != a) ? a : ((b != b) ? b : (a > b ? a : b)); }

template <class T> __device__ __forceinline__ T fr_fmax(T a, T b);
template <> __device__ __forceinline__ float fr_fmax<float>(float a, float b) { return __builtin_fmaxf(a, b); }
template <> __device__ __forceinline__ double fr_fmax<double>(double a, double b) { return __builtin_fmax(a, b); }

// x / s for many x and one s, with the result of the IEEE division in T.
// float: x / s = float(double(x) * (1.0 / double(s))). The product is within 2^-52 of
// the quotient, while the quotient of two 24-bit numbers is never closer than 2^-49
// (relative) to the midpoint of two floats unless it is a float itself, so the one
// rounding to float lands where the division's does; zero, infinity and NaN behave
// alike on both routes, and a subnormal quotient is rounded once by the conversion.
template <class T> struct FrDivisor;
template <> struct FrDivisor<float> {
    double r;
    __device__ __forceinline__ explicit FrDivisor(float s) : r(1.0 / (double)s) {}
    __device__ __forceinline__ float divide(float x) const { return (float)((double)x * r); }
};
template <> struct FrDivisor<double> {
    double s;
    __device__ __forceinline__ explicit FrDivisor(double s_) : s(s_) {}
    __device__ __forceinline__ double divide(double x) const { return x / s; }
};

struct FusedRowsParams {
    uint64_t rows, n;
    int64_t in_row_step, out_row_step;  // bytes
    const char* in;
    char* out;
    double eps;
};

// MODE 0 softmax, 1 layernorm. TPR lanes share a row, each holding NV vectors of V
// elements (TPR * NV * V >= n). Rows, vectors and the elements of a row's last vector beyond the data are masked.
// NT: non-temporal accesses, for arrays larger than the last-level cache.
template <class T, int MODE, int TPR, int NV, bool NT>
__global__ __launch_bounds__(kFrBlock) void fused_rows_kernel(FusedRowsParams p) {
    constexpr int V = 16 / (int)sizeof(T);
    constexpr int RPB = kFrBlock / TPR;  // rows per block
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    union Vec { u4 q; T t[V]; __device__ Vec() {} };
    const unsigned lane_r = threadIdx.x % TPR;
    const unsigned row_in_block = threadIdx.x / TPR;
    const uint64_t n_row_blocks = (p.rows + RPB - 1) / RPB;
    if constexpr (MODE == 0 && sizeof(T) == 4) float_tables_prepare();  // (the SFloat softmax reads the 2^x table)
    for (uint64_t rb = blockIdx.x; rb < n_row_blocks; rb += gridDim.x) {
        const uint64_t row = rb * RPB + row_in_block;
        const bool row_ok = row < p.rows;
        const char* src = p.in + (int64_t)(row_ok ? row : 0) * p.in_row_step;
        char* dst = p.out + (int64_t)(row_ok ? row : 0) * p.out_row_step;
        Vec x[NV];
        int cnt[NV];  // how many elements of the vector exist: V, none, or (the row's last vector) fewer
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const uint64_t col = ((uint64_t)k * TPR + lane_r) * V;
            const int64_t left = (int64_t)p.n - (int64_t)col;
            cnt[k] = row_ok ? (left >= V ? V : (left > 0 ? (int)left : 0)) : 0;
            // a lane without a whole vector re-reads the row's first one: no branch between the loads
            const u4* ld = reinterpret_cast<const u4*>(src + (cnt[k] == V ? col : 0) * sizeof(T));
            x[k].q = NT ? __builtin_nontemporal_load(ld) : *ld;
        }
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            if (cnt[k] > 0 && cnt[k] < V) {
                // part of a vector at the row's end: element by element, nothing read past the row
                const uint64_t col = ((uint64_t)k * TPR + lane_r) * V;
#pragma unroll
                for (int j = 0; j < V; ++j)
                    if (j < cnt[k]) x[k].t[j] = reinterpret_cast<const T*>(src)[col + j];
            }
        }
        auto put = [&](int k) {
            const uint64_t col = ((uint64_t)k * TPR + lane_r) * V;
            if (cnt[k] == V) {
                u4* st = reinterpret_cast<u4*>(dst + col * sizeof(T));
                if (NT) __builtin_nontemporal_store(x[k].q, st);
                else *st = x[k].q;
            } else {
#pragma unroll
                for (int j = 0; j < V; ++j)
                    if (j < cnt[k]) reinterpret_cast<T*>(dst)[col + j] = x[k].t[j];
            }
        };
        if constexpr (MODE == 0) {
            // Lanes without data hold -inf: neutral in the max, and exp(-inf - m) adds 0 to the sum.
            // The max keeps the larger non-NaN value per element and notes NaN apart (one maximum and
            // one compare per element); a NaN anywhere then replaces the row's max, as in the reduction.
            T m = -INFINITY;
            bool any_nan = false;
#pragma unroll
            for (int k = 0; k < NV; ++k) {
#pragma unroll
                for (int j = 0; j < V; ++j) {
                    const T v = j < cnt[k] ? x[k].t[j] : (T)-INFINITY;
                    x[k].t[j] = v;
                    any_nan |= (v != v);
                    m = fr_fmax(m, v);
                }
            }
            if (any_nan) m = (T)NAN;
            m = fr_allreduce<T, TPR>(m, [](T a, T b) { return fr_max_nan(a, b); });
            T s = 0;
#pragma unroll
            for (int k = 0; k < NV; ++k) {
#pragma unroll
                for (int j = 0; j < V; ++j) {
                    const T e = fr_exp<T>(x[k].t[j] - m);
                    x[k].t[j] = e;
                    s += e;
                }
            }
            s = fr_allreduce<T, TPR>(s, [](T a, T b) { return a + b; });
            const FrDivisor<T> by_s(s);
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                if (cnt[k] > 0) {
#pragma unroll
                    for (int j = 0; j < V; ++j) x[k].t[j] = by_s.divide(x[k].t[j]);
                    put(k);
                }
            }
        } else {
            // mean, then the squared deviations from it: two passes over registers
            T s = 0;
#pragma unroll
            for (int k = 0; k < NV; ++k) {
#pragma unroll
                for (int j = 0; j < V; ++j)
                    if (j < cnt[k]) s += x[k].t[j];
            }
            s = fr_allreduce<T, TPR>(s, [](T a, T b) { return a + b; });
            const T mean = s / (T)p.n;
            T q = 0;
#pragma unroll
            for (int k = 0; k < NV; ++k) {
#pragma unroll
                for (int j = 0; j < V; ++j) {
                    const T c = x[k].t[j] - mean;
                    x[k].t[j] = c;
                    if (j < cnt[k]) q += c * c;
                }
            }
            q = fr_allreduce<T, TPR>(q, [](T a, T b) { return a + b; });
            const T var = q / ((T)p.n - (T)1);
            const T sd = fr_sqrt<T>(var + (T)p.eps);
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                if (cnt[k] > 0) {
#pragma unroll
                    for (int j = 0; j < V; ++j) x[k].t[j] = x[k].t[j] / sd;
                    put(k);
                }
            }
        }
    }
}

template <class T, int MODE, int TPR, int NV>
void fr_launch_one(const FusedRowsParams& p, hipStream_t stream) {
    constexpr int RPB = kFrBlock / TPR;
    uint64_t grid = (p.rows + RPB - 1) / RPB;
    if (grid > 256u * 64u) grid = 256u * 64u;
    // one read and one write of the array: beyond the 256 MB last-level cache, stream past it
    const bool nt = stream_past_caches(2 * p.rows * p.n * sizeof(T));
    if (nt) hipLaunchKernelGGL((fused_rows_kernel<T, MODE, TPR, NV, true>), dim3((unsigned)grid), dim3(kFrBlock), 0, stream, p);
    else hipLaunchKernelGGL((fused_rows_kernel<T, MODE, TPR, NV, false>), dim3((unsigned)grid), dim3(kFrBlock), 0, stream, p);
}

// picks lanes per row and vectors per lane for the row length (four vectors per lane
// where the row allows, so that a lane has four loads in flight); false when the row
// is too long
template <class T, int MODE>
bool fr_launch(const FusedRowsParams& p, hipStream_t stream) {
    constexpr int V = 16 / (int)sizeof(T);
    const uint64_t nv = (p.n + V - 1) / V;  // vectors per row, the last one maybe partly there
    if (nv <= 8) fr_launch_one<T, MODE, 8, 1>(p, stream);
    else if (nv <= 16) fr_launch_one<T, MODE, 8, 2>(p, stream);
    else if (nv <= 32) fr_launch_one<T, MODE, 8, 4>(p, stream);
    else if (nv <= 64) fr_launch_one<T, MODE, 16, 4>(p, stream);
    else if (nv <= 128) fr_launch_one<T, MODE, 32, 4>(p, stream);
    else if (nv <= 256) fr_launch_one<T, MODE, 64, 4>(p, stream);
    else if (nv <= 512) fr_launch_one<T, MODE, 256, 2>(p, stream);
    else if (nv <= 1024) fr_launch_one<T, MODE, 256, 4>(p, stream);
    else if (nv <= 2048) fr_launch_one<T, MODE, 256, 8>(p, stream);
    else if (nv <= 4096 && sizeof(T) == 4) fr_launch_one<T, MODE, 256, 16>(p, stream);
    else return false;
    return true;
}

}  // namespace
}  // namespace cumo_hip

using namespace cumo_hip;

// type: 0 SFloat, 1 DFloat. mode: 0 softmax, 1 layernorm. Returns 1 when the launch
// was made, 0 when the shape is outside what the kernels take (rows shorter than one
// 128-bit vector, not aligned as their elements are, or too long): the caller
// composes the operations instead.
extern "C" int cumo_hip_fused_rows_kernel_launch(int type, int mode, const cumo_hip_fused_rows_t* d) {
    if (!d || d->rows == 0 || d->n == 0) return 1;
    const int es = type == 0 ? 4 : 8;
    const uint64_t v = 16 / es;
    if (type < 0 || type > 1 || mode < 0 || mode > 1) return 0;
    // rows need their element's alignment only (128-bit accesses work on any 4-byte boundary) and may end in
    // part of a vector, which goes element by element
    if (d->n < v) return 0;
    if (((uintptr_t)d->in % es) || ((uintptr_t)d->out % es) || (d->in_row_step % es) || (d->out_row_step % es)) return 0;
    FusedRowsParams p;
    p.rows = d->rows;
    p.n = d->n;
    p.in_row_step = d->in_row_step;
    p.out_row_step = d->out_row_step;
    p.in = d->in;
    p.out = d->out;
    p.eps = d->eps;
    hipStream_t stream = current_stream();
    bool ok;
    if (type == 0) ok = mode == 0 ? fr_launch<float, 0>(p, stream) : fr_launch<float, 1>(p, stream);
    else ok = mode == 0 ? fr_launch<double, 0>(p, stream) : fr_launch<double, 1>(p, stream);
    if (ok) cumo_cuda_runtime_check_kernel_launch();
    return ok ? 1 : 0;
}
