// cumsum / cumprod: inclusive scans along one run of a view.
//
// Replaces narray/gen/tmpl/cum_kernel.cu of the reference, which hands each run
// to thrust::inclusive_scan (one call per run, walked on the host:
// narray/gen/tmpl/cum.c:12-46). The operators are the reference's
// (types/real_accum_kernel.h:12-26, xint_macro_kernel.h:46-47); the nan forms
// treat NaN as "nothing yet", which makes them associative like the plain ones.
// Like a sum, a parallel float scan does not add strictly left to right.
//
// Two kernels:
//   scan_rows_kernel   one block per run, tile after tile with the running value
//                      carried along: many runs (an axis of a matrix), or short ones.
//   three launches     for few long runs: per-tile totals, a scan of the totals by
//                      one block, then every tile scans itself from its offset.
//                      Reads the input twice and writes once.
// Inside a tile each lane owns 8 consecutive elements: it scans them in registers,
// the lane totals are scanned across the wave with shuffles and the four wave
// totals through LDS. Everything is in a fixed order, so results do not change
// from launch to launch.
#include "common.h"

#include <cstring>

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
template <class T, class Op>
__device__ __forceinline__ void scan_tile(T (&v)[kScanPer], int cnt, T& carry, bool& has_carry) {
    __shared__ T wave_tot[kScanBlock / 64];
    __shared__ int wave_has[kScanBlock / 64];
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
    for (int j = 0; j < kScanBlock / 64; ++j) {
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

template <class T>
__device__ __forceinline__ void scan_load(const char* p, int64_t s, uint64_t first, int cnt, T (&v)[kScanPer]) {
    const int base = threadIdx.x * kScanPer;
    if (s == (int64_t)sizeof(T) && base + kScanPer <= cnt && ((reinterpret_cast<uintptr_t>(p) + (first + base) * sizeof(T)) & 15) == 0) {
        typedef uint32_t u4 __attribute__((ext_vector_type(4)));
        constexpr int NV = (int)(kScanPer * sizeof(T) / 16);
        union { T t[kScanPer]; u4 q[NV]; } u;
        const u4* src = reinterpret_cast<const u4*>(p + (first + base) * sizeof(T));
#pragma unroll
        for (int i = 0; i < NV; ++i) u.q[i] = src[i];
#pragma unroll
        for (int k = 0; k < kScanPer; ++k) v[k] = u.t[k];
        return;
    }
#pragma unroll
    for (int k = 0; k < kScanPer; ++k)
        if (base + k < cnt) v[k] = *reinterpret_cast<const T*>(p + (int64_t)(first + base + k) * s);
}

template <class T>
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
        for (int i = 0; i < NV; ++i) dst[i] = u.q[i];
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

// phase 1 of the three-launch form: the total of each tile. A tile of nothing but
// NaN under a nan operator has the total NaN, which the operator reads as "nothing".
template <class T, class Op>
__global__ __launch_bounds__(kScanBlock) void scan_tile_totals_kernel(const char* in, int64_t s_in, uint64_t n, T* totals) {
    const uint64_t first = (uint64_t)blockIdx.x * kScanTile;
    const uint64_t left = n - first;
    const int cnt = left < (uint64_t)kScanTile ? (int)left : kScanTile;
    T v[kScanPer];
    scan_load<T>(in, s_in, first, cnt, v);
    T carry = T();
    bool hc = false;
    scan_tile<T, Op>(v, cnt, carry, hc);
    if (threadIdx.x == 0) totals[blockIdx.x] = carry;
}

// phase 3: every tile scans itself, starting from the scanned total of the tiles before it
template <class T, class Op>
__global__ __launch_bounds__(kScanBlock) void scan_apply_kernel(const char* in, int64_t s_in, char* out, int64_t s_out, uint64_t n,
                                                                const T* scanned_totals) {
    const uint64_t first = (uint64_t)blockIdx.x * kScanTile;
    const uint64_t left = n - first;
    const int cnt = left < (uint64_t)kScanTile ? (int)left : kScanTile;
    T v[kScanPer];
    scan_load<T>(in, s_in, first, cnt, v);
    bool hc = blockIdx.x > 0;
    T carry = hc ? scanned_totals[blockIdx.x - 1] : T();
    scan_tile<T, Op>(v, cnt, carry, hc);
    scan_store<T>(out, s_out, first, cnt, v);
}

template <class T, class Op>
void scan_rows_launch(const ScanRowsParams& p, hipStream_t stream) {
    if (p.rows == 0 || p.n == 0) return;
    uint64_t grid = p.rows;
    if (grid > 65536) grid = 65536;
    hipLaunchKernelGGL((scan_rows_kernel<T, Op>), dim3((unsigned)grid), dim3(kScanBlock), 0, stream, p);
}

// One run of n elements. Short runs take one block; long ones the three launches.
template <class T, class Op>
int scan_run_launch(const char* p1, char* p2, ssize_t s1, ssize_t s2, uint64_t n) {
    if (n == 0) return 0;
    hipStream_t stream = current_stream();
    const uint64_t n_tiles = (n + kScanTile - 1) / kScanTile;
    if (n_tiles <= 8 || n_tiles > 0x7fffffffull) {
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
    T* totals = reinterpret_cast<T*>(cumo_cuda_runtime_malloc(sizeof(T) * n_tiles));
    if (!totals) return (int)hipErrorOutOfMemory;
    hipLaunchKernelGGL((scan_tile_totals_kernel<T, Op>), dim3((unsigned)n_tiles), dim3(kScanBlock), 0, stream, p1, (int64_t)s1, n, totals);
    ScanRowsParams p;
    std::memset(&p, 0, sizeof(p));
    p.rows = 1;
    p.n = n_tiles;
    p.s_in = p.s_out = (int64_t)sizeof(T);
    p.in = reinterpret_cast<const char*>(totals);
    p.out = reinterpret_cast<char*>(totals);
    scan_rows_launch<T, Op>(p, stream);
    hipLaunchKernelGGL((scan_apply_kernel<T, Op>), dim3((unsigned)n_tiles), dim3(kScanBlock), 0, stream, p1, (int64_t)s1, p2, (int64_t)s2, n,
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

}  // extern "C"
