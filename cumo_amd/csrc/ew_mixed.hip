// Arithmetic on two arrays of different element types, each one contiguous run, in one launch: every
// element is converted to the result's type on the way in, exactly as the cast the reference makes first
// would convert it (narray/gen/tmpl/binary.c:38-97 upcasts, then runs the result type's loop), and the
// result type's + - * / is applied. The cast into a temporary array -- a write and a read of the wider
// type for every element -- is what this saves: SFloat + DFloat moves 20 bytes an element instead of 36.
// Other layouts keep the two steps.
#include "common.h"
#include "cumo_hip_ndloop.h"
#include "ew_kernels.h"
#include "ew_ops.h"

namespace cumo_hip {
namespace {

constexpr int kMxBlock = 256;
// elements a vector: the result's 16 bytes (a lane's store is one 128-bit access next to its neighbours'; with four DFloat
// results a lane, every store instruction of a wave wrote every other 16 bytes of its span: SFloat + DFloat 0.69 of peak)
template <class TR> struct MxVec { static constexpr int value = 16 / (int)sizeof(TR); };

template <int OP, class T>
__device__ __forceinline__ T mixed_apply(T a, T b) {
    if (OP == 0) return a + b;
    if (OP == 1) return a - b;
    if (OP == 2) return a * b;
    return a / b;
}

template <int OP, class TA, class TB, class TR, bool NT, int kMxUnr>
__global__ __launch_bounds__(kMxBlock) void ew_mixed_flat_kernel(const char* __restrict__ px, const char* __restrict__ py,
                                                                 char* __restrict__ pz, uint64_t n) {
    constexpr int kMxVec = MxVec<TR>::value;
    const uint64_t i0 = ((uint64_t)blockIdx.x * (kMxBlock * kMxUnr) + threadIdx.x) * kMxVec;
    TA xv[kMxUnr][kMxVec];
    TB yv[kMxUnr][kMxVec];
    bool whole[kMxUnr];
#pragma unroll
    for (int u = 0; u < kMxUnr; ++u) {
        const uint64_t i = i0 + (uint64_t)u * (kMxBlock * kMxVec);
        whole[u] = i + kMxVec <= n;
        if (whole[u]) {
            raw_load<TA, kMxVec, NT>(px + i * sizeof(TA), xv[u]);
            raw_load<TB, kMxVec, NT>(py + i * sizeof(TB), yv[u]);
        }
    }
#pragma unroll
    for (int u = 0; u < kMxUnr; ++u) {
        const uint64_t i = i0 + (uint64_t)u * (kMxBlock * kMxVec);
        if (whole[u]) {
            TR zv[kMxVec];
#pragma unroll
            for (int j = 0; j < kMxVec; ++j) zv[j] = mixed_apply<OP, TR>((TR)xv[u][j], (TR)yv[u][j]);
            raw_store<TR, kMxVec, NT>(pz + i * sizeof(TR), zv);
        } else if (i < n) {
            // the run's last elements, fewer than a vector
            for (uint64_t k = i; k < n; ++k)
                reinterpret_cast<TR*>(pz)[k] = mixed_apply<OP, TR>((TR) reinterpret_cast<const TA*>(px)[k], (TR) reinterpret_cast<const TB*>(py)[k]);
        }
    }
}

template <int OP, class TA, class TB, class TR>
void mixed_launch(const char* x, const char* y, char* z, uint64_t n) {
    constexpr int kMxUnr = 4, kMxVec = MxVec<TR>::value;   // vectors a lane has in flight per operand
    const uint64_t per_block = (uint64_t)kMxBlock * kMxUnr * kMxVec;
    const dim3 g((unsigned)((n + per_block - 1) / per_block)), b(kMxBlock);
    const bool nt = stream_past_caches(n * (sizeof(TA) + sizeof(TB) + sizeof(TR)));
    if (nt) hipLaunchKernelGGL((ew_mixed_flat_kernel<OP, TA, TB, TR, true, kMxUnr>), g, b, 0, current_stream(), x, y, z, n);
    else hipLaunchKernelGGL((ew_mixed_flat_kernel<OP, TA, TB, TR, false, kMxUnr>), g, b, 0, current_stream(), x, y, z, n);
    cumo_cuda_runtime_check_kernel_launch();
}

// Int32 array op one DFloat number (a Ruby Float meets an Int32 array: the array is computed in DFloat,
// gen/def/int32.rb upcast table), the number on the right or, with LEFT, on the left.
template <int OP, bool LEFT, bool NT>
__global__ __launch_bounds__(kMxBlock) void ew_mixed_scalar_kernel(const char* __restrict__ px, double sv, char* __restrict__ pz, uint64_t n) {
    constexpr int U = 4, kMxVec = MxVec<double>::value;
    const uint64_t i0 = ((uint64_t)blockIdx.x * (kMxBlock * U) + threadIdx.x) * kMxVec;
    int32_t xv[U][kMxVec];
    bool whole[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint64_t i = i0 + (uint64_t)u * (kMxBlock * kMxVec);
        whole[u] = i + kMxVec <= n;
        if (whole[u]) raw_load<int32_t, kMxVec, NT>(px + i * sizeof(int32_t), xv[u]);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint64_t i = i0 + (uint64_t)u * (kMxBlock * kMxVec);
        if (whole[u]) {
            double zv[kMxVec];
#pragma unroll
            for (int j = 0; j < kMxVec; ++j)
                zv[j] = LEFT ? mixed_apply<OP, double>(sv, (double)xv[u][j]) : mixed_apply<OP, double>((double)xv[u][j], sv);
            raw_store<double, kMxVec, NT>(pz + i * sizeof(double), zv);
        } else if (i < n) {
            for (uint64_t k = i; k < n; ++k) {
                const double x = (double)reinterpret_cast<const int32_t*>(px)[k];
                reinterpret_cast<double*>(pz)[k] = LEFT ? mixed_apply<OP, double>(sv, x) : mixed_apply<OP, double>(x, sv);
            }
        }
    }
}

template <int OP, bool LEFT>
void mixed_scalar_launch(const char* x, double sv, char* z, uint64_t n) {
    const uint64_t per_block = (uint64_t)kMxBlock * 4 * MxVec<double>::value;
    const dim3 g((unsigned)((n + per_block - 1) / per_block)), b(kMxBlock);
    const bool nt = stream_past_caches(n * (sizeof(int32_t) + sizeof(double)));
    if (nt) hipLaunchKernelGGL((ew_mixed_scalar_kernel<OP, LEFT, true>), g, b, 0, current_stream(), x, sv, z, n);
    else hipLaunchKernelGGL((ew_mixed_scalar_kernel<OP, LEFT, false>), g, b, 0, current_stream(), x, sv, z, n);
    cumo_cuda_runtime_check_kernel_launch();
}

template <int OP>
bool mixed_by_types(int ta, int tb, const char* x, const char* y, char* z, uint64_t n) {
    // the result's type is the wider float of the two (gen/def/{sfloat,dfloat,int32}.rb: Int32 with SFloat is SFloat)
    if (ta == CUMO_HIP_SFLOAT && tb == CUMO_HIP_DFLOAT) mixed_launch<OP, float, double, double>(x, y, z, n);
    else if (ta == CUMO_HIP_DFLOAT && tb == CUMO_HIP_SFLOAT) mixed_launch<OP, double, float, double>(x, y, z, n);
    else if (ta == CUMO_HIP_INT32 && tb == CUMO_HIP_SFLOAT) mixed_launch<OP, int32_t, float, float>(x, y, z, n);
    else if (ta == CUMO_HIP_SFLOAT && tb == CUMO_HIP_INT32) mixed_launch<OP, float, int32_t, float>(x, y, z, n);
    else if (ta == CUMO_HIP_INT32 && tb == CUMO_HIP_DFLOAT) mixed_launch<OP, int32_t, double, double>(x, y, z, n);
    else if (ta == CUMO_HIP_DFLOAT && tb == CUMO_HIP_INT32) mixed_launch<OP, double, int32_t, double>(x, y, z, n);
    else return false;
    return true;
}

// Comparisons of two arrays of different element types into Bit: the flat Bit kernel of ew_kernels.h (four elements a
// lane, a group of eight lanes gathers a word, four words stored as one access) with an operator that converts both
// sides to the higher type first, as the cast the reference makes would (gen/tmpl/cond_binary.c:1-55).
template <int CMP, class TA, class TB, class TU>
struct OpCmpMixed { CUMO_HIP_OP_COMMON(TA, TB, uint32_t, 2, true, false)
    __device__ __forceinline__ bool operator()(TA xa, TB yb, uint32_t& z) const {
        const TU x = (TU)xa, y = (TU)yb;
        bool r;
        if (CMP == 0) r = x == y;
        else if (CMP == 1) r = x != y;
        else if (CMP == 2) r = x > y;
        else if (CMP == 3) r = x >= y;
        else if (CMP == 4) r = x < y;
        else r = x <= y;
        z = r ? 1u : 0u;
        return true; } };

template <int CMP, class TA, class TB, class TU>
void mixed_compare_launch(const char* x, const char* y, CUMO_BIT_DIGIT* z, uint64_t n) {
    typedef OpCmpMixed<CMP, TA, TB, TU> Op;
    constexpr int VB = 4;
    const uint64_t groups = (n + 127) / 128;
    const uint64_t blocks = (groups * (32 / VB) + kEwBlock - 1) / kEwBlock;
    const dim3 g((unsigned)blocks), b(kEwBlock);
    const bool nt = stream_past_caches(n * (sizeof(TA) + sizeof(TB)));
    if (nt) hipLaunchKernelGGL((ew_flat_bit_kernel<Op, VB, true>), g, b, 0, current_stream(), x, y, z, n, 0, Op{}, TA());
    else hipLaunchKernelGGL((ew_flat_bit_kernel<Op, VB, false>), g, b, 0, current_stream(), x, y, z, n, 0, Op{}, TA());
    cumo_cuda_runtime_check_kernel_launch();
}

template <int CMP>
bool mixed_compare_by_types(int ta, int tb, const char* x, const char* y, CUMO_BIT_DIGIT* z, uint64_t n) {
    if (ta == CUMO_HIP_SFLOAT && tb == CUMO_HIP_DFLOAT) mixed_compare_launch<CMP, float, double, double>(x, y, z, n);
    else if (ta == CUMO_HIP_DFLOAT && tb == CUMO_HIP_SFLOAT) mixed_compare_launch<CMP, double, float, double>(x, y, z, n);
    else if (ta == CUMO_HIP_INT32 && tb == CUMO_HIP_SFLOAT) mixed_compare_launch<CMP, int32_t, float, float>(x, y, z, n);
    else if (ta == CUMO_HIP_SFLOAT && tb == CUMO_HIP_INT32) mixed_compare_launch<CMP, float, int32_t, float>(x, y, z, n);
    else if (ta == CUMO_HIP_INT32 && tb == CUMO_HIP_DFLOAT) mixed_compare_launch<CMP, int32_t, double, double>(x, y, z, n);
    else if (ta == CUMO_HIP_DFLOAT && tb == CUMO_HIP_INT32) mixed_compare_launch<CMP, double, int32_t, double>(x, y, z, n);
    else return false;
    return true;
}

}  // namespace

bool mixed_flat_compare(int cmp, int ta, const char* x, int tb, const char* y, CUMO_BIT_DIGIT* z, uint64_t n) {
    if (n == 0 || n >= ((uint64_t)1 << 40)) return false;
    if ((((uintptr_t)x | (uintptr_t)y | (uintptr_t)z) & 15u) != 0) return false;
    switch (cmp) {
        case 0: return mixed_compare_by_types<0>(ta, tb, x, y, z, n);
        case 1: return mixed_compare_by_types<1>(ta, tb, x, y, z, n);
        case 2: return mixed_compare_by_types<2>(ta, tb, x, y, z, n);
        case 3: return mixed_compare_by_types<3>(ta, tb, x, y, z, n);
        case 4: return mixed_compare_by_types<4>(ta, tb, x, y, z, n);
        case 5: return mixed_compare_by_types<5>(ta, tb, x, y, z, n);
    }
    return false;
}

bool mixed_flat_binary(int op, int ta, const char* x, int tb, const char* y, char* z, uint64_t n) {
    if (n == 0 || n >= ((uint64_t)1 << 42)) return false;  // (the grid's x dimension: 2^31 blocks of 2^11 elements or more)
    if ((((uintptr_t)x | (uintptr_t)y | (uintptr_t)z) & 15u) != 0) return false;
    switch (op) {
        case 0: return mixed_by_types<0>(ta, tb, x, y, z, n);
        case 1: return mixed_by_types<1>(ta, tb, x, y, z, n);
        case 2: return mixed_by_types<2>(ta, tb, x, y, z, n);
        case 3: return mixed_by_types<3>(ta, tb, x, y, z, n);
    }
    return false;
}

bool mixed_flat_binary_s(int op, const char* x, double sv, bool scalar_is_left, char* z, uint64_t n) {
    if (n == 0 || n >= ((uint64_t)1 << 42)) return false;
    if ((((uintptr_t)x | (uintptr_t)z) & 15u) != 0) return false;
    switch (op * 2 + (scalar_is_left ? 1 : 0)) {
        case 0: mixed_scalar_launch<0, false>(x, sv, z, n); return true;
        case 1: mixed_scalar_launch<0, true>(x, sv, z, n); return true;
        case 2: mixed_scalar_launch<1, false>(x, sv, z, n); return true;
        case 3: mixed_scalar_launch<1, true>(x, sv, z, n); return true;
        case 4: mixed_scalar_launch<2, false>(x, sv, z, n); return true;
        case 5: mixed_scalar_launch<2, true>(x, sv, z, n); return true;
        case 6: mixed_scalar_launch<3, false>(x, sv, z, n); return true;
        case 7: mixed_scalar_launch<3, true>(x, sv, z, n); return true;
    }
    return false;
}

}  // namespace cumo_hip
