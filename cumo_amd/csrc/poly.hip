// x.poly(a0, a1, ..., an) = a0 + a1 x + ... + an x^n by Horner's rule, one launch for every element.
//
// Replaces narray/gen/tmpl/poly_kernel.cu of the reference with the same launcher symbols and
// arguments: every coefficient is an array descriptor of its own (a number arrives as a
// descriptor with zero steps). The reference copies the descriptors to device memory; here
// they ride in the kernel arguments, six coefficients a launch: a longer polynomial continues
// from the value the previous launch left in the result. Each step is the element type's own
// multiplication and addition, rounded separately (types/float_macro_kernel.h m_mul, m_add),
// Int32 wrapping.
#include "common.h"
#include "plan.h"

#include <type_traits>

namespace cumo_hip {
namespace {

constexpr int kPolyChunk = 6;

struct PolyParams {
    int ndim;
    int nc;       // coefficients in this launch, highest power first in c[]
    int from_z;   // 1: Horner continues from the value in z; 0: it starts from c[0] (or from x when nc == 0)
    uint64_t total;
    uint64_t shape[CUMO_NA_MAX_DIMENSION];
    int64_t step_x[CUMO_NA_MAX_DIMENSION], step_z[CUMO_NA_MAX_DIMENSION];
    int64_t step_c[kPolyChunk][CUMO_NA_MAX_DIMENSION];
    const char* x;
    char* z;
    const char* c[kPolyChunk];
};

template <class T>
__device__ __forceinline__ T poly_step(T x, T y, T a) {
    if constexpr (std::is_integral<T>::value) {
        return (T)((uint32_t)x * (uint32_t)y + (uint32_t)a);
    } else {
        const T m = x * y;  // compiled without contraction: two roundings, as the reference's m_mul then m_add
        return m + a;
    }
}

template <class T>
__global__ __launch_bounds__(256) void poly_kernel(PolyParams p) {
    for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < p.total; i += (uint64_t)gridDim.x * 256) {
        uint64_t r = i;
        int64_t ox = 0, oz = 0, oc[kPolyChunk];
#pragma unroll
        for (int k = 0; k < kPolyChunk; ++k) oc[k] = 0;
        for (int d = p.ndim - 1; d >= 0; --d) {
            const uint64_t n = p.shape[d];
            const uint64_t q = r / n;
            const int64_t j = (int64_t)(r - q * n);
            r = q;
            ox += j * p.step_x[d];
            oz += j * p.step_z[d];
#pragma unroll
            for (int k = 0; k < kPolyChunk; ++k) oc[k] += j * p.step_c[k][d];
        }
        const T xv = *reinterpret_cast<const T*>(p.x + ox);
        T y;
        int k = 0;
        if (p.from_z) {
            y = *reinterpret_cast<const T*>(p.z + oz);
        } else if (p.nc > 0) {
            y = *reinterpret_cast<const T*>(p.c[0] + oc[0]);
            k = 1;
        } else {
            y = xv;  // no coefficient at all answers x itself (poly_kernel.cu:11)
        }
#pragma unroll
        for (int q = 0; q < kPolyChunk; ++q) {
            if (q >= k && q < p.nc) y = poly_step<T>(xv, y, *reinterpret_cast<const T*>(p.c[q] + oc[q]));
        }
        *reinterpret_cast<T*>(p.z + oz) = y;
    }
}

// x and z one contiguous run each and every coefficient a single number: a 128-bit vector per lane
// (from any element boundary), the coefficients read once per lane.
struct PolyFlat {
    int nc, from_z;
    const char* c[kPolyChunk];
};

template <class T, bool NT>
__global__ __launch_bounds__(256) void poly_flat_kernel(const T* x, T* z, uint64_t n, PolyFlat p) {
    constexpr int V = 16 / sizeof(T);
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    union Vec {
        u4 q;
        T v[V];
        __device__ Vec() {}
    };
    T a[kPolyChunk];
#pragma unroll
    for (int k = 0; k < kPolyChunk; ++k) a[k] = k < p.nc ? *reinterpret_cast<const T*>(p.c[k]) : (T)0;
    const uint64_t nv = (n + V - 1) / V;
    for (uint64_t v = (uint64_t)blockIdx.x * 256 + threadIdx.x; v < nv; v += (uint64_t)gridDim.x * 256) {
        const uint64_t e = v * V;
        const bool whole = e + V <= n;
        Vec xs, ys;
        if (whole) {
            xs.q = NT ? __builtin_nontemporal_load(reinterpret_cast<const u4*>(x + e)) : *reinterpret_cast<const u4*>(x + e);
            if (p.from_z) ys.q = *reinterpret_cast<const u4*>(z + e);
        } else {
#pragma unroll
            for (int j = 0; j < V; ++j) {
                xs.v[j] = e + j < n ? x[e + j] : (T)0;
                ys.v[j] = (p.from_z && e + j < n) ? z[e + j] : (T)0;
            }
        }
#pragma unroll
        for (int j = 0; j < V; ++j) {
            T y;
            int k = 0;
            if (p.from_z) {
                y = ys.v[j];
            } else if (p.nc > 0) {
                y = a[0];
                k = 1;
            } else {
                y = xs.v[j];
            }
#pragma unroll
            for (int q = 0; q < kPolyChunk; ++q) {
                if (q >= k && q < p.nc) y = poly_step<T>(xs.v[j], y, a[q]);
            }
            ys.v[j] = y;
        }
        if (whole) {
            if (NT) __builtin_nontemporal_store(ys.q, reinterpret_cast<u4*>(z + e));
            else *reinterpret_cast<u4*>(z + e) = ys.q;
        } else {
#pragma unroll
            for (int j = 0; j < V; ++j)
                if (e + j < n) z[e + j] = ys.v[j];
        }
    }
}

// whether the operand's elements lie one after another in row-major order
inline bool poly_one_run(const cumo_na_iarray_t* a, const cumo_na_indexer_t* indexer, size_t elmsz) {
    int64_t want = (int64_t)elmsz;
    for (int d = indexer->ndim - 1; d >= 0; --d) {
        if (indexer->shape[d] == 1) continue;
        if ((int64_t)a->step[d] != want) return false;
        want *= (int64_t)indexer->shape[d];
    }
    return ((uintptr_t)a->ptr % alignof(uint32_t)) == 0 && ((uintptr_t)a->ptr % elmsz) == 0;
}

template <class T>
void poly_launch(const cumo_na_iarray_t* x, const cumo_na_iarray_t* coef, int ncoef, const cumo_na_iarray_t* z, const cumo_na_indexer_t* indexer) {
    if (indexer->total_size == 0) return;
    PolyParams p;
    p.ndim = indexer->ndim;
    p.total = indexer->total_size;
    for (int d = 0; d < CUMO_NA_MAX_DIMENSION; ++d) {
        p.shape[d] = d < indexer->ndim ? indexer->shape[d] : 1;
        p.step_x[d] = d < indexer->ndim ? x->step[d] : 0;
        p.step_z[d] = d < indexer->ndim ? z->step[d] : 0;
    }
    p.x = x->ptr;
    p.z = z->ptr;
    uint64_t grid = (p.total + 255) / 256;
    if (grid > 65536) grid = 65536;
    hipStream_t st = current_stream();
    // coefficients from the highest power down, kPolyChunk a launch
    int next = ncoef - 1;
    bool first = true;
    bool flat = !force_wide_indices() && p.total >= 1024 && poly_one_run(x, indexer, sizeof(T)) && poly_one_run(z, indexer, sizeof(T));
    for (int k = 0; k < ncoef && flat; ++k)
        for (int d = 0; d < indexer->ndim; ++d)
            if (indexer->shape[d] != 1 && coef[k].step[d] != 0) flat = false;
    if (flat) {
        const bool nt = stream_past_caches(p.total * sizeof(T) * 2);
        constexpr uint64_t V = 16 / sizeof(T);
        uint64_t g = ((p.total + V - 1) / V + 255) / 256;
        if (g > (uint64_t)kNumCU * 32) g = (uint64_t)kNumCU * 32;
        do {
            PolyFlat f;
            f.from_z = first ? 0 : 1;
            f.nc = 0;
            for (int k = 0; k < kPolyChunk; ++k) {
                f.c[k] = next >= 0 ? coef[next].ptr : nullptr;
                if (next >= 0) {
                    ++f.nc;
                    --next;
                }
            }
            if (nt) hipLaunchKernelGGL((poly_flat_kernel<T, true>), dim3((unsigned)g), dim3(256), 0, st, (const T*)x->ptr, (T*)z->ptr, p.total, f);
            else hipLaunchKernelGGL((poly_flat_kernel<T, false>), dim3((unsigned)g), dim3(256), 0, st, (const T*)x->ptr, (T*)z->ptr, p.total, f);
            first = false;
        } while (next >= 0);
        cumo_cuda_runtime_check_kernel_launch();
        return;
    }
    do {
        p.from_z = first ? 0 : 1;
        p.nc = 0;
        for (int k = 0; k < kPolyChunk; ++k) {
            const bool have = next >= 0;
            const cumo_na_iarray_t* a = have ? &coef[next] : nullptr;
            p.c[k] = have ? a->ptr : nullptr;
            for (int d = 0; d < CUMO_NA_MAX_DIMENSION; ++d) p.step_c[k][d] = (have && d < indexer->ndim) ? a->step[d] : 0;
            if (have) {
                ++p.nc;
                --next;
            }
        }
        hipLaunchKernelGGL((poly_kernel<T>), dim3((unsigned)grid), dim3(256), 0, st, p);
        first = false;
    } while (next >= 0);
    cumo_cuda_runtime_check_kernel_launch();
}

}  // namespace
}  // namespace cumo_hip

using namespace cumo_hip;

extern "C" {
void cumo_iter_sfloat_poly_kernel_launch(cumo_na_iarray_t* x, cumo_na_iarray_t* coef, int ncoef, cumo_na_iarray_t* z, cumo_na_indexer_t* indexer) {
    poly_launch<float>(x, coef, ncoef, z, indexer);
}
void cumo_iter_dfloat_poly_kernel_launch(cumo_na_iarray_t* x, cumo_na_iarray_t* coef, int ncoef, cumo_na_iarray_t* z, cumo_na_indexer_t* indexer) {
    poly_launch<double>(x, coef, ncoef, z, indexer);
}
void cumo_iter_int32_poly_kernel_launch(cumo_na_iarray_t* x, cumo_na_iarray_t* coef, int ncoef, cumo_na_iarray_t* z, cumo_na_indexer_t* indexer) {
    poly_launch<int32_t>(x, coef, ncoef, z, indexer);
}
}  // extern "C"
