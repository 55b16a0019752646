// A full / split SFloat sum that allocates nothing: for callers that cannot call
// hipMalloc (code under stream capture, tight serving loops, harnesses that forbid
// it). Same planner and same kernels as cumo_sfloat_sum_kernel_launch; the partial
// sums of a split reduction go to a fixed array in device memory instead of a block
// from the pool. No counterpart in the reference, whose split reductions always take
// their scratch from the memory pool (include/cumo/reduce_kernel.h:493-496).
#include "reduce_kernels.h"
#include "reduce_impls.h"

#include <mutex>

using namespace cumo_hip;

namespace {

constexpr size_t kScratchBytes = CUMO_HIP_NOALLOC_SCRATCH_BYTES;
constexpr int kMaxDevices = 64;

// One copy per GPU the library runs on, held until the process ends. Host code never
// uses this name as an address: the device address is looked up once per device.
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

std::mutex g_lock;
char* g_scratch_ptr[kMaxDevices];  // per device: address of that device's copy of `scratch`

thread_local size_t t_last_used = 0;

// The current device's copy of the array; nullptr after reporting an error, whose kind goes to *kind.
char* scratch_of_current_device(int* kind) {
    int dev = -1;
    *kind = CUMO_HIP_ERROR_RUNTIME;
    if (!hip_ok(hipGetDevice(&dev), "hipGetDevice")) return nullptr;
    if (dev < 0 || dev >= kMaxDevices) {
        *kind = CUMO_HIP_ERROR_ARGUMENT;
        report_error(CUMO_HIP_ERROR_ARGUMENT, 0, "cumo_hip_sfloat_sum_noalloc_kernel_launch: device ordinal out of range");
        return nullptr;
    }
    char* p;
    hipError_t st = hipSuccess;
    {
        std::lock_guard<std::mutex> hold(g_lock);
        p = g_scratch_ptr[dev];
        if (p == nullptr) {
            void* sym = nullptr;
            st = hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch));
            if (st == hipSuccess) g_scratch_ptr[dev] = p = static_cast<char*>(sym);
        }
    }
    // reported with the lock released: an installed handler may not return
    if (st != hipSuccess) {
        report_hip_error(st, "hipGetSymbolAddress(scratch)");
        return nullptr;
    }
    *kind = CUMO_HIP_OK;
    return p;
}

}  // namespace

extern "C" int cumo_hip_sfloat_sum_noalloc_kernel_launch(cumo_na_reduction_arg_t* arg) {
    t_last_used = 0;
    if (arg == nullptr) {
        report_error(CUMO_HIP_ERROR_ARGUMENT, 0, "cumo_hip_sfloat_sum_noalloc_kernel_launch: arg is NULL");
        return CUMO_HIP_ERROR_ARGUMENT;
    }
    int kind = CUMO_HIP_OK;
    char* p = scratch_of_current_device(&kind);
    if (p == nullptr) return kind;
    const RedScratch fixed = {p, kScratchBytes, 0};
    if (!reduce_launch(arg, nullptr, SumImpl<float, float, false, false>{0.0f}, 0, &fixed)) {
        report_error(CUMO_HIP_ERROR_ARGUMENT, 0,
                     "cumo_hip_sfloat_sum_noalloc_kernel_launch: the partial sums of this reduction do not fit the fixed "
                     "scratch array (CUMO_HIP_NOALLOC_SCRATCH_BYTES); use cumo_sfloat_sum_kernel_launch");
        return CUMO_HIP_ERROR_ARGUMENT;
    }
    t_last_used = fixed.used;
    return CUMO_HIP_OK;
}

extern "C" size_t cumo_hip_sfloat_sum_noalloc_scratch_used(void) { return t_last_used; }
