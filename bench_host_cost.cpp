// Per-operation cost of the host launch layer, measured from C so that no
// interpreter stands between the calls: tiny arrays (32 x 32 SFloat), operations
// issued back to back. Prints one JSON line. Built by cumo_amd/build.py into
// cumo_amd/bench_host_cost and run by bench.py.
//   ndloop_prepare      shape checks, broadcasting, dimension merging (no launch)
//   empty_launch        the runtime's own cost of launching a kernel that does nothing
//   empty_launch_1k     the same with a kilobyte of kernel arguments, as an elementwise launch has
//   launcher_add        cumo_iter_sfloat_add_kernel_launch with ready descriptors (plan + launch)
//   add_into_result     cumo_hip_na_binary("add") into a given result array
//   add_issue           the host side alone: 1000 such calls queued, timed before the device has drained them
//   add_alloc_free      the same with the result taken from and returned to the pool
//   sum_alloc_free      cumo_hip_na_reduce("sum") likewise
// Compiled with hipcc: the two do-nothing kernels live in this file, not in the library.
#include <hip/hip_runtime.h>

#include <chrono>
#include <cstdint>
#include <cstdio>
#include <cstring>

#include "cumo_hip.h"
#include "cumo_hip_ndloop.h"

// Kernels that do nothing, for what one launch costs on the library's current stream
// (the floor under the per-operation cost of the host layer): one without arguments and
// one that takes a kilobyte of them by value.
struct Kilobyte {
    uint64_t w[128];
};
__global__ void empty_kernel() {}
__global__ void empty_kernel_1k(Kilobyte k, uint64_t* sink) {
    if (sink) *sink = k.w[threadIdx.x & 127];  // never taken: sink is NULL
}
static void launch_empty_kernel(int with_arguments) {
    hipStream_t st = (hipStream_t)cumo_hip_get_stream();
    if (with_arguments) {
        Kilobyte k = {};
        hipLaunchKernelGGL(empty_kernel_1k, dim3(1), dim3(64), 0, st, k, (uint64_t*)nullptr);
    } else {
        hipLaunchKernelGGL(empty_kernel, dim3(1), dim3(64), 0, st);
    }
}

static double now() { return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count(); }

template <class F>
static double us_per_call(int n, int reps, F f) {
    double best = 1e30;
    for (int r = 0; r < reps; ++r) {
        cumo_hip_synchronize();
        const double t0 = now();
        for (int i = 0; i < n; ++i) f();
        cumo_hip_synchronize();
        const double t = (now() - t0) / n * 1e6;
        if (t < best) best = t;
    }
    return best;
}

int main() {
    size_t shape[2] = {32, 32};
    cumo_hip_narray_t x, y, z;
    std::memset(&x, 0, sizeof x);
    std::memset(&y, 0, sizeof y);
    std::memset(&z, 0, sizeof z);
    if (cumo_hip_na_alloc(&x, CUMO_HIP_SFLOAT, 2, shape) || cumo_hip_na_alloc(&y, CUMO_HIP_SFLOAT, 2, shape) ||
        cumo_hip_na_alloc(&z, CUMO_HIP_SFLOAT, 2, shape)) {
        std::fprintf(stderr, "bench_host_cost: allocation failed\n");
        return 1;
    }
    cumo_hip_na_fill(&x, 1.0);
    cumo_hip_na_fill(&y, 2.0);
    const int N = 20000;
    cumo_hip_ndfunc_t nf;
    std::memset(&nf, 0, sizeof nf);
    nf.nin = 2;
    nf.nout = 1;
    nf.out_type[0] = CUMO_HIP_SFLOAT;
    const cumo_hip_narray_t* in[2] = {&x, &y};
    cumo_hip_narray_t* out[1] = {&z};
    cumo_hip_loop_t lp;
    const double prepare = us_per_call(200000, 3, [&] { cumo_hip_na_ndloop_prepare(&nf, in, out, 0, &lp); });
    const double empty = us_per_call(N, 4, [&] { launch_empty_kernel(0); });
    const double empty_1k = us_per_call(N, 4, [&] { launch_empty_kernel(1); });
    cumo_na_indexer_t ix;
    cumo_na_iarray_t a1, a2, a3;
    cumo_hip_make_indexer(&lp, &ix);
    cumo_hip_make_iarray(&lp, 0, &a1);
    cumo_hip_make_iarray(&lp, 1, &a2);
    cumo_hip_make_iarray(&lp, 2, &a3);
    const double launcher = us_per_call(N, 4, [&] { cumo_iter_sfloat_add_kernel_launch(&a1, &a2, &a3, &ix, NULL); });
    const double add_into = us_per_call(N, 4, [&] { cumo_hip_na_binary("add", &x, &y, &z); });
    double add_issue = 1e30;
    for (int r = 0; r < 8; ++r) {
        cumo_hip_synchronize();
        const double t0 = now();
        for (int i = 0; i < 1000; ++i) cumo_hip_na_binary("add", &x, &y, &z);
        const double t = (now() - t0) / 1000 * 1e6;
        if (t < add_issue) add_issue = t;
    }
    cumo_hip_synchronize();
    const double add_alloc = us_per_call(N, 4, [&] {
        cumo_hip_narray_t r;
        std::memset(&r, 0, sizeof r);
        cumo_hip_na_binary("add", &x, &y, &r);
        cumo_cuda_runtime_free(r.ptr);
    });
    const double sum_alloc = us_per_call(N, 4, [&] {
        cumo_hip_narray_t r;
        std::memset(&r, 0, sizeof r);
        cumo_hip_na_reduce("sum", &x, 0, 0, 0, &r, NULL);
        cumo_cuda_runtime_free(r.ptr);
    });
    // the same on a stream of its own instead of the null stream
    void* st = cumo_hip_stream_create();
    cumo_hip_set_stream(st);
    const double empty_own = us_per_call(N, 4, [&] { launch_empty_kernel(0); });
    const double add_own = us_per_call(N, 4, [&] { cumo_hip_na_binary("add", &x, &y, &z); });
    cumo_hip_set_stream(NULL);
    cumo_hip_stream_destroy(st);
    const char* msg = NULL;
    if (cumo_hip_last_error(&msg)) {
        std::fprintf(stderr, "bench_host_cost: %s\n", msg ? msg : "error");
        return 1;
    }
    std::printf("{\"unit\": \"us per operation\", \"shape\": \"32x32 SFloat\", \"ndloop_prepare\": %.3f, \"empty_launch\": %.2f, \"empty_launch_1k\": %.2f, "
                "\"launcher_add\": %.2f, \"add_into_result\": %.2f, \"add_issue\": %.2f, \"add_alloc_free\": %.2f, \"sum_alloc_free\": %.2f, \"own_stream_empty_launch\": %.2f, \"own_stream_add_into_result\": %.2f}\n",
                prepare, empty, empty_1k, launcher, add_into, add_issue, add_alloc, sum_alloc, empty_own, add_own);
    return 0;
}
