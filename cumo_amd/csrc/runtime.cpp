// Runtime glue: error reporting, stream selection, the pinned error flag the
// Int32 division and abs kernels write through, and the synchronous copies the
// host uses to read results back.
//
// Replaces ext/cumo/cuda/runtime.c:16-68 of the reference. That file raises a
// Ruby exception from cumo_cuda_runtime_check_kernel_launch; this one cannot
// include ruby.h, so it calls the handler the host installed instead.
#include "common.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <atomic>
#include <mutex>

namespace cumo_hip {

static std::atomic<cumo_hip_error_handler_t> g_handler{nullptr};

struct LastError {
    int kind = 0;
    int status = 0;
    char message[512] = {0};
};
static thread_local LastError t_last;
static thread_local hipStream_t t_stream = nullptr;

void report_error(int kind, int hip_status, const char* message) {
    cumo_hip_error_handler_t h = g_handler.load();
    if (h) {
        h(kind, hip_status, message);  // may longjmp
        return;
    }
    // keep the first error until somebody reads it
    if (t_last.kind == 0) {
        t_last.kind = kind;
        t_last.status = hip_status;
        std::snprintf(t_last.message, sizeof(t_last.message), "%s", message ? message : "");
    }
}

void report_hip_error(hipError_t status, const char* what) {
    char buf[384];
    std::snprintf(buf, sizeof(buf), "%s: %s (error=%d)", what ? what : "hip", hipGetErrorString(status), (int)status);
    report_error(status == hipErrorOutOfMemory ? CUMO_HIP_ERROR_OUT_OF_MEMORY : CUMO_HIP_ERROR_RUNTIME, (int)status, buf);
}

hipStream_t current_stream() { return t_stream; }

bool force_wide_indices() {
    static const bool on = [] {
        const char* e = std::getenv("CUMO_HIP_FORCE_WIDE");
        return e != nullptr && e[0] != 0 && e[0] != '0';
    }();
    return on;
}

bool stream_past_caches(uint64_t bytes) {
    static const int mode = [] {
        const char* e = std::getenv("CUMO_HIP_NT");
        return e ? (std::atoi(e) != 0 ? 1 : 0) : -1;
    }();
    return mode < 0 ? bytes > kStreamNtBytes : mode != 0;
}

// Streams in use get a small number, for kernels that keep per-stream words in a
// fixed device array (tickets that launches on different streams must not share).
static std::mutex g_slot_lock;
static hipStream_t g_slot_stream[kStreamSlots];
static bool g_slot_used[kStreamSlots];

int stream_slot(hipStream_t stream) {
    std::lock_guard<std::mutex> hold(g_slot_lock);
    int free_slot = -1;
    for (int i = 0; i < kStreamSlots; ++i) {
        if (g_slot_used[i] && g_slot_stream[i] == stream) return i;
        if (!g_slot_used[i] && free_slot < 0) free_slot = i;
    }
    if (free_slot >= 0) {
        g_slot_used[free_slot] = true;
        g_slot_stream[free_slot] = stream;
    }
    return free_slot;
}

int stream_slot_release(hipStream_t stream) {
    std::lock_guard<std::mutex> hold(g_slot_lock);
    int held = -1;
    for (int i = 0; i < kStreamSlots; ++i) {
        if (g_slot_used[i] && g_slot_stream[i] == stream) {
            g_slot_used[i] = false;
            held = i;
        }
    }
    return held;
}

int device_compute_units() {
    static const int n = [] {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
            (void)hipGetLastError();
            return 0;
        }
        return cus;
    }();
    return n;
}

// The give-up word and counters of the kernels' bounded waits. The flag is pinned host memory
// the device writes through; the block the kernels read sits in device memory.
static std::mutex g_wait_lock;
static WaitCtl* g_wait_dev = nullptr;
static std::atomic<uint32_t*> g_wait_flag{nullptr};

WaitCtl* wait_ctl() {
    std::lock_guard<std::mutex> hold(g_wait_lock);
    if (g_wait_dev) return g_wait_dev;
    void* flag = nullptr;
    if (hipHostMalloc(&flag, 64, hipHostMallocMapped | hipHostMallocPortable) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    std::memset(flag, 0, 64);
    void* dev = nullptr;
    if (hipMalloc(&dev, sizeof(WaitCtl)) != hipSuccess) {
        (void)hipGetLastError();
        (void)hipHostFree(flag);
        return nullptr;
    }
    WaitCtl init;
    std::memset(&init, 0, sizeof(init));
    // CUMO_HIP_WAIT_LIMIT=0 (read once, for tests): every wait gives up at its first failed look
    const char* e = std::getenv("CUMO_HIP_WAIT_LIMIT");
    init.limit_scale = (e && e[0] == '0') ? 0u : 1u;
    init.host_flag = (uint32_t*)flag;
    if (hipMemcpy(dev, &init, sizeof(init), hipMemcpyHostToDevice) != hipSuccess) {
        (void)hipGetLastError();
        (void)hipFree(dev);
        (void)hipHostFree(flag);
        return nullptr;
    }
    g_wait_flag.store((uint32_t*)flag);
    g_wait_dev = (WaitCtl*)dev;
    return g_wait_dev;
}

static int wait_counts_read(uint32_t out[4]) {
    WaitCtl* dev;
    {
        std::lock_guard<std::mutex> hold(g_wait_lock);
        dev = g_wait_dev;
    }
    out[0] = out[1] = out[2] = out[3] = 0;
    if (!dev) return 0;  // no kernel with a wait was ever launched
    WaitCtl now;
    if (hipMemcpy(&now, dev, sizeof(now), hipMemcpyDeviceToHost) != hipSuccess) {
        (void)hipGetLastError();
        return -1;
    }
    for (int i = 0; i < 4; ++i) out[i] = now.gave_up[i];
    return 0;
}

bool wait_trouble_check() {
    uint32_t* flag = g_wait_flag.load();   // set once, before any kernel can write it
    if (!flag || *(volatile uint32_t*)flag == 0) return true;
    *(volatile uint32_t*)flag = 0;
    uint32_t c[4];
    char msg[256];
    if (wait_counts_read(c) == 0)
        std::snprintf(msg, sizeof(msg), "a kernel gave up waiting for another block's partial result; the results of that launch are not valid "
                      "(give-ups so far: reductions %u, scans %u, mulsum %u)", c[0], c[1], c[2]);
    else
        std::snprintf(msg, sizeof(msg), "a kernel gave up waiting for another block's partial result; the results of that launch are not valid");
    report_error(CUMO_HIP_ERROR_RUNTIME, 0, msg);
    return false;
}

}  // namespace cumo_hip

using namespace cumo_hip;

extern "C" {

int cumo_hip_wait_give_ups(uint32_t counts[4]) {
    if (!counts) return -1;
    return wait_counts_read(counts);
}

void cumo_hip_set_error_handler(cumo_hip_error_handler_t handler) { g_handler.store(handler); }

int cumo_hip_last_error(const char** message) {
    static thread_local char copy[512];
    int kind = t_last.kind;
    if (message) {
        std::memcpy(copy, t_last.message, sizeof(copy));
        *message = copy;
    }
    t_last.kind = 0;
    t_last.status = 0;
    t_last.message[0] = 0;
    return kind;
}

void cumo_hip_set_stream(void* hip_stream) { t_stream = (hipStream_t)hip_stream; }
void* cumo_hip_get_stream(void) { return (void*)t_stream; }

// a stream of the default priority that does not synchronise with the null stream
void* cumo_hip_stream_create(void) {
    hipStream_t st = nullptr;
    if (!hip_ok(hipStreamCreateWithFlags(&st, hipStreamNonBlocking), "hipStreamCreate")) return nullptr;
    return (void*)st;
}

// What the library keeps per stream (its slot of ticket and hand-over words, the look-back words
// of its scans, its arena of the pool) is given up; the stream itself stays the caller's.
void cumo_hip_stream_release(void* hip_stream) {
    if (!hip_stream) return;
    // what the stream still has queued may use its slot's words: drain it first
    hip_ok(hipStreamSynchronize((hipStream_t)hip_stream), "hipStreamSynchronize");
    scan_chain_words_drop_slot(stream_slot_release((hipStream_t)hip_stream));
    pool_retire_stream((hipStream_t)hip_stream);
}

void cumo_hip_stream_destroy(void* hip_stream) {
    if (!hip_stream) return;
    if (t_stream == (hipStream_t)hip_stream) t_stream = nullptr;
    cumo_hip_stream_release(hip_stream);
    hip_ok(hipStreamDestroy((hipStream_t)hip_stream), "hipStreamDestroy");
}

int cumo_hip_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return n;
}

void cumo_hip_synchronize(void) {
    if (hip_ok(hipStreamSynchronize(t_stream), "hipStreamSynchronize")) wait_trouble_check();
}

void cumo_hip_memcpy_h2d(void* dst, const void* src, size_t n) {
    if (n == 0) return;
    if (!hip_ok(hipMemcpyAsync(dst, src, n, hipMemcpyHostToDevice, t_stream), "hipMemcpyAsync(h2d)")) return;
    hip_ok(hipStreamSynchronize(t_stream), "hipStreamSynchronize");
}

void cumo_hip_memcpy_d2h(void* dst, const void* src, size_t n) {
    if (n == 0) return;
    if (!hip_ok(hipMemcpyAsync(dst, src, n, hipMemcpyDeviceToHost, t_stream), "hipMemcpyAsync(d2h)")) return;
    if (hip_ok(hipStreamSynchronize(t_stream), "hipStreamSynchronize")) wait_trouble_check();
}

// reference: cuda/runtime.c:16-20
void cumo_cuda_runtime_check_kernel_launch(void) {
    hipError_t st = hipGetLastError();
    if (st != hipSuccess) report_hip_error(st, "kernel launch");
}

// Pinned, device-mapped host words a kernel writes through when it rejects an
// element (reference: cuda/runtime.c:22-68). hipHostMalloc, not registration of
// existing memory.
static int* alloc_pinned_word(size_t bytes) {
    void* p = nullptr;
    if (!hip_ok(hipHostMalloc(&p, bytes, hipHostMallocMapped | hipHostMallocPortable), "hipHostMalloc")) return nullptr;
    std::memset(p, 0, bytes);
    return (int*)p;
}

int* cumo_cuda_runtime_error_flag_ptr(void) {
    static int* flag = nullptr;
    if (flag == nullptr) flag = alloc_pinned_word(sizeof(int));
    return flag;
}

int* cumo_cuda_runtime_error_flag_new(void) {
    int* flag = cumo_cuda_runtime_error_flag_ptr();
    if (flag) *flag = 0;
    return flag;
}

bool cumo_cuda_runtime_error_flag_get(int* flag) {
    if (!hip_ok(hipDeviceSynchronize(), "hipDeviceSynchronize")) return false;
    wait_trouble_check();
    return flag && (*(volatile int*)flag != 0);
}

size_t* cumo_cuda_runtime_error_item_ptr(void) {
    static size_t* item = nullptr;
    if (item == nullptr) item = (size_t*)alloc_pinned_word(sizeof(size_t));
    return item;
}

size_t* cumo_cuda_runtime_error_item_new(void) {
    size_t* item = cumo_cuda_runtime_error_item_ptr();
    if (item) *item = 0;
    return item;
}

}  // extern "C"

// Events on the stream the launchers use, for callers that time kernels
// (the benchmark): create, record on the current stream, elapsed (waits for
// the second event), destroy.
extern "C" {

void* cumo_hip_event_create(void) {
    hipEvent_t ev = nullptr;
    if (!hip_ok(hipEventCreate(&ev), "hipEventCreate")) return nullptr;
    return (void*)ev;
}

void cumo_hip_event_record(void* ev) { hip_ok(hipEventRecord((hipEvent_t)ev, t_stream), "hipEventRecord"); }

float cumo_hip_event_elapsed_ms(void* start, void* stop) {
    float ms = 0.f;
    if (!hip_ok(hipEventSynchronize((hipEvent_t)stop), "hipEventSynchronize")) return -1.f;
    if (!hip_ok(hipEventElapsedTime(&ms, (hipEvent_t)start, (hipEvent_t)stop), "hipEventElapsedTime")) return -1.f;
    return ms;
}

void cumo_hip_event_destroy(void* ev) {
    if (ev) (void)hipEventDestroy((hipEvent_t)ev);
}

}  // extern "C"
