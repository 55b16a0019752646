// Host read-back and ingest for arrays that live in plain device memory.
//
// The reference allocates managed memory (cuda/memory_pool_impl.cpp: cudaMallocManaged)
// and its host paths read and write array bytes with memcpy after a device
// synchronisation (narray/narray.c:1391-1560 from_binary / store_binary / to_binary,
// gen/tmpl/extract_cpu.c, narray.c:673-708 copy-on-write). Device memory from hipMalloc
// is not host-addressable, so those paths need an explicit transfer; this file is that
// transfer.
//
// A copy between pageable host memory and the device moves through a ring of pinned
// staging buffers (hipHostMalloc once, kept): while the DMA engine fills or drains one
// buffer over PCIe, a few host threads copy another between the ring and the caller's
// memory. The copies run on the library's current stream, so they are ordered after the
// kernels already queued there, and every call returns only when its bytes have
// arrived (the semantics of the synchronous memcpy the reference's host code assumes).
// Small copies take one staging buffer and no threads. Host memory that is already
// pinned goes straight to the DMA engine.
#include "common.h"

#include <pthread.h>

#include <atomic>
#include <condition_variable>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <thread>
#include <vector>

namespace cumo_hip {
namespace {

constexpr int kSlots = 4;
constexpr size_t kMinParallel = 1u << 20;  // below this a single memcpy beats waking threads

// ---- a few threads that do nothing but memcpy -------------------------------------
// Heap-allocated and never destroyed: the workers sleep on its condition variable until
// the process ends. After fork() the child has no workers; the atfork hook makes it
// start its own on first use.
struct CopyWorkers {
    struct Task {
        char* dst;
        const char* src;
        size_t n;
    };
    std::mutex mu;
    std::condition_variable wake, done;
    std::vector<Task> tasks;
    size_t pending = 0;
    int n_threads = 0;

    void run() {
        std::unique_lock<std::mutex> lk(mu);
        for (;;) {
            wake.wait(lk, [&] { return !tasks.empty(); });
            Task t = tasks.back();
            tasks.pop_back();
            lk.unlock();
            std::memcpy(t.dst, t.src, t.n);
            lk.lock();
            if (--pending == 0) done.notify_all();
        }
    }

    void start(int n) {
        for (int i = n_threads; i < n; ++i) std::thread([this] { run(); }).detach();
        if (n > n_threads) n_threads = n;
    }

    // dst[0, n) = src[0, n) split over the workers and the calling thread
    void copy(char* dst, const char* src, size_t n, int ways) {
        if (ways <= 1 || n < kMinParallel) {
            std::memcpy(dst, src, n);
            return;
        }
        size_t piece = ((n / (size_t)ways) + 4095) & ~(size_t)4095;
        size_t mine = piece < n ? piece : n;
        {
            std::lock_guard<std::mutex> lk(mu);
            for (size_t off = mine; off < n; off += piece) {
                tasks.push_back(Task{dst + off, src + off, (n - off < piece) ? n - off : piece});
                ++pending;
            }
        }
        wake.notify_all();
        std::memcpy(dst, src, mine);
        std::unique_lock<std::mutex> lk(mu);
        done.wait(lk, [&] { return pending == 0; });
    }
};

CopyWorkers* g_workers = nullptr;

struct Stage {
    std::mutex mu;  // one transfer at a time
    char* buf[kSlots] = {nullptr, nullptr, nullptr, nullptr};
    hipEvent_t ev[kSlots] = {nullptr, nullptr, nullptr, nullptr};
    size_t slot_bytes = 0;
    int threads = 0;
    bool ready = false;
    bool failed = false;
};
Stage* g_stage = nullptr;
std::once_flag g_stage_once;

void after_fork_in_child() {
    // the parent's threads and its locks' owners do not exist here
    g_workers = nullptr;
    g_stage = nullptr;  // pinned buffers are not inherited usefully either: start over
    new (&g_stage_once) std::once_flag();
}

long env_long(const char* name, long dflt, long lo, long hi) {
    const char* v = std::getenv(name);
    if (!v || !*v) return dflt;
    char* end = nullptr;
    long x = std::strtol(v, &end, 10);
    if (end == v) return dflt;
    return x < lo ? lo : (x > hi ? hi : x);
}

Stage* stage() {
    std::call_once(g_stage_once, [] {
        static bool hooked = false;
        if (!hooked) {
            pthread_atfork(nullptr, nullptr, after_fork_in_child);
            hooked = true;
        }
        g_stage = new Stage();
        g_stage->slot_bytes = (size_t)env_long("CUMO_HIP_STAGE_MIB", 8, 1, 256) << 20;
        g_stage->threads = (int)env_long("CUMO_HIP_COPY_THREADS", 4, 1, 16);
    });
    return g_stage;
}

// Inside the transfer lock nothing is reported: an installed error handler may leave
// by longjmp, which must not happen while the lock is held. Failures travel out as Err.
struct Err {
    hipError_t st = hipSuccess;
    const char* what = "";
    bool ok() const { return st == hipSuccess; }
    bool check(hipError_t e, const char* w) {
        if (e != hipSuccess && st == hipSuccess) {
            st = e;
            what = w;
        }
        return e == hipSuccess;
    }
};

// allocates the ring on first use
bool stage_ready(Stage* s, Err* err) {
    if (s->ready) return true;
    if (s->failed) return false;
    for (int i = 0; i < kSlots; ++i) {
        void* p = nullptr;
        if (!err->check(hipHostMalloc(&p, s->slot_bytes, hipHostMallocDefault), "hipHostMalloc(staging)") ||
            !err->check(hipEventCreateWithFlags(&s->ev[i], hipEventDisableTiming), "hipEventCreate(staging)")) {
            s->failed = true;
            return false;
        }
        s->buf[i] = (char*)p;
    }
    if (s->threads > 1) {
        if (!g_workers) g_workers = new CopyWorkers();
        g_workers->start(s->threads - 1);
    }
    s->ready = true;
    return true;
}

void host_copy(Stage* s, char* dst, const char* src, size_t n) {
    if (g_workers && s->threads > 1) g_workers->copy(dst, src, n, s->threads);
    else std::memcpy(dst, src, n);
}

bool host_is_pinned(const void* p) {
    hipPointerAttribute_t a;
    if (hipPointerGetAttributes(&a, p) != hipSuccess) {
        (void)hipGetLastError();  // ordinary host memory is "invalid value" to this query
        return false;
    }
    return a.type == hipMemoryTypeHost;
}

void to_host_locked(Stage* s, hipStream_t st, char* dst, const char* src, size_t n, Err* err) {
    if ((n >= s->slot_bytes && host_is_pinned(dst)) || !stage_ready(s, err)) {
        if (!err->ok()) return;
        // pinned memory, or no staging ring to be had: the runtime's own path
        if (err->check(hipMemcpyAsync(dst, src, n, hipMemcpyDeviceToHost, st), "hipMemcpyAsync(d2h)"))
            err->check(hipStreamSynchronize(st), "hipStreamSynchronize");
        return;
    }
    const size_t sb = s->slot_bytes;
    const size_t chunks = (n + sb - 1) / sb;
    if (chunks == 1) {
        // one buffer: wait for the stream itself rather than for an event recorded on it
        if (err->check(hipMemcpyAsync(s->buf[0], src, n, hipMemcpyDeviceToHost, st), "hipMemcpyAsync(d2h)") &&
            err->check(hipStreamSynchronize(st), "hipStreamSynchronize"))
            host_copy(s, dst, s->buf[0], n);
        return;
    }
    auto issue = [&](size_t c) -> bool {
        const size_t off = c * sb, len = (n - off < sb) ? n - off : sb;
        const int k = (int)(c % kSlots);
        return err->check(hipMemcpyAsync(s->buf[k], src + off, len, hipMemcpyDeviceToHost, st), "hipMemcpyAsync(d2h)") &&
               err->check(hipEventRecord(s->ev[k], st), "hipEventRecord");
    };
    bool ok = true;
    for (size_t c = 0; ok && c < chunks && c < (size_t)kSlots; ++c) ok = issue(c);
    for (size_t c = 0; ok && c < chunks; ++c) {
        const size_t off = c * sb, len = (n - off < sb) ? n - off : sb;
        const int k = (int)(c % kSlots);
        ok = err->check(hipEventSynchronize(s->ev[k]), "hipEventSynchronize");
        if (!ok) break;
        host_copy(s, dst + off, s->buf[k], len);
        if (c + kSlots < chunks) ok = issue(c + kSlots);
    }
    if (!ok) (void)hipStreamSynchronize(st);  // nothing may still be writing the ring
}

void from_host_locked(Stage* s, hipStream_t st, char* dst, const char* src, size_t n, Err* err) {
    if ((n >= s->slot_bytes && host_is_pinned(src)) || !stage_ready(s, err)) {
        if (!err->ok()) return;
        if (err->check(hipMemcpyAsync(dst, src, n, hipMemcpyHostToDevice, st), "hipMemcpyAsync(h2d)"))
            err->check(hipStreamSynchronize(st), "hipStreamSynchronize");
        return;
    }
    const size_t sb = s->slot_bytes;
    const size_t chunks = (n + sb - 1) / sb;
    bool ok = true;
    for (size_t c = 0; ok && c < chunks; ++c) {
        const size_t off = c * sb, len = (n - off < sb) ? n - off : sb;
        const int k = (int)(c % kSlots);
        if (c >= (size_t)kSlots) ok = err->check(hipEventSynchronize(s->ev[k]), "hipEventSynchronize");  // the DMA has drained this buffer
        if (!ok) break;
        host_copy(s, s->buf[k], src + off, len);
        ok = err->check(hipMemcpyAsync(dst + off, s->buf[k], len, hipMemcpyHostToDevice, st), "hipMemcpyAsync(h2d)") &&
             err->check(hipEventRecord(s->ev[k], st), "hipEventRecord");
    }
    // also after a failure: nothing may still be reading the ring when the next call reuses it
    err->check(hipStreamSynchronize(st), "hipStreamSynchronize");
}

int transfer(bool to_host, void* dst, const void* src, size_t n) {
    if (n == 0) return CUMO_HIP_OK;
    if (!dst || !src) {
        report_error(CUMO_HIP_ERROR_ARGUMENT, 0, to_host ? "copy_to_host: null pointer" : "copy_from_host: null pointer");
        return CUMO_HIP_ERROR_ARGUMENT;
    }
    hipStream_t st = current_stream();
    Stage* s = stage();
    Err err;
    s->mu.lock();
    if (to_host) to_host_locked(s, st, (char*)dst, (const char*)src, n, &err);
    else from_host_locked(s, st, (char*)dst, (const char*)src, n, &err);
    s->mu.unlock();
    if (err.ok()) {
        // the device has been waited for: a kernel that gave up a bounded wait is reported here
        if (to_host && !wait_trouble_check()) return CUMO_HIP_ERROR_RUNTIME;
        return CUMO_HIP_OK;
    }
    (void)hipGetLastError();  // reported here; must not show up again at the next launch check
    report_hip_error(err.st, err.what);  // may not return
    return err.st == hipErrorOutOfMemory ? CUMO_HIP_ERROR_OUT_OF_MEMORY : CUMO_HIP_ERROR_RUNTIME;
}

}  // namespace
}  // namespace cumo_hip

using namespace cumo_hip;

extern "C" {

// dst (host) = src (device), n bytes; returns when the bytes are in dst
int cumo_hip_copy_to_host(void* dst, const void* src, size_t n) { return transfer(true, dst, src, n); }

// dst (device) = src (host), n bytes; returns when the bytes are in dst
int cumo_hip_copy_from_host(void* dst, const void* src, size_t n) { return transfer(false, dst, src, n); }

}  // extern "C"
