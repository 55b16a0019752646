// Device memory pool over hipMalloc with stream-ordered reuse.
//
// Replaces cumo::internal::MemoryPool (reference: ext/cumo/cuda/memory_pool_impl.hpp:160-435,
// memory_pool_impl.cpp:16-353) and the extension's wrappers around it
// (ext/cumo/cuda/memory_pool.cpp:39-137). What is kept from there is the
// observable behaviour: sizes round up to 512 bytes, the smallest free chunk
// that fits is taken and split, a freed chunk merges with free neighbours of
// the same device allocation, an allocation failure frees every unsplit free
// block and retries once, and the counters used/free/total/n_free_blocks mean
// what they meant.
//
// What is different:
//  * an array of 2 MiB or more that is cut out of a larger free chunk starts on a
//    2 MiB boundary (the bytes before it stay a free chunk), so that large operands
//    keep the relative placement fresh device allocations have.
//  * plain hipMalloc, not managed memory: 288 GB of HBM is addressed directly
//    and nothing migrates; the host reads results back with explicit copies.
//  * each stream's arena is an ordered multimap keyed by chunk size, so best
//    fit is one lower_bound instead of a walk over a sparse bin vector, and the
//    byte counters are kept incrementally instead of by walking every chunk.
//  * reuse is stream ordered. A chunk freed from stream S goes back to S's
//    arena and can be handed out again on S at once: the kernels that used it
//    were queued on S before whatever the new owner queues. When S's arena has
//    nothing that fits, a chunk is taken from another stream's arena before
//    falling back to hipMalloc; the taking stream is made to wait (on the
//    device, hipStreamWaitEvent) for everything queued so far on the giving
//    stream, and the chunk moves arena for good. hipMalloc and hipFree, which
//    synchronise the device, stay off the steady-state path.
#include "common.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

namespace cumo_hip {
namespace {

constexpr size_t kRound = 512;  // hipMalloc alignment is at least this
// Arrays of at least this size start on a multiple of it when the pool cuts them out
// of a larger free chunk (a fresh device allocation of that size is aligned like this
// already). Measured reason: with two 128 MiB operands a strided-read / contiguous-write
// kernel ran 42.7 us when the operands were a multiple of 2 MiB apart and 45-47 us at
// 4 KiB or 1 MiB apart, the spread a chunk's position inside a reused block would give.
constexpr size_t kBigAlign = (size_t)2 << 20;
constexpr size_t kMaxAlloc = ~(size_t)0 - (kRound - 1);

struct Block;  // one hipMalloc

struct Chunk {
    char* ptr;
    size_t size;
    Block* block;
    Chunk* prev;  // address-ordered neighbours inside the same block
    Chunk* next;
    hipStream_t stream;
    bool in_use;
    std::multimap<size_t, Chunk*>::iterator where;  // valid while free
};

struct Block {
    char* base;
    size_t size;
};

typedef std::multimap<size_t, Chunk*> Arena;

// Backend: the device by default; tests swap in the host heap so that split,
// merge and accounting can be exercised on a machine without a GPU.
struct Backend {
    int (*alloc)(void** p, size_t n);  // 0 ok, 1 out of memory, <0 other hip error (negated)
    int (*release)(void* p);
};

int device_alloc(void** p, size_t n) {
    hipError_t st = hipMalloc(p, n);
    if (st == hipSuccess) return 0;
    (void)hipGetLastError();
    if (st == hipErrorOutOfMemory || st == hipErrorMemoryAllocation) return 1;
    return -(int)st;
}
int device_release(void* p) {
    hipError_t st = hipFree(p);
    if (st == hipSuccess || st == hipErrorDeinitialized) return 0;
    (void)hipGetLastError();
    return -(int)st;
}
int host_alloc(void** p, size_t n) {
    if (n > ((size_t)1 << 40)) return 1;
    void* q = nullptr;
    if (posix_memalign(&q, kRound, n) != 0) return 1;
    *p = q;
    return 0;
}
int host_release(void* p) { free(p); return 0; }

class Pool {
  public:
    std::mutex mu;
    std::unordered_map<hipStream_t, Arena> arenas;
    std::unordered_map<char*, Chunk*> in_use;
    size_t used_bytes = 0, free_bytes = 0, n_free = 0;
    size_t limit = 0;
    size_t device_calls = 0;
    Backend be{device_alloc, device_release};
    bool host_backend = false;

    static size_t rounded(size_t n) { return ((n + kRound - 1) / kRound) * kRound; }

    void arena_insert(Chunk* c) {
        c->where = arenas[c->stream].emplace(c->size, c);
        free_bytes += c->size;
        ++n_free;
    }
    void arena_erase(Chunk* c) {
        auto it = arenas.find(c->stream);
        it->second.erase(c->where);
        if (it->second.empty()) arenas.erase(it);
        free_bytes -= c->size;
        --n_free;
    }

    // smallest chunk >= size in the arena of `stream`
    Chunk* take_best_fit(hipStream_t stream, size_t size) {
        auto a = arenas.find(stream);
        if (a == arenas.end()) return nullptr;
        auto it = a->second.lower_bound(size);
        if (it == a->second.end()) return nullptr;
        Chunk* c = it->second;
        arena_erase(c);
        return c;
    }

    static size_t misalignment(const char* p) {
        const size_t r = (size_t)((uintptr_t)p % kBigAlign);
        return r ? kBigAlign - r : 0;
    }

    // c is free and outside the arenas: its first `head` bytes become a free chunk of their own
    void carve_head(Chunk* c, size_t head) {
        Chunk* h = new Chunk{c->ptr, head, c->block, c->prev, c, c->stream, false, {}};
        if (c->prev) c->prev->next = h;
        c->prev = h;
        c->ptr += head;
        c->size -= head;
        arena_insert(h);
    }

    // for size >= kBigAlign: the smallest chunk that holds `size` bytes from an aligned
    // address on, cut so that it starts there; an unaligned best fit when none does
    Chunk* take_aligned_fit(hipStream_t stream, size_t size) {
        auto a = arenas.find(stream);
        if (a == arenas.end()) return nullptr;
        int looked = 0;
        for (auto it = a->second.lower_bound(size); it != a->second.end() && looked < 64; ++it, ++looked) {
            Chunk* c = it->second;
            const size_t head = misalignment(c->ptr);
            if (head + size > c->size) continue;
            arena_erase(c);
            if (head) carve_head(c, head);
            return c;
        }
        return take_best_fit(stream, size);
    }

    // A chunk from another stream's arena. The caller orders the streams.
    Chunk* steal(hipStream_t stream, size_t size, hipStream_t* from) {
        Chunk* best = nullptr;
        for (auto& kv : arenas) {
            if (kv.first == stream) continue;
            auto it = kv.second.lower_bound(size);
            if (it == kv.second.end()) continue;
            if (!best || it->second->size < best->size) best = it->second;
        }
        if (!best) return nullptr;
        // Only whole blocks change stream: a split chunk's neighbours stay in
        // the old arena, and merging across arenas would break the ordering.
        if (best->prev || best->next) {
            best = nullptr;
            for (auto& kv : arenas) {
                if (kv.first == stream) continue;
                for (auto it = kv.second.lower_bound(size); it != kv.second.end(); ++it) {
                    Chunk* c = it->second;
                    if (!c->prev && !c->next) { if (!best || c->size < best->size) best = c; break; }
                }
            }
            if (!best) return nullptr;
        }
        *from = best->stream;
        arena_erase(best);
        best->stream = stream;
        return best;
    }

    void split(Chunk* c, size_t size) {
        if (c->size == size) return;
        Chunk* r = new Chunk{c->ptr + size, c->size - size, c->block, c, c->next, c->stream, false, {}};
        if (c->next) c->next->prev = r;
        c->next = r;
        c->size = size;
        arena_insert(r);
    }

    // hipFree every free chunk that is a whole block. Returns a negative hip
    // status if the device refused one.
    int release_unsplit(bool only_stream, hipStream_t stream) {
        std::vector<Chunk*> victims;
        for (auto& kv : arenas) {
            if (only_stream && kv.first != stream) continue;
            for (auto& e : kv.second) {
                Chunk* c = e.second;
                if (!c->prev && !c->next) victims.push_back(c);
            }
        }
        int rc = 0;
        for (Chunk* c : victims) {
            arena_erase(c);
            int r = be.release(c->block->base);
            if (r < 0 && rc == 0) rc = r;
            delete c->block;
            delete c;
        }
        return rc;
    }

    size_t held() const { return used_bytes + free_bytes; }
};

Pool g_pool;
bool g_enabled = true;
std::once_flag g_env_once;

void read_env() {
    const char* env = std::getenv("CUMO_MEMORY_POOL");  // reference: cuda/memory_pool.cpp:262-264
    if (env) {
        std::string v(env);
        g_enabled = !(v == "OFF" || v == "0" || v == "NO");
    }
}

}  // namespace

// A stream that is about to be destroyed (and has been drained): every chunk filed under
// it, free or in use, moves to the null stream's arena, so that nothing stays keyed by a
// dead handle (its free chunks could never be reused or ordered against otherwise).
void pool_retire_stream(hipStream_t stream) {
    if (stream == nullptr) return;
    Pool& p = g_pool;
    std::unique_lock<std::mutex> lock(p.mu);
    std::vector<Chunk*> moved;
    auto a = p.arenas.find(stream);
    if (a != p.arenas.end()) {
        for (auto& e : a->second) moved.push_back(e.second);
    }
    for (Chunk* c : moved) {
        p.arena_erase(c);
        c->stream = nullptr;
        p.arena_insert(c);
    }
    for (auto& kv : p.in_use) {
        if (kv.second->stream == stream) kv.second->stream = nullptr;
    }
}

}  // namespace cumo_hip

using namespace cumo_hip;

extern "C" {

int cumo_hip_pool_malloc(size_t size, void* hip_stream, void** out) {
    hipStream_t stream = (hipStream_t)hip_stream;
    *out = nullptr;
    if (size == 0) return CUMO_HIP_OK;  // reference: memory_pool_impl.cpp:114-120
    if (size > kMaxAlloc) return CUMO_HIP_ERROR_OUT_OF_MEMORY;
    size = Pool::rounded(size);

    Pool& p = g_pool;
    std::unique_lock<std::mutex> lock(p.mu);

    Chunk* c = size >= kBigAlign ? p.take_aligned_fit(stream, size) : p.take_best_fit(stream, size);
    if (!c) {
        hipStream_t from = nullptr;
        c = p.steal(stream, size, &from);
        if (c && !p.host_backend) {
            // everything queued so far on the giving stream must finish before
            // work queued from now on the taking stream touches the chunk
            hipEvent_t ev = nullptr;
            bool ok = hipEventCreateWithFlags(&ev, hipEventDisableTiming) == hipSuccess;
            ok = ok && hipEventRecord(ev, from) == hipSuccess;
            ok = ok && hipStreamWaitEvent(stream, ev, 0) == hipSuccess;
            if (ev) (void)hipEventDestroy(ev);
            if (!ok) {
                (void)hipGetLastError();
                (void)hipStreamSynchronize(from);
            }
        }
    }
    if (c) {
        const size_t head = size >= kBigAlign ? Pool::misalignment(c->ptr) : 0;
        if (head && head + size <= c->size) p.carve_head(c, head);  // a chunk taken over from another stream
        p.split(c, size);
    } else {
        if (p.limit && p.held() + size > p.limit) {
            p.release_unsplit(false, nullptr);
            if (p.held() + size > p.limit) return CUMO_HIP_ERROR_OUT_OF_MEMORY;
        }
        void* raw = nullptr;
        ++p.device_calls;
        int r = p.be.alloc(&raw, size);
        if (r == 1) {
            // reference: memory_pool_impl.cpp:167-186 -- give the device back
            // everything that is not split and try once more
            p.release_unsplit(false, nullptr);
            ++p.device_calls;
            r = p.be.alloc(&raw, size);
        }
        if (r == 1) return CUMO_HIP_ERROR_OUT_OF_MEMORY;
        if (r < 0) return CUMO_HIP_ERROR_RUNTIME;
        Block* b = new Block{(char*)raw, size};
        c = new Chunk{(char*)raw, size, b, nullptr, nullptr, stream, false, {}};
    }
    c->in_use = true;
    p.in_use.emplace(c->ptr, c);
    p.used_bytes += c->size;
    *out = c->ptr;
    return CUMO_HIP_OK;
}

int cumo_hip_pool_free(void* ptr) {
    if (!ptr) return CUMO_HIP_OK;
    Pool& p = g_pool;
    std::unique_lock<std::mutex> lock(p.mu);
    auto it = p.in_use.find((char*)ptr);
    if (it == p.in_use.end()) return CUMO_HIP_ERROR_ARGUMENT;
    Chunk* c = it->second;
    p.in_use.erase(it);
    c->in_use = false;
    p.used_bytes -= c->size;
    // merge with free neighbours of the same block (they are in the same
    // arena: a chunk only changes stream while it is a whole block)
    if (c->next && !c->next->in_use && c->next->stream == c->stream) {
        Chunk* n = c->next;
        p.arena_erase(n);
        c->size += n->size;
        c->next = n->next;
        if (n->next) n->next->prev = c;
        delete n;
    }
    if (c->prev && !c->prev->in_use && c->prev->stream == c->stream) {
        Chunk* q = c->prev;
        p.arena_erase(q);
        q->size += c->size;
        q->next = c->next;
        if (c->next) c->next->prev = q;
        delete c;
        c = q;
    }
    p.arena_insert(c);
    return CUMO_HIP_OK;
}

void cumo_hip_pool_free_all_blocks(void) {
    Pool& p = g_pool;
    int rc;
    {
        std::unique_lock<std::mutex> lock(p.mu);
        rc = p.release_unsplit(false, nullptr);
    }
    // memory the library holds outside the pool's books: the scans' kept look-back words
    scan_chain_words_drop_all();
    if (rc < 0) report_hip_error((hipError_t)(-rc), "hipFree");
}

size_t cumo_hip_pool_held_outside_bytes(void) { return scan_chain_words_held_bytes(); }

void cumo_hip_pool_free_all_blocks_stream(void* hip_stream) {
    Pool& p = g_pool;
    int rc;
    {
        std::unique_lock<std::mutex> lock(p.mu);
        rc = p.release_unsplit(true, (hipStream_t)hip_stream);
    }
    if (rc < 0) report_hip_error((hipError_t)(-rc), "hipFree");
}

size_t cumo_hip_pool_n_free_blocks(void) { std::unique_lock<std::mutex> l(g_pool.mu); return g_pool.n_free; }
size_t cumo_hip_pool_used_bytes(void) { std::unique_lock<std::mutex> l(g_pool.mu); return g_pool.used_bytes; }
size_t cumo_hip_pool_free_bytes(void) { std::unique_lock<std::mutex> l(g_pool.mu); return g_pool.free_bytes; }
size_t cumo_hip_pool_total_bytes(void) { std::unique_lock<std::mutex> l(g_pool.mu); return g_pool.used_bytes + g_pool.free_bytes; }
size_t cumo_hip_pool_device_malloc_calls(void) { std::unique_lock<std::mutex> l(g_pool.mu); return g_pool.device_calls; }

int cumo_hip_pool_enable(int on) {
    std::call_once(g_env_once, read_env);
    int prev = g_enabled ? 1 : 0;
    if (on >= 0) g_enabled = on != 0;
    return prev;
}

void cumo_hip_pool_retire_stream(void* hip_stream) { pool_retire_stream((hipStream_t)hip_stream); }

void cumo_hip_pool_set_limit(size_t bytes) { std::unique_lock<std::mutex> l(g_pool.mu); g_pool.limit = bytes; }

// Test hook: back the pool with the host heap (1) or the device (0). Only
// legal while the pool holds nothing.
int cumo_hip_pool_use_host_backend(int on) {
    Pool& p = g_pool;
    std::unique_lock<std::mutex> lock(p.mu);
    if (p.used_bytes || p.free_bytes) return CUMO_HIP_ERROR_ARGUMENT;
    p.host_backend = on != 0;
    p.be = on ? Backend{host_alloc, host_release} : Backend{device_alloc, device_release};
    return CUMO_HIP_OK;
}

// reference: cuda/memory_pool.cpp:64-96. The Ruby GC retry of the reference
// belongs to the host that owns a GC; it can be done from the error handler.
char* cumo_cuda_runtime_malloc(size_t size) {
    std::call_once(g_env_once, read_env);
    void* ptr = nullptr;
    if (!g_enabled) {
        if (size == 0) return nullptr;
        hipError_t st = hipMalloc(&ptr, size);
        if (st != hipSuccess) {
            (void)hipGetLastError();
            report_hip_error(st, "hipMalloc");
            return nullptr;
        }
        return (char*)ptr;
    }
    int rc = cumo_hip_pool_malloc(size, (void*)current_stream(), &ptr);
    if (rc == CUMO_HIP_OK) return (char*)ptr;
    char msg[192];
    if (rc == CUMO_HIP_ERROR_OUT_OF_MEMORY) {
        std::snprintf(msg, sizeof(msg), "out of memory to allocate %zu bytes (total %zu bytes)", size,
                      size + cumo_hip_pool_total_bytes());
    } else {
        std::snprintf(msg, sizeof(msg), "device allocation of %zu bytes failed", size);
    }
    report_error(rc, 0, msg);
    return nullptr;
}

static int runtime_free(char* ptr) {
    if (!ptr) return 0;
    // offer the pointer to the pool first whatever the enabled flag says now
    // (reference: cuda/memory_pool.cpp:98-117)
    if (cumo_hip_pool_free(ptr) == CUMO_HIP_OK) return 0;
    hipError_t st = hipFree(ptr);
    if (st == hipSuccess || st == hipErrorDeinitialized) return 0;
    (void)hipGetLastError();
    return (int)st;
}

void cumo_cuda_runtime_free(char* ptr) {
    int st = runtime_free(ptr);
    if (st) report_hip_error((hipError_t)st, "hipFree");
}

void cumo_cuda_runtime_free_no_raise(char* ptr) {
    int st = runtime_free(ptr);
    if (st) {
        std::fprintf(stderr, "cumo: failed to free device memory: %s (error=%d)\n",
                     hipGetErrorString((hipError_t)st), st);
    }
}

}  // extern "C"
