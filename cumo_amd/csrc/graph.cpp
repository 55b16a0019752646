// Replay of a recorded chain of operations as one HIP graph.
//
// The reference issues every array operation as its own launch; below about 10^5
// elements an operation costs its launch (about 2.4 us per kernel from the runtime
// here, the library's own work about 0.3 us on top), whatever the kernel does. A caller
// that repeats the same chain on the same arrays (an inner loop) records it once:
// between cumo_hip_graph_begin and cumo_hip_graph_end every launch the library makes
// goes into a stream capture instead of to the device, and cumo_hip_graph_launch then
// replays the whole chain with one submission. The reference has no counterpart.
//
// What a capture may hold: anything that only launches kernels. Operations that read
// something back to decide what to do (Int32 division and abs with their error flag,
// Bit#where / mask sizing their result, host read-back) end the capture with an error.
// Memory: arrays allocated inside the capture are the caller's as usual and every
// replay writes into them again; whatever is released inside the capture (the
// library's temporaries, the caller's intermediates) stays reserved for the graph until
// it is destroyed, because every replay uses it again. No memset node is recorded:
// the library clears memory with fill kernels.
#include "common.h"

#include <mutex>
#include <vector>

namespace cumo_hip {

namespace {
struct Graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    std::vector<char*> held;  // released inside the capture; given back on destroy
};
struct Capture {
    std::mutex mu;
    bool active = false;
    Graph* cur = nullptr;
    hipStream_t stream = nullptr;  // the library's capture stream (default priority), created once
    hipStream_t prev = nullptr;
};
Capture g_cap;
}  // namespace

// Called by the allocator: true when the pointer was taken over by the open capture.
bool capture_defer_free(char* ptr) {
    if (!g_cap.active) return false;
    std::lock_guard<std::mutex> lk(g_cap.mu);
    if (!g_cap.active || !g_cap.cur) return false;
    g_cap.cur->held.push_back(ptr);
    return true;
}

// Called by the allocator: inside a capture a block that was freed on another stream
// is taken without recording an event there (cumo_hip_graph_begin has waited for the
// whole device, and an event from outside the capture may not be waited on inside it).
bool capture_active() { return g_cap.active; }

}  // namespace cumo_hip

using namespace cumo_hip;

extern "C" {

void cumo_cuda_runtime_free(char* ptr);

int cumo_hip_graph_begin(void) {
    hipError_t st = hipSuccess;
    const char* what = "";
    int rc = CUMO_HIP_OK;
    g_cap.mu.lock();
    if (g_cap.active) {
        rc = CUMO_HIP_ERROR_ARGUMENT;
    } else {
        // everything queued so far is done before the capture starts: inputs are ready
        // and free blocks of any stream can be handed out without further ordering
        (void)hipGetLastError();  // an error somebody left unread must not be taken for a failed launch below
        st = hipDeviceSynchronize();
        what = "hipDeviceSynchronize";
        if (st == hipSuccess && !g_cap.stream) {
            st = hipStreamCreateWithFlags(&g_cap.stream, hipStreamNonBlocking);
            what = "hipStreamCreate";
        }
        if (st == hipSuccess) {
            st = hipStreamBeginCapture(g_cap.stream, hipStreamCaptureModeRelaxed);
            what = "hipStreamBeginCapture";
        }
        if (st == hipSuccess) {
            g_cap.prev = (hipStream_t)cumo_hip_get_stream();
            cumo_hip_set_stream((void*)g_cap.stream);
            g_cap.cur = new Graph();
            g_cap.active = true;
        } else {
            rc = CUMO_HIP_ERROR_RUNTIME;
        }
    }
    g_cap.mu.unlock();
    if (rc == CUMO_HIP_ERROR_ARGUMENT) report_error(rc, 0, "graph_begin: a capture is already open");
    else if (rc) report_hip_error(st, what);
    return rc;
}

void* cumo_hip_graph_end(void) {
    hipError_t st = hipSuccess;
    const char* what = "";
    Graph* g = nullptr;
    bool was_open = false;
    g_cap.mu.lock();
    if (g_cap.active) {
        was_open = true;
        g = g_cap.cur;
        g_cap.cur = nullptr;
        g_cap.active = false;
        st = hipStreamEndCapture(g_cap.stream, &g->graph);
        what = "hipStreamEndCapture (an operation inside the capture needed the host)";
        cumo_hip_set_stream((void*)g_cap.prev);
        if (st != hipSuccess) {
            // a capture that broke leaves its stream behind; the next one starts on a new stream
            (void)hipStreamDestroy(g_cap.stream);
            g_cap.stream = nullptr;
        }
        if (st == hipSuccess) {
            st = hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0);
            what = "hipGraphInstantiate";
        }
    }
    g_cap.mu.unlock();
    if (!was_open) {
        report_error(CUMO_HIP_ERROR_ARGUMENT, 0, "graph_end: no capture is open");
        return nullptr;
    }
    if (st != hipSuccess) {
        (void)hipGetLastError();
        // nothing was submitted: what the capture held goes back at once
        std::vector<char*> held;
        held.swap(g->held);
        if (g->graph) (void)hipGraphDestroy(g->graph);
        delete g;
        for (char* p : held) cumo_cuda_runtime_free_no_raise(p);
        report_hip_error(st, what);
        return nullptr;
    }
    return g;
}

// one replay, queued on the library's current stream
int cumo_hip_graph_launch(void* graph) {
    Graph* g = (Graph*)graph;
    if (!g || !g->exec) {
        report_error(CUMO_HIP_ERROR_ARGUMENT, 0, "graph_launch: not a graph");
        return CUMO_HIP_ERROR_ARGUMENT;
    }
    hipError_t st = hipGraphLaunch(g->exec, current_stream());
    if (st != hipSuccess) {
        report_hip_error(st, "hipGraphLaunch");
        return CUMO_HIP_ERROR_RUNTIME;
    }
    return CUMO_HIP_OK;
}

size_t cumo_hip_graph_node_count(void* graph) {
    Graph* g = (Graph*)graph;
    size_t n = 0;
    if (!g || !g->graph || hipGraphGetNodes(g->graph, nullptr, &n) != hipSuccess) return 0;
    return n;
}

// waits for the device (a replay may still be running), then releases the graph and
// the memory it kept reserved
void cumo_hip_graph_destroy(void* graph) {
    Graph* g = (Graph*)graph;
    if (!g) return;
    (void)hipDeviceSynchronize();
    if (g->exec) (void)hipGraphExecDestroy(g->exec);
    if (g->graph) (void)hipGraphDestroy(g->graph);
    std::vector<char*> held;
    held.swap(g->held);
    delete g;
    for (char* p : held) cumo_cuda_runtime_free_no_raise(p);
}

}  // extern "C"
