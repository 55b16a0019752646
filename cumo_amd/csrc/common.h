// Shared host-side plumbing of the library: error reporting, the per-thread
// stream, and the launch-check helper every launcher ends with.
#ifndef CUMO_HIP_COMMON_H
#define CUMO_HIP_COMMON_H

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include "cumo_hip.h"

namespace cumo_hip {

// Reports an error to the installed handler (which may not return) or latches
// it for cumo_hip_last_error. Callers must hold no C++ object with a
// destructor when they call it: a Ruby handler raises with longjmp.
void report_error(int kind, int hip_status, const char* message);
void report_hip_error(hipError_t status, const char* what);

hipStream_t current_stream();

// A number in [0, kStreamSlots) that belongs to this stream until it is destroyed
// through cumo_hip_stream_destroy, or -1 when every number is taken. Kernels that
// keep per-stream words in a fixed device array (tickets) index it with this.
constexpr int kStreamSlots = 64;
int stream_slot(hipStream_t stream);
int stream_slot_release(hipStream_t stream);  // the number it held, or -1

// pool.cpp: files everything the pool holds for a drained stream under the null stream.
void pool_retire_stream(hipStream_t stream);

// scan.hip: the regions of look-back words that streams keep from launch to launch. Dropped for
// a stream slot when its (drained) stream is retired, and all of them by free_all_blocks.
void scan_chain_words_drop_slot(int slot);
void scan_chain_words_drop_all();
size_t scan_chain_words_held_bytes();

// Device address of the reduction ticket words of a stream slot (zero between launches),
// nullptr after reporting an error. reduce_tickets.hip.
uint32_t* red_ticket_words(int slot);
// the slot's hand-over words for one launch of a full reduction, and that launch's number (never 0)
uint64_t* red_handover_words(int slot, uint32_t* launch_number);

// Bit counts through the reduction kernels (bit_count_reduce.hip): 1 when launched, 0 when the run or
// the loop is not one they take (the caller then uses the Bit kernels' own forms).
int bit_count_run_reduce(CUMO_BIT_DIGIT* a, size_t pos, uint64_t n, int count_false, uint64_t* out);
int bit_count_rows_reduce(const cumo_hip_bit_count_nd_t* counts);  // (stores the counts when counts->overwrite, adds them otherwise)
// Bit counts down the rows of a matrix whose rows start on word boundaries (bit_count_cols.hip): 1 when
// launched (stored or added as counts->overwrite says), 0 when the loop is not one it takes.
int bit_count_cols_words_launch(const cumo_hip_bit_count_nd_t* counts);

// x op y (op: 0 + 1 - 2 * 3 /) for two contiguous, 16-byte aligned runs of n elements of different types
// (SFloat / DFloat / Int32), converted to the result's type on the way in, into z of that type (ew_mixed.hip).
// False when the pair of types or the alignment is not one it takes; nothing is launched then.
bool mixed_flat_binary(int op, int ta, const char* x, int tb, const char* y, char* z, uint64_t n);
// the same for a contiguous Int32 run and one DFloat number (on the left when scalar_is_left), into a DFloat run
bool mixed_flat_binary_s(int op, const char* x, double sv, bool scalar_is_left, char* z, uint64_t n);

// x cmp y (cmp: 0 == 1 != 2 > 3 >= 4 < 5 <=) for two such runs into the bits of z from its first word on
bool mixed_flat_compare(int cmp, int ta, const char* x, int tb, const char* y, CUMO_BIT_DIGIT* z, uint64_t n);

// CUMO_HIP_FORCE_WIDE=1 (read once): every launch takes the 64-bit index arithmetic of the
// general kernels, whatever the array's size, and the lean kernels (which are 32-bit only)
// stand aside. For tests: the wide paths otherwise only run on arrays beyond 2^32 elements.
bool force_wide_indices();

// Whether a launch that moves `bytes` through memory once should use non-temporal
// accesses: from 48 MiB upward the data neither comes from nor is wanted in the caches,
// and keeping it out of them is measurably faster on operands that were not just
// touched. CUMO_HIP_NT=0 / 1 (read once) forces the answer.
constexpr uint64_t kStreamNtBytes = 48ull << 20;
bool stream_past_caches(uint64_t bytes);

// A kernel that waits for another block's word (the hand-over words of a split reduction, the
// look-back of a one-pass scan, the totals of a one-launch mulsum) waits a bounded number of
// looks. One that gives up cannot produce its result: it counts the event and raises the
// pinned host word, and the next point where the host waits for the device
// (wait_trouble_check) reports CUMO_HIP_ERROR_RUNTIME, the way a rejected element is
// reported through the pinned error flag (reference: cuda/runtime.c:22-47).
struct WaitCtl {
    uint32_t limit_scale;    // 0: give up at the first failed look (test knob); 1: the kernels' own limits
    uint32_t reserved;
    uint32_t* host_flag;     // pinned, device-mapped host word
    uint32_t gave_up[4];     // counts by family: see WaitFamily
};
enum WaitFamily { WAIT_REDUCE = 0, WAIT_SCAN = 1, WAIT_MULSUM = 2 };
// Device address of the block (allocated and filled on the first call; one per process),
// nullptr after reporting an error.
WaitCtl* wait_ctl();
// Host: reports and clears a raised give-up word. False when one was raised.
bool wait_trouble_check();
// Compute units of the current device (queried once).
int device_compute_units();

static inline bool hip_ok(hipError_t status, const char* what) {
    if (status == hipSuccess) return true;
    report_hip_error(status, what);
    return false;
}

}  // namespace cumo_hip

#endif
