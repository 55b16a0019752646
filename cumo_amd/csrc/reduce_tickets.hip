// The ticket words of the one-launch split reductions (reduce_stream.h): a fixed
// array in the library's device image, a stretch per stream slot, zero whenever no
// reduction of that stream is running (the block that counts in last puts the words
// it used back to zero). One copy per device; its address is looked up once per device.
#include "common.h"

#include <mutex>

namespace cumo_hip {

namespace {
constexpr uint32_t kTicketWords = 16384;  // = kRsTicketWords (reduce_stream.h)
constexpr int kMaxDevices = 64;
__device__ uint32_t g_red_tickets[kStreamSlots * kTicketWords];
// The hand-over words of the one-launch full reductions: 64-bit words {launch number, 32 bits of a
// partial result}, a stretch per stream slot. A word counts only when it carries the running
// launch's number, so the array never needs clearing (it starts as zeros; launch numbers start at 1).
constexpr uint32_t kHandoverWords = 8192;  // = kRsHandoverWords (reduce_stream.h)
__device__ uint64_t g_red_handover[kStreamSlots * kHandoverWords];
std::mutex g_lock;
uint32_t* g_base[kMaxDevices];
uint64_t* g_handover_base[kMaxDevices];
uint32_t g_launch_number[kMaxDevices][kStreamSlots];
}  // namespace

uint64_t* red_handover_words(int slot, uint32_t* launch_number) {
    if (slot < 0 || slot >= kStreamSlots) return nullptr;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return nullptr;
    }
    std::lock_guard<std::mutex> hold(g_lock);
    if (g_handover_base[dev] == nullptr) {
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_red_handover)) != hipSuccess) {
            (void)hipGetLastError();
            return nullptr;  // the caller takes the ticket form
        }
        g_handover_base[dev] = static_cast<uint64_t*>(p);
    }
    uint32_t& n = g_launch_number[dev][slot];
    n = (n == 0xffffffffu) ? 1u : n + 1u;  // never 0 (after 2^32 launches on one stream a number comes round again)
    *launch_number = n;
    return g_handover_base[dev] + (size_t)slot * kHandoverWords;
}

uint32_t* red_ticket_words(int slot) {
    if (slot < 0 || slot >= kStreamSlots) return nullptr;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return nullptr;
    }
    std::lock_guard<std::mutex> hold(g_lock);
    if (g_base[dev] == nullptr) {
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_red_tickets)) != hipSuccess) {
            (void)hipGetLastError();
            return nullptr;  // the caller falls back to the two-launch form
        }
        g_base[dev] = static_cast<uint32_t*>(p);
    }
    return g_base[dev] + (size_t)slot * kTicketWords;
}

}  // namespace cumo_hip
