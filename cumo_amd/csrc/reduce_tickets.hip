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
std::mutex g_lock;
uint32_t* g_base[kMaxDevices];
}  // namespace

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
