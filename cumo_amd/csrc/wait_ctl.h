// Device side of the bounded waits: the look limit and what a wait does when it gives up.
#ifndef CUMO_HIP_WAIT_CTL_H
#define CUMO_HIP_WAIT_CTL_H

#include "common.h"

namespace cumo_hip {

// the limit of looks for this launch: the kernel's own, or 0 under the test knob
__device__ __forceinline__ uint32_t wait_limit(const WaitCtl* ctl, uint32_t own) {
    return ctl->limit_scale ? own : 0u;
}

// Called by one lane of a wait that gave up. The result of the launch is not valid from here
// on; the kernel still runs to its end with whatever the word held.
__device__ __forceinline__ void wait_gave_up(WaitCtl* ctl, int family) {
    __hip_atomic_fetch_add(&ctl->gave_up[family], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(ctl->host_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

}  // namespace cumo_hip

#endif
