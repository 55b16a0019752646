// Division of a 31-bit number by a fixed divisor as one multiply and one shift:
// with s = ceil(log2 d) and M = ceil(2^(31+s) / d) (which fits 32 bits),
// n / d = (n * M) >> (31 + s) for every n < 2^31 (Granlund and Montgomery, "Division
// by invariant integers using multiplication", with N = 31).
#pragma once
#ifndef CUMO_HIP_HOST_CHECK  // (a CPU build of the element functions defines the qualifiers away)
#include <hip/hip_runtime.h>
#endif

#include <cstdint>

namespace cumo_hip {

struct Div31 {
    uint32_t mul, shift;
};

inline Div31 div31_make(uint32_t d) {
    uint32_t s = 0;
    while (s < 31 && (1u << s) < d) ++s;
    const unsigned __int128 one = 1;
    const unsigned __int128 m = ((one << (31 + s)) + d - 1) / d;
    return Div31{(uint32_t)m, 31 + s};
}

__device__ __forceinline__ uint32_t div31(uint32_t n, Div31 d) { return (uint32_t)(((uint64_t)n * d.mul) >> d.shift); }

}  // namespace cumo_hip
