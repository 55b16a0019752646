// all? / any? along the rows of a Bit matrix whose rows start on word boundaries, straight into
// the packed Bit result: a block owns one word of the result and the 32 rows behind its bits,
// a wave reads its eight of them two at a time with 128-bit loads and stops a row's reading once
// it is decided. The reference launches one reduction per row from a host walk
// (gen/tmpl_bit/bit_reduce.c:106-146 over tmpl_bit/bit_reduce_kernel.cu:5-77).
#include "common.h"

using namespace cumo_hip;

namespace {

constexpr int kWaves = 4;   // a block of 4 waves per word of the result: eight rows a wave

typedef uint32_t q4u __attribute__((ext_vector_type(4)));

template <bool NT>
__device__ __forceinline__ uint4 load_q(const uint4* p) {
    if (NT) {
        const q4u v = __builtin_nontemporal_load(reinterpret_cast<const q4u*>(p));
        return make_uint4(v.x, v.y, v.z, v.w);
    }
    return *p;
}

// `found` of a row: some word has a bit set after the flip (all?: a clear bit, any?: a set bit). Two rows at a
// time (the same row twice when there is no second: its answer is not used). Every load of a step is
// unconditional, so that all of them are in flight together: a position past the row's end is pulled back to
// its last vector, and looking at a word twice changes nothing here.
template <bool NT, int U>
__device__ __forceinline__ void rows_found(const uint32_t* r0, const uint32_t* r1, uint32_t full_words, uint32_t tail_mask, uint32_t flip,
                                           bool vec, uint32_t& found0, uint32_t& found1) {
    const uint32_t lane = threadIdx.x & 63u;
    uint32_t a0 = 0, a1 = 0;
    if (vec && full_words >= 4) {
        const uint32_t nv = full_words >> 2;
        const uint4* q0 = reinterpret_cast<const uint4*>(r0);
        const uint4* q1 = reinterpret_cast<const uint4*>(r1);
        for (uint32_t i = lane; i < nv; i += 64u * U) {
            uint4 v0[U], v1[U];
#pragma unroll
            for (int k = 0; k < U; ++k) {
                const uint32_t j = min(i + 64u * k, nv - 1);
                v0[k] = load_q<NT>(q0 + j);
                v1[k] = load_q<NT>(q1 + j);
            }
#pragma unroll
            for (int k = 0; k < U; ++k) {
                a0 |= (v0[k].x ^ flip) | (v0[k].y ^ flip) | (v0[k].z ^ flip) | (v0[k].w ^ flip);
                a1 |= (v1[k].x ^ flip) | (v1[k].y ^ flip) | (v1[k].z ^ flip) | (v1[k].w ^ flip);
            }
            // both rows decided: nothing further down them can change the answer
            if (__builtin_amdgcn_ballot_w64(a0 != 0) != 0 && __builtin_amdgcn_ballot_w64(a1 != 0) != 0) break;
        }
        const uint32_t w = (nv << 2) + lane;  // the words after the last whole vector
        if (w < full_words) {
            a0 |= r0[w] ^ flip;
            a1 |= r1[w] ^ flip;
        }
    } else if (full_words > 0) {
        for (uint32_t i = lane; i < full_words; i += 64u * U) {
            uint32_t v0[U], v1[U];
#pragma unroll
            for (int k = 0; k < U; ++k) {
                const uint32_t j = min(i + 64u * k, full_words - 1);
                v0[k] = r0[j];
                v1[k] = r1[j];
            }
#pragma unroll
            for (int k = 0; k < U; ++k) {
                a0 |= v0[k] ^ flip;
                a1 |= v1[k] ^ flip;
            }
            if (__builtin_amdgcn_ballot_w64(a0 != 0) != 0 && __builtin_amdgcn_ballot_w64(a1 != 0) != 0) break;
        }
    }
    if (tail_mask != 0 && lane == 0) {
        a0 |= (r0[full_words] ^ flip) & tail_mask;
        a1 |= (r1[full_words] ^ flip) & tail_mask;
    }
    found0 = __builtin_amdgcn_ballot_w64(a0 != 0) != 0 ? 1u : 0u;
    found1 = __builtin_amdgcn_ballot_w64(a1 != 0) != 0 ? 1u : 0u;
}

// Word b of `out` holds the results of rows 32 b - shift ... 32 b - shift + 31 (those inside [0, rows)).
template <bool NT, int U>
__global__ __launch_bounds__(kWaves * 64) void bit_anyall_rows_kernel(const uint32_t* __restrict__ in, uint64_t rows, int64_t row_words,
                                                                      uint32_t full_words, uint32_t tail_mask, uint32_t all,
                                                                      uint32_t* __restrict__ out, uint32_t shift, uint32_t vec) {
    __shared__ uint32_t s_found[32];
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t flip = all ? 0xffffffffu : 0u;
    const int64_t first = (int64_t)blockIdx.x * 32 - (int64_t)shift;
    // a wave takes its rows two at a time: wave, wave + kWaves; wave + 2 kWaves, wave + 3 kWaves; ...
    for (int pair = 0; pair < 32 / (2 * kWaves); ++pair) {
        const int slot = (int)wave + 2 * kWaves * pair;
        const int64_t ra = first + slot, rb = ra + kWaves;
        const bool have_a = ra >= 0 && (uint64_t)ra < rows;
        const bool have_b = rb >= 0 && (uint64_t)rb < rows;
        uint32_t fa = 0, fb = 0;
        if (have_a || have_b) {
            const uint32_t* pa = in + (have_a ? ra : rb) * row_words;
            const uint32_t* pb = in + (have_b ? rb : ra) * row_words;
            rows_found<NT, U>(pa, pb, full_words, tail_mask, flip, vec != 0, fa, fb);
            if (!have_a) fa = 0;
            if (!have_b) fb = 0;
        }
        if ((threadIdx.x & 63u) == 0) {
            s_found[slot] = fa;
            s_found[slot + kWaves] = fb;
        }
    }
    __syncthreads();
    if (threadIdx.x < 32) {
        const int64_t r = first + threadIdx.x;
        const bool have = r >= 0 && (uint64_t)r < rows;
        const uint32_t f = s_found[threadIdx.x];
        const uint32_t bit = all ? (f ^ 1u) : f;
        // (only the lower half of the wave is active: the ballots cover its 32 lanes)
        const uint32_t valid = (uint32_t)__builtin_amdgcn_ballot_w64(have);
        const uint32_t word = (uint32_t)__builtin_amdgcn_ballot_w64(have && bit != 0);
        if (threadIdx.x == 0) {
            if (valid == 0xffffffffu) {
                out[blockIdx.x] = word;
            } else if (valid != 0) {
                // the word's other bits belong to neighbours of the result
                atomicAnd(&out[blockIdx.x], ~valid | word);
                atomicOr(&out[blockIdx.x], word);
            }
        }
    }
}

}  // namespace

extern "C" int cumo_hip_bit_anyall_rows_kernel_launch(CUMO_BIT_DIGIT* in, size_t pos, uint64_t rows, int64_t row_step, uint64_t n, int all,
                                                      CUMO_BIT_DIGIT* out, size_t out_pos) {
    if (in == nullptr || out == nullptr || rows == 0 || n == 0) return 0;
    if ((pos % 32) != 0 || (row_step % 32) != 0 || force_wide_indices()) return 0;
    // a row per half wave-pass: short rows leave lanes idle and few rows leave compute units idle;
    // the counts along the rows serve those shapes
    if (n < 4096 || n >= (1ull << 36) || rows < 4096) return 0;
    const uint32_t* base = in + pos / 32;
    const int64_t row_words = row_step / 32;
    const uint32_t full_words = (uint32_t)(n / 32);
    const uint32_t tail = (uint32_t)(n % 32);
    const uint32_t tail_mask = tail ? ((1u << tail) - 1u) : 0u;
    const uint32_t vec = ((reinterpret_cast<uintptr_t>(base) % 16) == 0 && (row_words % 4) == 0) ? 1u : 0u;
    uint32_t* dst = out + out_pos / 32;
    const uint32_t shift = (uint32_t)(out_pos % 32);
    const uint64_t blocks = (shift + rows + 31) / 32;
    if (blocks > 0x7fffffffull) return 0;
    const bool nt = stream_past_caches(rows * (n / 8));
    hipStream_t stream = current_stream();
    const dim3 g((unsigned)blocks), b(kWaves * 64);
    // eight vectors of a row in flight per lane where the rows are long enough to have them, else four
    const bool deep = full_words >= 8 * 4 * 64;
#define CUMO_ANYALL_LAUNCH(NT, U)                                                                                                      \
    hipLaunchKernelGGL((bit_anyall_rows_kernel<NT, U>), g, b, 0, stream, base, rows, row_words, full_words, tail_mask, all ? 1u : 0u, dst, \
                       shift, vec)
    if (nt && deep) CUMO_ANYALL_LAUNCH(true, 8);
    else if (nt) CUMO_ANYALL_LAUNCH(true, 4);
    else if (deep) CUMO_ANYALL_LAUNCH(false, 8);
    else CUMO_ANYALL_LAUNCH(false, 4);
#undef CUMO_ANYALL_LAUNCH
    cumo_cuda_runtime_check_kernel_launch();
    return 1;
}
