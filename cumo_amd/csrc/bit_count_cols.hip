// count_true / count_false down the rows of a Bit matrix (the counted dimension is the
// slow one, the kept one runs along the words), for rows that start on word boundaries.
//
// The reference has no kernel for this: its ndloop walks the outputs on the host and
// launches tmpl_bit/bit_count_kernel.cu:4-78 once per output (narray/ndloop.c:1569-1613),
// one thread per bit and one 64-bit atomicAdd per set bit.
//
// Here a lane owns one word of a row (32 columns) and walks a stretch of rows with sixteen
// rows' loads in flight. The sixteen words are not counted bit by bit: they go through a
// tree of carry-save adders (three words in, a sum word and a carry word out, three
// instructions) into a counter that stands upright in registers, bit q of every column's
// count in plane q. That is about four vector instructions per word instead of the
// twenty-four a byte-sliced count needs, which alone would take as long as the rows take to
// arrive. The stretches of a block (its groups of lanes) add their upright counters in a
// binary tree through LDS, still as planes; only then a thread per column reads its count
// off the planes. The blocks of a column group leave their counts in scratch, and the one
// that counts in last (a ticket per column group) adds them up in order and writes the
// results: no zero-fill launch before and no atomics on the results. count_false counts the
// set bits too and takes them from the number of rows at the end.
#include "bit_common.h"

#include <cstdlib>

using namespace cumo_hip;

namespace {

constexpr uint32_t kTicketWordsPerSlot = 16384;   // what red_ticket_words() hands out per stream slot (reduce_tickets.hip)
constexpr int kVcRows = 16;            // rows a lane has in flight
constexpr uint32_t kVcStretch = 240;   // rows between two additions to the long counter: 15 groups of 16, so planes 4..7 count to 15
constexpr int kVcPlanes = 8;           // planes of the short counter: up to 255 rows
constexpr int kVcBlockPlanes = 14;     // planes of a group's and a block's counter: up to 16383 rows
constexpr int kVcBufferWord3 = 0x00020000;   // buffer descriptor, last word: raw 32-bit data, no swizzle, no bounds beyond num_records
constexpr int kVcAuxNt = 2;                  // buffer load cache policy: non-temporal

struct BitCountColsVc {
    const uint32_t* in;       // word of (row 0, column 0) of the first outer index
    char* out;
    uint32_t* partial;        // [n_outer][parts][col_blocks][columns of a block], when parts > 1
    uint32_t* tickets;        // [n_outer * col_blocks], zero between launches
    uint32_t cols, words, col_blocks, rows, rows_per_group, parts, n_outer;
    int64_t s_red_w, s_outer_w;   // steps in words
    int64_t o_outer, o_col;       // result steps in bytes
    int overwrite, count_false;
};

// a + b + c of three words as a sum word and a carry word (three instructions: xor, bit-select, xor)
#define CUMO_CSA(h, l, a, b, c)                      \
    do {                                             \
        const uint32_t a_ = (a);                     \
        const uint32_t u_ = a_ ^ (b);                \
        const uint32_t c_ = (c);                     \
        h = (u_ & c_) | (~u_ & a_);                  \
        l = u_ ^ c_;                                 \
    } while (0)

// Sixteen words of one column group into the short counter.
__device__ __forceinline__ void vc_add16(uint32_t (&pl)[kVcPlanes], const uint32_t (&x)[kVcRows]) {
    uint32_t ones = pl[0], twos = pl[1], fours = pl[2], eights = pl[3];
    uint32_t ta, tb, fa, fb, ea, eb, sixteens;
    CUMO_CSA(ta, ones, ones, x[0], x[1]);
    CUMO_CSA(tb, ones, ones, x[2], x[3]);
    CUMO_CSA(fa, twos, twos, ta, tb);
    CUMO_CSA(ta, ones, ones, x[4], x[5]);
    CUMO_CSA(tb, ones, ones, x[6], x[7]);
    CUMO_CSA(fb, twos, twos, ta, tb);
    CUMO_CSA(ea, fours, fours, fa, fb);
    CUMO_CSA(ta, ones, ones, x[8], x[9]);
    CUMO_CSA(tb, ones, ones, x[10], x[11]);
    CUMO_CSA(fa, twos, twos, ta, tb);
    CUMO_CSA(ta, ones, ones, x[12], x[13]);
    CUMO_CSA(tb, ones, ones, x[14], x[15]);
    CUMO_CSA(fb, twos, twos, ta, tb);
    CUMO_CSA(eb, fours, fours, fa, fb);
    CUMO_CSA(sixteens, eights, eights, ea, eb);
    pl[0] = ones; pl[1] = twos; pl[2] = fours; pl[3] = eights;
    // the carry out of the tree counts sixteen: add it into the planes above
    uint32_t carry = sixteens;
#pragma unroll
    for (int q = 4; q < kVcPlanes; ++q) {
        const uint32_t t = pl[q] & carry;
        pl[q] ^= carry;
        carry = t;
    }
}

// LANES lanes across (a word each), BLOCK / LANES stretches of rows deep.
template <int BLOCK, int LANES>
__global__ __launch_bounds__(BLOCK) void bit_count_cols_vc_kernel(BitCountColsVc p) {
    constexpr unsigned NG = BLOCK / LANES;         // groups of lanes, each with a stretch of rows of its own
    constexpr unsigned BC = LANES * 32;            // columns across the block
    constexpr unsigned CPT = BC / BLOCK;           // columns a thread reads off the planes
    static_assert((NG & (NG - 1)) == 0 && BC % BLOCK == 0, "the groups meet in a binary tree; whole columns per thread");
    __shared__ uint32_t planes[NG / 2][kVcBlockPlanes][LANES];   // the counters of the groups that hand theirs over
    __shared__ uint32_t total_planes[kVcBlockPlanes][LANES];
    __shared__ int s_last;
    static_assert(LANES == 64, "a group is a wave: its rows are the same for every lane, so row addresses are scalar");
    const unsigned lane = threadIdx.x & 63u;
    const unsigned group = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t cb = blockIdx.x % p.col_blocks;
    const uint32_t b2 = blockIdx.x / p.col_blocks;
    const uint32_t part = b2 % p.parts;
    const uint32_t o = b2 / p.parts;
    const uint32_t cw = cb * (unsigned)LANES + lane;          // this lane's word of the row
    const uint32_t cwc = cw < p.words ? cw : p.words - 1;     // (a lane past the row's end reads the last word again; its columns are never written)
    const uint64_t first_row = ((uint64_t)part * NG + group) * p.rows_per_group;
    const uint32_t r0 = first_row < p.rows ? (uint32_t)first_row : p.rows;
    const uint32_t r1 = r0 + p.rows_per_group < p.rows ? r0 + p.rows_per_group : p.rows;
    // Buffer loads: a row's offset is a scalar operand and the lane adds its word's 32-bit
    // offset, so a load needs no vector arithmetic for its address. The descriptor's base is the
    // first row of the stretch in hand (the launcher has checked that a stretch spans less than 2 GiB).
    const uint32_t* plane0 = p.in + (int64_t)o * p.s_outer_w;
    const int lane_off = (int)(cwc * 4u);
    const int row_bytes = (int)(p.s_red_w * 4);

    uint32_t acc[kVcBlockPlanes];   // this group's stretch
#pragma unroll
    for (int q = 0; q < kVcBlockPlanes; ++q) acc[q] = 0u;
    for (uint32_t ra = r0; ra < r1; ra += kVcStretch) {
        const uint32_t rb = ra + kVcStretch < r1 ? ra + kVcStretch : r1;
        const __amdgpu_buffer_rsrc_t rsrc =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t*>(plane0 + (int64_t)ra * p.s_red_w), 0, -1, kVcBufferWord3);
        uint32_t pl[kVcPlanes];
#pragma unroll
        for (int q = 0; q < kVcPlanes; ++q) pl[q] = 0u;
        uint32_t r = ra;
        for (; r + kVcRows <= rb; r += kVcRows) {
            // every load of the step goes out before anything waits for one
            uint32_t x[kVcRows];
            const int step_off = (int)(r - ra) * row_bytes;
#pragma unroll
            for (int u = 0; u < kVcRows; ++u) x[u] = __builtin_amdgcn_raw_buffer_load_b32(rsrc, lane_off, step_off + u * row_bytes, kVcAuxNt);
            __builtin_amdgcn_sched_barrier(0);
            vc_add16(pl, x);
        }
        if (r < rb) {
            // the stretch's last rows: a row past the end is loaded again from the last row and dropped
            uint32_t x[kVcRows];
#pragma unroll
            for (int u = 0; u < kVcRows; ++u) {
                const uint32_t rr = r + u < rb ? r + u : rb - 1;
                x[u] = __builtin_amdgcn_raw_buffer_load_b32(rsrc, lane_off, (int)(rr - ra) * row_bytes, kVcAuxNt);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < kVcRows; ++u) x[u] = (r + u < rb) ? x[u] : 0u;
            vc_add16(pl, x);
        }
        // acc += pl: full adders down the planes
        uint32_t carry = 0u;
#pragma unroll
        for (int q = 0; q < kVcBlockPlanes; ++q) {
            const uint32_t b = q < kVcPlanes ? pl[q] : 0u;
            uint32_t h, l;
            CUMO_CSA(h, l, acc[q], b, carry);
            acc[q] = l;
            carry = h;
        }
    }
    // the groups' counters meet in a binary tree through LDS
#pragma unroll
    for (unsigned half = NG / 2; half >= 1; half >>= 1) {
        if (group >= half && group < 2 * half) {
#pragma unroll
            for (int q = 0; q < kVcBlockPlanes; ++q) planes[group - half][q][lane] = acc[q];
        }
        __syncthreads();
        if (group < half) {
            uint32_t carry = 0u;
#pragma unroll
            for (int q = 0; q < kVcBlockPlanes; ++q) {
                uint32_t h, l;
                CUMO_CSA(h, l, acc[q], planes[group][q][lane], carry);
                acc[q] = l;
                carry = h;
            }
        }
        __syncthreads();
    }
    if (group == 0) {
#pragma unroll
        for (int q = 0; q < kVcBlockPlanes; ++q) total_planes[q][lane] = acc[q];
    }
    __syncthreads();
    // a thread per column: the column's count from its bit of every plane
    const uint32_t col0 = cb * BC;
    const uint64_t block_r0 = (uint64_t)part * NG * p.rows_per_group;
    const uint64_t block_r1 = block_r0 + (uint64_t)NG * p.rows_per_group < p.rows ? block_r0 + (uint64_t)NG * p.rows_per_group : p.rows;
    const uint32_t rows_here = block_r0 < block_r1 ? (uint32_t)(block_r1 - block_r0) : 0u;
    uint32_t mine[CPT];
#pragma unroll
    for (unsigned k = 0; k < CPT; ++k) {
        const unsigned i = threadIdx.x + k * BLOCK;
        const unsigned w = i >> 5, j = i & 31u;
        uint32_t c = 0u;
#pragma unroll
        for (int q = 0; q < kVcBlockPlanes; ++q) c |= ((total_planes[q][w] >> j) & 1u) << q;
        mine[k] = p.count_false ? rows_here - c : c;
    }
    if (p.parts == 1) {
#pragma unroll
        for (unsigned k = 0; k < CPT; ++k) {
            const uint32_t col = col0 + threadIdx.x + k * BLOCK;
            if (col < p.cols) {
                unsigned long long* dst = reinterpret_cast<unsigned long long*>(p.out + (int64_t)o * p.o_outer + (int64_t)col * p.o_col);
                *dst = p.overwrite ? (unsigned long long)mine[k] : *dst + mine[k];
            }
        }
        return;
    }
    // several blocks share these columns: the counts go to scratch, written through at agent scope,
    // and the block that counts in last adds them up
    uint32_t* scratch = p.partial + (((size_t)o * p.parts + part) * p.col_blocks + cb) * BC;
#pragma unroll
    for (unsigned k = 0; k < CPT; ++k)
        __hip_atomic_store(scratch + threadIdx.x + k * BLOCK, mine[k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);   // this thread's stores are acknowledged
    __syncthreads();                 // ... and every thread's
    if (threadIdx.x == 0) {
        uint32_t* t = p.tickets + (size_t)o * p.col_blocks + cb;
        int last = 0;
        if (__hip_atomic_fetch_add(t, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == p.parts - 1) {
            __hip_atomic_store(t, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            last = 1;
        }
        s_last = last;
    }
    __syncthreads();
    if (!s_last) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    const uint32_t* all = p.partial + ((size_t)o * p.parts * p.col_blocks + cb) * BC;
    const size_t part_step = (size_t)p.col_blocks * BC;
    // sixteen blocks' counts of every column of this thread asked for at once: one after the other
    // they cost a trip to memory each, and this block is the only one left running for its columns
    unsigned long long total[CPT];
#pragma unroll
    for (unsigned k = 0; k < CPT; ++k) total[k] = 0;
    for (uint32_t q0 = 0; q0 < p.parts; q0 += 16) {
        uint32_t v[CPT][16];
#pragma unroll
        for (unsigned k = 0; k < CPT; ++k)
#pragma unroll
            for (uint32_t u = 0; u < 16; ++u) {
                const uint32_t q = q0 + u < p.parts ? q0 + u : p.parts - 1;
                v[k][u] = all[(size_t)q * part_step + threadIdx.x + k * BLOCK];
            }
#pragma unroll
        for (unsigned k = 0; k < CPT; ++k)
#pragma unroll
            for (uint32_t u = 0; u < 16; ++u) total[k] += q0 + u < p.parts ? v[k][u] : 0u;
    }
#pragma unroll
    for (unsigned k = 0; k < CPT; ++k) {
        const uint32_t col = col0 + threadIdx.x + k * BLOCK;
        if (col >= p.cols) continue;
        unsigned long long* dst = reinterpret_cast<unsigned long long*>(p.out + (int64_t)o * p.o_outer + (int64_t)col * p.o_col);
        *dst = p.overwrite ? total[k] : *dst + total[k];
    }
}

// geometry for blocks of BLOCK / LANES groups of LANES lanes; false when the launch does not fit
template <int BLOCK, int LANES>
bool vc_geometry(BitCountColsVc& p, uint64_t want_blocks, uint64_t* blocks) {
    constexpr uint32_t NG = BLOCK / LANES;
    p.col_blocks = (p.words + (uint32_t)LANES - 1) / (uint32_t)LANES;
    const uint64_t across = (uint64_t)p.col_blocks * p.n_outer;
    uint64_t parts = (want_blocks + across - 1) / across;
    const uint64_t most = ((uint64_t)p.rows + 32 * NG - 1) / (32 * NG);   // stretches of 32 rows or more
    if (parts > most) parts = most;
    if (parts < 1) parts = 1;
    p.rows_per_group = (uint32_t)(((uint64_t)p.rows + parts * NG - 1) / (parts * NG));
    p.parts = (uint32_t)(((uint64_t)p.rows + (uint64_t)p.rows_per_group * NG - 1) / ((uint64_t)p.rows_per_group * NG));
    if ((uint64_t)p.rows_per_group * NG >= (1u << kVcBlockPlanes)) return false;   // a block's counter would run over
    // offsets inside a stretch of rows are 32-bit operands of the loads
    if (((uint64_t)kVcStretch + kVcRows) * (uint64_t)p.s_red_w * 4 + (uint64_t)p.words * 4 >= 0x7fffffffull) return false;
    *blocks = across * p.parts;
    return *blocks <= 0x7fffffffull && across <= kTicketWordsPerSlot;
}

}  // namespace

namespace cumo_hip {

// 1 when launched (the results are then stored or added as d->overwrite says, with no zero-fill
// needed), 0 when the loop is not one this form takes
int bit_count_cols_words_launch(const cumo_hip_bit_count_nd_t* d) {
    if (d->red_ndim != 1 || d->out_ndim < 1 || d->out_ndim > 2 || force_wide_indices()) return 0;
    const int L = d->out_ndim - 1;
    if (d->in_out_step[L] != 1 || d->in_red_step[0] <= 0 || d->out_shape[L] < 64 || d->red_shape[0] < 2) return 0;
    if (d->out_shape[L] >= 0x7fffffffull || d->red_shape[0] >= 0x7fffffffull) return 0;
    if (L == 1 && (d->in_out_step[0] < 0 || d->out_shape[0] >= 0x10000ull)) return 0;
    // rows (and planes) that start on word boundaries
    if ((d->pos & 31) != 0 || (d->in_red_step[0] & 31) != 0 || (L == 1 && (d->in_out_step[0] & 31) != 0)) return 0;
    BitCountColsVc p;
    std::memset(&p, 0, sizeof(p));
    p.in = d->in + (d->pos >> 5);
    p.out = d->out;
    p.cols = (uint32_t)d->out_shape[L];
    p.words = (p.cols + 31u) / 32u;
    p.rows = (uint32_t)d->red_shape[0];
    p.n_outer = L == 1 ? (uint32_t)d->out_shape[0] : 1u;
    p.s_red_w = d->in_red_step[0] >> 5;
    p.s_outer_w = L == 1 ? (d->in_out_step[0] >> 5) : 0;
    p.o_outer = L == 1 ? d->out_step[0] : 0;
    p.o_col = d->out_step[L];
    p.overwrite = d->overwrite;
    p.count_false = d->count_false;
    // A block is LANES lanes across and 1024 / LANES stretches of rows deep: the rows are cut
    // inside the block, where the stretches meet in LDS, rather than across blocks, whose counts
    // have to go through memory -- few blocks per column group, and many column groups to share
    // the adding-up at the end. CUMO_HIP_BIT_COLS_LANES=32|64 and CUMO_HIP_BIT_COLS_BLOCKS (read
    // once) fix the shape of a block and the number of blocks aimed at.
    static const int forced_lanes = [] {
        const char* e = std::getenv("CUMO_HIP_BIT_COLS_LANES");
        return e ? std::atoi(e) : 0;
    }();
    static const int forced_blocks = [] {
        const char* e = std::getenv("CUMO_HIP_BIT_COLS_BLOCKS");
        return e ? std::atoi(e) : 0;
    }();
    const uint64_t want_blocks = forced_blocks > 0 ? (uint64_t)forced_blocks : (uint64_t)kNumCU;
    (void)forced_lanes;
    const int lanes = 64;
    uint64_t blocks = 0;
    if (!vc_geometry<1024, 64>(p, want_blocks, &blocks)) return 0;
    hipStream_t stream = current_stream();
    if (p.parts > 1) {
        p.tickets = red_ticket_words(stream_slot(stream));
        if (p.tickets == nullptr) return 0;
        const size_t bytes = sizeof(uint32_t) * (size_t)blocks * lanes * 32;
        p.partial = reinterpret_cast<uint32_t*>(cumo_cuda_runtime_malloc(bytes));
        if (p.partial == nullptr) return 0;
    }
    const dim3 g((unsigned)blocks), b(1024);
    hipLaunchKernelGGL((bit_count_cols_vc_kernel<1024, 64>), g, b, 0, stream, p);
    // stream-ordered reuse: whoever gets the scratch next can only touch it from later work on this stream
    if (p.partial) cumo_cuda_runtime_free(reinterpret_cast<char*>(p.partial));
    cumo_cuda_runtime_check_kernel_launch();
    return 1;
}

}  // namespace cumo_hip
