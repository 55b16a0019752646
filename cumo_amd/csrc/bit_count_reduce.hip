// count_true / count_false of long contiguous runs of bits through the reduction kernels: the run's
// words are a reduce axis of 32-bit elements, an element's value is its number of set (or clear) bits,
// and the first and last word of the axis are masked to the bits that belong to the run. This gives
// the counts what the sums have: 128-bit loads with four in flight, an axis shared by up to 2048
// blocks whose accumulators are handed over inside the one launch, and rows shared by 2^k lanes.
// (The reference counts with one thread per bit and an atomicAdd per set bit:
// narray/gen/tmpl_bit/bit_count_kernel.cu:15-24.)
#include "reduce_kernels.h"
#include "reduce_impls.h"

using namespace cumo_hip;

namespace {

template <bool COUNT_FALSE, bool ADD>
struct PopcountImpl {
    typedef uint32_t In;
    typedef uint64_t Acc;
    static constexpr bool USES_INDEX = true;
    static constexpr int NOUT = 1;
    uint32_t first_mask, last_mask;  // the bits of the axis' first and last word that count
    int64_t last;                    // position of the last word along the axis
    __device__ __forceinline__ Acc identity() const { return 0; }
    __device__ __forceinline__ void accumulate(In x, int64_t idx, Acc& acc) const {
        if (COUNT_FALSE) x = ~x;
        if (idx == 0) x &= first_mask;
        if (idx == last) x &= last_mask;
        acc += (Acc)__popc(x);
    }
    CUMO_HIP_ACCUMULATE_N_BY_ELEMENT
    __device__ __forceinline__ void combine(const Acc& next, Acc& acc) const { acc += next; }
    __device__ __forceinline__ void store(const Acc& acc, char* out, char*) const {
        if (ADD) *reinterpret_cast<uint64_t*>(out) += acc;
        else *reinterpret_cast<uint64_t*>(out) = acc;
    }
};

template <bool ADD>
bool launch(cumo_na_reduction_arg_t* arg, uint32_t first_mask, uint32_t last_mask, int64_t last, bool count_false) {
    if (count_false) return reduce_launch(arg, nullptr, PopcountImpl<true, ADD>{first_mask, last_mask, last}, 1);
    return reduce_launch(arg, nullptr, PopcountImpl<false, ADD>{first_mask, last_mask, last}, 1);
}

inline uint32_t low_mask(unsigned n) { return n >= 32 ? 0xffffffffu : ((1u << n) - 1u); }

}  // namespace

// *out = the number of set (or clear) bits of bits [pos, pos + n) of a (pos < 32). Returns 1 when
// launched, 0 when the run is one for the ticket kernel (short) or cannot go this way.
int cumo_hip::bit_count_run_reduce(CUMO_BIT_DIGIT* a, size_t pos, uint64_t n, int count_false, uint64_t* out) {
    if (n < (1ull << 24) || pos >= 32 || force_wide_indices()) return 0;
    const uint64_t nw = (pos + n + 31) / 32;
    cumo_na_reduction_arg_t arg;
    std::memset(&arg, 0, sizeof(arg));
    arg.in.ptr = reinterpret_cast<char*>(a);
    arg.in.step[0] = 4;
    arg.in_indexer.ndim = 1;
    arg.in_indexer.shape[0] = nw;
    arg.in_indexer.total_size = nw;
    arg.out.ptr = reinterpret_cast<char*>(out);
    arg.out_indexer.ndim = 0;
    arg.out_indexer.total_size = 1;
    const uint32_t first_mask = ~low_mask((unsigned)pos);
    const uint32_t last_mask = low_mask((unsigned)((pos + n - 1) % 32) + 1);
    return launch<false>(&arg, first_mask, last_mask, (int64_t)nw - 1, count_false != 0) ? 1 : 0;
}

// Counts along the innermost dimension, added onto the results (or stored, with `overwrite`), where every run is whole words: the
// runs start on words (pos and the kept dimensions' steps are multiples of 32), run along the bits and
// are a multiple of 32 long. Returns 1 when launched, 0 when the loop is not of that kind.
int cumo_hip::bit_count_rows_reduce(const cumo_hip_bit_count_nd_t* d) {
    if (!d || d->red_ndim != 1 || d->out_ndim < 1 || d->out_ndim + 1 > CUMO_NA_MAX_DIMENSION || force_wide_indices()) return 0;
    if (d->in_red_step[0] != 1 || (d->red_shape[0] % 32) != 0 || d->red_shape[0] < 2048 || (d->pos % 32) != 0) return 0;
    cumo_na_reduction_arg_t arg;
    std::memset(&arg, 0, sizeof(arg));
    size_t outs = 1;
    for (int k = 0; k < d->out_ndim; ++k) {
        if ((d->in_out_step[k] % 32) != 0) return 0;
        arg.in.step[k] = d->in_out_step[k] / 8;  // bits -> bytes
        arg.out.step[k] = d->out_step[k];
        arg.in_indexer.shape[k] = d->out_shape[k];
        arg.out_indexer.shape[k] = d->out_shape[k];
        outs *= d->out_shape[k];
    }
    const size_t nw = d->red_shape[0] / 32;
    arg.in.ptr = reinterpret_cast<char*>(d->in + d->pos / 32);
    arg.in.step[d->out_ndim] = 4;
    arg.in_indexer.ndim = (unsigned char)(d->out_ndim + 1);
    arg.in_indexer.shape[d->out_ndim] = nw;
    arg.in_indexer.total_size = outs * nw;
    arg.out.ptr = d->out;
    arg.out_indexer.ndim = (unsigned char)d->out_ndim;
    arg.out_indexer.total_size = outs;
    if (outs == 0 || nw == 0) return 0;
    if (d->overwrite) return launch<false>(&arg, 0xffffffffu, 0xffffffffu, (int64_t)nw - 1, d->count_false != 0) ? 1 : 0;
    return launch<true>(&arg, 0xffffffffu, 0xffffffffu, (int64_t)nw - 1, d->count_false != 0) ? 1 : 0;
}
