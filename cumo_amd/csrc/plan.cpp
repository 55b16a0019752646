// Launch planner (host only). See plan.h.
//
// The reference contracts dimensions in ndloop (narray/ndloop.c:870-932) and
// then still pays a 64-bit divide and modulo per dimension per element in the
// kernel (include/cumo/indexer.h:239-257). Here the contraction is redone on
// the descriptors the launcher receives (the host iterators do not always run
// it, e.g. reductions: narray/ndloop.c:1480-1518), the dimension that runs
// along memory is found per operand, and the kernel is told which dimension to
// put its lanes on and how wide a vector access every operand tolerates.
#include "plan.h"

#include <cstdlib>
#include <cstring>

namespace cumo_hip {

static inline uint64_t mag(int64_t s) { return s < 0 ? (uint64_t)(-s) : (uint64_t)s; }

// dimension with the smallest non-zero |step|, the later one on a tie; -1 if
// the operand is a broadcast scalar
static int fastest_dim(int ndim, const int64_t* step) {
    int best = -1;
    for (int d = 0; d < ndim; ++d) {
        if (step[d] == 0) continue;
        if (best < 0 || mag(step[d]) <= mag(step[best])) best = d;
    }
    return best;
}

static void move_to(int ndim, uint64_t* shape, int64_t (*step)[kMaxDim], int nops, int from, int to) {
    // rotate dimension `from` to position `to` (to >= from), keeping the order of the rest
    uint64_t s = shape[from];
    int64_t st[kMaxOperands];
    for (int o = 0; o < nops; ++o) st[o] = step[o][from];
    for (int d = from; d < to; ++d) {
        shape[d] = shape[d + 1];
        for (int o = 0; o < nops; ++o) step[o][d] = step[o][d + 1];
    }
    shape[to] = s;
    for (int o = 0; o < nops; ++o) step[o][to] = st[o];
    (void)ndim;
}

void plan_elementwise(int ndim, const size_t* shape, int nops, const EwOperand* ops, EwPlan* plan) {
    std::memset(plan, 0, sizeof(*plan));
    plan->tr_dim = -1;
    plan->vec = 1;
    plan->vec_loose = 1;
    uint64_t total = 1;
    for (int d = 0; d < ndim; ++d) total *= shape[d];
    plan->total = total;
    if (total == 0) {
        plan->kind = EW_EMPTY;
        return;
    }

    // 1. drop size-1 dims, 2. merge neighbours every operand walks with one stride
    int n = 0;
    uint64_t* sh = plan->shape;
    int64_t(*st)[kMaxDim] = plan->step;
    for (int d = 0; d < ndim; ++d) {
        if (shape[d] == 1) continue;
        bool merge = n > 0;
        if (merge) {
            for (int o = 0; o < nops; ++o) {
                if (st[o][n - 1] != (int64_t)ops[o].step[d] * (int64_t)shape[d]) { merge = false; break; }
            }
        }
        if (merge) {
            sh[n - 1] *= shape[d];
            for (int o = 0; o < nops; ++o) st[o][n - 1] = ops[o].step[d];
        } else {
            sh[n] = shape[d];
            for (int o = 0; o < nops; ++o) st[o][n] = ops[o].step[d];
            ++n;
        }
    }
    if (n == 0) {
        n = 1;
        sh[0] = 1;
        for (int o = 0; o < nops; ++o) st[o][0] = 0;
    }
    plan->ndim = n;
    plan->kind = EW_ROWS;

    // 3. which dim do the lanes run along: the one the written operand walks fastest
    const int out = nops - 1;
    int F = fastest_dim(n, st[out]);
    if (F < 0) {
        for (int o = 0; o < nops && F < 0; ++o) F = fastest_dim(n, st[o]);
        if (F < 0) F = n - 1;
    }
    // an input that walks another dim faster wants a tile transpose
    int G = -1;
    for (int o = 0; o < out; ++o) {
        if (ops[o].elmsz == 0) continue;
        if (st[o][F] == 0) continue;
        int f = fastest_dim(n, st[o]);
        if (f >= 0 && f != F && mag(st[o][f]) < mag(st[o][F])) {
            if (mag(st[o][f]) == (uint64_t)ops[o].elmsz) { G = f; break; }
        }
    }
    bool transpose = false;
    if (G >= 0 && ops[out].elmsz != 0 && mag(st[out][F]) == (uint64_t)ops[out].elmsz &&
        st[out][F] > 0 && sh[F] >= 16 && sh[G] >= 16) {
        // every operand has to be walkable by one of the two tile orientations
        transpose = true;
        for (int o = 0; o < out; ++o) {
            if (ops[o].elmsz == 0) { transpose = false; break; }
        }
    }
    plan->fast_dim = F;
    if (transpose) {
        plan->kind = EW_TRANSPOSE;
        plan->tr_dim = G;
        // order: ..., G, F
        move_to(n, sh, st, nops, F, n - 1);
        int g = (G > F) ? G - 1 : G;
        move_to(n, sh, st, nops, g, n - 2);
        return;
    }
    move_to(n, sh, st, nops, F, n - 1);

    // 4. vector width
    int min_elmsz = 16;
    for (int o = 0; o < nops; ++o) {
        if (ops[o].elmsz > 0 && ops[o].elmsz < min_elmsz) min_elmsz = ops[o].elmsz;
    }
    if (min_elmsz == 16) min_elmsz = 4;
    const int L = n - 1;
    plan->vec_loose = 1;
    for (int loose = 1; loose >= 0; --loose)
    for (int vec = 16 / min_elmsz; vec > 1; vec >>= 1) {
        bool ok = sh[L] >= (uint64_t)vec;
        for (int o = 0; o < nops && ok; ++o) {
            const int es = ops[o].elmsz;
            if (es == 0) {
                // Bit operand: rows start on word boundaries, lanes own whole nibbles
                if (st[o][L] == 0) { ok = (o != out); continue; }
                if (st[o][L] != 1 || (ops[o].bitpos % 32) != 0) { ok = false; break; }
                for (int d = 0; d < L; ++d) if (st[o][d] % 32) { ok = false; break; }
                if (n > 1 && (sh[L] % 32) != 0 && o == out) {
                    // a short last word would be shared with the next row only if rows
                    // abut, which word-aligned outer steps already exclude
                }
                continue;
            }
            if (st[o][L] == 0) { if (o == out) ok = false; continue; }
            // an input that runs backwards along the rows is read by vectors too (the row kernel turns a vector's
            // elements round); its vectors start wherever the view's last element puts them: element alignment
            const bool backwards = o != out && es >= 4 && st[o][L] == -(int64_t)es && !loose;
            if (st[o][L] != es && !backwards) { ok = false; break; }
            int align = vec * es;
            if (align > 16) align = 16;
            if ((loose && o != out && es >= 4) || backwards) align = es;
            if (((uintptr_t)ops[o].ptr % align) != 0) { ok = false; break; }
            for (int d = 0; d < L; ++d) if (st[o][d] % align) { ok = false; break; }
        }
        // rows that are not a whole number of vectors would leave the next row unaligned
        if (ok && n > 1 && (sh[L] % vec) != 0) ok = false;
        if (ok) {
            if (loose) plan->vec_loose = vec;
            else plan->vec = vec;
            break;
        }
    }
}

// ---------------------------------------------------------------------------

static int ceil_pow2(uint64_t x) {
    int p = 1;
    while ((uint64_t)p < x && p < (1 << 30)) p <<= 1;
    return p;
}

void plan_reduce(const cumo_na_reduction_arg_t* arg, const cumo_na_iarray_t* out2, int in_elmsz, int accum_bytes,
                 ReducePlan* plan, bool allow_tail) {
    std::memset(plan, 0, sizeof(*plan));
    plan->vec = 1;
    plan->n_split = 1;
    plan->local_split_bits = 0;
    plan->threads_per_row = 1;
    const int in_ndim = arg->in_indexer.ndim;
    const int out_ndim_in = arg->out_indexer.ndim;
    const uint64_t out_total = arg->out_indexer.total_size;
    const uint64_t in_total = arg->in_indexer.total_size;
    plan->out_total = out_total;
    if (out_total == 0) {
        plan->kind = RED_EMPTY;
        return;
    }
    // an empty reduce axis still answers the identity for every output
    plan->red_total = in_total / out_total;

    // output dims: drop size 1, merge where input, output (and second output) agree
    int no = 0;
    for (int d = 0; d < out_ndim_in; ++d) {
        uint64_t s = arg->in_indexer.shape[d];
        if (s == 1) continue;
        int64_t a = arg->in.step[d], b = arg->out.step[d], c = out2 ? out2->step[d] : 0;
        if (no > 0 && plan->in_out_step[no - 1] == a * (int64_t)s && plan->out_step[no - 1] == b * (int64_t)s &&
            plan->out2_step[no - 1] == c * (int64_t)s) {
            plan->out_shape[no - 1] *= s;
            plan->in_out_step[no - 1] = a;
            plan->out_step[no - 1] = b;
            plan->out2_step[no - 1] = c;
        } else {
            plan->out_shape[no] = s;
            plan->in_out_step[no] = a;
            plan->out_step[no] = b;
            plan->out2_step[no] = c;
            ++no;
        }
    }
    plan->out_ndim = no;
    // reduce dims
    int nr = 0;
    for (int d = out_ndim_in; d < in_ndim; ++d) {
        uint64_t s = arg->in_indexer.shape[d];
        if (s == 1) continue;
        int64_t a = arg->in.step[d];
        if (nr > 0 && plan->in_red_step[nr - 1] == a * (int64_t)s) {
            plan->red_shape[nr - 1] *= s;
            plan->in_red_step[nr - 1] = a;
        } else {
            plan->red_shape[nr] = s;
            plan->in_red_step[nr] = a;
            ++nr;
        }
    }
    plan->red_ndim = nr;

    const uint64_t N = plan->red_total;
    const uint64_t rs = nr > 0 ? mag(plan->in_red_step[nr - 1]) : 0;
    const uint64_t os = no > 0 ? mag(plan->in_out_step[no - 1]) : 0;

    // lanes go along whichever of the two innermost axes runs along memory
    const bool col = os != 0 && (rs == 0 || os < rs) && plan->out_shape[no - 1] >= 16;
    if (col) {
        plan->kind = RED_COL;
        const int L = no - 1;
        int vec = 16 / in_elmsz;
        for (; vec > 1; vec >>= 1) {
            // the input is only read: a 128-bit global load needs no more than the element's alignment
            const int align = in_elmsz >= 4 ? in_elmsz : vec * in_elmsz;
            // (outputs along one dimension may end in part of a vector where the caller's kernel sees to it)
            const bool whole = (plan->out_shape[L] % vec) == 0 || (allow_tail && no <= 2 && plan->out_shape[L] >= (uint64_t)vec * 16);
            bool ok = plan->in_out_step[L] == in_elmsz && whole && ((uintptr_t)arg->in.ptr % align) == 0;
            for (int d = 0; d < L && ok; ++d) ok = (plan->in_out_step[d] % align) == 0;
            for (int d = 0; d < nr && ok; ++d) ok = (plan->in_red_step[d] % align) == 0;
            if (ok) break;
        }
        plan->vec = vec < 1 ? 1 : vec;
        plan->red_tail = plan->vec > 1 ? (int)(plan->out_shape[L] % (uint64_t)plan->vec) : 0;
        // few outputs and a long axis: cut the axis across blocks
        uint64_t threads = (out_total / plan->out_shape[L]) * ((plan->out_shape[L] + plan->vec - 1) / plan->vec);
        uint64_t blocks = (threads + 255) / 256;
        if (blocks < (uint64_t)kNumCU * 2 && N >= 128) {
            uint64_t want = ((uint64_t)kNumCU * 4 + blocks - 1) / blocks;
            uint64_t fits = N / 32;
            uint64_t s = want < fits ? want : fits;
            if (s > 1024) s = 1024;
            // Up to 16 ways inside the block (combined through LDS, no second launch). Beyond that a
            // second launch over the partial results is needed anyway, and then the block stays wider
            // (four ways inside, 64 vectors of every row it reads) and the rest is cut across blocks:
            // 16 ways inside leave a block 16 vectors of a row, 256 bytes at a time (column sums of
            // a 4096 x 4096 DFloat: 30.4 us that way, 27.2 us this way; of a 4096 x 4095 one, which
            // the general kernels take: 41 -> 29 us).
            int bits = 0;
            if (s > 16) {
                // a second launch folds: the block is as wide as the outputs allow (up to 256 vectors, 4 KiB of every
                // row it reads), what is left of its 256 lanes shares the axis, and the axis is cut across enough
                // blocks to fill the device (1024 of them) while a lane's part of it keeps 32 positions
                // (at least four blocks side by side where that leaves them 64 vectors: the fold of more than
                // 256 parts costs more than the wider block gains)
                uint64_t wide = 64;
                while (wide < 256 && wide * 8 <= threads) wide <<= 1;
                while (wide > 16 && wide / 2 >= threads) wide >>= 1;
                while ((256u >> bits) > wide) ++bits;
                const uint64_t col_blocks = (threads + wide - 1) / wide;
                uint64_t parts = ((uint64_t)kNumCU * 4 + col_blocks - 1) / col_blocks;
                if (parts > (fits >> bits)) parts = fits >> bits;
                if (parts > 1024) parts = 1024;
                if (parts < 1) parts = 1;
                s = parts << bits;
            } else {
                while (bits < 4 && (2ull << bits) <= s) ++bits;
            }
            plan->local_split_bits = bits;
            s = (s + (1ull << bits) - 1) >> bits;
            if (s >= 2) plan->n_split = (int)s;
        }
        (void)accum_bytes;
        return;
    }

    plan->kind = RED_ROW;
    int vec = 16 / in_elmsz;
    for (; vec > 1; vec >>= 1) {
        const int align = in_elmsz >= 4 ? in_elmsz : vec * in_elmsz;  // read-only: the element's alignment is enough
        // (a single long axis may end in part of a vector where the caller folds that part by itself)
        const bool whole = nr > 0 && ((plan->red_shape[nr - 1] % vec) == 0 ||
                                      (allow_tail && nr == 1 && plan->red_shape[0] >= (uint64_t)vec * 16));
        bool ok = nr > 0 && plan->in_red_step[nr - 1] == in_elmsz && whole && ((uintptr_t)arg->in.ptr % align) == 0;
        for (int d = 0; d < nr - 1 && ok; ++d) ok = (plan->in_red_step[d] % align) == 0;
        for (int d = 0; d < no && ok; ++d) ok = (plan->in_out_step[d] % align) == 0;
        if (ok) break;
    }
    plan->vec = vec < 1 ? 1 : vec;
    plan->red_tail = (plan->vec > 1 && nr == 1) ? (int)(plan->red_shape[0] % (uint64_t)plan->vec) : 0;

    // lanes per output: enough that each lane still has a few accesses to overlap
    uint64_t per_lane = (uint64_t)plan->vec * 4;
    // an accumulator of more than two elements' width (running moments) makes the fold across
    // lanes the expensive part: fewer lanes, each with twice the elements. (Value + index is
    // two elements wide and prefers the full count: C3 argmax(axis:2) 23.2 -> 22.6 us.)
    if (accum_bytes > 2 * in_elmsz) per_lane *= 2;
    int tpr = ceil_pow2((N + per_lane - 1) / per_lane);
    if (N >= 8192) tpr = 256;
    else if (tpr > 64) tpr = 64;
    if (tpr < 1) tpr = 1;
    // rows of 16 KiB and more: a whole block per row (every lane still has four 128-bit loads to
    // overlap, and a block reads one long run instead of four rows at once). Measured on SFloat
    // [8192,4096] (fresh operands): mean 22.9 -> 21.3 us, var 24.1 -> 22.2 us.
    // (An accumulator wider than an element makes the fold across the block dear: then only
    // from 16 elements per lane on. DFloat [8192,2048] var: 25.6 us with a wave per row, 35.4 us
    // with a block.)
    if (tpr == 64 && N * (uint64_t)in_elmsz >= 16384 && (accum_bytes <= in_elmsz || N >= 4096)) tpr = 256;
    plan->threads_per_row = tpr;

    uint64_t blocks = (out_total * (uint64_t)tpr + 255) / 256;
    if (blocks < (uint64_t)kNumCU * 2 && N >= 16384) {
        uint64_t want = ((uint64_t)kNumCU * 8 + blocks - 1) / blocks;
        uint64_t fits = N / 8192;
        uint64_t s = want < fits ? want : fits;
        if (s > 2048) s = 2048;
        if (s >= 2) {
            plan->n_split = (int)s;
            plan->threads_per_row = 256;
        }
    }
}

}  // namespace cumo_hip

using namespace cumo_hip;

extern "C" {

int cumo_hip_plan_elementwise(const cumo_na_indexer_t* indexer, int n_operands, const cumo_na_iarray_t* const* operands,
                              const int* elmsz, const size_t* bitpos, cumo_hip_ew_plan_t* out) {
    if (n_operands < 1 || n_operands > kMaxOperands) return CUMO_HIP_ERROR_ARGUMENT;
    EwOperand ops[kMaxOperands];
    for (int o = 0; o < n_operands; ++o) {
        ops[o].ptr = operands[o]->ptr;
        ops[o].step = operands[o]->step;
        ops[o].elmsz = elmsz[o];
        ops[o].bitpos = bitpos ? bitpos[o] : 0;
    }
    EwPlan p;
    plan_elementwise(indexer->ndim, indexer->shape, n_operands, ops, &p);
    std::memset(out, 0, sizeof(*out));
    out->kind = p.kind;
    out->ndim = p.ndim;
    out->vec = p.vec;
    out->fast_dim = p.fast_dim;
    out->tr_dim = p.tr_dim;
    for (int d = 0; d < p.ndim; ++d) {
        out->shape[d] = p.shape[d];
        for (int o = 0; o < n_operands; ++o) out->step[o][d] = p.step[o][d];
    }
    return CUMO_HIP_OK;
}

int cumo_hip_plan_reduce(const cumo_na_reduction_arg_t* arg, int in_elmsz, int accum_bytes, cumo_hip_reduce_plan_t* out) {
    ReducePlan p;
    plan_reduce(arg, nullptr, in_elmsz, accum_bytes, &p);
    std::memset(out, 0, sizeof(*out));
    out->kind = p.kind;
    out->vec = p.vec;
    out->threads_per_row = p.threads_per_row;
    out->n_split = p.n_split;
    out->out_ndim = p.out_ndim;
    out->red_ndim = p.red_ndim;
    out->out_total = p.out_total;
    out->red_total = p.red_total;
    for (int d = 0; d < kMaxDim; ++d) {
        out->out_shape[d] = p.out_shape[d];
        out->red_shape[d] = p.red_shape[d];
        out->in_out_step[d] = p.in_out_step[d];
        out->in_red_step[d] = p.in_red_step[d];
        out->out_step[d] = p.out_step[d];
    }
    return CUMO_HIP_OK;
}

}  // extern "C"
