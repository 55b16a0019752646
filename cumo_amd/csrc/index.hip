// Index-array views: the arithmetic on device index arrays that builds them, the
// 1-D indexed copy, and the gather / scatter between a view with index arrays and a
// contiguous buffer that ndloop stages such operands through.
//
// Replaces narray/index_kernel.cu:10-173, narray/data_kernel.cu:11-20,22-45,134-164
// and narray/ndloop_kernel.cu:11-93 of the reference with the same launcher symbols.
// These are small integer kernels: one element per thread, grid-stride, 256-thread
// blocks; the gather / scatter decomposes the flat position once per element over the
// loop dimensions and moves 4- and 8-byte elements as one access each.
#include "common.h"
#include "div31.h"

#include <cstring>

namespace cumo_hip {
namespace {

constexpr int kIxBlock = 256;

inline unsigned ix_grid(uint64_t n) {
    uint64_t g = (n + kIxBlock - 1) / kIxBlock;
    if (g > 65536) g = 65536;
    return (unsigned)(g ? g : 1);
}

#define IX_LOOP(n) for (uint64_t i = (uint64_t)blockIdx.x * kIxBlock + threadIdx.x; i < (n); i += (uint64_t)gridDim.x * kIxBlock)

// one generic kernel for the index-array arithmetic: OP picks the expression
enum {
    IX_MUL_STRIDE,          // idx[i] = idx[i] * s1
    IX_THROUGH,             // idx[i] = idx1[idx[i]]
    IX_LAST_MUL_STRIDE,     // idx[i] = (last - idx[i]) * s1
    IX_THROUGH_BEG_STEP,    // idx[i] = idx1[beg + step*i]
    IX_BEG_STEP_STRIDE,     // idx[i] = (beg + step*i) * s1
    IX_ADD_BEG_STEP_STRIDE, // idx[i] += (beg + step*i) * s1
    IX_ADD_IDX_STRIDE,      // idx[i] += idx1[i] * s1
    IX_ADD_THROUGH_IDX,     // idx[i] += idx1[idx2[i]]
    IX_ADD_THROUGH_BEG_STEP,// idx[i] += idx1[beg + step*i]
    IX_ADD_LAST_MUL_STRIDE, // idx[i] += (last - idx[i]) * s1
    IX_DIAG_II,             // idx[i] = idx1[i+k0] + idx2[i+k1]
    IX_DIAG_IS,             // idx[i] = idx1[i+k0] + s1*(i+k1)
    IX_DIAG_SI              // idx[i] = s1*(i+k0) + idx2[i+k1]
};

template <int OP>
__global__ __launch_bounds__(kIxBlock) void index_arith_kernel(size_t* idx, const size_t* idx1, const size_t* idx2, size_t a, ssize_t step, ssize_t s1,
                                                               size_t k1, uint64_t n) {
    IX_LOOP(n) {
        size_t v = 0;
        switch (OP) {
            case IX_MUL_STRIDE: v = idx[i] * (size_t)s1; break;
            case IX_THROUGH: v = idx1[idx[i]]; break;
            case IX_LAST_MUL_STRIDE: v = (a - idx[i]) * (size_t)s1; break;
            case IX_THROUGH_BEG_STEP: v = idx1[a + (size_t)(step * (ssize_t)i)]; break;
            case IX_BEG_STEP_STRIDE: v = (a + (size_t)(step * (ssize_t)i)) * (size_t)s1; break;
            case IX_ADD_BEG_STEP_STRIDE: v = idx[i] + (a + (size_t)(step * (ssize_t)i)) * (size_t)s1; break;
            case IX_ADD_IDX_STRIDE: v = idx[i] + idx1[i] * (size_t)s1; break;
            case IX_ADD_THROUGH_IDX: v = idx[i] + idx1[idx2[i]]; break;
            case IX_ADD_THROUGH_BEG_STEP: v = idx[i] + idx1[a + (size_t)(step * (ssize_t)i)]; break;
            case IX_ADD_LAST_MUL_STRIDE: v = idx[i] + (a - idx[i]) * (size_t)s1; break;
            case IX_DIAG_II: v = idx1[i + a] + idx2[i + k1]; break;
            case IX_DIAG_IS: v = idx1[i + a] + (size_t)(s1 * (ssize_t)(i + k1)); break;
            case IX_DIAG_SI: v = (size_t)(s1 * (ssize_t)(i + a)) + idx2[i + k1]; break;
        }
        idx[i] = v;
    }
}

template <int OP>
void index_arith(size_t* idx, const size_t* idx1, const size_t* idx2, size_t a, ssize_t step, ssize_t s1, size_t k1, uint64_t n) {
    if (n == 0) return;
    hipLaunchKernelGGL((index_arith_kernel<OP>), dim3(ix_grid(n)), dim3(kIxBlock), 0, current_stream(), idx, idx1, idx2, a, step, s1, k1, n);
    cumo_cuda_runtime_check_kernel_launch();
}

__device__ __forceinline__ void ix_move(char* dst, const char* src, size_t elmsz) {
    if (elmsz == 4) *reinterpret_cast<uint32_t*>(dst) = *reinterpret_cast<const uint32_t*>(src);
    else if (elmsz == 8) *reinterpret_cast<uint64_t*>(dst) = *reinterpret_cast<const uint64_t*>(src);
    else for (size_t b = 0; b < elmsz; ++b) dst[b] = src[b];
}

__global__ __launch_bounds__(kIxBlock) void copy_bytes_indexed_kernel(const char* p1, char* p2, ssize_t s1, ssize_t s2, const size_t* idx1,
                                                                      const size_t* idx2, uint64_t n, size_t elmsz) {
    IX_LOOP(n) {
        const char* a = p1 + (idx1 ? (ssize_t)idx1[i] : (ssize_t)i * s1);
        char* b = p2 + (idx2 ? (ssize_t)idx2[i] : (ssize_t)i * s2);
        ix_move(b, a, elmsz);
    }
}

struct StridxView {
    int ndim;
    uint64_t total;
    uint64_t shape[CUMO_NA_MAX_DIMENSION];
    Div31 div[CUMO_NA_MAX_DIMENSION];
    int64_t stride[CUMO_NA_MAX_DIMENSION];      // used when index[d] == nullptr
    const size_t* index[CUMO_NA_MAX_DIMENSION]; // byte offsets per position of the dimension
    char* ptr;
};

// offset of the element (or row) with flat position r over dimensions [0, ndim)
template <bool SMALL>
__device__ __forceinline__ int64_t stridx_offset(const StridxView& v, int ndim, uint64_t r64) {
    int64_t off = 0;
    if (SMALL) {
        uint32_t r = (uint32_t)r64;
        for (int d = ndim - 1; d >= 0; --d) {
            uint32_t k = r;
            if (d > 0) {
                const uint32_t q = div31(r, v.div[d]);
                k = r - q * (uint32_t)v.shape[d];
                r = q;
            }
            off += v.index[d] ? (int64_t)v.index[d][k] : (int64_t)k * v.stride[d];
        }
    } else {
        uint64_t r = r64;
        for (int d = ndim - 1; d >= 0; --d) {
            const uint64_t m = v.shape[d];
            const uint64_t q = r / m;
            const uint64_t k = r - q * m;
            r = q;
            off += v.index[d] ? (int64_t)v.index[d][k] : (int64_t)k * v.stride[d];
        }
    }
    return off;
}

template <int ES> struct IxWord;
template <> struct IxWord<4> { typedef uint32_t type; };
template <> struct IxWord<8> { typedef uint64_t type; };

// TO_BUFFER: buf[i] = view element i (gather); else view element i = buf[i] (scatter).
// ES: element size moved as one access (4, 8) or 0 for any size as bytes. SMALL: fewer
// than 2^31 elements. A thread takes four elements a block apart, computes the four
// offsets, then issues the four reads together.
template <bool TO_BUFFER, int ES, bool SMALL>
__global__ __launch_bounds__(kIxBlock) void stridx_buffer_kernel(StridxView v, char* buf, size_t elmsz) {
    constexpr int U = 4;
    const uint64_t span = (uint64_t)kIxBlock * U;
    for (uint64_t base = (uint64_t)blockIdx.x * span + threadIdx.x; base < v.total; base += (uint64_t)gridDim.x * span) {
        int64_t off[U];
        uint64_t pos[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint64_t i = base + (uint64_t)u * kIxBlock;
            pos[u] = i < v.total ? i : v.total - 1;  // past the end: re-read the last element, store nothing
            off[u] = stridx_offset<SMALL>(v, v.ndim, pos[u]);
        }
        if constexpr (ES != 0) {
            typedef typename IxWord<ES>::type W;
            W val[U];
#pragma unroll
            for (int u = 0; u < U; ++u) val[u] = *reinterpret_cast<const W*>(TO_BUFFER ? v.ptr + off[u] : buf + pos[u] * ES);
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (base + (uint64_t)u * kIxBlock < v.total) *reinterpret_cast<W*>(TO_BUFFER ? buf + pos[u] * ES : v.ptr + off[u]) = val[u];
            }
        } else {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (base + (uint64_t)u * kIxBlock < v.total) {
                    const char* src = TO_BUFFER ? v.ptr + off[u] : buf + pos[u] * elmsz;
                    char* dst = TO_BUFFER ? buf + pos[u] * elmsz : v.ptr + off[u];
                    for (size_t b = 0; b < elmsz; ++b) dst[b] = src[b];
                }
            }
        }
    }
}

// The last dimension is contiguous in the view: rows of row_bytes (a whole number of 4-byte
// words) move whole, as 128-bit vectors and up to three words after them where the row's
// address in the view is a 4-byte boundary, byte by byte otherwise. A row is cut into
// segments of at most seg_vecs vectors; LPR lanes share one segment, four vectors each
// per step. v.ndim counts the outer dimensions only. NT, for copies that stream past the
// caches: non-temporal stores, and non-temporal loads from the buffer (touched exactly
// once; rows read from the view may repeat, so those loads stay cached).
struct StridxRows {
    uint32_t units;      // rows * segs_per_row  (< 2^31)
    uint32_t segs_per_row;
    Div31 seg_div;
    uint32_t row_vecs;   // whole 16-byte vectors of a row
    uint32_t seg_vecs;
    uint32_t tail_words; // 4-byte words of a row after its whole vectors (0..3)
    uint64_t row_bytes;
};

typedef uint32_t ix_u4 __attribute__((ext_vector_type(4)));

template <bool TO_BUFFER, int LPR, bool NT>
__global__ __launch_bounds__(kIxBlock) void stridx_rows_kernel(StridxView v, StridxRows g, char* buf) {
    constexpr int UPB = kIxBlock / LPR;  // units per block
    const uint32_t lane = threadIdx.x % LPR;
    const uint32_t n_blocks = (g.units + UPB - 1) / UPB;
    for (uint32_t ub = blockIdx.x; ub < n_blocks; ub += gridDim.x) {
        const uint32_t unit = ub * UPB + threadIdx.x / LPR;
        if (unit >= g.units) continue;
        uint32_t row = unit, seg = 0;
        if (g.segs_per_row > 1) {
            row = div31(unit, g.seg_div);
            seg = unit - row * g.segs_per_row;
        }
        const int64_t off = stridx_offset<true>(v, v.ndim, row);
        const uint32_t first = seg * g.seg_vecs;
        const uint32_t nv = min(g.seg_vecs, g.row_vecs - first);
        char* in_view = v.ptr + off + (uint64_t)first * 16;
        char* in_buf = buf + (uint64_t)row * g.row_bytes + (uint64_t)first * 16;
        const char* src = TO_BUFFER ? in_view : in_buf;
        char* dst = TO_BUFFER ? in_buf : in_view;
        // (a 128-bit access works on any 4-byte boundary)
        if (((uintptr_t)in_view & 3) == 0) {
            if (seg + 1 == g.segs_per_row && lane < g.tail_words) {
                // the words of the row after its last whole vector
                const uint64_t at = (uint64_t)(g.row_vecs - first) * 16 + (uint64_t)lane * 4;
                *reinterpret_cast<uint32_t*>(dst + at) = *reinterpret_cast<const uint32_t*>(src + at);
            }
            const ix_u4* s4 = reinterpret_cast<const ix_u4*>(src);
            ix_u4* d4 = reinterpret_cast<ix_u4*>(dst);
            for (uint32_t b = 0; b < nv; b += 4 * LPR) {
                ix_u4 x[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const ix_u4* ld = s4 + min(b + k * LPR + lane, nv - 1);
                    x[k] = (NT && !TO_BUFFER) ? __builtin_nontemporal_load(ld) : *ld;
                }
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    if (b + k * LPR + lane < nv) {
                        if (NT) __builtin_nontemporal_store(x[k], d4 + (b + k * LPR + lane));
                        else d4[b + k * LPR + lane] = x[k];
                    }
                }
            }
        } else {
            const uint32_t nb = nv * 16 + ((seg + 1 == g.segs_per_row) ? g.tail_words * 4 : 0);
            for (uint32_t b = lane; b < nb; b += LPR) dst[b] = src[b];
        }
    }
}

template <bool TO_BUFFER>
void stridx_buffer_launch(const cumo_na_iarray_stridx_t* a, const cumo_na_indexer_t* indexer, char* buf, size_t elmsz) {
    if (indexer->total_size == 0 || elmsz == 0) return;
    StridxView v;
    std::memset(&v, 0, sizeof(v));
    v.ndim = indexer->ndim;
    v.total = indexer->total_size;
    const bool small = v.total < (1ull << 31);
    for (int d = 0; d < indexer->ndim; ++d) {
        v.shape[d] = indexer->shape[d];
        if (small) v.div[d] = div31_make((uint32_t)indexer->shape[d]);
        if (CUMO_SDX_IS_INDEX(a->stridx[d])) v.index[d] = CUMO_SDX_GET_INDEX(a->stridx[d]);
        else v.stride[d] = CUMO_SDX_GET_STRIDE(a->stridx[d]);
    }
    v.ptr = a->ptr;
    hipStream_t stream = current_stream();
    // whole rows: the last dimension runs contiguously in the view
    const int last = v.ndim - 1;
    if (small && v.ndim >= 1 && !v.index[last] && v.stride[last] == (int64_t)elmsz && ((uintptr_t)buf & 3) == 0) {
        const uint64_t row_bytes = v.shape[last] * elmsz;
        if (row_bytes % 4 == 0 && row_bytes >= 256) {
            StridxRows g;
            g.row_vecs = (uint32_t)(row_bytes / 16);
            g.tail_words = (uint32_t)((row_bytes % 16) / 4);
            g.row_bytes = row_bytes;
            g.seg_vecs = 1024;
            g.segs_per_row = (g.row_vecs + g.seg_vecs - 1) / g.seg_vecs;
            const uint64_t rows = v.total / v.shape[last];
            const uint64_t units = rows * g.segs_per_row;
            if (units < (1ull << 31)) {
                g.units = (uint32_t)units;
                g.seg_div = div31_make(g.segs_per_row);
                v.ndim = last;  // the kernel walks the outer dimensions only
                v.total = rows;
                const int lpr = g.row_vecs <= 64 ? 16 : (g.row_vecs <= 256 ? 64 : 256);
                const uint64_t upb = kIxBlock / lpr;
                uint64_t grid = (units + upb - 1) / upb;
                if (grid > 256u * 64u) grid = 256u * 64u;
                // one read and one write of every byte: past the 256 MB last-level cache, stream by it
                const bool nt = stream_past_caches(2 * rows * row_bytes);
#define IX_ROWS(L, N) hipLaunchKernelGGL((stridx_rows_kernel<TO_BUFFER, L, N>), dim3((unsigned)grid), dim3(kIxBlock), 0, stream, v, g, buf)
                if (lpr == 16) { if (nt) IX_ROWS(16, true); else IX_ROWS(16, false); }
                else if (lpr == 64) { if (nt) IX_ROWS(64, true); else IX_ROWS(64, false); }
                else { if (nt) IX_ROWS(256, true); else IX_ROWS(256, false); }
#undef IX_ROWS
                cumo_cuda_runtime_check_kernel_launch();
                return;
            }
        }
    }
    uint64_t grid = (v.total + (uint64_t)kIxBlock * 4 - 1) / ((uint64_t)kIxBlock * 4);
    if (grid > 65536) grid = 65536;
    const dim3 gd((unsigned)grid), bd(kIxBlock);
    // single accesses of 4 or 8 bytes need the addresses aligned: offsets are whole
    // elements in any view the host layer builds, so the base pointers decide
    const bool aligned = (((uintptr_t)a->ptr | (uintptr_t)buf) % (elmsz ? elmsz : 1)) == 0;
    const int es = (aligned && (elmsz == 4 || elmsz == 8)) ? (int)elmsz : 0;
#define IX_GO(ES, SM) hipLaunchKernelGGL((stridx_buffer_kernel<TO_BUFFER, ES, SM>), gd, bd, 0, stream, v, buf, elmsz)
    if (small) {
        if (es == 4) IX_GO(4, true); else if (es == 8) IX_GO(8, true); else IX_GO(0, true);
    } else {
        if (es == 4) IX_GO(4, false); else if (es == 8) IX_GO(8, false); else IX_GO(0, false);
    }
#undef IX_GO
    cumo_cuda_runtime_check_kernel_launch();
}

}  // namespace
}  // namespace cumo_hip

using namespace cumo_hip;

extern "C" {

// narray/index_kernel.cu:87-173
void cumo_na_index_aref_nadata_index_stride_kernel_launch(size_t* idx, ssize_t s1, uint64_t n) { index_arith<IX_MUL_STRIDE>(idx, nullptr, nullptr, 0, 0, s1, 0, n); }
void cumo_na_index_aref_naview_index_index_kernel_launch(size_t* idx, size_t* idx1, uint64_t n) { index_arith<IX_THROUGH>(idx, idx1, nullptr, 0, 0, 0, 0, n); }
void cumo_na_index_aref_naview_index_stride_last_kernel_launch(size_t* idx, ssize_t s1, size_t last, uint64_t n) { index_arith<IX_LAST_MUL_STRIDE>(idx, nullptr, nullptr, last, 0, s1, 0, n); }
void cumo_na_index_aref_naview_index_stride_kernel_launch(size_t* idx, ssize_t s1, uint64_t n) { index_arith<IX_MUL_STRIDE>(idx, nullptr, nullptr, 0, 0, s1, 0, n); }
void cumo_na_index_aref_naview_index_index_beg_step_kernel_launch(size_t* idx, size_t* idx1, size_t beg, ssize_t step, uint64_t n) { index_arith<IX_THROUGH_BEG_STEP>(idx, idx1, nullptr, beg, step, 0, 0, n); }
void cumo_na_index_at_nadata_index_stride_add_kernel_launch(size_t* idx, size_t* idx1, ssize_t s1, uint64_t n) { index_arith<IX_ADD_IDX_STRIDE>(idx, idx1, nullptr, 0, 0, s1, 0, n); }
void cumo_na_index_at_nadata_index_beg_step_stride_kernel_launch(size_t* idx, size_t beg, ssize_t step, ssize_t s1, uint64_t n) { index_arith<IX_BEG_STEP_STRIDE>(idx, nullptr, nullptr, beg, step, s1, 0, n); }
void cumo_na_index_at_nadata_index_beg_step_stride_add_kernel_launch(size_t* idx, size_t beg, ssize_t step, ssize_t s1, uint64_t n) { index_arith<IX_ADD_BEG_STEP_STRIDE>(idx, nullptr, nullptr, beg, step, s1, 0, n); }
void cumo_na_index_at_naview_index_index_index_add_kernel_launch(size_t* idx, size_t* idx1, size_t* idx2, uint64_t n) { index_arith<IX_ADD_THROUGH_IDX>(idx, idx1, idx2, 0, 0, 0, 0, n); }
void cumo_na_index_at_naview_index_index_beg_step_add_kernel_launch(size_t* idx, size_t* idx1, size_t beg, ssize_t step, uint64_t n) { index_arith<IX_ADD_THROUGH_BEG_STEP>(idx, idx1, nullptr, beg, step, 0, 0, n); }
void cumo_na_index_at_naview_index_stride_last_add_kernel_launch(size_t* idx, ssize_t s1, size_t last, uint64_t n) { index_arith<IX_ADD_LAST_MUL_STRIDE>(idx, nullptr, nullptr, last, 0, s1, 0, n); }

// narray/data_kernel.cu:134-164
void cumo_iter_copy_bytes_kernel_launch(char* p1, char* p2, ssize_t s1, ssize_t s2, size_t* idx1, size_t* idx2, uint64_t n, ssize_t elmsz) {
    if (n == 0) return;
    hipLaunchKernelGGL(copy_bytes_indexed_kernel, dim3(ix_grid(n)), dim3(kIxBlock), 0, current_stream(), (const char*)p1, p2, s1, s2, (const size_t*)idx1,
                       (const size_t*)idx2, n, (size_t)elmsz);
    cumo_cuda_runtime_check_kernel_launch();
}
void cumo_na_diagonal_index_index_kernel_launch(size_t* idx, size_t* idx0, size_t* idx1, size_t k0, size_t k1, uint64_t n) { index_arith<IX_DIAG_II>(idx, idx0, idx1, k0, 0, 0, k1, n); }
void cumo_na_diagonal_index_stride_kernel_launch(size_t* idx, size_t* idx0, ssize_t s1, size_t k0, size_t k1, uint64_t n) { index_arith<IX_DIAG_IS>(idx, idx0, nullptr, k0, 0, s1, k1, n); }
void cumo_na_diagonal_stride_index_kernel_launch(size_t* idx, ssize_t s0, size_t* idx1, size_t k0, size_t k1, uint64_t n) { index_arith<IX_DIAG_SI>(idx, nullptr, idx1, k0, 0, s0, k1, n); }

// narray/ndloop_kernel.cu:46-93
void cumo_ndloop_copy_from_buffer_kernel_launch(cumo_na_iarray_stridx_t* a, cumo_na_indexer_t* indexer, char* buf, size_t elmsz) {
    stridx_buffer_launch<false>(a, indexer, buf, elmsz);
}
void cumo_ndloop_copy_to_buffer_kernel_launch(cumo_na_iarray_stridx_t* a, cumo_na_indexer_t* indexer, char* buf, size_t elmsz) {
    stridx_buffer_launch<true>(a, indexer, buf, elmsz);
}

}  // extern "C"
