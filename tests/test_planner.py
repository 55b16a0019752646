"""Launch planner decisions, host only: which dimension the lanes run along, what
merges, when 128-bit accesses are allowed, when a reduction is split."""
import ctypes as C

import numpy as np
import pytest

from cumo_amd import _lib
from cumo_amd._lib import EwPlan, IArray, Indexer, ReducePlan, ReductionArg

P = C.POINTER
BASE = 0x7F0000000000  # a 4 KiB-aligned fake device address; nothing is dereferenced


def ew_plan(shape, operands, elmsz, bitpos=None):
    ix = Indexer()
    ix.ndim = len(shape)
    ix.total_size = int(np.prod(shape)) if shape else 1
    for d, s in enumerate(shape):
        ix.shape[d] = s
    arrs = []
    for ptr, steps in operands:
        a = IArray()
        a.ptr = ptr
        for d, s in enumerate(steps):
            a.step[d] = s
        arrs.append(a)
    ptrs = (P(IArray) * len(arrs))(*[C.pointer(a) for a in arrs])
    es = (C.c_int * len(arrs))(*elmsz)
    bp = (C.c_size_t * len(arrs))(*(bitpos or [0] * len(arrs)))
    plan = EwPlan()
    assert _lib.lib.cumo_hip_plan_elementwise(C.byref(ix), len(arrs), ptrs, es, bp, C.byref(plan)) == 0
    return plan


def test_contiguous_collapses_to_one_dim_vectorised():
    p = ew_plan((64, 32, 16), [(BASE, (2048, 64, 4)), (BASE + 4096 * 64, (2048, 64, 4)), (BASE + 4096 * 128, (2048, 64, 4))], [4, 4, 4])
    assert (p.kind, p.ndim, p.vec) == (1, 1, 4)
    assert p.shape[0] == 64 * 32 * 16
    p = ew_plan((4096, 4096), [(BASE, (32768, 8)), (BASE + (1 << 30), (32768, 8))], [8, 8])
    assert (p.kind, p.ndim, p.vec) == (1, 1, 2)


def test_row_broadcast_keeps_two_dims_and_vectorises():
    # A[4096,4096] + r[1,4096] (f64): r has steps (0, 8), nothing merges, 128-bit still fine
    p = ew_plan((4096, 4096), [(BASE, (32768, 8)), (BASE + (1 << 30), (0, 8)), (BASE + (1 << 31), (32768, 8))], [8, 8, 8])
    assert (p.kind, p.ndim, p.vec) == (1, 2, 2)
    # S[.., 512, 512] - m[.., 512, 1] (f32): merges to [262144, 512], m broadcast along the row
    p = ew_plan((32, 16, 512, 512), [(BASE, (16 * 512 * 2048, 512 * 2048, 2048, 4)), (BASE + (1 << 32), (16 * 2048, 2048, 4, 0)),
                                     (BASE + (1 << 33), (16 * 512 * 2048, 512 * 2048, 2048, 4))], [4, 4, 4])
    assert (p.kind, p.ndim, p.vec) == (1, 2, 4)
    assert list(p.shape[:2]) == [32 * 16 * 512, 512]
    assert list(p.step[1][:2]) == [4, 0]


def test_misaligned_or_strided_falls_back_to_scalar_access():
    p = ew_plan((1000,), [(BASE + 4, (4,)), (BASE + 8192, (4,))], [4, 4])
    assert p.vec == 1
    p = ew_plan((1000,), [(BASE, (8,)), (BASE + 8192, (4,))], [4, 4])   # every other element
    assert p.vec == 1
    p = ew_plan((10, 1001), [(BASE, (4004, 4)), (BASE + (1 << 20), (4004, 4))], [4, 4])  # merges: one run of 10010
    assert (p.ndim, p.vec) == (1, 4)  # one run: the ragged tail is handled inside the kernel
    p = ew_plan((10, 1001), [(BASE, (8000, 4)), (BASE + (1 << 20), (4004, 4))], [4, 4])  # rows of 1001 floats, padded source
    assert p.ndim == 2 and p.vec == 1


def test_transposed_input_asks_for_the_tile_kernel():
    # V = M.transpose[true, (0..-1).step(2)] of M[8192,8192] f32: V[i,j] = M[2j,i]
    p = ew_plan((8192, 4096), [(BASE, (4, 65536)), (BASE + (1 << 30), (16384, 4))], [4, 4])
    assert p.kind == 2
    assert p.ndim == 2
    # after the permutation the last dim is the output's fast one
    assert p.step[1][1] == 4 and p.step[0][0] == 4
    # plain transposed operand on both sides: lanes follow the output, no tile needed when both agree
    p = ew_plan((100, 200), [(BASE, (4, 400)), (BASE + (1 << 20), (4, 400))], [4, 4])
    assert p.kind == 1 and p.shape[p.ndim - 1] == 100


def test_size_one_dims_drop_and_empty():
    p = ew_plan((1, 5, 1, 7, 1), [(BASE, (0, 28, 0, 4, 0)), (BASE + 4096, (0, 28, 0, 4, 0))], [4, 4])
    assert p.ndim == 1 and p.shape[0] == 35
    p = ew_plan((3, 0, 4), [(BASE, (0, 16, 4)), (BASE, (0, 16, 4))], [4, 4])
    assert p.kind == 0
    p = ew_plan((), [(BASE, ()), (BASE + 64, ())], [4, 4])
    assert p.kind == 1 and p.ndim == 1 and p.shape[0] == 1


def test_bit_output_vector_needs_word_alignment():
    p = ew_plan((33554432,), [(BASE, (4,)), (BASE + (1 << 30), (1,))], [4, 0], [0, 0])
    assert p.vec == 4
    p = ew_plan((33554432,), [(BASE, (4,)), (BASE + (1 << 30), (1,))], [4, 0], [0, 5])
    assert p.vec == 1
    p = ew_plan((100, 96), [(BASE, (800, 4)), (BASE + (1 << 30), (96, 1))], [4, 0], [0, 0])  # strided source rows, packed bit rows
    assert p.ndim == 2 and p.vec == 4
    p = ew_plan((100, 100), [(BASE, (800, 4)), (BASE + (1 << 30), (100, 1))], [4, 0], [0, 0])  # bit rows not word aligned
    assert p.vec == 1


def red_plan(shape, steps, out_ndim, out_steps, elmsz=4, accum=4, ptr=BASE):
    arg = ReductionArg()
    arg.in_.ptr = ptr
    arg.out.ptr = BASE + (1 << 34)
    arg.in_indexer.ndim = len(shape)
    arg.in_indexer.total_size = int(np.prod(shape))
    for d, (s, st) in enumerate(zip(shape, steps)):
        arg.in_indexer.shape[d] = s
        arg.in_.step[d] = st
    arg.out_indexer.ndim = out_ndim
    arg.out_indexer.total_size = int(np.prod(shape[:out_ndim])) if out_ndim else 1
    for d in range(out_ndim):
        arg.out_indexer.shape[d] = shape[d]
        arg.out.step[d] = out_steps[d]
    plan = ReducePlan()
    assert _lib.lib.cumo_hip_plan_reduce(C.byref(arg), elmsz, accum, C.byref(plan)) == 0
    return plan


def test_reduce_row_plans():
    # [64,512,1024] f32 over the last axis: one wave per row, 128-bit loads
    p = red_plan((64, 512, 1024), (512 * 4096, 4096, 4), 2, (2048, 4))
    assert (p.kind, p.vec, p.threads_per_row, p.n_split) == (1, 4, 64, 1)
    assert p.out_ndim == 1 and p.out_total == 32768 and p.red_total == 1024
    # [4096,4096] f64 rows
    p = red_plan((4096, 4096), (32768, 8), 1, (8,), elmsz=8, accum=8)
    assert (p.kind, p.vec) == (1, 2) and p.threads_per_row in (64, 256)
    # short rows share a wave
    p = red_plan((100000, 8), (32, 4), 1, (4,))
    assert p.kind == 1 and p.threads_per_row == 1
    # full reduction of 2^25 elements is split
    p = red_plan((64 * 512 * 1024,), (4,), 0, ())
    assert p.kind == 1 and p.n_split > 1 and p.threads_per_row == 256 and p.out_total == 1


def test_reduce_column_plans():
    # [64,512,1024] over axis 0: reduce dims go last, so the descriptor is (512,1024,64)
    p = red_plan((512, 1024, 64), (4096, 4, 512 * 4096), 2, (4096, 4))
    assert (p.kind, p.vec, p.n_split) == (2, 4, 1)
    assert p.out_ndim == 1 and p.out_total == 524288
    # few outputs, long axis: split across blocks
    p = red_plan((64, 1 << 20), (4, 256), 1, (4,))
    assert p.kind == 2 and p.n_split > 1


def test_reduce_generic_shapes_plan_without_error():
    p = red_plan((5, 7, 9, 11), (-4 * 693, 396, -44, 8), 2, (28, 4))
    assert p.kind in (1, 2) and p.vec == 1
    p = red_plan((0, 5), (20, 4), 1, (4,))
    assert p.kind == 0
    p = red_plan((5, 0), (0, 4), 1, (4,))  # empty axis: every output still gets the identity
    assert p.kind != 0 and p.red_total == 0
