"""The host launch layer without a GPU: broadcasting, reduce dimensions moved
last, result shapes, loop contraction and the descriptors built from a prepared
loop. What is expected follows the reference's ndloop
(ext/cumo/narray/ndloop.c:421-451 trans_map, 493-516 broadcast rule, 870-940
contraction, 750-863 result shapes) and cumo_na_make_* (indexer.h:114-220).
Results are allocated from the pool's host backend, and the iterator is a
Python callback, so nothing is launched."""
import ctypes as C

import pytest

from cumo_amd import _lib
from cumo_amd._lib import (ITER_FUNC, NDF_FLAT_REDUCE, NDF_KEEP_DIM, Indexer, IArray, BitIArray, BitIArrayStridx, Loop,
                           NArrayDesc, NdFunc, ReductionArg)

L = _lib.lib
SF, DF, I32, I64, U64, BIT = range(6)
ELMSZ = {SF: 4, DF: 8, I32: 4, I64: 8, U64: 8, BIT: 1}
P = C.POINTER


@pytest.fixture(autouse=True)
def host_pool():
    L.cumo_hip_pool_free_all_blocks()
    assert L.cumo_hip_pool_use_host_backend(1) == 0
    yield
    L.cumo_hip_pool_free_all_blocks()
    assert L.cumo_hip_pool_total_bytes() == 0, "a test leaked pool memory"
    assert L.cumo_hip_pool_use_host_backend(0) == 0
    L.cumo_hip_last_error(None)


def view(type_, shape, strides=None, offset=0, ptr=0x10000):
    d = NArrayDesc()
    d.type, d.ndim, d.ptr, d.offset = type_, len(shape), ptr, offset
    if strides is None:
        strides, s = [0] * len(shape), ELMSZ[type_]
        for k in range(len(shape) - 1, -1, -1):
            strides[k] = s
            s *= shape[k]
    for k, (n, st) in enumerate(zip(shape, strides)):
        d.shape[k], d.stride[k] = n, st
    return d


def prepare(ins, out_types, reduce=0, flag=0, outs=None):
    nf = NdFunc()
    nf.flag, nf.nin, nf.nout = flag, len(ins), len(out_types)
    for k, t in enumerate(out_types):
        nf.out_type[k] = t
    in_arr = (P(NArrayDesc) * len(ins))(*[C.pointer(d) for d in ins])
    outs = outs if outs is not None else [NArrayDesc() for _ in out_types]
    out_arr = (P(NArrayDesc) * max(1, len(outs)))(*[C.pointer(d) for d in outs])
    lp = Loop()
    rc = L.cumo_hip_na_ndloop_prepare(C.byref(nf), in_arr, out_arr, reduce, C.byref(lp))
    return rc, lp, outs


def release(outs):
    for d in outs:
        if d.ptr:
            L.cumo_cuda_runtime_free(d.ptr)


def last_error():
    msg = C.c_char_p()
    kind = L.cumo_hip_last_error(C.byref(msg))
    return kind, (msg.value or b"").decode()


def test_broadcast_row_vector_keeps_two_dimensions():
    # C2: f64 [4096,4096] + [1,4096]
    a, r = view(DF, (4096, 4096)), view(DF, (1, 4096), ptr=0x9000000)
    rc, lp, outs = prepare([a, r], [DF])
    assert rc == 0 and (lp.narg, lp.ndim, lp.reduce_dim) == (3, 2, 0)
    assert list(lp.n[:2]) == [4096, 4096]
    assert list(lp.args[0].step[:2]) == [32768, 8]
    assert list(lp.args[1].step[:2]) == [0, 8]          # the row repeats
    assert list(lp.args[2].step[:2]) == [32768, 8]
    z = outs[0]
    assert (z.type, z.ndim, list(z.shape[:2]), list(z.stride[:2]), z.offset) == (DF, 2, [4096, 4096], [32768, 8], 0)
    assert z.ptr and L.cumo_hip_pool_used_bytes() == 4096 * 4096 * 8
    release(outs)


def test_contiguous_operands_contract_to_one_dimension():
    x, y = view(SF, (8, 16, 32)), view(SF, (8, 16, 32), ptr=0x80000)
    rc, lp, outs = prepare([x, y], [SF])
    assert rc == 0 and lp.ndim == 1 and lp.n[0] == 8 * 16 * 32
    assert [lp.args[j].step[0] for j in range(3)] == [4, 4, 4]
    release(outs)
    # a sliced middle dimension stops the merge there, the outer pair still merges with nothing
    xs = view(SF, (8, 8, 32), strides=(2048, 256, 4))
    rc, lp, outs = prepare([xs], [SF])
    assert rc == 0 and lp.ndim == 2
    assert list(lp.n[:lp.ndim]) == [64, 32]            # dims 0 and 1 merge (2048 == 256*8), dim 2 does not (256 != 4*32)
    assert list(lp.args[0].step[:2]) == [256, 4] and list(lp.args[1].step[:2]) == [128, 4]
    release(outs)


def test_size_one_dimensions_drop_and_scalars_loop_once():
    x = view(DF, (1, 5, 1), strides=(40, 8, 8))
    rc, lp, outs = prepare([x], [DF])
    assert rc == 0 and lp.ndim == 1 and lp.n[0] == 5 and lp.args[0].step[0] == 8
    assert list(outs[0].shape[:3]) == [1, 5, 1]
    release(outs)
    s = view(DF, ())
    rc, lp, outs = prepare([s], [DF])
    assert rc == 0 and lp.ndim == 1 and lp.n[0] == 1 and outs[0].ndim == 0
    release(outs)


def test_shape_mismatch_reports_shape_error_like_the_reference():
    rc, lp, outs = prepare([view(SF, (3, 4)), view(SF, (3, 5))], [SF])
    assert rc == 4
    kind, text = last_error()
    assert kind == 4 and text == "shape1[1](=4) != shape2[1](=5)"
    assert not outs[0].ptr
    # lower-rank operands align at the last dimension
    rc, lp, outs = prepare([view(SF, (2, 3, 4)), view(SF, (3, 1))], [SF])
    assert rc == 0 and list(outs[0].shape[:3]) == [2, 3, 4]
    assert list(lp.n[:lp.ndim]) == [2, 3, 4] and list(lp.args[1].step[:3]) == [0, 4, 0]
    release(outs)


def test_reduce_dimensions_move_last():
    x = view(SF, (2, 3, 4))
    rc, lp, outs = prepare([x], [SF], reduce=0b010, flag=NDF_FLAT_REDUCE)
    assert rc == 0 and (lp.ndim, lp.reduce_dim) == (3, 1)
    assert list(lp.n[:3]) == [2, 4, 3]
    assert list(lp.args[0].step[:3]) == [48, 4, 16]
    assert list(lp.args[1].step[:3]) == [16, 4, 0]
    assert (outs[0].ndim, list(outs[0].shape[:2])) == (2, [2, 4])
    arg = ReductionArg()
    L.cumo_hip_make_reduction_arg(C.byref(lp), C.byref(arg))
    assert (arg.in_indexer.ndim, arg.in_indexer.total_size, list(arg.in_indexer.shape[:3])) == (3, 24, [2, 4, 3])
    assert (arg.out_indexer.ndim, arg.out_indexer.total_size, list(arg.out_indexer.shape[:2])) == (2, 8, [2, 4])
    assert arg.in_.ptr == 0x10000 and list(arg.in_.step[:3]) == [48, 4, 16]
    assert arg.out.ptr == outs[0].ptr and list(arg.out.step[:3]) == [16, 4, 0]
    release(outs)


def test_reduce_keepdims_and_full_reduction():
    x = view(DF, (2, 3, 4))
    rc, lp, outs = prepare([x], [DF], reduce=0b101, flag=NDF_FLAT_REDUCE | NDF_KEEP_DIM)
    assert rc == 0 and (outs[0].ndim, list(outs[0].shape[:3])) == (3, [1, 3, 1])
    assert (lp.ndim, lp.reduce_dim) == (3, 2) and list(lp.n[:3]) == [3, 2, 4]
    assert list(lp.args[0].step[:3]) == [32, 96, 8] and list(lp.args[1].step[:3]) == [8, 0, 0]
    release(outs)
    # every dimension reduced on a contiguous array: one run
    rc, lp, outs = prepare([x], [DF], reduce=0b111, flag=NDF_FLAT_REDUCE)
    assert rc == 0 and (lp.ndim, lp.reduce_dim, lp.n[0]) == (1, 1, 24) and outs[0].ndim == 0
    assert L.cumo_hip_pool_used_bytes() == 512    # one 8-byte result, rounded up by the pool
    release(outs)
    # neighbouring reduce dimensions merge, kept ones merge, the two groups never do
    y = view(SF, (4, 5, 6, 7))
    rc, lp, outs = prepare([y], [SF], reduce=0b1100, flag=NDF_FLAT_REDUCE)
    assert rc == 0 and (lp.ndim, lp.reduce_dim) == (2, 1) and list(lp.n[:2]) == [20, 42]
    release(outs)
    # a reduced dimension of size 1 still leaves one reduce dimension
    w = view(SF, (5, 1))
    rc, lp, outs = prepare([w], [SF], reduce=0b10, flag=NDF_FLAT_REDUCE)
    assert rc == 0 and (lp.ndim, lp.reduce_dim) == (2, 1) and list(lp.n[:2]) == [5, 1]
    release(outs)


def test_reduce_flag_errors():
    x = view(SF, (2, 3))
    rc, _, outs = prepare([x], [SF], reduce=0b100, flag=NDF_FLAT_REDUCE)
    assert rc == 8 and last_error()[0] == 8
    rc, _, outs = prepare([x], [SF], reduce=0b01, flag=0)
    assert rc == 3 and last_error()[0] == 3


def test_given_result_is_checked_not_allocated():
    x = view(SF, (3, 4))
    good = view(SF, (3, 4), ptr=0x500000)
    rc, lp, _ = prepare([x], [SF], outs=[good])
    assert rc == 0 and lp.args[1].ptr == 0x500000 and L.cumo_hip_pool_used_bytes() == 0
    rc, _, _ = prepare([x], [SF], outs=[view(SF, (4, 3), ptr=0x500000)])
    assert rc == 4 and last_error()[0] == 4
    rc, _, _ = prepare([x], [SF], outs=[view(DF, (3, 4), ptr=0x500000)])
    assert rc == 6 and last_error()[0] == 6
    # a strided result view keeps its own steps
    strided = view(SF, (3, 4), strides=(64, 8), offset=16, ptr=0x500000)
    rc, lp, _ = prepare([x], [SF], outs=[strided])
    assert rc == 0 and lp.args[1].ptr == 0x500010 and list(lp.args[1].step[:2]) == [64, 8] and lp.ndim == 2


def test_bit_views_carry_bit_positions():
    b = view(BIT, (10, 70), strides=(96, 1), offset=37, ptr=0x7000)
    rc, lp, outs = prepare([b], [BIT])
    assert rc == 0 and lp.args[0].ptr == 0x7000 and lp.args[0].bitpos == 37 and lp.args[0].elmsz == 0
    assert list(lp.args[0].step[:2]) == [96, 1] and list(lp.args[1].step[:2]) == [70, 1]
    assert L.cumo_hip_pool_used_bytes() == 512 and L.cumo_hip_na_storage_bytes(BIT, 700) == 88
    ia, sx = BitIArray(), BitIArrayStridx()
    L.cumo_hip_make_bit_iarray(C.byref(lp), 0, C.byref(ia))
    L.cumo_hip_make_bit_iarray_stridx(C.byref(lp), 0, C.byref(sx))
    assert (ia.ptr, ia.pos, list(ia.step[:2])) == (0x7000, 37, [96, 1])
    assert (sx.pos, sx.stridx[0], sx.stridx[1], sx.stridx[5]) == (37, (96 << 1) | 1, (1 << 1) | 1, 1)
    release(outs)


def test_negative_steps_and_make_descriptors():
    x = view(I32, (6, 5), strides=(-20, 4), offset=100)
    rc, lp, outs = prepare([x], [I32])
    assert rc == 0 and lp.args[0].ptr == 0x10000 + 100 and list(lp.args[0].step[:2]) == [-20, 4]
    ix, ia = Indexer(), IArray()
    L.cumo_hip_make_indexer(C.byref(lp), C.byref(ix))
    L.cumo_hip_make_iarray(C.byref(lp), 0, C.byref(ia))
    assert (ix.ndim, ix.total_size, list(ix.shape[:2])) == (2, 30, [6, 5])
    assert ia.ptr == 0x10000 + 100 and list(ia.step[:3]) == [-20, 4, 0]
    release(outs)


def run_ndloop(ins, out_types, reduce=0, flag=0):
    seen = []

    def it(lp):
        seen.append((lp.contents.ndim, list(lp.contents.n[:lp.contents.ndim]), lp.contents.reduce_dim))

    nf = NdFunc()
    nf.func, nf.flag, nf.nin, nf.nout = ITER_FUNC(it), flag, len(ins), len(out_types)
    for k, t in enumerate(out_types):
        nf.out_type[k] = t
    in_arr = (P(NArrayDesc) * len(ins))(*[C.pointer(d) for d in ins])
    outs = [NArrayDesc() for _ in out_types]
    out_arr = (P(NArrayDesc) * max(1, len(outs)))(*[C.pointer(d) for d in outs])
    rc = L.cumo_hip_na_ndloop(C.byref(nf), in_arr, out_arr, reduce, None)
    release(outs)
    return rc, seen, outs


def test_iterator_is_called_once_and_not_for_empty_loops():
    rc, seen, _ = run_ndloop([view(SF, (3, 4)), view(SF, (4,))], [SF])
    assert rc == 0 and seen == [(2, [3, 4], 0)]
    rc, seen, outs = run_ndloop([view(SF, (3, 0)), view(SF, (1,))], [SF])
    assert rc == 0 and seen == [] and list(outs[0].shape[:2]) == [3, 0]
    # an empty reduce axis with outputs to fill still reaches the iterator
    rc, seen, outs = run_ndloop([view(SF, (3, 0))], [SF], reduce=0b10, flag=NDF_FLAT_REDUCE)
    assert rc == 0 and seen == [(2, [3, 0], 1)]


def test_operation_front_ends_fail_before_any_launch():
    x, z = view(SF, (3, 4)), NArrayDesc()
    assert L.cumo_hip_na_binary(b"no_such_op", C.byref(x), C.byref(x), C.byref(z)) == 6
    kind, text = last_error()
    assert kind == 6 and "no_such_op" in text
    assert L.cumo_hip_na_binary(b"bit_and", C.byref(x), C.byref(x), C.byref(z)) == 6 and last_error()[0] == 6
    i = view(I32, (3, 4))
    assert L.cumo_hip_na_unary(b"floor", C.byref(i), C.byref(z)) == 6 and last_error()[0] == 6
    assert L.cumo_hip_na_reduce(b"mean", C.byref(i), 0, 0, 0, C.byref(z), None) == 6 and last_error()[0] == 6
    b = view(BIT, (8,))
    assert L.cumo_hip_na_binary(b"add", C.byref(b), C.byref(x), C.byref(z)) == 6 and last_error()[0] == 6
    assert L.cumo_hip_na_bit_binary(b"and", C.byref(x), C.byref(b), C.byref(z)) == 6 and last_error()[0] == 6
    # reference: narray/narray.c:1704-1716
    e = view(SF, (0, 4))
    assert L.cumo_hip_na_reduce(b"sum", C.byref(e), 0, 0, 0, C.byref(z), None) == 4
    assert last_error() == (4, "cannot reduce empty NArray")
    assert L.cumo_hip_na_reduce(b"sum", C.byref(x), 0b100, 0, 0, C.byref(z), None) == 8 and last_error()[0] == 8
    assert L.cumo_hip_na_compare(b"gt", C.byref(x), C.byref(view(SF, (5,))), C.byref(z)) == 4 and last_error()[0] == 4
    assert not z.ptr and L.cumo_hip_pool_used_bytes() == 0
