"""The launcher boundary itself, the way the Ruby extension's generated host
iterators call it: descriptors filled by hand (not by this library's launch
layer), with dimensions left un-merged, size-1 dimensions kept, steps of 0 for
repeated operands and negative steps, exactly as
ext/cumo/include/cumo/indexer.h:114-220 would build them. Results are compared
with numpy on the same views (single IEEE operations, integer work: bit-exact)."""
import ctypes as C

import numpy as np
import pytest

from helpers import assert_bits_equal, assert_reduction_close

pytestmark = pytest.mark.gpu

P = C.POINTER


def dev(arr):
    """Uploads a numpy array; returns (device pointer, keep-alive)."""
    from cumo_amd import _lib
    a = np.ascontiguousarray(arr)
    p = _lib.call(_lib.lib.cumo_cuda_runtime_malloc, max(a.nbytes, 4))
    _lib.call(_lib.lib.cumo_hip_memcpy_h2d, p, a.ctypes.data, a.nbytes)
    return p


def fetch(ptr, shape, dtype):
    from cumo_amd import _lib
    out = np.empty(shape, dtype=dtype)
    _lib.call(_lib.lib.cumo_hip_memcpy_d2h, out.ctypes.data, ptr, out.nbytes)
    return out


def free(*ptrs):
    from cumo_amd import _lib
    for p in ptrs:
        _lib.lib.cumo_cuda_runtime_free(p)


def indexer(shape):
    from cumo_amd import _lib
    ix = _lib.Indexer()
    ix.ndim = len(shape)
    ix.total_size = int(np.prod(shape)) if len(shape) else 1
    for d, n in enumerate(shape):
        ix.shape[d] = n
    return ix


def iarray(ptr, steps):
    from cumo_amd import _lib
    ia = _lib.IArray()
    ia.ptr = ptr
    for d, s in enumerate(steps):
        ia.step[d] = s
    return ia


def test_binary_add_uncontracted_five_dimensions_with_repeat():
    from cumo_amd import _lib
    rng = np.random.default_rng(5)
    shape = (3, 1, 4, 2, 5)
    x = rng.standard_normal(shape, dtype=np.float32)
    y = rng.standard_normal((4, 1, 5), dtype=np.float32)        # repeats along dims 0, 1 and 3
    px, py = dev(x), dev(y)
    pz = _lib.call(_lib.lib.cumo_cuda_runtime_malloc, x.nbytes)
    ix = indexer(shape)
    a1 = iarray(px, x.strides)
    a2 = iarray(py, (0, 0, y.strides[0], 0, y.strides[2]))
    a3 = iarray(pz, x.strides)
    f = _lib.fn("cumo_iter_sfloat_add_kernel_launch", None, [P(_lib.IArray)] * 3 + [P(_lib.Indexer), P(C.c_int)])
    _lib.call(f, C.byref(a1), C.byref(a2), C.byref(a3), C.byref(ix), None)
    assert_bits_equal(fetch(pz, shape, np.float32), x + y.reshape(1, 1, 4, 1, 5))
    # the scalar form: 10 - x
    fs = _lib.fn("cumo_iter_sfloat_sub_s_kernel_launch", None,
                 [P(_lib.IArray), C.c_float, P(_lib.IArray), P(_lib.Indexer), P(C.c_int), C.c_int])
    _lib.call(fs, C.byref(a1), C.c_float(10.0), C.byref(a3), C.byref(ix), None, 1)
    assert_bits_equal(fetch(pz, shape, np.float32), np.float32(10.0) - x)
    free(px, py, pz)


def test_negative_steps_and_view_offset_in_ptr():
    from cumo_amd import _lib
    h = np.arange(7 * 9, dtype=np.int32).reshape(7, 9)
    v = h[::-2, 1:8:3]                                           # shape (4, 3), steps (-72, 12)
    ph = dev(h)
    pz = _lib.call(_lib.lib.cumo_cuda_runtime_malloc, 4 * 12)
    off = v.__array_interface__["data"][0] - h.__array_interface__["data"][0]
    a1 = iarray(ph + off, v.strides)
    a2 = iarray(pz, (12, 4))
    ix = indexer(v.shape)
    f = _lib.fn("cumo_iter_int32_store_int32_kernel_launch", None, [P(_lib.IArray), P(_lib.IArray), P(_lib.Indexer)])
    _lib.call(f, C.byref(a2), C.byref(a1), C.byref(ix))          # a1 of the launcher is the destination
    assert_bits_equal(fetch(pz, v.shape, np.int32), np.ascontiguousarray(v))
    g = _lib.fn("cumo_iter_copy_bytes_indexer_kernel_launch", None, [P(_lib.IArray), P(_lib.IArray), P(_lib.Indexer), C.c_ssize_t])
    _lib.call(_lib.lib.cumo_hip_memset, pz, 0, 48)
    _lib.call(g, C.byref(a1), C.byref(a2), C.byref(ix), 4)       # here a1 is the source
    assert_bits_equal(fetch(pz, v.shape, np.int32), np.ascontiguousarray(v))
    free(ph, pz)


def test_reduction_arg_with_reduce_dimensions_last():
    from cumo_amd import _lib
    rng = np.random.default_rng(6)
    h = rng.standard_normal((6, 7, 8))
    ph = dev(h)
    pz = _lib.call(_lib.lib.cumo_cuda_runtime_malloc, 8 * 48)
    arg = _lib.ReductionArg()
    # reduce dim 1: the loop order is [6, 8 | 7] (indexer.h:189-220)
    arg.in_.ptr = ph
    for k, (n, s) in enumerate(((6, 448), (8, 8), (7, 64))):
        arg.in_indexer.shape[k] = n
        arg.in_.step[k] = s
    arg.in_indexer.ndim, arg.in_indexer.total_size = 3, 336
    arg.out.ptr = pz
    arg.out.step[0], arg.out.step[1] = 64, 8
    arg.out_indexer.ndim, arg.out_indexer.total_size = 2, 48
    arg.out_indexer.shape[0], arg.out_indexer.shape[1] = 6, 8
    for name, want in (("sum", h.sum(axis=1)), ("max", h.max(axis=1)), ("min", h.min(axis=1))):
        f = _lib.fn("cumo_dfloat_%s_kernel_launch" % name, None, [P(_lib.ReductionArg)])
        _lib.call(f, C.byref(arg))
        got = fetch(pz, (6, 8), np.float64)
        if name == "sum":
            assert_reduction_close(got, want, 7, scale=np.abs(h).sum(axis=1))
        else:
            assert_bits_equal(got, want, name)
    # argmax answers the position along the reduced axis, as Int32 or Int64 by symbol
    pi = _lib.call(_lib.lib.cumo_cuda_runtime_malloc, 8 * 48)
    arg.out.ptr = pi
    arg.out.step[0], arg.out.step[1] = 32, 4
    f = _lib.fn("cumo_dfloat_argmax_int32_kernel_launch", None, [P(_lib.ReductionArg)])
    _lib.call(f, C.byref(arg))
    assert_bits_equal(fetch(pi, (6, 8), np.int32), h.argmax(axis=1).astype(np.int32))
    arg.out.step[0], arg.out.step[1] = 64, 8
    f = _lib.fn("cumo_dfloat_argmin_int64_kernel_launch", None, [P(_lib.ReductionArg)])
    _lib.call(f, C.byref(arg))
    assert_bits_equal(fetch(pi, (6, 8), np.int64), h.argmin(axis=1).astype(np.int64))
    free(ph, pz, pi)


def test_compare_into_bits_at_a_bit_offset():
    from cumo_amd import _lib
    rng = np.random.default_rng(7)
    x = rng.standard_normal((5, 37), dtype=np.float32)
    px = dev(x)
    nwords = 16
    pw = dev(np.full(nwords, 0xFFFFFFFF, dtype=np.uint32))       # untouched bits must stay set
    a1 = iarray(px, x.strides)
    a3 = _lib.BitIArray()
    a3.ptr, a3.pos = pw, 13
    a3.step[0], a3.step[1] = 37, 1
    ix = indexer(x.shape)
    f = _lib.fn("cumo_iter_sfloat_gt_s_kernel_launch", None,
                [P(_lib.IArray), C.c_float, P(_lib.BitIArray), P(_lib.Indexer), C.c_int])
    _lib.call(f, C.byref(a1), C.c_float(0.25), C.byref(a3), C.byref(ix), 0)
    words = fetch(pw, (nwords,), np.uint32)
    bits = np.unpackbits(words.view(np.uint8), bitorder="little")
    want = np.ones(nwords * 32, dtype=np.uint8)
    want[13:13 + x.size] = (x > np.float32(0.25)).reshape(-1)
    assert (bits == want).all()
    # count_true over that run adds onto the destination (tmpl_bit/bit_count_kernel.cu:4-78)
    pc = dev(np.array([1000], dtype=np.uint64))
    g = _lib.fn("cumo_iter_bit_count_true_stride_kernel_launch", None,
                [C.c_size_t, C.c_void_p, C.c_void_p, C.c_ssize_t, C.c_uint64])
    _lib.call(g, 13, pc, pw, 1, x.size)
    assert int(fetch(pc, (1,), np.uint64)[0]) == 1000 + int((x > np.float32(0.25)).sum())
    free(px, pw, pc)


@pytest.mark.parametrize("pos", [0, 128, 256 + 128, 96, 5])
@pytest.mark.parametrize("n", [1, 127, 128, 129, 255, 1000, 128 * 300, 128 * 300 + 77])
def test_flat_compare_into_bits_positions_and_ragged_ends(pos, n):
    """One contiguous run compared into a Bit run that starts on a 128-bit unit (the
    lean kernel) or anywhere else (the general one): every bit before and after the
    run must keep its value, whichever kernel stores the ragged last words."""
    from cumo_amd import _lib
    rng = np.random.default_rng(1000 + pos + n)
    x = rng.integers(-3, 4, size=n).astype(np.float32)
    y = rng.integers(-3, 4, size=n).astype(np.float32)
    x[rng.integers(0, n)] = np.nan
    px, py = dev(x), dev(y)
    nwords = (pos + n + 31) // 32 + 8
    for fillv in (0xFFFFFFFF, 0):
        pw = dev(np.full(nwords, fillv, dtype=np.uint32))
        a1, a2 = iarray(px, (4,)), iarray(py, (4,))
        a3 = _lib.BitIArray()
        a3.ptr, a3.pos = pw, pos
        a3.step[0] = 1
        ix = indexer((n,))
        f = _lib.fn("cumo_iter_sfloat_le_kernel_launch", None, [P(_lib.IArray), P(_lib.IArray), P(_lib.BitIArray), P(_lib.Indexer)])
        _lib.call(f, C.byref(a1), C.byref(a2), C.byref(a3), C.byref(ix))
        bits = np.unpackbits(fetch(pw, (nwords,), np.uint32).view(np.uint8), bitorder="little")
        want = np.full(nwords * 32, 1 if fillv else 0, dtype=np.uint8)
        with np.errstate(invalid="ignore"):
            want[pos:pos + n] = x <= y
        assert (bits == want).all(), (pos, n, fillv, "array <= array")
        # scalar on the left: 1 > x
        fs = _lib.fn("cumo_iter_sfloat_gt_s_kernel_launch", None,
                     [P(_lib.IArray), C.c_float, P(_lib.BitIArray), P(_lib.Indexer), C.c_int])
        _lib.call(fs, C.byref(a1), C.c_float(1.0), C.byref(a3), C.byref(ix), 1)
        bits = np.unpackbits(fetch(pw, (nwords,), np.uint32).view(np.uint8), bitorder="little")
        with np.errstate(invalid="ignore"):
            want[pos:pos + n] = np.float32(1.0) > x
        assert (bits == want).all(), (pos, n, fillv, "scalar > array")
        free(pw)
    # DFloat: two elements per lane, sixteen lanes per word
    xd = x.astype(np.float64)
    pd = dev(xd)
    pw = dev(np.full(nwords, 0xFFFFFFFF, dtype=np.uint32))
    a1 = iarray(pd, (8,))
    a3 = _lib.BitIArray()
    a3.ptr, a3.pos = pw, pos
    a3.step[0] = 1
    ix = indexer((n,))
    fd = _lib.fn("cumo_iter_dfloat_lt_s_kernel_launch", None,
                 [P(_lib.IArray), C.c_double, P(_lib.BitIArray), P(_lib.Indexer), C.c_int])
    _lib.call(fd, C.byref(a1), C.c_double(0.5), C.byref(a3), C.byref(ix), 0)
    bits = np.unpackbits(fetch(pw, (nwords,), np.uint32).view(np.uint8), bitorder="little")
    want = np.ones(nwords * 32, dtype=np.uint8)
    with np.errstate(invalid="ignore"):
        want[pos:pos + n] = xd < 0.5
    assert (bits == want).all(), (pos, n, "dfloat")
    free(px, py, pd, pw)


def test_int32_divide_by_zero_sets_the_pinned_flag_and_skips_the_store():
    from cumo_amd import _lib
    x = np.array([7, 8, 9, 10], dtype=np.int32)
    y = np.array([2, 0, 3, 0], dtype=np.int32)
    px, py = dev(x), dev(y)
    pz = dev(np.full(4, -1, dtype=np.int32))
    ix = indexer((4,))
    a1, a2, a3 = iarray(px, (4,)), iarray(py, (4,)), iarray(pz, (4,))
    flag = _lib.lib.cumo_cuda_runtime_error_flag_new()
    f = _lib.fn("cumo_iter_int32_div_kernel_launch", None, [P(_lib.IArray)] * 3 + [P(_lib.Indexer), P(C.c_int)])
    _lib.call(f, C.byref(a1), C.byref(a2), C.byref(a3), C.byref(ix), flag)
    assert _lib.call(_lib.lib.cumo_cuda_runtime_error_flag_get, flag) is True
    assert fetch(pz, (4,), np.int32).tolist() == [3, -1, 3, -1]
    free(px, py, pz)


def test_zero_total_size_is_a_no_op():
    from cumo_amd import _lib
    ix = indexer((0, 5))
    a = iarray(None, (20, 4))
    f = _lib.fn("cumo_iter_sfloat_add_kernel_launch", None, [P(_lib.IArray)] * 3 + [P(_lib.Indexer), P(C.c_int)])
    _lib.call(f, C.byref(a), C.byref(a), C.byref(a), C.byref(ix), None)
    _lib.call(_lib.lib.cumo_hip_synchronize)
