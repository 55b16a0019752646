"""The rest of the Bit template set and the stores around it, through the C-ABI with
hand-built arguments, against numpy bit for bit: all? / any? (tmpl_bit/bit_reduce.c:1-3),
Bit fill (tmpl_bit/fill.c:1-2), number -> Bit (tmpl_bit/store_from.c:2), store_array
(tmpl_bit/store_array.c:1-5, tmpl/store_array.c:2-5), the same-type store between views
with index arrays (tmpl/store_from.c:5); then the reference's own cases for them
(test/narray_test.rb:2725-2815, test/bit_test.rb:38-40,70-72,164-166) through the mirror."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

P = C.POINTER
SZ, SSZ, U64, VP = C.c_size_t, C.c_ssize_t, C.c_uint64, C.c_void_p


def lib():
    from cumo_amd import _lib
    return _lib


def dev(a):
    L = lib()
    a = np.ascontiguousarray(a)
    p = L.call(L.lib.cumo_cuda_runtime_malloc, max(a.nbytes, 8))
    if a.nbytes:
        L.call(L.lib.cumo_hip_memcpy_h2d, p, a.ctypes.data, a.nbytes)
    return p


def fetch(p, n, dtype):
    L = lib()
    out = np.empty(n, dtype=dtype)
    if out.nbytes:
        L.call(L.lib.cumo_hip_memcpy_d2h, out.ctypes.data, p, out.nbytes)
    return out


def free(*ps):
    for p in ps:
        lib().lib.cumo_cuda_runtime_free(p)


def pack(bits, total_bits=None):
    """LSB-first 32-bit words (template.h:110-138)."""
    bits = np.asarray(bits, dtype=np.uint8)
    n = bits.size if total_bits is None else total_bits
    buf = np.zeros(((n + 31) // 32) * 32, dtype=np.uint8)
    buf[:bits.size] = bits
    return np.packbits(buf, bitorder="little").view(np.uint32)


def unpack(words, n):
    return np.unpackbits(np.asarray(words, dtype=np.uint32).view(np.uint8), bitorder="little")[:n]


def indexer(shape):
    L = lib()
    ix = L.Indexer()
    ix.ndim = len(shape)
    ix.total_size = int(np.prod(shape)) if len(shape) else 1
    for d, n in enumerate(shape):
        ix.shape[d] = n
    return ix


def stride_sdx(s):
    return (int(s) << 1) | 1


@pytest.mark.parametrize("n", [1, 31, 32, 33, 64, 100, 20000, (1 << 20) + 77])
def test_all_any_of_one_contiguous_run(n):
    L = lib()
    rng = np.random.default_rng(n)
    for which, init in (("all_p", 1), ("any_p", 0)):
        f = L.fn("cumo_iter_bit_%s_contiguous_reduce_kernel_launch" % which, None, [VP, SZ, VP, SZ, U64])
        g = L.fn("cumo_iter_bit_%s_reduce_kernel_launch" % which, None, [VP, SZ, SSZ, VP, VP, SZ, U64])
        for p1 in (0, 13, 32, 45):
            for odd_at in (None, 0, n // 2, n - 1):
                bits = np.full(p1 + n + 40, 1 - init, dtype=np.uint8)   # everything around the run would flip the answer
                bits[p1:p1 + n] = init
                if odd_at is not None:
                    bits[p1 + odd_at] = 1 - init
                pa = dev(pack(bits))
                out = np.array([0xffffffff if init else 0, 0x5a5a5a5a], dtype=np.uint32)
                for launcher in ("words", "gather"):
                    po = dev(out)
                    if launcher == "words":
                        L.call(f, pa, p1, po, 7, n)
                    else:
                        L.call(g, pa, p1, 1, None, po, 7, n)
                    got = fetch(po, 2, np.uint32)
                    want = out.copy()
                    answer = init if odd_at is None else 1 - init
                    want[0] = (want[0] & ~np.uint32(1 << 7)) | np.uint32(answer << 7)
                    assert (got == want).all(), (which, launcher, n, p1, odd_at, got, want)
                    free(po)
                free(pa)


def test_all_any_strided_indexed_and_elementwise():
    L = lib()
    rng = np.random.default_rng(7)
    n = 20000
    src = rng.integers(0, 2, size=3 * n + 50).astype(np.uint8)
    pa = dev(pack(src))
    picked = ((np.arange(n) * 7 + 3) % n).astype(np.uint64)
    pidx = dev(picked)
    for which, init in (("all_p", 1), ("any_p", 0)):
        g = L.fn("cumo_iter_bit_%s_reduce_kernel_launch" % which, None, [VP, SZ, SSZ, VP, VP, SZ, U64])
        e = L.fn("cumo_iter_bit_%s_elementwise_kernel_launch" % which, None, [VP, SZ, SSZ, VP, VP, SZ, SSZ, VP, U64])
        for (p1, s1, idx, sel) in ((5, 2, None, src[5:5 + 2 * n:2]), (3 * n + 20, -3, None, src[3 * n + 20::-3][:n]), (11, 0, pidx, src[11 + picked.astype(np.int64)])):
            for force in (False, True):
                s = src.copy()
                if force:   # make the whole selection equal to init so that the answer stays
                    pos = (11 + picked.astype(np.int64)) if idx is not None else (p1 + s1 * np.arange(n))
                    s[pos] = init
                    pb = dev(pack(s))
                else:
                    pb = pa
                seln = s[(11 + picked.astype(np.int64)) if idx is not None else (p1 + s1 * np.arange(n))]
                po = dev(np.array([0xffffffff if init else 0], dtype=np.uint32))
                L.call(g, pb, p1, s1, idx, po, 31, n)
                got = (int(fetch(po, 1, np.uint32)[0]) >> 31) & 1
                want = int(seln.all()) if init else int(seln.any())
                assert got == want, (which, p1, s1, force)
                free(po)
                if force:
                    free(pb)
        # elementwise: out[j] (a strided run of result bits) folds column j of a 2-d bit matrix, row by row
        rows, cols = 5, 700
        m = rng.integers(0, 2, size=(rows, cols)).astype(np.uint8)
        if init:
            m[:, ::3] = 1
        else:
            m[:, ::3] = 0
        pm = dev(pack(m.reshape(-1)))
        res_bits = np.full(3 * cols + 9, init, dtype=np.uint8)
        po = dev(pack(res_bits))
        for r in range(rows):
            L.call(e, pm, r * cols, 1, None, po, 9, 3, None, cols)
        got = unpack(fetch(po, (3 * cols + 9 + 31) // 32, np.uint32), 3 * cols + 9)
        want = res_bits.copy()
        want[9::3][:cols] = m.all(axis=0) if init else m.any(axis=0)
        assert (got == want).all(), which
        free(pm, po)
    free(pa, pidx)


@pytest.mark.parametrize("n,p3", [(1, 0), (5, 30), (32, 0), (33, 31), (64, 64), (1000, 7), (100003, 45)])
def test_bit_fill_contiguous_and_general(n, p3):
    L = lib()
    f = L.fn("cumo_iter_bit_fill_contiguous_kernel_launch", None, [VP, SZ, U64, C.c_uint])
    g = L.fn("cumo_iter_bit_fill_kernel_launch", None, [P(L.BitIArrayStridx), C.c_uint, P(L.Indexer)])
    total = p3 + n + 50
    rng = np.random.default_rng(n + p3)
    for y in (0, 1):
        before = rng.integers(0, 2, size=total).astype(np.uint8)
        pa = dev(pack(before))
        L.call(f, pa, p3, n, 0xffffffff if y else 0)
        want = before.copy()
        want[p3:p3 + n] = y
        assert (unpack(fetch(pa, (total + 31) // 32, np.uint32), total) == want).all()
        free(pa)
    # general form: a 2-d view with a step of 3 bits along the rows and an index array along the columns
    rows, cols = 6, 41
    total = 7 + rows * 200
    colidx = (np.arange(cols) * 4 + 1).astype(np.uint64)
    pidx = dev(colidx)
    before = rng.integers(0, 2, size=total).astype(np.uint8)
    for y in (0, 1):
        pa = dev(pack(before))
        a3 = L.BitIArrayStridx()
        a3.ptr, a3.pos = pa, 7
        a3.stridx[0] = stride_sdx(200)
        a3.stridx[1] = pidx          # a device pointer: bit 0 clear
        ix = indexer((rows, cols))
        L.call(g, C.byref(a3), y, C.byref(ix))
        want = before.copy()
        for r in range(rows):
            want[7 + r * 200 + colidx.astype(np.int64)] = y
        assert (unpack(fetch(pa, (total + 31) // 32, np.uint32), total) == want).all()
        free(pa)
    free(pidx)


@pytest.mark.parametrize("tname,dtype", [("sfloat", np.float32), ("dfloat", np.float64), ("int32", np.int32), ("int64", np.int64), ("uint64", np.uint64)])
def test_number_to_bit_store(tname, dtype):
    L = lib()
    f = L.fn("cumo_iter_bit_store_%s_kernel_launch" % tname, None, [P(L.BitIArrayStridx), P(L.IArrayStridx), P(L.Indexer)])
    rng = np.random.default_rng(len(tname))
    esz = np.dtype(dtype).itemsize
    for n, pos, step in ((1, 0, 1), (40, 3, 1), (64, 32, 1), (1000, 61, 2), (100003, 5, 1), (1 << 20, 0, 1)):
        vals = rng.integers(-2, 3, size=n * step).astype(dtype)
        if dtype in (np.float32, np.float64):
            vals[::7] = dtype(-0.0)       # -0 is zero
            vals[3::11] = np.nan          # NaN != 0 is true
            vals[5::13] = 1e-30
        total = pos + n + 40
        before = rng.integers(0, 2, size=total).astype(np.uint8)
        pa, pv = dev(pack(before)), dev(vals)
        a1, a2 = L.BitIArrayStridx(), L.IArrayStridx()
        a1.ptr, a1.pos = pa, pos
        a1.stridx[0] = stride_sdx(1)
        a2.ptr = pv
        a2.stridx[0] = stride_sdx(esz * step)
        ix = indexer((n,))
        L.call(f, C.byref(a1), C.byref(a2), C.byref(ix))
        want = before.copy()
        want[pos:pos + n] = (vals[::step] != 0).astype(np.uint8)
        assert (unpack(fetch(pa, (total + 31) // 32, np.uint32), total) == want).all(), (tname, n, pos, step)
        free(pa, pv)
    # 2-d: destination rows 100 bits apart walked backwards, source columns through an index array
    rows, cols = 9, 37
    vals = rng.integers(-1, 2, size=(rows, 64)).astype(dtype)
    colidx = (rng.permutation(64)[:cols] * esz).astype(np.uint64)
    total = 1000
    before = rng.integers(0, 2, size=total).astype(np.uint8)
    pa, pv, pidx = dev(pack(before)), dev(vals), dev(colidx)
    a1, a2 = L.BitIArrayStridx(), L.IArrayStridx()
    a1.ptr, a1.pos = pa, 850
    a1.stridx[0], a1.stridx[1] = stride_sdx(-100), stride_sdx(2)
    a2.ptr = pv
    a2.stridx[0] = stride_sdx(64 * esz)
    a2.stridx[1] = pidx
    ix = indexer((rows, cols))
    L.call(f, C.byref(a1), C.byref(a2), C.byref(ix))
    want = before.copy()
    for r in range(rows):
        want[850 - 100 * r + 2 * np.arange(cols)] = (vals[r, (colidx // esz).astype(np.int64)] != 0)
    assert (unpack(fetch(pa, (total + 31) // 32, np.uint32), total) == want).all()
    free(pa, pv, pidx)


def test_bit_store_array_launchers():
    L = lib()
    rng = np.random.default_rng(21)
    n = 5000
    stage_bits = rng.integers(0, 2, size=n).astype(np.uint8)
    pz = dev(pack(stage_bits))
    total = 3 * n + 100
    before = rng.integers(0, 2, size=total).astype(np.uint8)
    idx = (rng.permutation(total - 10)[:n]).astype(np.uint64)
    pidx = dev(idx)
    cases = [
        ("contiguous", [VP, SZ, VP, U64], lambda pa: (pa, 37, pz, n), lambda w: w.__setitem__(slice(37, 37 + n), stage_bits)),
        ("stride", [VP, SZ, SSZ, VP, U64], lambda pa: (pa, 3 * n + 20, -3, pz, n), lambda w: w.__setitem__(3 * n + 20 - 3 * np.arange(n), stage_bits)),
        ("index", [VP, SZ, VP, VP, U64], lambda pa: (pa, 9, pidx, pz, n), lambda w: w.__setitem__(9 + idx.astype(np.int64), stage_bits)),
        ("stride_scalar", [VP, SZ, SSZ, C.c_uint, U64], lambda pa: (pa, 40, 2, 1, n), lambda w: w.__setitem__(40 + 2 * np.arange(n), 1)),
        ("stride_scalar", [VP, SZ, SSZ, C.c_uint, U64], lambda pa: (pa, 41, 1, 0, n), lambda w: w.__setitem__(slice(41, 41 + n), 0)),
        ("index_scalar", [VP, SZ, VP, C.c_uint, U64], lambda pa: (pa, 2, pidx, 0, n), lambda w: w.__setitem__(2 + idx.astype(np.int64), 0)),
    ]
    for name, sig, args, apply in cases:
        f = L.fn("cumo_iter_bit_store_array_%s_kernel_launch" % name, None, sig)
        pa = dev(pack(before))
        L.call(f, *args(pa))
        want = before.copy()
        apply(want)
        assert (unpack(fetch(pa, (total + 31) // 32, np.uint32), total) == want).all(), name
        free(pa)
    free(pz, pidx)


@pytest.mark.parametrize("tname,dtype,ctype", [("sfloat", np.float32, C.c_float), ("dfloat", np.float64, C.c_double), ("int32", np.int32, C.c_int32)])
def test_typed_stridx_store_and_store_array(tname, dtype, ctype):
    L = lib()
    rng = np.random.default_rng(31)
    esz = np.dtype(dtype).itemsize
    # dst[rowidx, ::-2] = src[:, colidx]
    rows, cols = 11, 23
    src = rng.integers(-50, 50, size=(rows, 64)).astype(dtype)
    dst0 = rng.integers(-50, 50, size=(40, 70)).astype(dtype)
    rowidx = rng.permutation(40)[:rows]
    colidx = rng.permutation(64)[:cols]
    ps, pd = dev(src), dev(dst0)
    pri, pci = dev((rowidx * 70 * esz).astype(np.uint64)), dev((colidx * esz).astype(np.uint64))
    a1, a2 = L.IArrayStridx(), L.IArrayStridx()
    a1.ptr = pd + 69 * esz
    a1.stridx[0] = pri
    a1.stridx[1] = stride_sdx(-2 * esz)
    a2.ptr = ps
    a2.stridx[0] = stride_sdx(64 * esz)
    a2.stridx[1] = pci
    ix = indexer((rows, cols))
    f = L.fn("cumo_iter_%s_store_%s_stridx_kernel_launch" % (tname, tname), None, [P(L.IArrayStridx), P(L.IArrayStridx), P(L.Indexer)])
    L.call(f, C.byref(a1), C.byref(a2), C.byref(ix))
    want = dst0.copy()
    want[rowidx[:, None], 69 - 2 * np.arange(cols)[None, :]] = src[:, colidx]
    got = fetch(pd, dst0.size, dtype).reshape(dst0.shape)
    assert (got.view(np.uint8) == want.view(np.uint8)).all()
    free(ps, pd, pri, pci)
    # store_array: a staged host array into a strided / indexed run, or one value
    n = 3000
    z = rng.integers(-9, 9, size=n).astype(dtype)
    base = rng.integers(-9, 9, size=4 * n).astype(dtype)
    idx = (rng.permutation(4 * n)[:n] * esz).astype(np.uint64)
    pz, pidx = dev(z), dev(idx)
    for name, sig, args, apply in (
            ("stride", [VP, SSZ, VP, U64], lambda pb: (pb + 5 * esz, 3 * esz, pz, n), lambda w: w.__setitem__(5 + 3 * np.arange(n), z)),
            ("index", [VP, VP, VP, U64], lambda pb: (pb, pidx, pz, n), lambda w: w.__setitem__((idx // esz).astype(np.int64), z)),
            ("stride_scalar", [VP, SSZ, ctype, U64], lambda pb: (pb + (4 * n - 1) * esz, -esz, ctype(7), n), lambda w: w.__setitem__(4 * n - 1 - np.arange(n), 7)),
            ("index_scalar", [VP, VP, ctype, U64], lambda pb: (pb, pidx, ctype(-3), n), lambda w: w.__setitem__((idx // esz).astype(np.int64), -3))):
        g = L.fn("cumo_iter_%s_store_array_%s_kernel_launch" % (tname, name), None, sig)
        pb = dev(base)
        L.call(g, *args(pb))
        want = base.copy()
        apply(want)
        assert (fetch(pb, base.size, dtype).view(np.uint8) == want.view(np.uint8)).all(), name
        free(pb)
    free(pz, pidx)


@pytest.mark.parametrize("n", [1, 5, 31, 32, 33, 64, 95, 1000, 100003, (1 << 21) + 19])
def test_bit_store_bit_contiguous(n):
    # tmpl_bit/store_bit.c:2 / store_bit_kernel.cu:38-47: word pointers + bit offsets below 32,
    # only the n named bits of the receiver change
    L = lib()
    f = L.fn("cumo_iter_bit_store_bit_contiguous_kernel_launch", None, [VP, SZ, VP, SZ, U64])
    rng = np.random.default_rng(n)
    for p1, p3 in ((0, 0), (0, 13), (13, 0), (7, 7), (31, 1), (1, 31), (19, 30)):
        src = rng.integers(0, 2, size=p1 + n + 70).astype(np.uint8)
        before = rng.integers(0, 2, size=p3 + n + 70).astype(np.uint8)
        pa, pz = dev(pack(src)), dev(pack(before))
        L.call(f, pa, p1, pz, p3, n)
        want = before.copy()
        want[p3:p3 + n] = src[p1:p1 + n]
        got = unpack(fetch(pz, (before.size + 31) // 32, np.uint32), before.size)
        assert (got == want).all(), (n, p1, p3, np.flatnonzero(got != want)[:8])
        free(pa, pz)


def test_bit_store_bit_general_views():
    # tmpl_bit/store_bit.c:1 / store_bit_kernel.cu:1-19: both operands through their own
    # stride-or-index entries: reversed, stepped, 2-d with a column index array, broadcast source
    L = lib()
    g = L.fn("cumo_iter_bit_store_bit_kernel_launch", None, [P(L.BitIArrayStridx), P(L.BitIArrayStridx), P(L.Indexer)])
    rng = np.random.default_rng(11)

    def run(shape, spos, ssteps, dpos, dsteps, nsrc, ndst, sidx=None, didx=None):
        src = rng.integers(0, 2, size=nsrc).astype(np.uint8)
        before = rng.integers(0, 2, size=ndst).astype(np.uint8)
        pa, pz = dev(pack(src)), dev(pack(before))
        a1, a3 = L.BitIArrayStridx(), L.BitIArrayStridx()
        a1.ptr, a1.pos, a3.ptr, a3.pos = pa, spos, pz, dpos
        held = []
        for d in range(len(shape)):
            for a, steps, idx in ((a1, ssteps, sidx), (a3, dsteps, didx)):
                if idx is not None and idx[0] == d:
                    p = dev(idx[1].astype(np.uint64))
                    held.append(p)
                    a.stridx[d] = p
                else:
                    a.stridx[d] = stride_sdx(steps[d])
        ix = indexer(shape)
        L.call(g, C.byref(a1), C.byref(a3), C.byref(ix))
        want = before.copy()
        for pos in np.ndindex(*shape):
            so, do = spos, dpos
            for d, i in enumerate(pos):
                so += int(sidx[1][i]) if sidx is not None and sidx[0] == d else ssteps[d] * i
                do += int(didx[1][i]) if didx is not None and didx[0] == d else dsteps[d] * i
            want[do] = src[so]
        got = unpack(fetch(pz, (ndst + 31) // 32, np.uint32), ndst)
        assert (got == want).all(), (shape, spos, ssteps, dpos, dsteps, np.flatnonzero(got != want)[:8])
        free(pa, pz, *held)

    for n in (1, 33, 64, 65, 777):
        run((n,), 3, (1,), 5 + n - 1, (-1,), n + 10, n + 10)               # receiver reversed
        run((n,), 2 * n + 1, (-2,), 9, (3,), 2 * n + 5, 3 * n + 12)         # source reversed with step 2, receiver step 3
        run((n,), 17, (0,), 1, (1,), 40, n + 40)                            # one source bit broadcast
    run((37, 45), 4, (100, 2), 11, (45, 1), 37 * 100 + 20, 37 * 45 + 30)    # 2-d, rows of the receiver end to end at offset 11
    run((6, 41), 7, (200, 0), 3, (300, 0), 7 + 6 * 200, 3 + 6 * 300,        # index arrays along the columns of both
        sidx=(1, (np.arange(41) * 4 + 1) % 190), didx=(1, (np.arange(41) * 7 + 2)))
    run((3, 4, 5, 6, 7), 0, (840, 210, 42, 7, 1), 6, (900, 215, 43, 7, 1), 2520, 2800)   # 5-d (past the unrolled cases)


def test_bit_store_bit_empty():
    L = lib()
    f = L.fn("cumo_iter_bit_store_bit_contiguous_kernel_launch", None, [VP, SZ, VP, SZ, U64])
    g = L.fn("cumo_iter_bit_store_bit_kernel_launch", None, [P(L.BitIArrayStridx), P(L.BitIArrayStridx), P(L.Indexer)])
    before = np.array([0xdeadbeef, 0x01234567], dtype=np.uint32)
    pa, pz = dev(before), dev(before)
    L.call(f, pa, 3, pz, 5, 0)
    a1, a3 = L.BitIArrayStridx(), L.BitIArrayStridx()
    a1.ptr, a3.ptr = pa, pz
    a1.stridx[0] = a3.stridx[0] = stride_sdx(1)
    ix = indexer((0,))
    L.call(g, C.byref(a1), C.byref(a3), C.byref(ix))
    assert (fetch(pz, 2, np.uint32) == before).all()
    free(pa, pz)


# ---- the reference's own cases, through the mirror ---------------------------------------------
def test_reversed_bit_views_all_any_and_store():
    # test/narray_test.rb:2725-2746
    import cumo_amd
    for n in (8, 32, 33, 64, 65, 200):
        xs = np.array([1 if i % 3 == 0 else 0 for i in range(n)], dtype=np.uint8)
        a = cumo_amd.Bit.cast(xs)
        rev = a[::-1]
        assert rev.to_numpy().tolist() == xs[::-1].tolist()
        assert rev.all_p() is False and rev.any_p() is True
        dst = cumo_amd.Bit.zeros(n)
        dst[::-1].store(a)
        assert dst.to_numpy().tolist() == xs[::-1].tolist()


def test_bit_reduction_along_an_axis_of_a_reversed_view():
    # test/narray_test.rb:2748-2759
    import cumo_amd
    rows, cols = 7, 33
    xs = np.array([1 if i % 3 == 0 else 0 for i in range(rows * cols)], dtype=np.uint8)
    a = cumo_amd.Bit.cast(xs).reshape(rows, cols)
    rev = a[:, ::-1]
    grid = xs.reshape(rows, cols)[:, ::-1]
    assert rev.all_p(axis=1).to_numpy().tolist() == grid.all(axis=1).astype(int).tolist()
    assert rev.any_p(axis=0).to_numpy().tolist() == grid.any(axis=0).astype(int).tolist()


def test_bit_reductions_over_long_arrays_and_views():
    # test/narray_test.rb:2761-2790 (the indexed view of the reference is covered by the raw launcher test above)
    import cumo_amd
    n = 20000
    views = (("flat", slice(None)), ("offset 13", slice(13, n)), ("offset 32", slice(32, n)), ("step 2", slice(0, n, 2)))
    for zero_at in (None, 0, n // 2, n - 1):
        xs = np.ones(n, dtype=np.uint8)
        if zero_at is not None:
            xs[zero_at] = 0
        a = cumo_amd.Bit.cast(xs)
        b = ~a
        for label, sl in views:
            want_all = bool(xs[sl].all())
            assert a[sl].all_p() is want_all, (label, zero_at)
            assert b[sl].any_p() is (not want_all), (label, zero_at)
            assert b[sl].none_p() is want_all, (label, zero_at)


def test_bit_reductions_along_an_axis():
    # test/narray_test.rb:2792-2815
    import cumo_amd
    rows, cols = 6, 20000
    xs = np.array([0 if i % 20001 == 0 else 1 for i in range(rows * cols)], dtype=np.uint8)
    a = cumo_amd.Bit.cast(xs).reshape(rows, cols)
    grid = xs.reshape(rows, cols)
    assert a.all_p(axis=1).to_numpy().tolist() == grid.all(axis=1).astype(int).tolist()
    assert a.any_p(axis=1).to_numpy().tolist() == grid.any(axis=1).astype(int).tolist()
    assert a.all_p(axis=0).to_numpy().tolist() == grid.all(axis=0).astype(int).tolist()
    k = a.all_p(axis=1, keepdims=True)
    assert k.shape == (rows, 1) and k.to_numpy().reshape(-1).tolist() == grid.all(axis=1).astype(int).tolist()
    v = a[:, ::2]
    want = grid[:, ::2]
    assert v.all_p(axis=1).to_numpy().tolist() == want.all(axis=1).astype(int).tolist()
    assert (~v).all_p(axis=1).to_numpy().tolist() == (~want.astype(bool)).all(axis=1).astype(int).tolist()
    # many short runs take the count form (one launch whatever the shape)
    m = np.random.default_rng(3).integers(0, 2, size=(300, 40)).astype(np.uint8)
    m[::7] = 1
    m[3::11] = 0
    bm = cumo_amd.Bit.cast(m)
    assert bm.all_p(axis=1).to_numpy().tolist() == m.all(axis=1).astype(int).tolist()
    assert bm.any_p(axis=1).to_numpy().tolist() == m.any(axis=1).astype(int).tolist()
    assert bm.none_p(axis=1).to_numpy().tolist() == (~m.any(axis=1)).astype(int).tolist()


def test_bit_cast_from_device_arrays_fill_and_empty():
    import cumo_amd
    rng = np.random.default_rng(9)
    for cls, dtype in ((cumo_amd.SFloat, np.float32), (cumo_amd.DFloat, np.float64), (cumo_amd.Int32, np.int32)):
        h = rng.integers(-1, 2, size=(37, 53)).astype(dtype)
        d = cls.cast(h)
        assert (cumo_amd.Bit.cast(d).to_numpy() == (h != 0)).all()
        assert (cumo_amd.Bit.cast(d[::2, ::-3]).to_numpy() == (h[::2, ::-3] != 0)).all()
        assert (cumo_amd.Bit.cast(d.transpose()).to_numpy() == (h.T != 0)).all()
    b = cumo_amd.Bit.zeros(5, 70)
    b.fill(1)
    assert b.to_numpy().all()
    b[1:4, 3:67:2].fill(0)
    want = np.ones((5, 70), dtype=np.uint8)
    want[1:4, 3:67:2] = 0
    assert (b.to_numpy() == want).all()
    b[:, 64:].fill(False)
    want[:, 64:] = 0
    assert (b.to_numpy() == want).all()
    with pytest.raises(ValueError):
        b.fill(2)
    # an empty array answers false to all three (tmpl_bit/bit_reduce.c:132-134, none_p.c)
    e = cumo_amd.Bit.zeros(0)
    assert e.all_p() is False and e.any_p() is False
