"""Host read-back and ingest: the staged transfers and the array methods over them
(to_binary / from_binary / store_binary / aref_cpu / extract_cpu, to_numpy / cast).
Bytes in, bytes out: every check is bit-exact. The literal cases follow
test/narray_test.rb (to_binary / from_binary / store_binary) of the reference."""
import ctypes as C

import numpy as np
import pytest

from helpers import assert_bits_equal

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n", [0, 1, 3, 4095, 4096, 1 << 20, (8 << 20) - 1, 8 << 20, (8 << 20) + 1, (40 << 20) + 12345, 100 << 20])
def test_staged_copies_round_trip(n):
    """Sizes around the staging buffer (8 MiB), beyond the ring (4 buffers) and odd tails."""
    from cumo_amd import _lib
    rng = np.random.default_rng(n & 0xffff)
    src = rng.integers(0, 256, n, dtype=np.uint8)
    p = _lib.call(_lib.lib.cumo_cuda_runtime_malloc, max(n, 1))
    assert _lib.call(_lib.lib.cumo_hip_copy_from_host, p, src.ctypes.data, n) == 0
    back = np.zeros(n, dtype=np.uint8)
    assert _lib.call(_lib.lib.cumo_hip_copy_to_host, back.ctypes.data, p, n) == 0
    assert (back == src).all()
    if n > 100:
        # a device offset and a host offset that are not aligned to anything
        part = np.zeros(n - 50, dtype=np.uint8)
        assert _lib.call(_lib.lib.cumo_hip_copy_to_host, part.ctypes.data + 3, p + 7, n - 57) == 0
        assert (part[3:n - 54] == src[7:n - 50]).all() and not part[:3].any() and not part[n - 54:].any()
    _lib.lib.cumo_cuda_runtime_free(p)


def test_copies_are_ordered_after_queued_kernels():
    import cumo_amd
    rng = np.random.default_rng(1)
    h = rng.standard_normal(1 << 24).astype(np.float32)
    x = cumo_amd.SFloat.cast(h)
    y = x
    for _ in range(20):
        y = y + 1.0
    want = h.copy()
    for _ in range(20):
        want = want + np.float32(1.0)
    assert_bits_equal(y.to_numpy(), want)
    # ingest into memory a kernel has just read, then compute on it again
    x.store_binary((h * 2).tobytes())
    assert_bits_equal((x + 0.0).to_numpy(), h * 2 + np.float32(0.0))


@pytest.mark.parametrize("cls_name,dtype", [("SFloat", np.float32), ("DFloat", np.float64), ("Int32", np.int32)])
def test_binary_strings_and_views(cls_name, dtype):
    import cumo_amd
    cls = getattr(cumo_amd, cls_name)
    src = np.array([[1, 2, 3], [5, 7, 11]], dtype=dtype)
    a = cls.cast(src)
    assert a.to_binary() == src.tobytes()
    assert a.byte_size() == src.nbytes
    assert cls.from_binary(src.tobytes()).to_a() == [1, 2, 3, 5, 7, 11]
    assert cls.from_binary(src.tobytes(), [3, 2]).to_a() == [[1, 2], [3, 5], [7, 11]]
    assert cls.from_binary(src.tobytes() + b"xx", 4).to_a() == [1, 2, 3, 5]
    with pytest.raises(ValueError):
        cls.from_binary(src.tobytes(), [4, 2])
    with pytest.raises(ValueError):
        cls.from_binary(b"")
    # views: transposed, strided, reversed, a single row
    assert a.transpose().to_binary() == np.ascontiguousarray(src.T).tobytes()
    assert a[:, ::2].to_binary() == np.ascontiguousarray(src[:, ::2]).tobytes()
    assert a.reverse().to_binary() == np.ascontiguousarray(src[::-1, ::-1]).tobytes()
    assert a[1].to_binary() == src[1].tobytes()
    # store_binary: whole array, with an offset, into a view, too short
    b = cls.zeros(2, 3)
    assert b.store_binary(b"\0" * 5 + src.tobytes(), 5) == src.nbytes
    assert_bits_equal(b.to_numpy(), src)
    t = cls.zeros(3, 2)
    t.transpose().store_binary(src.tobytes())
    assert_bits_equal(t.to_numpy(), np.ascontiguousarray(src.T))
    with pytest.raises(ValueError):
        b.store_binary(src.tobytes()[:-1])
    with pytest.raises(ValueError):
        b.store_binary(src.tobytes(), 200)
    # single elements
    assert a.aref_cpu(1, 2) == 11 and a.aref_cpu(-1, -3) == 5
    assert a.transpose().aref_cpu(2, 0) == 3
    assert a[1, 1].extract_cpu() == 7
    assert a.sum().extract_cpu() == 29
    with pytest.raises(IndexError):
        a.aref_cpu(2, 0)
    rng = np.random.default_rng(8)
    big = rng.integers(-1000, 1000, (3000, 1500)).astype(dtype)
    d = cls.cast(big)
    assert_bits_equal(d.to_numpy(), big)
    assert_bits_equal(d.transpose()[::3, 5:].to_numpy(), big.T[::3, 5:])
    assert d[::7].to_binary() == np.ascontiguousarray(big[::7]).tobytes()


def test_bit_arrays_cross_packed():
    import cumo_amd
    rng = np.random.default_rng(4)
    for shape in ((5,), (8,), (3, 11), (64, 64), (1000, 37)):
        h = rng.integers(0, 2, shape).astype(np.uint8)
        b = cumo_amd.Bit.cast(h)
        assert_bits_equal(b.to_numpy(), h)
        packed = np.packbits(h.reshape(-1), bitorder="little").tobytes()
        got = b.to_binary()
        assert len(got) == len(packed)
        mask_last = (1 << (h.size % 8)) - 1 if h.size % 8 else 0xff
        assert got[:-1] == packed[:-1] and (got[-1] & mask_last) == packed[-1]
        assert b.byte_size() == (h.size + 7) // 8
        c = cumo_amd.Bit.from_binary(packed, list(shape))
        assert_bits_equal(c.to_numpy(), h)
        if len(shape) == 2:
            assert_bits_equal(b.transpose().to_numpy(), h.T)
            assert_bits_equal(b[1:, 3:].to_numpy(), h[1:, 3:])
            z = cumo_amd.Bit.cast(np.zeros(shape, dtype=np.uint8))
            sub = h[1:, 3:]
            z[1:, 3:].store_binary(np.packbits(sub.reshape(-1), bitorder="little").tobytes())
            want = np.zeros(shape, dtype=np.uint8)
            want[1:, 3:] = sub
            assert_bits_equal(z.to_numpy(), want)
            assert b.aref_cpu(2, 5) == int(h[2, 5]) and b.aref_cpu(-1, -1) == int(h[-1, -1])


def test_reference_cases_zero_dimensional_and_bit_views_with_an_offset():
    import struct
    import cumo_amd
    # narray_alt_coverage_test.rb:751-758
    a = cumo_amd.DFloat.cast(3.5)
    packed = struct.pack("d", 3.5)
    assert a.to_binary() == packed
    assert a.transpose().to_binary() == packed
    assert a.reshape(1).to_binary() == packed
    # narray_alt_coverage_test.rb:784-794
    bits = [1 if (i * 7 % 5) == 0 else 0 for i in range(200)]
    b = cumo_amd.Bit.cast(np.array(bits, dtype=np.uint8))
    for i in (0, 1, 3, 8, 11, 16, 63, 64, 65, 100):
        v = b[i:i + 21]
        assert v.to_a() == bits[i:i + 21]
        unpacked = np.unpackbits(np.frombuffer(v.to_binary(), dtype=np.uint8), bitorder="little")[:21].tolist()
        assert unpacked == bits[i:i + 21]
    # narray_test.rb:1082-1150: round trips through a string, the string left as it was
    rng = np.random.default_rng(6)
    for cls, dt in ((cumo_amd.SFloat, np.float32), (cumo_amd.DFloat, np.float64), (cumo_amd.Int32, np.int32)):
        h = rng.integers(0, 10, (2, 5)).astype(dt)
        x = cls.cast(h)
        data = x.to_binary()
        keep = bytes(data)
        r = cls.from_binary(data, [2, 5])
        assert_bits_equal(r.to_numpy(), h)
        r[0, 0] = r[0, 0] + 1
        assert r.aref_cpu(0, 0) == h[0, 0] + 1 and data == keep
        s = cls.zeros(2, 5)
        assert s.store_binary(b"ab" + data, 2) == h.nbytes
        assert_bits_equal(s.to_numpy(), h)
