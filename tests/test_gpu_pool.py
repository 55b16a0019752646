"""The memory pool over real device memory (the host-heap tests cover the
bookkeeping): blocks come from hipMalloc, are reused without a device call,
reuse is ordered by the stream, and the out-of-memory path raises what the
reference raises (ext/cumo/cuda/memory_pool.cpp:64-96,
test/cuda/memory_pool_test.rb:16-72)."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def clean_pool():
    import cumo_amd
    cumo_amd.synchronize()
    cumo_amd.MemoryPool.free_all_blocks()
    yield
    from cumo_amd import _lib
    _lib.lib.cumo_hip_pool_set_limit(0)
    cumo_amd.MemoryPool.free_all_blocks()


def test_reuse_without_device_call_and_counters():
    import cumo_amd
    from cumo_amd import _lib
    L = _lib.lib
    base_used = L.cumo_hip_pool_used_bytes()
    a = cumo_amd.SFloat.new(1000)                 # 4000 bytes -> 4096
    assert L.cumo_hip_pool_used_bytes() - base_used == 4096
    p = a._buf.ptr
    calls = L.cumo_hip_pool_device_malloc_calls()
    del a
    assert L.cumo_hip_pool_used_bytes() == base_used and L.cumo_hip_pool_free_bytes() >= 4096
    b = cumo_amd.SFloat.new(1024)
    assert b._buf.ptr == p and L.cumo_hip_pool_device_malloc_calls() == calls
    del b
    cumo_amd.MemoryPool.free_all_blocks()
    assert L.cumo_hip_pool_total_bytes() == base_used


def test_stream_ordered_reuse_keeps_results_right():
    import cumo_amd
    n = 1 << 22
    x = cumo_amd.SFloat.cast(np.arange(n, dtype=np.float32))
    ptrs = set()
    for k in range(20):
        t = x + float(k)          # result block
        u = t * 2.0               # second block; t is released right after the launch that reads it
        ptrs.add(t._buf.ptr)
        del t
        got = u.to_numpy()
        assert got[12345] == np.float32((12345 + k) * 2.0) and got[-1] == np.float32((n - 1 + k) * 2.0)
        del u
    assert len(ptrs) <= 2, "blocks are expected to be reused"


def test_out_of_memory_raises_like_the_reference():
    import cumo_amd
    from cumo_amd import _lib
    L = _lib.lib
    L.cumo_hip_pool_set_limit(L.cumo_hip_pool_total_bytes() + (1 << 20))
    with pytest.raises(cumo_amd.OutOfMemoryError) as ei:
        cumo_amd.SFloat.new(1 << 20)              # 4 MiB over a 1 MiB allowance
    assert "out of memory to allocate 4194304 bytes" in str(ei.value)
    small = cumo_amd.SFloat.new(1 << 10)          # still serviceable
    assert small._buf.ptr
    # the failure inside a launch-layer call leaves nothing allocated behind
    used = L.cumo_hip_pool_used_bytes()
    x = cumo_amd.SFloat.new(1 << 17)              # 512 KiB fits
    with pytest.raises(cumo_amd.OutOfMemoryError):
        x + x + x                                  # needs two more 512 KiB blocks at once; the allowance holds one
    del x
    assert L.cumo_hip_pool_used_bytes() == used


def test_pool_disabled_goes_straight_to_the_device():
    import cumo_amd
    from cumo_amd import _lib
    L = _lib.lib
    assert cumo_amd.MemoryPool.enabled()
    cumo_amd.MemoryPool.disable()
    try:
        total = L.cumo_hip_pool_total_bytes()
        a = cumo_amd.DFloat.cast(np.ones(1000))
        assert L.cumo_hip_pool_total_bytes() == total
        assert float((a + a).sum()) == 2000.0
        del a
    finally:
        cumo_amd.MemoryPool.enable()


def test_two_streams_share_the_pool_without_mixing_results():
    """Work alternates between the null stream and a stream of the library's own making; arrays
    released on one stream are taken over by allocations on the other (whole blocks change
    stream behind an event). Every result must be what the same operations give on one stream."""
    import cumo_amd
    from cumo_amd import _lib
    L = _lib.lib
    rng = np.random.default_rng(77)
    n = 1 << 20
    hx = rng.standard_normal(n).astype(np.float32)
    x = cumo_amd.SFloat.cast(hx)
    own = L.cumo_hip_stream_create()
    assert own
    try:
        want = hx
        got = x
        for it in range(12):
            L.cumo_hip_set_stream(own if it % 2 == 0 else None)
            if it:
                # what the other stream produced must be complete before this stream reads it
                L.cumo_hip_set_stream(None if it % 2 == 0 else own)
                cumo_amd.synchronize()
                L.cumo_hip_set_stream(own if it % 2 == 0 else None)
            tmp = got * 1.5            # a temporary that is released at once, on this stream
            got = tmp + float(it)
            del tmp
            want = want * np.float32(1.5) + np.float32(it)
            cumo_amd.MemoryPool.free_all_blocks() if it == 5 else None
        cumo_amd.synchronize()
        L.cumo_hip_set_stream(None)
        assert (got.to_numpy().view(np.uint32) == want.view(np.uint32)).all()
    finally:
        L.cumo_hip_set_stream(None)
        L.cumo_hip_synchronize()
        L.cumo_hip_stream_destroy(own)
    _lib.check()


def test_look_back_words_of_scans_are_counted_and_given_back():
    """One-pass scans keep a region of words per stream outside the pool's books. It shows in
    cumo_hip_pool_held_outside_bytes, goes back to the driver with free_all_blocks and when
    the stream is released, and later scans on the stream still give the right answer."""
    import cumo_amd
    from cumo_amd import _lib
    L = _lib.lib
    held = _lib.fn("cumo_hip_pool_held_outside_bytes", C.c_size_t, [])
    release = _lib.fn("cumo_hip_stream_release", None, [C.c_void_p])
    assert held() == 0                      # (the fixture has just called free_all_blocks)
    n = (1 << 22) + 5
    hx = np.random.default_rng(5).integers(-3, 4, n).astype(np.float32)
    want = np.cumsum(hx.astype(np.float64)).astype(np.float32)   # small integers: exact in any order
    x = cumo_amd.SFloat.cast(hx)
    assert (x.cumsum().to_numpy() == want).all()
    on_null = held()
    assert on_null > 0
    own = L.cumo_hip_stream_create()
    assert own
    try:
        cumo_amd.synchronize()
        L.cumo_hip_set_stream(own)
        assert (x.cumsum().to_numpy() == want).all()
        assert held() > on_null             # a second region, for the second stream
        cumo_amd.synchronize()
        release(own)                        # the caller keeps the stream, the library forgets it
        assert held() == on_null
        assert (x.cumsum().to_numpy() == want).all()   # the stream is taken up again from nothing
        assert held() > on_null
        cumo_amd.synchronize()
    finally:
        L.cumo_hip_set_stream(None)
        L.cumo_hip_stream_destroy(own)
    assert held() == on_null
    cumo_amd.MemoryPool.free_all_blocks()
    assert held() == 0
    assert (x.cumsum().to_numpy() == want).all()
    _lib.check()
