"""Memory pool logic on the host heap (no GPU): the assertions follow the
reference's own pool harness, ext/cumo/cuda/memory_pool_impl_test.cpp:29-835
(rounding, best fit, split, merge, free_all_blocks, counters, out of memory,
huge sizes, threads)."""
import ctypes as C
import threading

import pytest

from cumo_amd import _lib

L = _lib.lib
ROUND = 512


@pytest.fixture(autouse=True)
def host_pool():
    L.cumo_hip_pool_free_all_blocks()
    assert L.cumo_hip_pool_total_bytes() == 0, "another test left allocations behind"
    assert L.cumo_hip_pool_use_host_backend(1) == 0
    L.cumo_hip_pool_set_limit(0)
    yield
    L.cumo_hip_pool_free_all_blocks()
    L.cumo_hip_pool_set_limit(0)
    assert L.cumo_hip_pool_total_bytes() == 0
    assert L.cumo_hip_pool_use_host_backend(0) == 0


def malloc(n, stream=None):
    p = C.c_void_p()
    rc = L.cumo_hip_pool_malloc(n, stream, C.byref(p))
    return rc, p.value


def test_rounding_and_counters():
    rc, p = malloc(1)
    assert rc == 0 and p
    assert L.cumo_hip_pool_used_bytes() == ROUND
    assert L.cumo_hip_pool_free_bytes() == 0
    rc, q = malloc(ROUND + 1)
    assert L.cumo_hip_pool_used_bytes() == 3 * ROUND
    assert L.cumo_hip_pool_free(p) == 0
    assert (L.cumo_hip_pool_used_bytes(), L.cumo_hip_pool_free_bytes(), L.cumo_hip_pool_total_bytes()) == (2 * ROUND, ROUND, 3 * ROUND)
    assert L.cumo_hip_pool_n_free_blocks() == 1
    assert L.cumo_hip_pool_free(q) == 0
    assert L.cumo_hip_pool_n_free_blocks() == 2
    assert L.cumo_hip_pool_used_bytes() == 0


def test_zero_size_and_unknown_pointer():
    rc, p = malloc(0)
    assert rc == 0 and p is None
    assert L.cumo_hip_pool_free(None) == 0
    assert L.cumo_hip_pool_free(C.c_void_p(12345 * 512)) == 3  # not ours: nothing freed


def test_reuse_same_size_without_device_call():
    rc, p = malloc(4 * ROUND)
    calls = L.cumo_hip_pool_device_malloc_calls()
    L.cumo_hip_pool_free(p)
    rc, q = malloc(4 * ROUND)
    assert q == p
    assert L.cumo_hip_pool_device_malloc_calls() == calls
    L.cumo_hip_pool_free(q)


def test_best_fit_split_and_merge():
    rc, big = malloc(8 * ROUND)
    L.cumo_hip_pool_free(big)
    rc, a = malloc(2 * ROUND)          # split off the head
    assert a == big
    assert L.cumo_hip_pool_free_bytes() == 6 * ROUND and L.cumo_hip_pool_n_free_blocks() == 1
    rc, b = malloc(3 * ROUND)          # split the remainder again
    assert b == big + 2 * ROUND
    rc, c = malloc(3 * ROUND)          # exact fit of what is left
    assert c == big + 5 * ROUND
    assert L.cumo_hip_pool_free_bytes() == 0
    # free the middle, then the head: they merge; then the tail: one block again
    L.cumo_hip_pool_free(b)
    L.cumo_hip_pool_free(a)
    assert L.cumo_hip_pool_n_free_blocks() == 1 and L.cumo_hip_pool_free_bytes() == 5 * ROUND
    L.cumo_hip_pool_free(c)
    assert L.cumo_hip_pool_n_free_blocks() == 1 and L.cumo_hip_pool_free_bytes() == 8 * ROUND
    rc, again = malloc(8 * ROUND)
    assert again == big
    L.cumo_hip_pool_free(again)


def test_best_fit_takes_the_smallest_that_fits():
    rc, a = malloc(10 * ROUND)
    rc, b = malloc(4 * ROUND)
    rc, c = malloc(6 * ROUND)
    for p in (a, b, c):
        L.cumo_hip_pool_free(p)
    rc, x = malloc(5 * ROUND)
    assert x == c                      # 6 is the smallest block >= 5
    rc, y = malloc(4 * ROUND)
    assert y == b
    L.cumo_hip_pool_free(x)
    L.cumo_hip_pool_free(y)


def test_free_all_blocks_keeps_split_chunks():
    rc, big = malloc(8 * ROUND)
    rc, other = malloc(2 * ROUND)
    L.cumo_hip_pool_free(big)
    L.cumo_hip_pool_free(other)
    rc, head = malloc(3 * ROUND)       # big is split now: head in use, 5 free
    assert head == big
    L.cumo_hip_pool_free_all_blocks()  # only `other` is a whole free block
    assert L.cumo_hip_pool_free_bytes() == 5 * ROUND
    assert L.cumo_hip_pool_n_free_blocks() == 1
    L.cumo_hip_pool_free(head)
    L.cumo_hip_pool_free_all_blocks()
    assert L.cumo_hip_pool_total_bytes() == 0


def test_streams_have_their_own_arenas():
    s1, s2 = C.c_void_p(0x10), C.c_void_p(0x20)
    rc, a = malloc(4 * ROUND, s1)
    L.cumo_hip_pool_free(a)
    rc, b = malloc(4 * ROUND, s1)      # same stream: immediate reuse
    assert b == a
    L.cumo_hip_pool_free(b)
    L.cumo_hip_pool_free_all_blocks_stream(s2)   # nothing of s2 to free
    assert L.cumo_hip_pool_free_bytes() == 4 * ROUND
    calls = L.cumo_hip_pool_device_malloc_calls()
    rc, c = malloc(2 * ROUND, s2)      # another stream takes the whole block over rather than going to the device
    assert c == a and L.cumo_hip_pool_device_malloc_calls() == calls
    L.cumo_hip_pool_free(c)
    L.cumo_hip_pool_free_all_blocks_stream(s1)
    assert L.cumo_hip_pool_free_bytes() == 4 * ROUND  # it lives in s2's arena now, merged back
    L.cumo_hip_pool_free_all_blocks_stream(s2)
    assert L.cumo_hip_pool_total_bytes() == 0


def test_out_of_memory_frees_cached_blocks_then_reports():
    L.cumo_hip_pool_set_limit(16 * ROUND)
    rc, a = malloc(10 * ROUND)
    L.cumo_hip_pool_free(a)
    rc, b = malloc(12 * ROUND)         # does not fit beside the cached 10: the cache is released first
    assert rc == 0
    assert L.cumo_hip_pool_total_bytes() == 12 * ROUND
    rc, c = malloc(8 * ROUND)
    assert rc == 2 and c is None       # CUMO_HIP_ERROR_OUT_OF_MEMORY
    L.cumo_hip_pool_free(b)
    # a size that cannot be rounded without wrapping is out of memory, not a tiny chunk
    rc, d = malloc(2 ** 64 - 1)
    assert rc == 2 and d is None
    rc, e = malloc(2 ** 62)
    assert rc == 2 and e is None


def test_threads():
    errors = []

    def worker(seed):
        import random
        rnd = random.Random(seed)
        held = []
        for _ in range(400):
            if held and rnd.random() < 0.5:
                if L.cumo_hip_pool_free(held.pop(rnd.randrange(len(held)))) != 0:
                    errors.append("free failed")
            else:
                rc, p = malloc(rnd.randrange(1, 20) * ROUND)
                if rc != 0 or not p:
                    errors.append("malloc failed")
                else:
                    held.append(p)
        for p in held:
            L.cumo_hip_pool_free(p)

    ts = [threading.Thread(target=worker, args=(i,)) for i in range(8)]
    for t in ts:
        t.start()
    for t in ts:
        t.join()
    assert not errors
    assert L.cumo_hip_pool_used_bytes() == 0
    # everything merged back: every free block is a whole device allocation
    n = L.cumo_hip_pool_n_free_blocks()
    L.cumo_hip_pool_free_all_blocks()
    assert L.cumo_hip_pool_total_bytes() == 0, n


def test_large_allocations_are_cut_on_two_mebibyte_boundaries(host_pool):
    """An array of 2 MiB or more taken out of a larger free chunk starts on a 2 MiB
    boundary; what lies before it stays free and everything merges back."""
    MIB = 1 << 20
    rc, block = malloc(9 * MIB + ROUND)   # the host heap gives no particular alignment
    assert rc == 0
    L.cumo_hip_pool_free(block)
    assert L.cumo_hip_pool_n_free_blocks() == 1
    rc, a = malloc(4 * MIB)
    assert rc == 0 and a % (2 * MIB) == 0
    assert block <= a < block + 2 * MIB
    rc, b = malloc(2 * MIB)
    assert rc == 0 and b % (2 * MIB) == 0 and b == a + 4 * MIB
    rc, small = malloc(ROUND)                 # small requests keep taking the best fit as it lies
    assert rc == 0
    for q in (a, b, small):
        assert L.cumo_hip_pool_free(q) == 0
    assert L.cumo_hip_pool_n_free_blocks() == 1 and L.cumo_hip_pool_used_bytes() == 0
    assert L.cumo_hip_pool_free_bytes() == 9 * MIB + ROUND
    rc, again = malloc(9 * MIB + ROUND)       # the whole block again, from its start
    assert rc == 0 and again == block
    L.cumo_hip_pool_free(again)
