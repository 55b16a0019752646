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


# ---- the rest of the reference's harness (memory_pool_impl_test.cpp:404-835) -----------------
def test_malloc_with_zero_takes_no_cached_chunk():
    # TestMallocWithZero (:413-423)
    rc, p1 = malloc(4 * ROUND)
    L.cumo_hip_pool_free(p1)
    rc, z = malloc(0)
    assert rc == 0 and z is None
    assert L.cumo_hip_pool_used_bytes() == 0 and L.cumo_hip_pool_free_bytes() == 4 * ROUND
    rc, again = malloc(4 * ROUND)
    assert again == p1
    L.cumo_hip_pool_free(again)


def test_malloc_with_huge_size_is_refused_not_wrapped():
    # TestMallocWithHugeSize (:425-437): sizes that cannot be rounded up without wrapping
    rc, p1 = malloc(4 * ROUND)
    L.cumo_hip_pool_free(p1)
    size_max = (1 << 64) - 1
    for n in (size_max, size_max - 1, size_max - (ROUND - 2)):
        rc, p = malloc(n)
        assert rc == 2 and p is None, n          # OutOfMemoryError
    assert L.cumo_hip_pool_used_bytes() == 0 and L.cumo_hip_pool_free_bytes() == 4 * ROUND
    rc, again = malloc(4 * ROUND)
    assert again == p1
    L.cumo_hip_pool_free(again)


def test_free_reports_ownership_and_double_free():
    # TestFreeDoubly, TestFreeReportsOwnership (:455-486)
    rc, p = malloc(4 * ROUND)
    assert L.cumo_hip_pool_free(p) == 0
    assert L.cumo_hip_pool_free(p) == 3          # already returned: not owned any more, nothing corrupted
    assert L.cumo_hip_pool_free(None) == 0        # NULL is a no-op, as free(3)
    assert L.cumo_hip_pool_free(C.c_void_p(p + 1)) == 3
    # a buffer from outside the pool stays the caller's to free
    raw = (C.c_char * ROUND)()
    assert L.cumo_hip_pool_free(C.c_void_p(C.addressof(raw))) == 3
    # a chunk that is not at the head of its block is owned just as much
    rc, head = malloc(2 * ROUND)
    rc, tail = malloc(2 * ROUND)
    assert head == p and tail == p + 2 * ROUND
    assert L.cumo_hip_pool_free(tail) == 0
    assert L.cumo_hip_pool_free(tail) == 3
    assert L.cumo_hip_pool_free(head) == 0
    assert L.cumo_hip_pool_used_bytes() == 0 and L.cumo_hip_pool_n_free_blocks() == 1


def test_malloc_split_and_free_merge_in_both_orders():
    # TestMallocSplit, TestFreeMerge, TestFreeDifferentSize (:488-531)
    rc, p1 = malloc(4 * ROUND)
    L.cumo_hip_pool_free(p1)
    for first in ("tail", "head"):
        rc, head = malloc(2 * ROUND)
        rc, tail = malloc(2 * ROUND)
        assert head == p1 and tail == p1 + 2 * ROUND
        for q in ((tail, head) if first == "tail" else (head, tail)):
            L.cumo_hip_pool_free(q)
        rc, p2 = malloc(4 * ROUND)
        assert p2 == p1
        L.cumo_hip_pool_free(p2)
    rc, p3 = malloc(8 * ROUND)
    assert p3 != p1
    L.cumo_hip_pool_free(p3)


def test_free_all_blocks_without_malloc_and_per_stream():
    # TestFreeAllBlocksWithoutMalloc (:542-544) and the per-stream cases the reference carries
    # as comments (:559-590)
    L.cumo_hip_pool_free_all_blocks()
    s = C.c_void_p(0x1000)                         # any handle names an arena on the host backend
    rc, p1 = malloc(4 * ROUND)
    rc, p2 = malloc(4 * ROUND, s)                  # while p1 is held: a block of its own
    assert p2 != p1
    L.cumo_hip_pool_free(p1)                       # (a free whole block would have moved to the asking stream's arena instead)
    L.cumo_hip_pool_free(p2)
    assert L.cumo_hip_pool_n_free_blocks() == 2
    L.cumo_hip_pool_free_all_blocks_stream(None)    # the null stream's arena only
    assert L.cumo_hip_pool_n_free_blocks() == 1 and L.cumo_hip_pool_free_bytes() == 4 * ROUND
    calls = L.cumo_hip_pool_device_malloc_calls()
    rc, p4 = malloc(4 * ROUND, s)                  # still cached for its own stream
    assert p4 == p2 and L.cumo_hip_pool_device_malloc_calls() == calls
    L.cumo_hip_pool_free(p4)
    L.cumo_hip_pool_free_all_blocks_stream(s)
    assert L.cumo_hip_pool_total_bytes() == 0


def test_byte_counters_with_two_streams():
    # TestGetUsedBytes / FreeBytes / TotalBytes and their stream forms (:592-660)
    s = C.c_void_p(0x2000)
    rc, p1 = malloc(4 * ROUND)
    rc, hold = malloc(ROUND)
    L.cumo_hip_pool_free(p1)
    L.cumo_hip_pool_free(hold)
    # the other stream takes the smallest whole free block that fits, for good
    rc, p2 = malloc(ROUND, s)
    assert p2 == hold
    assert L.cumo_hip_pool_used_bytes() == ROUND
    assert L.cumo_hip_pool_free_bytes() == 4 * ROUND
    assert L.cumo_hip_pool_total_bytes() == 5 * ROUND
    L.cumo_hip_pool_free(p2)
    rc, a = malloc(2 * ROUND)
    rc, b = malloc(4 * ROUND)
    L.cumo_hip_pool_free(a)
    L.cumo_hip_pool_free(b)
    rc, c = malloc(ROUND)
    assert L.cumo_hip_pool_total_bytes() == L.cumo_hip_pool_used_bytes() + L.cumo_hip_pool_free_bytes()
    L.cumo_hip_pool_free(c)
    assert L.cumo_hip_pool_used_bytes() == 0


def test_concurrent_split_and_merge_with_stamps():
    # TestConcurrentSplitAndMerge (:742-787): every thread splits chunks off one big free block,
    # stamps them, checks the stamps and frees them next to chunks other threads still hold
    threads, per_thread, rounds = 8, 16, 50
    total = ROUND * threads * per_thread * 2
    rc, big = malloc(total)
    L.cumo_hip_pool_free(big)
    assert L.cumo_hip_pool_n_free_blocks() == 1
    corrupted = []

    def worker(t):
        for _ in range(rounds):
            ptrs = []
            for k in range(per_thread):
                rc, p = malloc(ROUND)
                if rc != 0:
                    corrupted.append("malloc")
                    return
                C.memset(p, (t * per_thread + k + 1) & 0xff, ROUND)
                ptrs.append(p)
            for k, p in enumerate(ptrs):
                if C.string_at(p, ROUND) != bytes([(t * per_thread + k + 1) & 0xff]) * ROUND:
                    corrupted.append((t, k))
                L.cumo_hip_pool_free(p)

    ts = [threading.Thread(target=worker, args=(t,)) for t in range(threads)]
    for t in ts:
        t.start()
    for t in ts:
        t.join()
    assert not corrupted
    assert L.cumo_hip_pool_used_bytes() == 0
    assert L.cumo_hip_pool_n_free_blocks() == 1 and L.cumo_hip_pool_free_bytes() == total


def test_concurrent_first_use():
    # TestConcurrentPools (:789-807)
    def worker():
        for _ in range(200):
            rc, p = malloc(ROUND)
            assert rc == 0 and p
            L.cumo_hip_pool_free(p)
    ts = [threading.Thread(target=worker) for _ in range(8)]
    for t in ts:
        t.start()
    for t in ts:
        t.join()
    assert L.cumo_hip_pool_used_bytes() == 0


def test_a_failing_free_does_not_abort(capfd):
    # TestFailingFreeDoesNotAbort (:821-833): the no-raise release of a pointer nobody owns
    # reports and returns (the reference's destructor must not terminate the process)
    junk = (C.c_char * 64)()
    _lib.lib.cumo_cuda_runtime_free_no_raise(C.c_void_p(C.addressof(junk)))
    msg = C.c_char_p()
    _lib.lib.cumo_hip_last_error(C.byref(msg))       # whatever the device call left behind is cleared
    err = capfd.readouterr().err
    assert "failed to free" in err or err == ""      # no GPU: hipFree may be a no-op error path


def test_retired_stream_chunks_move_to_the_null_stream():
    # a destroyed stream's arena must not stay keyed by the dead handle: its chunks are filed
    # under the null stream, where they are reused
    h = C.c_void_p(0x3000)                             # the host backend needs no real stream
    rc, p = malloc(4 * ROUND, h)
    L.cumo_hip_pool_free(p)
    rc, held = malloc(2 * ROUND, h)                   # one chunk still in use on that stream
    retire = _lib.fn("cumo_hip_pool_retire_stream", None, [C.c_void_p])
    retire(h)
    calls = L.cumo_hip_pool_device_malloc_calls()
    rc, q = malloc(2 * ROUND)                          # null stream: takes the retired arena's free chunk
    assert rc == 0 and L.cumo_hip_pool_device_malloc_calls() == calls
    L.cumo_hip_pool_free(q)
    L.cumo_hip_pool_free(held)
    assert L.cumo_hip_pool_used_bytes() == 0 and L.cumo_hip_pool_n_free_blocks() == 1
