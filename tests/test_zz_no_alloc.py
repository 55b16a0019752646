"""The entry point that allocates nothing: cumo_hip_sfloat_sum_noalloc_kernel_launch
against cumo_sfloat_sum_kernel_launch on the same descriptors, through the C-ABI.
Same planner and kernels, so the results must agree bit for bit; the partial sums
of a split reduction live in a fixed array inside the library instead of a block
from the pool. Two calls in a row, the second on a smaller input (the array keeps
the first call's partial sums), then a shape whose partial sums do not fit."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

P = C.POINTER
SCRATCH_BYTES = 256 << 10   # CUMO_HIP_NOALLOC_SCRATCH_BYTES


def _dev(a):
    from cumo_amd import _lib
    p = _lib.call(_lib.lib.cumo_cuda_runtime_malloc, max(a.nbytes, 4))
    _lib.call(_lib.lib.cumo_hip_memcpy_h2d, p, a.ctypes.data, a.nbytes)
    return p


def _fetch(p, n):
    from cumo_amd import _lib
    out = np.empty(n, dtype=np.float32)
    _lib.call(_lib.lib.cumo_hip_memcpy_d2h, out.ctypes.data, p, out.nbytes)
    return out


def _arg(pin, pout, out_shape, red_shape, in_steps, out_steps):
    """Reduction descriptor with the kept dimensions first (indexer.h:189-220)."""
    from cumo_amd import _lib
    arg = _lib.ReductionArg()
    shape = tuple(out_shape) + tuple(red_shape)
    arg.in_.ptr = pin
    for k, (n, s) in enumerate(zip(shape, in_steps)):
        arg.in_indexer.shape[k] = n
        arg.in_.step[k] = s
    arg.in_indexer.ndim = len(shape)
    arg.in_indexer.total_size = int(np.prod(shape))
    arg.out.ptr = pout
    for k, (n, s) in enumerate(zip(out_shape, out_steps)):
        arg.out_indexer.shape[k] = n
        arg.out.step[k] = s
    arg.out_indexer.ndim = len(out_shape)
    arg.out_indexer.total_size = int(np.prod(out_shape)) if out_shape else 1
    return arg


def _plan(arg):
    from cumo_amd import _lib
    plan = _lib.ReducePlan()
    assert _lib.lib.cumo_hip_plan_reduce(C.byref(arg), 4, 4, C.byref(plan)) == 0
    return plan


def _both(h, out_shape, red_shape, in_steps, out_steps):
    """Runs the pool-backed launcher and the one that allocates nothing on the same
    input; returns (reference bits, no-alloc bits, status, device mallocs during the
    no-alloc call, pool bytes taken during it, plan)."""
    from cumo_amd import _lib
    lib = _lib.lib
    n_out = int(np.prod(out_shape)) if out_shape else 1
    pin = _dev(h)
    p1 = _lib.call(lib.cumo_cuda_runtime_malloc, 4 * n_out)
    p2 = _lib.call(lib.cumo_cuda_runtime_malloc, 4 * n_out)
    _lib.call(lib.cumo_hip_memset, p1, 0xff, 4 * n_out)
    _lib.call(lib.cumo_hip_memset, p2, 0xff, 4 * n_out)
    ref = _lib.fn("cumo_sfloat_sum_kernel_launch", None, [P(_lib.ReductionArg)])
    noalloc = _lib.fn("cumo_hip_sfloat_sum_noalloc_kernel_launch", C.c_int, [P(_lib.ReductionArg)])
    a1 = _arg(pin, p1, out_shape, red_shape, in_steps, out_steps)
    a2 = _arg(pin, p2, out_shape, red_shape, in_steps, out_steps)
    plan = _plan(a1)
    _lib.call(ref, C.byref(a1))
    mallocs, used = lib.cumo_hip_pool_device_malloc_calls(), lib.cumo_hip_pool_used_bytes()
    status = noalloc(C.byref(a2))
    plan.scratch_used = int(_lib.fn("cumo_hip_sfloat_sum_noalloc_scratch_used", C.c_size_t, [])())
    d_mallocs = lib.cumo_hip_pool_device_malloc_calls() - mallocs
    d_used = lib.cumo_hip_pool_used_bytes() - used
    msg = C.c_char_p()
    kind = lib.cumo_hip_last_error(C.byref(msg))
    assert kind == status, (kind, status, msg.value)
    want, got = _fetch(p1, n_out), _fetch(p2, n_out)
    for p in (pin, p1, p2):
        lib.cumo_cuda_runtime_free(p)
    return want.view(np.uint32), got.view(np.uint32), status, d_mallocs, d_used, plan


def test_two_calls_in_a_row_second_one_smaller():
    rng = np.random.default_rng(11)
    # a full sum: one output, the axis cut into chunks whose partial sums go through the scratch
    for n in ((1 << 22) + 13, (1 << 18) + 3):
        h = rng.uniform(-1, 1, n).astype(np.float32)
        want, got, status, d_mallocs, d_used, plan = _both(h, (), (n,), (4,), ())
        # (the launcher plans with its own options, so the exported plan does not say whether the
        # axis was cut: what the launch handed to its kernels does)
        assert plan.scratch_used >= 8, "the case must exercise the scratch"
        assert status == 0
        assert d_mallocs == 0 and d_used == 0
        assert (want == got).all(), (n, want, got)
        assert abs(float(got.view(np.float32)[0]) - float(h.astype(np.float64).sum())) <= 1e-5 * np.log2(n) * np.abs(h).sum()
    # few outputs across memory with a long axis (split column reduction), then a smaller one of the kind
    for rows, cols in ((8192, 64), (2048, 32)):
        h = rng.standard_normal((rows, cols)).astype(np.float32)
        want, got, status, d_mallocs, d_used, plan = _both(h, (cols,), (rows,), (4, 4 * cols), (4,))
        assert status == 0 and d_mallocs == 0 and d_used == 0
        assert plan.scratch_used >= 8, "the case must exercise the scratch"
        assert (want == got).all(), (rows, cols)
    # no scratch needed at all: row sums
    h = rng.standard_normal((300, 1000)).astype(np.float32)
    want, got, status, d_mallocs, d_used, plan = _both(h, (300,), (1000,), (4000, 4), (4,))
    assert plan.scratch_used == 0 and status == 0 and d_mallocs == 0 and d_used == 0
    assert (want == got).all()


def test_partial_sums_beyond_the_fixed_array_are_refused():
    from cumo_amd import _lib
    rng = np.random.default_rng(12)
    # search the planner for a shape whose partial sums exceed the array: many outputs, each split
    found = None
    for rows, cols in ((1 << 14, 3072), (1 << 15, 5120), (1 << 14, 1 << 13), (1 << 15, 1 << 12), (1 << 13, 1 << 14), (1 << 16, 1 << 11)):
        probe = _arg(0x1000, 0x2000, (cols,), (rows,), (4, 4 * cols), (4,))
        plan = _plan(probe)
        if plan.n_split > 1 and 4 * cols * plan.n_split > SCRATCH_BYTES:
            found = (rows, cols)
            break
    if found is None:
        pytest.skip("the planner splits none of the probed shapes beyond the fixed array")
    rows, cols = found
    h = rng.standard_normal((rows, cols)).astype(np.float32)
    want, got, status, d_mallocs, d_used, plan = _both(h, (cols,), (rows,), (4, 4 * cols), (4,))
    assert status == 3          # CUMO_HIP_ERROR_ARGUMENT, nothing launched
    assert plan.scratch_used == 0
    assert d_mallocs == 0 and d_used == 0
    assert (got == 0xffffffff).all(), "a refused call must not write the result"
    # and the entry point still works afterwards
    h = rng.uniform(-1, 1, 1 << 20).astype(np.float32)
    want, got, status, *_ = _both(h, (), (h.size,), (4,), ())
    assert status == 0 and (want == got).all()
