"""The 64-bit index arithmetic of the general kernels. It only runs by itself on arrays
beyond 2^32 elements, so (1) the view and reduction suites run once more in a child
process with CUMO_HIP_FORCE_WIDE=1, which makes every launch take it, and (2) arrays of
more than 2^32 elements go through sum / max / argmax / argmin for real: filled on the
device, a few elements stored, the expected answers known in closed form; index results
are Int64 there (reference: narray/gen/tmpl/accum_arg.c:92-110)."""
import os
import subprocess
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_view_and_reduction_suites_with_wide_indices_forced():
    env = dict(os.environ, CUMO_HIP_FORCE_WIDE="1")
    picked = ["tests/test_gpu_reduce.py::test_float_reductions_every_axis", "tests/test_gpu_reduce.py::test_random_float_sums",
              "tests/test_gpu_reduce.py::test_nan_rules", "tests/test_gpu_reduce.py::test_int32_reductions",
              "tests/test_gpu_reduce.py::test_min_max_keep_the_zero_that_came_first",
              "tests/test_gpu_elementwise.py::test_float_binary_over_views", "tests/test_gpu_elementwise.py::test_broadcast_shapes",
              "tests/test_gpu_elementwise.py::test_many_dims_and_permuted_views", "tests/test_gpu_elementwise.py::test_compare_into_bit",
              "tests/test_gpu_elementwise.py::test_casts_and_copies"]
    p = subprocess.run([sys.executable, "-m", "pytest", "-x", "-q", "-m", "gpu", "-p", "no:cacheprovider", "--timeout", "120",
                        "--timeout-method", "thread"] + picked, cwd=ROOT, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    tail = "\n".join(p.stdout.strip().splitlines()[-15:])
    assert p.returncode == 0, tail
    assert " passed" in tail and "failed" not in tail, tail


def test_reductions_of_more_than_2_to_the_32_elements():
    import cumo_amd
    n = (1 << 32) + 4096 + 12
    x = cumo_amd.SFloat.zeros(n)
    marks = {3: 5.0, 10: -2.0, (1 << 32) + 17: 7.0, (1 << 32) + 100: 7.0, n - 1: -2.0, 1 << 31: 0.25}
    for i, v in marks.items():
        x[i:i + 1].fill(v)
    assert float(x.sum()) == sum(marks.values())
    assert float(x.max()) == 7.0 and float(x.min()) == -2.0
    am, an = x.argmax(), x.argmin()
    assert isinstance(am, cumo_amd.Int64) and isinstance(an, cumo_amd.Int64)
    assert int(am) == (1 << 32) + 17       # the lower of the two equal maxima
    assert int(an) == 10
    assert int(x.max_index()) == (1 << 32) + 17 and int(x.min_index()) == 10
    # a view that starts beyond 2^32 elements and walks backwards
    tail = x[:(1 << 32) - 1:-1]
    assert tail.size == 4096 + 12
    assert float(tail.sum()) == 7.0 + 7.0 - 2.0
    assert int(tail.argmax()) == n - 1 - ((1 << 32) + 100)   # reversed: the later element comes first
    del x, tail
    cumo_amd.MemoryPool.free_all_blocks()


def test_row_and_column_reductions_with_more_than_2_to_the_31_outputs_or_positions():
    import cumo_amd
    cols = (1 << 31) + 8
    x = cumo_amd.SFloat.zeros(2, cols)
    x[0, 5:6].fill(3.0)
    x[1, 5:6].fill(4.0)
    x[1, cols - 1:cols].fill(9.0)
    x[0, (1 << 31) + 2:(1 << 31) + 3].fill(-1.0)
    # axis 1: two rows of more than 2^31 elements each
    s = x.sum(axis=1).to_numpy()
    assert s.tolist() == [2.0, 13.0]
    a = x.argmax(axis=1)
    assert a.to_numpy().tolist() == [5, cols - 1]
    # axis 0: more than 2^31 outputs (the general column kernel, 64-bit output indices)
    c = x.sum(axis=0)
    assert c.shape == (cols,)
    assert float(c[5:6].sum()) == 7.0 and float(c[cols - 1:].sum()) == 9.0 and float(c[(1 << 31) + 2:(1 << 31) + 3].sum()) == -1.0
    assert float(c.sum()) == 15.0
    m = x.max(axis=0)
    assert float(m[cols - 1:].max()) == 9.0 and float(m.sum()) == 4.0 + 9.0
    del x, c, m
    cumo_amd.MemoryPool.free_all_blocks()
