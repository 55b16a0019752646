"""A bounded wait that gives up must be REPORTED, not folded into a silently wrong result.

With CUMO_HIP_WAIT_LIMIT=0 (read once per process) every wait inside a kernel gives up at
its first failed look. The blocks that publish still run to their end, so every kernel
exits normally; only the waiting blocks stop waiting. The next call that waits for the
device must then report CUMO_HIP_ERROR_RUNTIME (the pinned-flag contract of the reference,
cuda/runtime.c:22-47), and cumo_hip_wait_give_ups must count the event. Without the knob
the same work reports nothing and the counts stay at zero."""
import os
import subprocess
import sys
import textwrap

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CHILD = textwrap.dedent("""
    import ctypes as C, sys
    import numpy as np
    import cumo_amd
    from cumo_amd import _lib
    L = _lib.lib
    L.cumo_hip_wait_give_ups.restype = C.c_int
    L.cumo_hip_wait_give_ups.argtypes = [C.POINTER(C.c_uint32 * 4)]

    def counts():
        c = (C.c_uint32 * 4)()
        assert L.cumo_hip_wait_give_ups(C.byref(c)) == 0
        return list(c)

    def reported(work):
        '''Runs work() (launches only), then waits for the device; the text of the error the wait reports, or None.'''
        work()
        try:
            cumo_amd.synchronize()
            _lib.check()
        except _lib.RuntimeError_ as e:
            return str(e)
        return None

    which = sys.argv[1]
    rng = np.random.default_rng(0)
    x = cumo_amd.SFloat.cast(rng.integers(-8, 8, 1 << 24).astype(np.float32))
    y = cumo_amd.SFloat.cast(rng.integers(-8, 8, 1 << 24).astype(np.float32))
    keep = []
    cumo_amd.synchronize(); _lib.check()
    before = counts()
    out = {}
    out['reduce'] = reported(lambda: keep.append(x.sum()))                 # full sum: hand-over words, one launch
    out['scan'] = reported(lambda: keep.append(x.cumsum()))                # one long run: chained look-back
    m = cumo_amd.SFloat.cast(rng.integers(-8, 8, (8192, 2048)).astype(np.float32))
    out['scan_cols'] = reported(lambda: keep.append(m.cumsum(axis=0)))     # down the rows: chained strips
    out['mulsum'] = reported(lambda: keep.append(x.mulsum(y)))             # one-launch dot product
    after = counts()
    print('RESULT', repr(out), before, after)
    if which == 'knob':
        assert before == [0, 0, 0, 0], before
        for k, v in out.items():
            assert v is not None and 'gave up' in v, (k, v)
        assert after[0] > 0 and after[1] > 0 and after[2] > 0, after
        # the error is reported once per raised flag, and a later clean launch reports nothing
        small = cumo_amd.SFloat.cast(np.arange(8, dtype=np.float32))
        assert reported(lambda: keep.append(small + small)) is None
    else:
        assert all(v is None for v in out.values()), out
        assert after == [0, 0, 0, 0], after
        assert float(keep[0].to_numpy()) == float(x.to_numpy().astype(np.float64).sum())
    print('CHILD OK')
""")


def run_child(which, env_extra):
    env = dict(os.environ, **env_extra)
    env["PYTHONPATH"] = ROOT + os.pathsep + env.get("PYTHONPATH", "")
    p = subprocess.run([sys.executable, "-c", CHILD, which], cwd=ROOT, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                       text=True, timeout=300)
    tail = "\n".join(p.stdout.strip().splitlines()[-12:])
    assert p.returncode == 0 and "CHILD OK" in p.stdout, tail


def test_a_wait_that_gives_up_is_reported_at_the_next_sync():
    run_child("knob", {"CUMO_HIP_WAIT_LIMIT": "0"})


def test_no_give_up_without_the_knob():
    run_child("plain", {})
