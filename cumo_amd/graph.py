"""A chain of array operations recorded once and replayed with one submission.

    with cumo_amd.Graph() as g:        # nothing runs inside the block
        t = 2.5 * x
        y = t + b
        s = y.sum()
    g.launch()                         # one run of the chain: t, y, s now hold results
    x.store(new_values); g.launch()    # again, from x's current contents

Everything inside the block must be launch-only (include/cumo_hip.h, cumo_hip_graph_*):
an operation that needs the host in the middle raises, and the block then leaves no
graph behind. The arrays made inside the block are ordinary arrays that every replay
rewrites; they may be read between replays like any other.
"""
from . import _lib
from ._lib import call

_L = _lib.lib


class Graph:
    def __init__(self):
        self._h = None

    def __enter__(self):
        call(_L.cumo_hip_graph_begin)
        return self

    def __exit__(self, etype, evalue, tb):
        h = _L.cumo_hip_graph_end()
        if etype is not None:
            # the failing operation has been reported already; drop what end() adds
            _L.cumo_hip_last_error(None)
            if h:
                _L.cumo_hip_graph_destroy(h)
            return False
        _lib.check()
        self._h = h
        return False

    @property
    def nodes(self):
        return int(_L.cumo_hip_graph_node_count(self._h)) if self._h else 0

    def launch(self, times=1):
        if not self._h:
            raise ValueError("no recorded graph")
        for _ in range(times):
            _L.cumo_hip_graph_launch(self._h)
        _lib.check()

    def close(self):
        if self._h:
            _L.cumo_hip_graph_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
