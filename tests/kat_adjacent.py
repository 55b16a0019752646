"""Known answers for pow, clip, maximum/minimum, mulsum and cumsum/cumprod,
transcribed from the reference's own tests (test/narray_test.rb, cited per case),
and two engines that run them: the CPU oracle and the device path. A case is a
function of an engine and an element type name that yields (got, want, cite)
triples; `want` is a literal from the reference test or, where that test
compares two of the library's own answers, the other answer."""
import math
import os
import sys

import numpy as np

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))

NP = {"sfloat": np.float32, "dfloat": np.float64, "int32": np.int32}
NAN = math.nan


class OperationFailed(Exception):
    """What either engine raises for Cumo::NArray::OperationError."""


# ---------------------------------------------------------------------------
# engines
# ---------------------------------------------------------------------------
class OracleArray:
    def __init__(self, eng, a):
        self.eng, self.a = eng, a

    def to_list(self):
        return self.a.tolist()

    def view(self, key):
        return OracleArray(self.eng, self.a[key])

    def transpose(self):
        return OracleArray(self.eng, self.a.T)

    def reshape(self, *shape):
        return OracleArray(self.eng, self.a.reshape(shape))


class OracleEngine:
    name = "oracle"

    def __init__(self):
        import numo_oracle
        self.o = numo_oracle

    def arr(self, tname, data):
        return OracleArray(self, np.array(data, dtype=NP[tname]))

    def _raw(self, b, like):
        if isinstance(b, OracleArray):
            return b.a
        return b

    def clip(self, x, lo, hi):
        def bound(b):
            if isinstance(b, OracleArray):
                return b.a.astype(x.a.dtype)
            return b
        try:
            return OracleArray(self, self.o.clip(np.ascontiguousarray(x.a), bound(lo), bound(hi)))
        except self.o.FlagError:
            raise OperationFailed()
        except ValueError as e:
            if "not given" in str(e):
                raise
            raise

    def clip_scalars_checked(self, x, lo, hi):
        # two numeric bounds are compared by the caller before anything runs (clip.c:222)
        if np.asarray(lo, dtype=x.a.dtype) > np.asarray(hi, dtype=x.a.dtype):
            raise OperationFailed()
        return self.clip(x, lo, hi)

    def pow(self, x, y):
        o = self.o
        if isinstance(x, OracleArray) and isinstance(y, OracleArray):
            if y.a.dtype == np.int32 and x.a.dtype != np.int32:
                return OracleArray(self, o.pow_int(x.a, y.a))
            up = np.result_type(x.a.dtype, y.a.dtype)
            if x.a.dtype == np.int32 and y.a.dtype == np.int32:
                up = np.int32
            return OracleArray(self, o.binary("pow", np.ascontiguousarray(x.a.astype(up)), np.ascontiguousarray(y.a.astype(up))))
        if isinstance(x, OracleArray):
            if isinstance(y, int):
                if x.a.dtype == np.int32:
                    return OracleArray(self, o.binary("pow", np.ascontiguousarray(x.a), y))
                return OracleArray(self, o.pow_int(x.a, y))
            a = x.a if x.a.dtype != np.int32 else x.a.astype(np.float64)
            return OracleArray(self, o.binary("pow", np.ascontiguousarray(a), float(y)))
        # number ** array
        if y.a.dtype == np.int32:
            if isinstance(x, int):
                return OracleArray(self, o.binary("pow", x, np.ascontiguousarray(y.a), scalar_is_left=True))
            return OracleArray(self, o.pow_int(np.float64(x), y.a))
        return OracleArray(self, o.binary("pow", float(x), np.ascontiguousarray(y.a), scalar_is_left=True))

    def cum(self, op, x, axis=None, nan=False):
        return OracleArray(self, self.o.cum(op, x.a, axis=axis, nan=nan))

    def mulsum(self, x, y, axis=None, keepdims=False, nan=False):
        return OracleArray(self, np.asarray(self.o.mulsum(x.a, y.a, axis=axis, keepdims=keepdims, nan=nan)))

    def mul_sum(self, x, y, axis=None):
        """(x * y).sum(axis:) as the reference tests write it; exact for the small integers they use"""
        prod = self.o.binary("mul", np.ascontiguousarray(np.broadcast_to(x.a, np.broadcast_shapes(x.a.shape, y.a.shape))),
                             np.ascontiguousarray(np.broadcast_to(y.a, np.broadcast_shapes(x.a.shape, y.a.shape))))
        return OracleArray(self, np.asarray(self.o.reduce("sum", prod, axis=axis)))

    def ewcomp(self, op, tname, a, b, nan=False):
        dt = NP[tname]
        ra = a.a.astype(dt) if isinstance(a, OracleArray) else np.array(a, dtype=dt)
        rb = b.a.astype(dt) if isinstance(b, OracleArray) else np.array(b, dtype=dt)
        shape = np.broadcast_shapes(ra.shape, rb.shape)
        ra = np.ascontiguousarray(np.broadcast_to(ra, shape))
        rb = np.ascontiguousarray(np.broadcast_to(rb, shape))
        return OracleArray(self, self.o.binary(op + ("_nan" if nan and dt != np.int32 else ""), ra, rb))


class DeviceArray:
    def __init__(self, eng, a):
        self.eng, self.a = eng, a

    def to_list(self):
        return self.a.to_numpy().tolist()

    def view(self, key):
        return DeviceArray(self.eng, self.a[key])

    def transpose(self):
        return DeviceArray(self.eng, self.a.transpose())

    def reshape(self, *shape):
        return DeviceArray(self.eng, self.a.reshape(*shape))


class DeviceEngine:
    name = "device"

    def __init__(self):
        import cumo_amd
        self.m = cumo_amd

    def cls(self, tname):
        return {"sfloat": self.m.SFloat, "dfloat": self.m.DFloat, "int32": self.m.Int32}[tname]

    def arr(self, tname, data):
        return DeviceArray(self, self.cls(tname).cast(np.array(data, dtype=NP[tname])))

    def _u(self, b):
        return b.a if isinstance(b, DeviceArray) else b

    def clip(self, x, lo, hi):
        from cumo_amd._lib import OperationError
        try:
            return DeviceArray(self, x.a.clip(self._u(lo), self._u(hi)))
        except OperationError:
            raise OperationFailed()

    clip_scalars_checked = clip

    def pow(self, x, y):
        return DeviceArray(self, self._u(x) ** self._u(y))

    def ewcomp(self, op, tname, a, b, nan=False):
        return DeviceArray(self, getattr(self.cls(tname), op)(self._u(a), self._u(b), nan=nan))

    def cum(self, op, x, axis=None, nan=False):
        return DeviceArray(self, getattr(x.a, op)(axis=axis, nan=nan))

    def mulsum(self, x, y, axis=None, keepdims=False, nan=False):
        return DeviceArray(self, x.a.mulsum(y.a, axis=axis, keepdims=keepdims, nan=nan))

    def mul_sum(self, x, y, axis=None):
        return DeviceArray(self, (x.a * y.a).sum(axis=axis))


# ---------------------------------------------------------------------------
# cases
# ---------------------------------------------------------------------------
def case_clip(E, t):
    a = E.arr(t, list(range(10)))
    yield E.clip(a, 1, 8).to_list(), [1, 1, 2, 3, 4, 5, 6, 7, 8, 8], "narray_test.rb:680"
    yield E.clip(a, None, 8).to_list(), [0, 1, 2, 3, 4, 5, 6, 7, 8, 8], "narray_test.rb:681"
    yield E.clip(a, 3, None).to_list(), [3, 3, 3, 3, 4, 5, 6, 7, 8, 9], "narray_test.rb:682"
    yield E.clip(a, E.arr(t, [3, 4, 1, 1, 1, 4, 4, 4, 4, 4]), 8).to_list(), [3, 4, 2, 3, 4, 5, 6, 7, 8, 8], "narray_test.rb:687"
    yield E.clip(a, 1, E.arr(t, [9, 9, 9, 5, 5, 5, 5, 5, 5, 5])).to_list(), [1, 1, 2, 3, 4, 5, 5, 5, 5, 5], "narray_test.rb:688"
    yield E.clip(a, E.arr(t, [2] * 10), E.arr(t, [7] * 10)).to_list(), [2, 2, 2, 3, 4, 5, 6, 7, 7, 7], "narray_test.rb:689"
    m = E.arr(t, list(range(12))).reshape(3, 4)
    yield E.clip(m.view((slice(1, 3), slice(1, 3))), 6, 9).to_list(), [[6, 6], [9, 9]], "narray_test.rb:700"
    yield E.clip(m.transpose(), 2, 8).to_list(), [[2, 4, 8], [2, 5, 8], [2, 6, 8], [3, 7, 8]], "narray_test.rb:701"
    yield E.clip(m.view((slice(None), slice(None, None, -1))), 2, 8).to_list(), [[3, 2, 2, 2], [7, 6, 5, 4], [8, 8, 8, 8]], "narray_test.rb:702"
    big = E.arr(t, [i % 100 for i in range(100000)])
    c = E.clip(big, 20, 80).to_list()
    yield [min(c), max(c)], [20, 80], "narray_test.rb:709-710"
    yield c[:25], [20] * 21 + [21, 22, 23, 24], "narray_test.rb:711"
    # a numeric bound answers what the same bound as an array answers (728-733); the
    # element type converts 1.5 / 7.5 the way m_num_to_data does
    lo, hi = (1.5, 7.5) if t != "int32" else (1, 7)
    yield E.clip(a, lo, hi).to_list(), E.clip(a, E.arr(t, [lo] * 10), E.arr(t, [hi] * 10)).to_list(), "narray_test.rb:730"
    yield E.clip(a, lo, None).to_list(), E.clip(a, E.arr(t, [lo] * 10), None).to_list(), "narray_test.rb:731"
    yield E.clip(a, None, hi).to_list(), E.clip(a, None, E.arr(t, [hi] * 10)).to_list(), "narray_test.rb:732"
    deep = E.arr(t, list(range(512))).reshape(*([2] * 9))
    yield (E.clip(deep, 1, 2).to_list(), E.clip(deep, E.arr(t, [1] * 512).reshape(*([2] * 9)), E.arr(t, [2] * 512).reshape(*([2] * 9))).to_list(),
           "narray_test.rb:737")


def case_clip_nan_bounds(E, t):
    a = E.arr(t, list(range(6)))
    nan = E.arr(t, [NAN] * 6)
    yield E.clip(a, NAN, 4).to_list(), E.clip(a, nan, 4).to_list(), "narray_test.rb:745"
    yield E.clip(a, 1, NAN).to_list(), E.clip(a, 1, nan).to_list(), "narray_test.rb:746"


def case_clip_raises(E, t):
    a = E.arr(t, list(range(10)))
    for fn, cite in ((lambda: E.clip_scalars_checked(a, 6, 3), "narray_test.rb:716"),
                     (lambda: E.clip(a, E.arr(t, [6] * 10), E.arr(t, [3] * 10)), "narray_test.rb:716 (array bounds)")):
        try:
            fn()
            raised = False
        except OperationFailed:
            raised = True
        yield raised, True, cite
    try:
        E.clip(a, None, None)
        raised = False
    except ValueError:
        raised = True
    yield raised, True, "narray_test.rb:717"


def case_ewcomp(E, t):
    a = E.arr(t, [1, 2, 3, 5, 7, 11])
    b = E.arr(t, [11, 10, 9, 7, 5, 1])   # 12 - a
    yield E.ewcomp("maximum", t, a, b).to_list(), [11, 10, 9, 7, 7, 11], "narray_test.rb:210"
    yield E.ewcomp("minimum", t, a, b).to_list(), [1, 2, 3, 5, 5, 1], "narray_test.rb:211"
    yield E.ewcomp("maximum", t, a, 5).to_list(), [5, 5, 5, 5, 7, 11], "narray_test.rb:212"
    yield E.ewcomp("minimum", t, a, 5).to_list(), [1, 2, 3, 5, 5, 5], "narray_test.rb:213"


def case_pow(E, t):
    a = E.arr(t, [1, 2, 3, 4])
    yield E.pow(a, 0).to_list(), [1, 1, 1, 1], "narray_test.rb:4726"
    yield E.pow(a, 1).to_list(), [1, 2, 3, 4], "narray_test.rb:4727"
    yield E.pow(a, 3).to_list(), [1, 8, 27, 64], "narray_test.rb:4728"
    yield E.pow(a, E.arr("int32", [3] * 4)).to_list(), E.pow(a, 3).to_list(), "narray_test.rb:4472"
    deep = E.arr(t, list(range(1, 513))).reshape(*([2] * 9))
    yield E.pow(deep, E.arr("int32", [2] * 512).reshape(*([2] * 9))).to_list(), E.pow(deep, 2).to_list(), "narray_test.rb:4475"
    yield E.pow(E.arr(t, [2] * 4), a).to_list(), E.pow(2, a).to_list(), "narray_test.rb:4820"
    if t != "int32":
        yield E.pow(a, E.arr(t, [2.5] * 4)).to_list(), E.pow(a, 2.5).to_list(), "narray_test.rb:4481"
        yield E.pow(deep, E.arr(t, [0.5] * 512).reshape(*([2] * 9))).to_list(), E.pow(deep, 0.5).to_list(), "narray_test.rb:4483"


def _running(values, op):
    out, acc = [], None
    for v in values:
        acc = v if acc is None else op(acc, v)
        out.append(acc)
    return out


def _running_skip_nan(values, op):
    # narray_test.rb:2876-2888
    acc = values[0]
    out = [acc]
    for y in values[1:]:
        if acc != acc:
            acc = y
        elif y == y:
            acc = op(acc, y)
        out.append(acc)
    return out


def case_cum_long_and_views(E, t):
    # values that keep every partial result exact, so association cannot matter (narray_test.rb:2895-2924)
    n = 20000
    adds = [(i % 3) + 1 for i in range(n)]
    muls = [2 if i % 4 < 2 else 0.5 for i in range(n)]
    views = [("flat", slice(None)), ("offset 13", slice(13, n)), ("step 2", slice(0, n, 2)), ("reversed", slice(None, None, -1))]
    a = E.arr(t, adds)
    for label, sl in views:
        yield E.cum("cumsum", a.view(sl)).to_list(), _running(adds[sl], lambda x, y: x + y), "narray_test.rb:2913 " + label
    if t != "int32":
        b = E.arr(t, muls)
        for label, sl in views:
            yield E.cum("cumprod", b.view(sl)).to_list(), _running(muls[sl], lambda x, y: x * y), "narray_test.rb:2921 " + label


def case_cum_axis(E, t):
    rows, cols = 6, 20000
    adds = [(i % 3) + 1 for i in range(rows * cols)]
    muls = [2 if i % 4 < 2 else 0.5 for i in range(rows * cols)]
    a = E.arr(t, adds).reshape(rows, cols)
    yield E.cum("cumsum", a, axis=1).to_list(), [_running(adds[r * cols:(r + 1) * cols], lambda x, y: x + y) for r in range(rows)], "narray_test.rb:2934"
    down = [_running([adds[r * cols + c] for r in range(rows)], lambda x, y: x + y) for c in range(cols)]
    yield E.cum("cumsum", a, axis=0).to_list(), [[down[c][r] for c in range(cols)] for r in range(rows)], "narray_test.rb:2937"
    b = E.arr(t, muls).reshape(rows, cols)
    yield E.cum("cumprod", b, axis=1).to_list(), [_running(muls[r * cols:(r + 1) * cols], lambda x, y: x * y) for r in range(rows)], "narray_test.rb:2941"


def case_cum_nan(E, t):
    for n in (64, 20000):
        for at in (0, 1, n // 2, n - 1):
            adds = [(i % 3) + 1.0 for i in range(n)]
            muls = [2.0 if i % 4 < 2 else 0.5 for i in range(n)]
            adds[at] = NAN
            muls[at] = NAN
            lbl = " n=%d at=%d" % (n, at)
            a, b = E.arr(t, adds), E.arr(t, muls)
            yield E.cum("cumsum", a).to_list(), _running(adds, lambda x, y: x + y), "narray_test.rb:2956" + lbl
            yield E.cum("cumsum", a, nan=True).to_list(), _running_skip_nan(adds, lambda x, y: x + y), "narray_test.rb:2957" + lbl
            yield E.cum("cumprod", b).to_list(), _running(muls, lambda x, y: x * y), "narray_test.rb:2961" + lbl
            yield E.cum("cumprod", b, nan=True).to_list(), _running_skip_nan(muls, lambda x, y: x * y), "narray_test.rb:2962" + lbl


def case_mulsum(E, t):
    a, b = E.arr(t, [1, 2, 3]), E.arr(t, [2, 3, 4])
    yield E.mulsum(a, b).to_list(), 1 * 2 + 2 * 3 + 3 * 4, "narray_test.rb:756"
    if t != "int32":
        yield E.mulsum(E.arr(t, [NAN, 2, 3]), b, nan=True).to_list(), 0 + 2 * 3 + 3 * 4, "narray_test.rb:764"

    def small(shape):
        n = 1
        for v in shape:
            n *= v
        return E.arr(t, [i % 4 + 1 for i in range(n)]).reshape(*shape)
    for shape in ([3], [3, 1], [1, 3], [3, 2], [2, 3], [3, 1, 1], [2, 3, 1], [2, 1, 3], [2, 3, 4]):
        x = small(shape)
        for axis in range(-len(shape), len(shape)):
            yield E.mulsum(x, x, axis=axis).to_list(), E.mul_sum(x, x, axis=axis).to_list(), "narray_test.rb:776 %r axis %d" % (shape, axis)
    x = small([3, 1])
    yield E.mulsum(x, x).to_list(), E.mul_sum(x, x).to_list(), "narray_test.rb:782"
    for shape in ([3, 1], [3, 2], [2, 3], [2, 3, 1], [2, 3, 4]):
        x = small(shape)
        two = E.arr(t, [2]).reshape(*([1] * len(shape)))
        for axis in range(len(shape)):
            yield E.mulsum(x, two, axis=axis).to_list(), E.mul_sum(x, two, axis=axis).to_list(), "narray_test.rb:790 %r axis %d" % (shape, axis)
    x = small([6])
    r = x.view(slice(None, None, -1))
    yield E.mulsum(r, r, axis=0).to_list(), E.mul_sum(x, x, axis=0).to_list(), "narray_test.rb:797"
    y = small([3, 2])
    ry = y.view((slice(None, None, -1), slice(None)))
    yield E.mulsum(ry, ry, axis=0).to_list(), E.mul_sum(y, y, axis=0).to_list(), "narray_test.rb:799"


CASES = [
    ("clip", case_clip, ("sfloat", "dfloat", "int32")),
    ("clip_nan_bounds", case_clip_nan_bounds, ("sfloat", "dfloat")),
    ("clip_raises", case_clip_raises, ("sfloat", "dfloat", "int32")),
    ("ewcomp", case_ewcomp, ("sfloat", "dfloat", "int32")),
    ("pow", case_pow, ("sfloat", "dfloat", "int32")),
    ("cum_long_and_views", case_cum_long_and_views, ("sfloat", "dfloat", "int32")),
    ("cum_axis", case_cum_axis, ("dfloat",)),
    ("cum_nan", case_cum_nan, ("dfloat", "sfloat")),
    ("mulsum", case_mulsum, ("sfloat", "dfloat", "int32")),
]


def all_cases():
    out = []
    for name, fn, types in CASES:
        for t in types:
            out.append((name, fn, t))
    return out


def same(got, want):
    """Exact match of nested lists, NaN equal to NaN."""
    g = np.asarray(got, dtype=np.float64)
    w = np.asarray(want, dtype=np.float64)
    if g.shape != w.shape:
        return False
    return bool(((g == w) | (np.isnan(g) & np.isnan(w))).all())


def run(E, name, fn, t):
    for got, want, cite in fn(E, t):
        assert same(got, want), "%s %s %s [%s]: got %r want %r" % (E.name, name, t, cite, got, want)
