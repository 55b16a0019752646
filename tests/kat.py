"""Runs the known-answer cases of tests/golden/reference_kats.json against an
engine: the CPU oracle or the device path. The fixture holds literals from the
reference's own tests; this file only decodes them."""
import json
import math
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
NP = {"sfloat": np.float32, "dfloat": np.float64, "int32": np.int32}
REDUCTIONS = {"sum", "prod", "mean", "var", "stddev", "rms", "min", "max", "ptp", "min_index", "max_index", "argmin", "argmax"}
COMPARES = {"eq", "ne", "gt", "ge", "lt", "le"}


def _num(v):
    if isinstance(v, str):
        return {"nan": math.nan, "inf": math.inf, "-inf": -math.inf, "-0.0": -0.0}[v]
    return v


def _decode(v):
    if isinstance(v, list):
        return [_decode(x) for x in v]
    return _num(v)


def load_cases():
    with open(os.path.join(HERE, "golden", "reference_kats.json")) as f:
        cases = json.load(f)["cases"]
    out = []
    for c in cases:
        for t in c["types"]:
            out.append((t, c))
    return out


def case_id(tc):
    t, c = tc
    return "%s-%s-%s" % (t, c["op"], c["cite"].split(":")[-1])


def make_input(t, c):
    dt = NP[t]
    if "gen" in c:
        shape = tuple(c["shape"])
        n = int(np.prod(shape))
        if c["gen"] == "seq":
            return np.arange(n, dtype=dt).reshape(shape)
        if c["gen"] == "mod3":
            return (np.arange(n) % 3).astype(dt).reshape(shape)
        if c["gen"] == "fill":
            return np.full(shape, c["value"], dtype=dt)
        raise ValueError(c["gen"])
    return np.array(_decode(c["data"]), dtype=dt)


def check(t, c, got):
    """got: numpy array or scalar produced by the engine."""
    want = np.array(_decode(c["expect"]), dtype=np.float64)
    got = np.asarray(got)
    assert got.shape == want.shape, (c["cite"], got.shape, want.shape)
    g = got.astype(np.float64)
    nan = np.isnan(want)
    assert (np.isnan(g) == nan).all(), (c["cite"], got, want)
    if c.get("signed_zero"):
        assert (np.signbit(g) == np.signbit(want)).all(), (c["cite"], got, want)
    rel = c.get("rel", 0.0)
    with np.errstate(invalid="ignore"):
        ok = nan | (g == want) | (np.abs(g - want) <= rel * np.abs(want))
    assert ok.all(), (c["cite"], got, want)


def run_oracle(t, c, oracle):
    x = make_input(t, c)
    op = c["op"]
    if op in REDUCTIONS:
        return oracle.reduce(op, x, axis=_axis(c), keepdims=c.get("keepdims", False), nan=c.get("nan", False))
    if op in COMPARES:
        if "scalar" in c:
            return oracle.compare(op, x, c["scalar"])
        return oracle.compare(op, x, np.array(_decode(c["other"]), dtype=x.dtype))
    if op == "minus":
        return oracle.unary(op, x)
    if "scalar" in c:
        return oracle.binary(op, x, c["scalar"])
    y = np.array(_decode(c["other"]), dtype=x.dtype)
    if c.get("other_transpose"):
        y = y.T
    return oracle.binary(op, x, y)


def _axis(c):
    a = c.get("axis")
    return tuple(a) if isinstance(a, list) else a


def run_device(t, c, cumo):
    cls = {"sfloat": cumo.SFloat, "dfloat": cumo.DFloat, "int32": cumo.Int32}[t]
    x = cls.cast(make_input(t, c))
    op = c["op"]
    if op in REDUCTIONS:
        kw = {"axis": _axis(c), "keepdims": c.get("keepdims", False)}
        if t != "int32" or op not in ("sum", "prod", "min", "max", "ptp", "min_index", "max_index", "argmin", "argmax"):
            kw["nan"] = c.get("nan", False)
        elif c.get("nan"):
            kw["nan"] = True
        return getattr(x, op)(**kw).to_numpy()
    if op in COMPARES:
        if "scalar" in c:
            return getattr(x, op)(c["scalar"]).to_numpy()
        return getattr(x, op)(cls.cast(np.array(_decode(c["other"]), dtype=NP[t]))).to_numpy()
    if op == "minus":
        return (-x).to_numpy()
    pyop = {"add": "__add__", "sub": "__sub__", "mul": "__mul__", "div": "__truediv__"}[op]
    if "scalar" in c:
        return getattr(x, pyop)(c["scalar"]).to_numpy()
    y = cls.cast(np.array(_decode(c["other"]), dtype=NP[t]))
    if c.get("other_transpose"):
        y = y.transpose()
    return getattr(x, pyop)(y).to_numpy()
