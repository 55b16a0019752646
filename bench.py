#!/usr/bin/env python3
"""Benchmark of the array hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--all-configs] [--no-cpu]

The last stdout line is ONE compact JSON line (headline, roofline, cpu_baseline and a
per-op map of fractions of peak); the full per-op tables go to gpurun_out/bench_full.json
(--full-out). A "step" is one pass of the headline workload (BASELINE.json
configs[1]: DFloat broadcast add + row reductions) with the inputs already resident
in HBM: C = A + r; C.sum(axis:1); C.max(axis:1) -- three launches through the
C-ABI. `value` is algorithmic bytes per step / seconds per step in GB/s, where
algorithmic bytes count every distinct input element once and every output element
once (the reference's own convention, bench/cumo_probe.rb:74-232).

Every GPU figure is taken with ROTATED buffers: consecutive launches (or steps) take
turns over several distinct sets of operands and results, so that at least 1 GiB of
other data passes between two uses of a buffer and nothing is served by the 256 MB
last-level cache -- sustained HBM. The same measurement on one set of buffers, back
to back, is printed beside it (`value_replay`, `frac_replay`).

`roofline` covers the dominant kernel of the step (the broadcast add, 256 MiB of
the step's 512 MiB), timed per launch with HIP events on the stream the launchers
use. `cpu_baseline` times the Numo-shaped single-thread C loops of the oracle on the
same workload on this machine's host cores. `per_config` lists every op of the five
BASELINE configs (filled with --all-configs, which the default run also does with
few iterations).

Everything runs on one GPU; --gpus N with N > 1 exits with a message.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth
ADD_KERNEL = "ew_rows2_lean_kernel<OpAdd<double>, 2, 5>"
# HBM bytes per launch of the C2 broadcast add come from two rocprofv3 --pmc runs of this
# file (FETCH_SIZE, then WRITE_SIZE; KiB per dispatch), each scaled by the same counter's
# reading for --pmc-calibration's plain 256 MiB copy. The summary of those runs is kept in
# this file, and the line that starts with TRAFFIC_KEY carries the figure; it is read from
# there (never typed in here), and reported as null when the summary is absent.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "ew_rows2_lean_add_f64_c2_hbm_traffic.txt")
TRAFFIC_KEY = "traffic_bytes_per_launch"


def read_traffic_bytes():
    try:
        with open(TRAFFIC_PROFILE) as f:
            for line in f:
                if line.startswith(TRAFFIC_KEY):
                    return int(line.split("=")[1].split()[0])
    except (OSError, ValueError, IndexError):
        pass
    return None


METRIC = "achieved HBM GB/s (% of MI355X peak) and GElem/s vs Numo CPU, per config"
MIB = 1 << 20


# ---------------------------------------------------------------------------
# synthetic inputs (host generated, seeded; neither library's own rand is usable
# because Cumo draws from Philox and Numo from SFMT)
# ---------------------------------------------------------------------------
def inputs_c1(n=1 << 20):
    rng = np.random.default_rng(0)
    return {"x": rng.uniform(-1, 1, n).astype(np.float32), "b": rng.uniform(-1, 1, n).astype(np.float32)}


def inputs_c2(n=4096):
    rng = np.random.default_rng(1)
    return {"A": rng.standard_normal((n, n)), "r": rng.standard_normal((1, n))}


def inputs_c3(shape=(64, 512, 1024)):
    rng = np.random.default_rng(2)
    u = rng.random(shape, dtype=np.float32)
    return {"T": (np.floor(u * 128) / 16 - 4).astype(np.float32)}  # multiples of 1/16 in [-4, 4): ties


def inputs_c4(n=8192):
    rng = np.random.default_rng(3)
    m = rng.standard_normal((n, n), dtype=np.float32)
    i = np.random.default_rng(4).integers(0, 1000, size=(n, n), dtype=np.int32)
    return {"M": m, "I": i}


def inputs_next(shape=(8192, 4096)):
    rng = np.random.default_rng(5)
    return {"x": rng.standard_normal(shape, dtype=np.float32), "y": rng.standard_normal(shape, dtype=np.float32),
            "rows": rng.integers(0, shape[0], shape[0]), "perm": rng.permutation(shape[0]),
            "d": rng.standard_normal(shape), "i": rng.integers(-1000, 1000, size=shape).astype(np.int32)}


def inputs_c5(s_shape=(32, 16, 512, 512), x_shape=(8192, 4096)):
    rng = np.random.default_rng(4)
    s = rng.standard_normal(s_shape, dtype=np.float32) * np.float32(2.0)  # N(0,2) read as sigma = 2
    x = rng.standard_normal(x_shape, dtype=np.float32)
    return {"S": s, "X": x}


# ---------------------------------------------------------------------------
# the five configs as chains of ops; every entry: (label, fn(env) -> result stored under label, bytes, elements)
# ---------------------------------------------------------------------------
def config_ops(name, cumo, host):
    """Returns (env, ops). env holds the device-resident inputs; ops is a list of
    (label, callable(env), algorithmic_bytes, elements)."""
    NM = cumo.NMath
    if name in ("c1", "c1_large"):
        n = host["x"].size
        env = {"x": cumo.SFloat.cast(host["x"]), "b": cumo.SFloat.cast(host["b"])}
        return env, [
            ("t=2.5*x", lambda e: e.__setitem__("t", 2.5 * e["x"]), 8 * n, n),
            ("y=t+b", lambda e: e.__setitem__("y", e["t"] + e["b"]), 12 * n, n),
            ("s=y.sum", lambda e: e.__setitem__("s", e["y"].sum()), 4 * n + 4, n),
        ]
    if name in ("c2", "c2_large"):
        n = host["A"].shape[0]
        env = {"A": cumo.DFloat.cast(host["A"]), "r": cumo.DFloat.cast(host["r"])}
        full, vec = 8 * n * n, 8 * n
        return env, [
            ("C=A+r", lambda e: e.__setitem__("C", e["A"] + e["r"]), 2 * full + vec, n * n),
            ("C.sum(axis:1)", lambda e: e.__setitem__("sum", e["C"].sum(axis=1)), full + vec, n * n),
            ("C.max(axis:1)", lambda e: e.__setitem__("max", e["C"].max(axis=1)), full + vec, n * n),
        ]
    if name in ("c3", "c3_large"):
        t = host["T"]
        env = {"T": cumo.SFloat.cast(t)}
        nb, n = t.nbytes, t.size
        ops = []
        for red in ("sum", "mean", "max", "min"):
            for axis, out in ((0, t.shape[1] * t.shape[2]), (2, t.shape[0] * t.shape[1]), (None, 1)):
                label = "T.%s(%s)" % (red, "axis:%d" % axis if axis is not None else "")
                ops.append((label, (lambda r, a, l: lambda e: e.__setitem__(l, getattr(e["T"], r)(axis=a)))(red, axis, label), nb + 4 * out, n))
        for red in ("argmax", "argmin"):
            label = "T.%s(axis:2)" % red
            ops.append((label, (lambda r, l: lambda e: e.__setitem__(l, getattr(e["T"], r)(axis=2)))(red, label), nb + 4 * t.shape[0] * t.shape[1], n))
        return env, ops
    if name == "c4":
        m, i = host["M"], host["I"]
        env = {"M": cumo.SFloat.cast(m), "I": cumo.Int32.cast(i)}
        env["V"] = env["M"].transpose()[:, ::2]   # V = M.transpose[true, (0..-1).step(2)]: V[i,j] = M[2j,i]
        nv = env["V"].size
        rows = len(range(0, i.shape[0], 3))
        return env, [
            ("E0=NMath.exp(V)", lambda e: e.__setitem__("E0", NM.exp(e["V"])), 8 * nv, nv),
            ("E=E0-1.0", lambda e: e.__setitem__("E", e["E0"] - 1.0), 8 * nv, nv),
            ("mask=E>0.5", lambda e: e.__setitem__("mask", e["E"] > 0.5), 4 * nv + nv // 8, nv),
            ("mask.count_true", lambda e: e.__setitem__("cnt", e["mask"].count_true()), nv // 8 + 8, nv),
            ("I[(0..-1).step(3),true].copy", lambda e: e.__setitem__("Ic", e["I"][::3].copy()), 2 * 4 * rows * i.shape[1], rows * i.shape[1]),
            # not an op of the config: the same transposed view copied with no arithmetic, the ceiling for E0
            ("tcopy=V.copy (ceiling of exp(V))", lambda e: e.__setitem__("Vc", e["V"].copy()), 8 * nv, nv),
        ]
    if name == "c5":
        s, x = host["S"], host["X"]
        env = {"S": cumo.SFloat.cast(s), "X": cumo.SFloat.cast(x)}
        ns, nx = s.size, x.size
        rs, rx = ns // s.shape[-1], x.shape[0]
        return env, [
            ("m=S.max(axis:-1,keepdims)", lambda e: e.__setitem__("m", e["S"].max(axis=-1, keepdims=True)), 4 * ns + 4 * rs, ns),
            ("d=S-m", lambda e: e.__setitem__("d", e["S"] - e["m"]), 8 * ns + 4 * rs, ns),
            ("e=NMath.exp(d)", lambda e: e.__setitem__("e", NM.exp(e["d"])), 8 * ns, ns),
            ("z=e.sum(axis:-1,keepdims)", lambda e: e.__setitem__("z", e["e"].sum(axis=-1, keepdims=True)), 4 * ns + 4 * rs, ns),
            ("p=e/z", lambda e: e.__setitem__("p", e["e"] / e["z"]), 8 * ns + 4 * rs, ns),
            ("mean=X.mean(axis:-1,keepdims)", lambda e: e.__setitem__("mean", e["X"].mean(axis=-1, keepdims=True)), 4 * nx + 4 * rx, nx),
            ("var=X.var(axis:-1,keepdims)", lambda e: e.__setitem__("var", e["X"].var(axis=-1, keepdims=True)), 4 * nx + 4 * rx, nx),
            ("c=X-mean", lambda e: e.__setitem__("c", e["X"] - e["mean"]), 8 * nx + 4 * rx, nx),
            ("v=var+1e-5", lambda e: e.__setitem__("v", e["var"] + 1e-5), 8 * rx, rx),
            ("sd=NMath.sqrt(v)", lambda e: e.__setitem__("sd", NM.sqrt(e["v"])), 8 * rx, rx),
            ("n=c/sd", lambda e: e.__setitem__("n", e["c"] / e["sd"]), 8 * nx + 4 * rx, nx),
            # the same two composites as one launch each (library additions beside the chain above):
            # one read and one write of the array
            ("Fused.softmax(S)", lambda e: e.__setitem__("pf", cumo.Fused.softmax(e["S"])), 8 * ns, ns),
            ("Fused.layernorm(X,1e-5)", lambda e: e.__setitem__("nf", cumo.Fused.layernorm(e["X"], 1e-5)), 8 * nx, nx),
        ]
    if name == "next":
        x, y = host["x"], host["y"]
        env = {"x": cumo.SFloat.cast(x), "y": cumo.SFloat.cast(y), "b": cumo.SFloat.cast(y)}
        env["mask"] = env["x"] > 0.5
        env["d"] = cumo.DFloat.cast(host["d"])
        env["i"] = cumo.Int32.cast(host["i"])
        env["rows"] = host["rows"]
        env["perm"] = host["perm"]
        n, nb = x.size, x.nbytes
        r, c = x.shape
        cnt = int((x > 0.5).sum())
        return env, [
            ("x.mulsum(y,axis:1)", lambda e: e.__setitem__("dot", e["x"].mulsum(e["y"], axis=1)), 2 * nb + 4 * r, n),
            ("x.clip(-1,1)", lambda e: e.__setitem__("cl", e["x"].clip(-1.0, 1.0)), 2 * nb, n),
            ("SFloat.maximum(x,y)", lambda e: e.__setitem__("mx", cumo.SFloat.maximum(e["x"], e["y"])), 3 * nb, n),
            ("x**3", lambda e: e.__setitem__("p3", e["x"] ** 3), 2 * nb, n),
            ("x.cumsum(axis:1)", lambda e: e.__setitem__("cs", e["x"].cumsum(axis=1)), 2 * nb, n),
            ("mask.where", lambda e: e.__setitem__("wh", e["mask"].where()), n // 8 + 4 * cnt, n),
            ("x[mask]", lambda e: e.__setitem__("xm", e["x"][e["mask"]]), n // 8 + 4 * cnt + 4 * cnt, n),
            # rows drawn with replacement: repeated rows are read from cache, and some 37% of the rows are never
            # read; the permutation beside it reads every row once, as the scatter writes every row once
            ("x[rows,true] (gather)", lambda e: e.__setitem__("g", e["x"][e["rows"]]), 2 * nb + 8 * r, n),
            ("x[perm,true] (gather, every row once)", lambda e: e.__setitem__("g", e["x"][e["perm"]]), 2 * nb + 8 * r, n),
            ("b[perm,true]=x (scatter)", lambda e: e["b"].__setitem__(e["perm"], e["x"]), 2 * nb + 8 * r, n),
            # two element types: the bytes the operation is defined over (each input once, the result once)
            ("x+d (SFloat+DFloat)", lambda e: e.__setitem__("xd", e["x"] + e["d"]), 5 * nb, n),
            ("i*0.5 (Int32 by Float)", lambda e: e.__setitem__("ih", e["i"] * 0.5), 3 * nb, n),
            ("x>d into Bit", lambda e: e.__setitem__("xgd", e["x"] > e["d"]), 3 * nb + n // 8, n),
        ]
    if name == "odd":
        # the hot-path operations on a matrix whose rows are not a whole number of 128-bit vectors (4095 SFloat:
        # every row after the first starts off a 16-byte boundary)
        x, y, r = host["x"], host["y"], host["r"]
        env = {"x": cumo.SFloat.cast(x), "y": cumo.SFloat.cast(y), "r": cumo.SFloat.cast(r), "perm": host["perm"]}
        n, nb = x.size, x.nbytes
        rows, cols = x.shape
        return env, [
            ("A+r (row vector)", lambda e: e.__setitem__("c", e["x"] + e["r"]), 2 * nb + 4 * cols, n),
            ("A+B", lambda e: e.__setitem__("c", e["x"] + e["y"]), 3 * nb, n),
            ("A>r into Bit", lambda e: e.__setitem__("m", e["x"] > e["r"]), nb + n // 8, n),
            ("A.transpose + 1", lambda e: e.__setitem__("t", e["x"].transpose() + 1.0), 2 * nb, n),
            ("A.sum(axis:1)", lambda e: e.__setitem__("s", e["x"].sum(axis=1)), nb + 4 * rows, n),
            ("A.max(axis:1)", lambda e: e.__setitem__("s", e["x"].max(axis=1)), nb + 4 * rows, n),
            ("A.sum(axis:0)", lambda e: e.__setitem__("s0", e["x"].sum(axis=0)), nb + 4 * cols, n),
            ("A.sum", lambda e: e.__setitem__("s1", e["x"].sum()), nb, n),
            ("A.mulsum(B,axis:1)", lambda e: e.__setitem__("d", e["x"].mulsum(e["y"], axis=1)), 2 * nb + 4 * rows, n),
            ("Fused.softmax(A)", lambda e: e.__setitem__("p", cumo.Fused.softmax(e["x"])), 2 * nb, n),
            ("Fused.layernorm(A)", lambda e: e.__setitem__("l", cumo.Fused.layernorm(e["x"], 1e-5)), 2 * nb, n),
            ("A[perm,true]", lambda e: e.__setitem__("g", e["x"][e["perm"]]), 2 * nb + 8 * rows, n),
            ("A.cumsum(axis:1)", lambda e: e.__setitem__("c1", e["x"].cumsum(axis=1)), 2 * nb, n),
            ("A.cumsum(axis:0)", lambda e: e.__setitem__("c0", e["x"].cumsum(axis=0)), 2 * nb, n),
        ]
    if name in ("bit", "bit_large"):
        # Bit arrays of 2^29 bits (64 MiB; 2^31 bits, 256 MiB, for bit_large) and the stores between Bit and SFloat [8192,4096]
        a, b, x = host["a"], host["b"], host.get("x")
        env = {"a": cumo.Bit.cast(a), "b": cumo.Bit.cast(b)}
        env["t"] = env["a"] | ~env["a"]
        n = a.size
        rows, cols = a.shape
        casts = []
        if x is not None:
            env["x"] = cumo.SFloat.cast(x)
            env["m"] = env["x"] > 0.0
            nx = x.size
            casts = [
                ("SFloat.cast(m) (Bit -> SFloat)", lambda e: e.__setitem__("f", e["m"]._cast_to(cumo.SFloat)), nx // 8 + 4 * nx, nx),
                ("Bit.cast(x) (SFloat -> Bit)", lambda e: e.__setitem__("g", e["x"]._cast_to(cumo.Bit)), nx // 8 + 4 * nx, nx),
            ]
        return env, [
            ("a & b", lambda e: e.__setitem__("c", e["a"] & e["b"]), 3 * n // 8, n),
            ("~a", lambda e: e.__setitem__("c", ~e["a"]), 2 * n // 8, n),
            ("a[true,1..-1] ^ b[true,0..-2]", lambda e: e.__setitem__("v", e["a"][:, 1:] ^ e["b"][:, :-1]), 3 * n // 8, n),
            ("a.count_true", lambda e: e.__setitem__("k", e["a"].count_true()), n // 8, n),
            ("a.count_true(axis:1)", lambda e: e.__setitem__("k1", e["a"].count_true(axis=1)), n // 8 + 8 * rows, n),
            ("a.count_true(axis:0)", lambda e: e.__setitem__("k0", e["a"].count_true(axis=0)), n // 8 + 8 * cols, n),
            # on an array with every bit set: a row of `a` is decided by its first words and the kernel stops reading it there
            ("t.all?(axis:1) (t all set: every word is read)", lambda e: e.__setitem__("p", e["t"].all_p(axis=1)), n // 8, n),
        ] + casts
    if name == "nmath":
        # NMath beyond exp / sqrt, the Float power and the scans on 2^26 elements (256 MiB SFloat,
        # 512 MiB DFloat per array); arguments positive so that every function is defined
        x = host["x"]
        n = x.size
        env = {"xs": cumo.SFloat.cast(x), "xd": cumo.DFloat.cast(x.astype(np.float64))}
        env["xs2"] = env["xs"].reshape(8192, n // 8192)
        ops = []
        for fname in ("log", "sin", "cos", "tan", "tanh", "erf", "asinh", "atan", "exp", "sqrt", "log1p", "sinh", "erfc", "cbrt"):
            ops.append(("NMath.%s(SFloat)" % fname, (lambda f: lambda e: e.__setitem__("r", getattr(NM, f)(e["xs"])))(fname), 8 * n, n))
        for fname in ("log", "sin", "tanh", "erf", "exp", "sqrt", "erfc", "asinh", "log1p"):
            ops.append(("NMath.%s(DFloat)" % fname, (lambda f: lambda e: e.__setitem__("rd", getattr(NM, f)(e["xd"])))(fname), 16 * n, n))
        ops += [
            # (2.5 is a whole number of halves: squarings and a square root; 2.7 takes the general power)
            ("SFloat**2.5", lambda e: e.__setitem__("r", e["xs"] ** 2.5), 8 * n, n),
            ("SFloat**2.7", lambda e: e.__setitem__("r", e["xs"] ** 2.7), 8 * n, n),
            ("DFloat**2.5", lambda e: e.__setitem__("rd", e["xd"] ** 2.5), 16 * n, n),
            ("SFloat.cumsum (one run of 2^26)", lambda e: e.__setitem__("r", e["xs"].cumsum()), 8 * n, n),
            ("SFloat[8192,8192].cumsum(axis:0)", lambda e: e.__setitem__("r2", e["xs2"].cumsum(axis=0)), 8 * n, n),
            ("SFloat[8192,8192].cumsum(axis:1)", lambda e: e.__setitem__("r2", e["xs2"].cumsum(axis=1)), 8 * n, n),
        ]
        return env, ops
    raise ValueError(name)


def inputs_odd(shape=(8192, 4095)):
    rng = np.random.default_rng(7)
    return {"x": rng.standard_normal(shape, dtype=np.float32), "y": rng.standard_normal(shape, dtype=np.float32),
            "r": rng.standard_normal((1, shape[1]), dtype=np.float32), "perm": rng.permutation(shape[0])}


def inputs_bit(shape=(16384, 32768)):
    rng = np.random.default_rng(8)
    return {"a": rng.integers(0, 2, size=shape, dtype=np.uint8), "b": rng.integers(0, 2, size=shape, dtype=np.uint8),
            "x": rng.standard_normal((8192, 4096), dtype=np.float32)}


def inputs_bit_large(shape=(32768, 65536)):
    # (bits unpacked from random bytes: 2^31 draws of one bit each would take most of a minute)
    rng = np.random.default_rng(9)
    n = shape[0] * shape[1]
    return {k: np.unpackbits(np.frombuffer(rng.bytes(n // 8), dtype=np.uint8)).reshape(shape) for k in ("a", "b")}


def inputs_nmath(n=1 << 26):
    rng = np.random.default_rng(6)
    return {"x": rng.uniform(0.05, 3.0, n).astype(np.float32)}


HOST_INPUTS = {
    "c1": inputs_c1, "c1_large": lambda: inputs_c1(1 << 26), "c2": inputs_c2, "c3": inputs_c3, "c4": inputs_c4, "c5": inputs_c5,
    "c2_large": lambda: inputs_c2(8192), "c3_large": lambda: inputs_c3((256, 512, 1024)), "next": inputs_next,
    "nmath": inputs_nmath, "odd": inputs_odd, "bit": inputs_bit, "bit_large": inputs_bit_large,
}
WORKLOAD_TEXT = {
    "c1": "C1 SFloat axpy + full sum, n=2^20",
    "c1_large": "C1 at n=2^26 (256 MiB per array)",
    "c2_large": "C2 at 8192 x 8192 (512 MiB per matrix)",
    "c3_large": "C3 at [256,512,1024] (512 MiB)",
    "next": "operations beside the five configs on SFloat [8192,4096]: mulsum, clip, maximum, integer power, cumsum, where, a[mask], row gather and scatter through index arrays, arithmetic and comparison of two element types",
    "odd": "the hot-path operations on SFloat [8192,4095]: rows that are not a whole number of 128-bit vectors and start off 16-byte boundaries",
    "bit": "Bit [16384,32768] (64 MiB): logic on whole arrays and on windows, counts of the whole, along rows and down columns, all?; stores between Bit and SFloat [8192,4096]",
    "bit_large": "the Bit logic and counts at [32768,65536] (256 MiB), where a launch's fixed start and drain weigh a quarter of what they do at 64 MiB",
    "nmath": "NMath functions, Float power and cumsum on 2^26 elements (SFloat 256 MiB, DFloat 512 MiB per array), arguments uniform in [0.05, 3)",
    "c2": "C2 DFloat broadcast add + row reduce: A f64 [4096,4096] + r [1,4096]; C.sum(axis:1); C.max(axis:1)",
    "c3": "C3 SFloat axis reductions on [64,512,1024]",
    "c4": "C4 strided/transposed views on SFloat [8192,8192] + Int32 stride-3 row slice copy",
    "c5": "C5 softmax [32,16,512,512] + layernorm statistics [8192,4096] composed from array ops",
}


class Timer:
    def __init__(self, lib):
        self.lib = lib
        self.e0 = lib.cumo_hip_event_create()
        self.e1 = lib.cumo_hip_event_create()

    def time(self, fn):
        self.lib.cumo_hip_event_record(self.e0)
        fn()
        self.lib.cumo_hip_event_record(self.e1)
        return self.lib.cumo_hip_event_elapsed_ms(self.e0, self.e1)

    def close(self):
        self.lib.cumo_hip_event_destroy(self.e0)
        self.lib.cumo_hip_event_destroy(self.e1)


ROTATE_BYTES = 1 << 30   # memory touched between two uses of one buffer in the rotated figures
ROTATE_MAX_SETS = 9      # 128 MiB operations: eight other sets (1 GiB) between two uses of a set


def rotation_sets(nbytes):
    """How many distinct operand/result sets an operation of `nbytes` algorithmic bytes
    is rotated over, so that at least ROTATE_BYTES of other data pass through the caches
    between two uses of a buffer (the last-level cache holds 256 MB)."""
    need = -(-ROTATE_BYTES // max(int(nbytes), 1)) + 1
    return max(2, min(ROTATE_MAX_SETS, need))


def measure_config(name, cumo, lib, iters, warmup, replay_too=True):
    """Every op of a config, timed two ways with HIP events on the launch stream:
    `rotated` -- consecutive launches take turns over K distinct sets of operands and
    results (K device copies of the inputs, K results), so a launch finds none of its
    data in a cache: sustained HBM; and `replay` -- the same call on the same buffers
    back to back, which at 128-256 MiB is helped by the 256 MB last-level cache.
    `frac_of_peak`, `gbps`, `gelem_s` are the rotated figures."""
    host = HOST_INPUTS[name]()
    sets = [config_ops(name, cumo, host)]
    for _ in range(max(rotation_sets(o[2]) for o in sets[0][1]) - 1):
        sets.append(config_ops(name, cumo, host))
    del host
    from cumo_amd import _lib
    timer = Timer(lib)
    rows = []
    batch = 10
    n_ops = len(sets[0][1])
    for i in range(n_ops):
        label, _, nbytes, nelem = sets[0][1][i]
        # the op runs once per set through the host mirror, which records the library
        # calls it makes; the timed region issues exactly those C-ABI calls again (into
        # the result the first call allocated) between two events on the launch stream,
        # so the figure is the library's and not the Python mirror's. Every set runs the
        # op (later ops of the chain need its result), the rotation uses the first K.
        per_set = []
        keep = []
        for env, ops in sets:
            with _lib.record() as calls:
                ops[i][1](env)
            keep.append(calls)  # holds the temporaries the operation released
            # launches that rewrite an index array in place (positions -> byte offsets) belong to
            # building the view, not to the copy, and must not run twice on the same array
            per_set.append([c for c in calls if not c[0].__name__.startswith("cumo_na_index_")])
        k = rotation_sets(nbytes)
        rot = per_set[:k]
        state = [0]

        # where / a[mask] size their own result: every timed call gets an empty result descriptor, as a caller's
        # would be, and the result of the set's previous turn is released after it (replaying the recorded call as it
        # stands would hand the library a result of the right length, which no caller has before the call)
        sizing = ("cumo_hip_na_where", "cumo_hip_na_mask")
        owned = [[None] * len(r) for r in rot]
        first = {}  # (set, call) -> the result the recorded call allocated (the mirror's array owns it)

        def rotated(times):
            j = state[0]
            for _ in range(times):
                for c, (f, a) in enumerate(rot[j]):
                    if f.__name__ in sizing:
                        z = a[-1]._obj
                        first.setdefault((j, c), z.ptr)
                        z.ptr = None
                        f(*a)
                        if owned[j][c]:
                            lib.cumo_cuda_runtime_free(owned[j][c])
                        owned[j][c] = z.ptr
                    else:
                        f(*a)
                j = j + 1 if j + 1 < k else 0
            state[0] = j
            _lib.check()

        rotated(max(warmup, k))
        if i == 0:
            # the device has idled while the host prepared the inputs: bring it back to its
            # sustained state (clocks, the pool's blocks mapped) before the first op is timed,
            # or the first two or three ops of a config read 10-20% slow
            t0 = time.perf_counter()
            while time.perf_counter() - t0 < 0.3:
                rotated(batch)
                lib.cumo_hip_synchronize()
        ts = sorted(timer.time(lambda: rotated(batch)) / batch for _ in range(iters))
        for row_owned in owned:
            for ptr in row_owned:
                if ptr:
                    lib.cumo_cuda_runtime_free(ptr)
        for (j, c), ptr in first.items():
            rot[j][c][1][-1]._obj.ptr = ptr  # the replay leg below writes into the recorded result again
        del keep
        med, best = ts[len(ts) // 2], ts[0]
        row_replay = {}
        if replay_too:
            _lib.replay(per_set[0], warmup)
            tr = sorted(timer.time(lambda: _lib.replay(per_set[0], batch)) / batch for _ in range(iters))
            med_replay = tr[len(tr) // 2]
            row_replay = {"ms_median_replay": round(med_replay, 5), "frac_replay": round(nbytes / (med_replay * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
        rows.append({
            "op": label, "bytes": int(nbytes), "sets": k, "rotation_bytes": int(nbytes) * k,
            "ms_median": round(med, 5), "ms_best": round(best, 5),
            "gbps": round(nbytes / (med * 1e-3) / 1e9, 1), "frac_of_peak": round(nbytes / (med * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "gelem_s": round(nelem / (med * 1e-3) / 1e9, 2), **row_replay,
        })
    timer.close()
    for env, _ in sets:
        env.clear()
    # the pool keeps its blocks from one config to the next, as it does in a long-running process
    return rows


def measure_host_io(lib, mib=256, reps=5):
    """Read-back and ingest of one contiguous array between pageable host memory and the
    device: the library's staged copies beside the runtime's own pageable path (what a
    plain hipMemcpy gives). PCIe-bound: GB/s here are not comparable with the HBM figures."""
    from cumo_amd import _lib
    n = mib << 20
    h = np.random.default_rng(0).integers(0, 255, n, dtype=np.uint8)
    back = np.empty_like(h)
    p = _lib.call(lib.cumo_cuda_runtime_malloc, n)
    out = {"bytes": n, "unit": "GB/s", "host_memory": "pageable"}
    for name, f in (("ingest_staged", lambda: lib.cumo_hip_copy_from_host(p, h.ctypes.data, n)),
                    ("ingest_runtime_memcpy", lambda: lib.cumo_hip_memcpy_h2d(p, h.ctypes.data, n)),
                    ("readback_staged", lambda: lib.cumo_hip_copy_to_host(back.ctypes.data, p, n)),
                    ("readback_runtime_memcpy", lambda: lib.cumo_hip_memcpy_d2h(back.ctypes.data, p, n))):
        f()
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            f()
            ts.append(time.perf_counter() - t0)
        ts.sort()
        out[name] = round(n / ts[len(ts) // 2] / 1e9, 2)
    _lib.check()
    if not (back == h).all():
        raise SystemExit("bench: host round trip returned different bytes")
    lib.cumo_cuda_runtime_free(p)
    return out


def measure_host_cost():
    """Per-operation cost of the C host layer on tiny arrays, from the C driver built next to
    the library (bench_host_cost.cpp): no interpreter between the calls."""
    import subprocess
    tool = os.path.join(ROOT, "cumo_amd", "bench_host_cost")
    if not os.path.exists(tool):
        return {"skipped": "cumo_amd/bench_host_cost is not built (python cumo_amd/build.py)"}
    p = subprocess.run([tool], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
    if p.returncode:
        return {"failed": p.stderr.strip()[-300:]}
    return json.loads(p.stdout.strip().splitlines()[-1])


def cpu_baseline_c2(budget_s=12.0):
    """Numo-shaped single-thread C loops (the oracle's row loops) on the same C2
    workload, on this machine's host cores. A bounded number of passes."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import numo_oracle as oracle
    lib = oracle.lib
    h = inputs_c2()
    a, r = h["A"], h["r"]
    n = a.shape[0]
    c = np.empty_like(a)
    s = np.empty(n)
    m = np.empty(n)
    vp = lambda x: C.c_void_p(x.ctypes.data)
    SZ, SSZ = C.c_size_t, C.c_ssize_t
    lib.numo_rows_binary.restype = C.c_int
    lib.numo_rows_reduce.restype = C.c_int

    def one_pass():
        lib.numo_rows_binary(b"add", 1, SZ(n), SZ(n), vp(a), SSZ(8 * n), SSZ(8), vp(r), SSZ(0), SSZ(8), vp(c), SSZ(8 * n), SSZ(8))
        lib.numo_rows_reduce(b"sum", 1, SZ(n), SZ(n), vp(c), SSZ(8 * n), vp(s))
        lib.numo_rows_reduce(b"max", 1, SZ(n), SZ(n), vp(c), SSZ(8 * n), vp(m))

    one_pass()
    t0 = time.perf_counter()
    passes = 0
    while passes < 2 or (time.perf_counter() - t0 < budget_s and passes < 600):
        one_pass()
        passes += 1
    dt = (time.perf_counter() - t0) / passes
    nbytes = 4 * 8 * n * n + 3 * 8 * n
    return {
        "value": round(nbytes / dt / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
        "sample": "%d passes of the full C2 step (A+r, row sum, row max on 4096x4096 f64), Numo-shaped single-thread C loops "
                  "(oracle/numo_oracle.c numo_rows_*), gcc -O2, 1 of %d host cores; %.1f ms per pass" % (passes, os.cpu_count() or 0, dt * 1e3),
        "ms_per_step": round(dt * 1e3, 3),
    }


FINAL_LINE_MAX = 6000  # bytes: the last stdout line must stay small enough for any log tail to hold it whole


def compact(out):
    """The result as the last stdout line carries it: every headline field, `roofline` and
    `cpu_baseline` whole, and of the per-op tables only `op -> fraction of HBM peak`
    (3 decimals). The full tables go to a file (write_full)."""
    c = {k: v for k, v in out.items() if k not in ("per_config", "host_io", "host_cost")}
    if "per_config" in out:
        c["per_config"] = {name: {o["op"]: round(o["frac_of_peak"], 3) for o in cfg["ops"]}
                           for name, cfg in out["per_config"].items()}
    hc = out.get("host_cost")
    if isinstance(hc, dict) and "launcher_add" in hc:
        c["host_cost_us"] = {k: hc[k] for k in ("empty_launch", "launcher_add", "add_alloc_free", "sum_alloc_free") if k in hc}
    return c


def final_line(out, full_path=None):
    """One JSON line of at most FINAL_LINE_MAX bytes. Should the compact form ever outgrow
    that, the per-op map is dropped first: the headline, roofline and cpu_baseline always fit."""
    c = compact(out)
    if full_path:
        c["full_results"] = full_path
    line = json.dumps(c)
    if len(line) > FINAL_LINE_MAX:
        c.pop("per_config", None)
        c["per_config_omitted"] = "see full_results"
        line = json.dumps(c)
    if len(line) > FINAL_LINE_MAX:
        raise SystemExit("bench: the result line is %d bytes, over the %d-byte limit" % (len(line), FINAL_LINE_MAX))
    return line


def write_full(out, path):
    """Every table of the run (per-op timings, host transfer rates, host cost) as indented
    JSON. Returns the path relative to this file's folder, or None when it cannot be written."""
    try:
        os.makedirs(os.path.dirname(path), exist_ok=True)
        with open(path, "w") as f:
            json.dump(out, f, indent=1)
            f.write("\n")
        return os.path.relpath(path, ROOT)
    except OSError:
        return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--full-out", default=os.path.join(ROOT, "gpurun_out", "bench_full.json"),
                    help="file that receives the full per-op tables (the last stdout line holds a compact form)")
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--all-configs", action="store_true", help="measure every op of all five configs with full iteration counts")
    ap.add_argument("--configs", default="", help="comma-separated subset for per_config (c1,c1_large,c2,c2_large,c3,c3_large,c4,c5,next,nmath,odd,bit,bit_large)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-per-config", action="store_true")
    ap.add_argument("--rotated-only", action="store_true",
                    help="leave out the same-buffer replay legs, so that a kernel trace of this command holds rotated launches only")
    ap.add_argument("--no-extras", action="store_true", help="skip the host transfer and host-cost measurements")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="also launch a plain contiguous copy of known size (256 MiB in, 256 MiB out) five times, so that a "
                         "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE run of this command can scale its counters by it")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus %d is not supported (the path has no cross-GPU stage)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import cumo_amd
    from cumo_amd import _lib
    lib = _lib.lib
    lib.cumo_cuda_runtime_free.argtypes = [C.c_void_p]
    if cumo_amd.device_count() < 1:
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)

    # ---- headline step: C2 -------------------------------------------------------
    host = inputs_c2()
    n = host["A"].shape[0]
    K = ROTATE_MAX_SETS
    sets = [config_ops("c2", cumo_amd, host) for _ in range(K)]
    env, ops = sets[0]
    step_bytes = sum(o[2] for o in ops)

    # The timed step is the chain as the extension's C host side runs it: three
    # calls into the library's host launch layer (broadcast, result allocation
    # from the pool, descriptors, launch). Only the Ruby VM above it is missing.
    # Consecutive steps take turns over K device copies of the inputs, and a step's
    # three results are released K steps later, so every buffer a step touches was
    # last used more than 1 GiB of traffic ago: nothing but the chain's own
    # producer -> consumer reuse (C is read right after it is written) can come
    # from a cache.
    NA = _lib.NArrayDesc
    descs = [(e["A"]._desc(), e["r"]._desc()) for e, _ in sets]
    na_binary, na_reduce, na_free = lib.cumo_hip_na_binary, lib.cumo_hip_na_reduce, lib.cumo_cuda_runtime_free
    ref = C.byref
    ring = [None] * K
    turn = [0]

    def step(rotate=True):
        j = turn[0] if rotate else 0
        old = ring[j]
        if old is not None:
            na_free(old[1].ptr)
            na_free(old[2].ptr)
            na_free(old[0].ptr)
        dA, dr = descs[j]
        zc, zs, zm = NA(), NA(), NA()
        na_binary(b"add", ref(dA), ref(dr), ref(zc))
        na_reduce(b"sum", ref(zc), 2, 0, 0, ref(zs), None)
        na_reduce(b"max", ref(zc), 2, 0, 0, ref(zm), None)
        ring[j] = (zc, zs, zm)
        if rotate:
            turn[0] = j + 1 if j + 1 < K else 0

    def timed_steps(rotate):
        for _ in range(max(args.warmup, K if rotate else 0)):
            step(rotate)
        _lib.check()
        cumo_amd.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step(rotate)
        cumo_amd.synchronize()
        dt = time.perf_counter() - t0
        _lib.check()
        return dt

    wall = timed_steps(True)
    ms_per_step = wall / args.steps * 1e3
    value = step_bytes / (wall / args.steps) / 1e9
    wall_replay = timed_steps(False) if not args.rotated_only else None   # the same step on one set of buffers, back to back
    for old in ring:
        if old is not None:
            for z in old:
                na_free(z.ptr)
    ring = None

    # the same step driven by the Python host mirror (descriptor building in
    # Python per op), for the record
    def py_step(j):
        e, o = sets[j % K]
        for _, fn, _, _ in o:
            fn(e)
    for j in range(K):
        py_step(j)
    cumo_amd.synchronize()
    t0 = time.perf_counter()
    for j in range(args.steps):
        py_step(j)
    cumo_amd.synchronize()
    ms_per_step_python_host = (time.perf_counter() - t0) / args.steps * 1e3

    # dominant kernel, per launch: HIP events on the launch stream around batches of
    # launches that take turns over the K sets (rotated: sustained HBM) and around
    # batches of the same launch on one set (replay: last-level cache helps)
    add_sets = []
    for e, o in sets:
        with _lib.record() as add_calls:
            o[0][1](e)
        add_sets.append(add_calls)
    timer = Timer(lib)
    add_bytes = ops[0][2]
    batch = 10
    pos = [0]

    def rotated(times):
        j = pos[0]
        for _ in range(times):
            for f, a in add_sets[j]:
                f(*a)
            j = j + 1 if j + 1 < K else 0
        pos[0] = j

    rotated(K)
    ts = sorted(timer.time(lambda: rotated(batch)) / batch for _ in range(max(20, args.steps)))
    avg_replay_ms = None
    if not args.rotated_only:
        _lib.replay(add_sets[0], 3)
        tr = sorted(timer.time(lambda: _lib.replay(add_sets[0], batch)) / batch for _ in range(max(20, args.steps)))
        avg_replay_ms = sum(tr) / len(tr)
    timer.close()
    avg_ms = sum(ts) / len(ts)
    achieved = add_bytes / (avg_ms * 1e-3) / 1e9
    roofline = {
        "bound": "hbm", "kernel": ADD_KERNEL + " (C = A + r, f64 4096x4096 + 1x4096)",
        "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
        "bytes_per_launch": int(add_bytes), "avg_launch_ms": round(avg_ms, 5), "median_launch_ms": round(ts[len(ts) // 2], 5),
        "method": "launches take turns over %d operand/result sets (%.2f GiB between two uses of a buffer)" % (K, (K - 1) * add_bytes / 2**30),
        "traffic": read_traffic_bytes(),
    }
    if avg_replay_ms is not None:
        roofline["frac_replay"] = round(add_bytes / (avg_replay_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
        roofline["avg_launch_ms_replay"] = round(avg_replay_ms, 5)
    del add_sets
    for e, _ in sets:
        e.clear()
    del sets, env, ops
    cumo_amd.MemoryPool.free_all_blocks()

    if args.pmc_calibration:
        src = cumo_amd.SFloat.zeros(1 << 26)
        for _ in range(5):
            dst = src.copy()  # ew_flat_kernel<OpCast<unsigned int, unsigned int>, 4, true>: reads 256 MiB, writes 256 MiB
        cumo_amd.synchronize()
        del src, dst
        cumo_amd.MemoryPool.free_all_blocks()

    per_config = {}
    if not args.no_per_config:
        names = [c for c in args.configs.split(",") if c] or ["c1", "c2", "c3", "c4", "c5", "c1_large", "c2_large", "c3_large", "next", "nmath", "odd", "bit", "bit_large"]
        iters, warm = (30, 5) if args.all_configs else (7, 2)
        for name in names:
            per_config[name] = {"workload": WORKLOAD_TEXT[name], "ops": measure_config(name, cumo_amd, lib, iters, warm, not args.rotated_only)}

    out = {
        "metric": METRIC, "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "value_replay": round(step_bytes / (wall_replay / args.steps) / 1e9, 1) if wall_replay else None, "ms_per_step_python_host": round(ms_per_step_python_host, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f64", "data": "synthetic",
        "config": {"workload": WORKLOAD_TEXT["c2"], "rotation": "steps take turns over %d device copies of the inputs; results are released %d steps later" % (K, K), "bytes_per_step": int(step_bytes), "launches_per_step": 3,
                   "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4), "gelem_per_s": round(3 * 4096 * 4096 / (wall / args.steps) / 1e9, 2)},
        "roofline": roofline,
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline_c2()
    if per_config:
        out["per_config"] = per_config
        if not args.no_extras:
            out["host_io"] = measure_host_io(lib)
            out["host_cost"] = measure_host_cost()
    full_path = write_full(out, args.full_out)
    print(final_line(out, full_path))


if __name__ == "__main__":
    main()
