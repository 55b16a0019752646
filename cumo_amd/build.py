"""Builds cumo_amd/libcumo_hip.so (gfx950) from cumo_amd/csrc with hipcc.

One hipcc invocation per translation unit, run in parallel, then one link. The
library is kept in-tree next to this file; nothing is installed.

    python cumo_amd/build.py [-j N] [--force]

(run as a script, not with -m: importing the package loads the library)
"""
import argparse
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libcumo_hip.so")
HOST_COST_TOOL = os.path.join(HERE, "bench_host_cost")

ARCH = "gfx950"
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
COMMON = [
    "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fvisibility=hidden", "-fvisibility-inlines-hidden",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
    "-Wall", "-Wno-unused-function", "-Wno-deprecated-declarations",
]
# device code: no packed FP32 forms
# --offload-compress: the device code of every unit is stored compressed in the library (a third of
# the size; the runtime unpacks it once when the library is loaded)
DEVICE = ["--offload-arch=" + ARCH, "--offload-compress", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def sources():
    out = []
    for name in sorted(os.listdir(CSRC)):
        if name.endswith(".hip") or name.endswith(".cpp"):
            out.append(os.path.join(CSRC, name))
    return out


def deps_newer_than(obj):
    """True when the source or any header the object was compiled from (its .d file, written
    by -MD) is newer than the object, or when that list is missing."""
    dep = obj + ".d"
    try:
        m = os.path.getmtime(obj)
        with open(dep) as f:
            text = f.read()
    except OSError:
        return True
    text = text.replace("\\\n", " ")
    files = text.split(":", 1)[1].split() if ":" in text else []
    if not files:
        return True
    for path in files:
        try:
            if os.path.getmtime(path) > m:
                return True
        except OSError:
            return True
    return False


def compile_one(src, force):
    obj = os.path.join(OBJ, os.path.basename(src) + ".o")
    if not force and not deps_newer_than(obj):
        return obj, "", 0
    dep = ["-MD", "-MF", obj + ".d"]
    if src.endswith(".hip"):
        cmd = [HIPCC] + DEVICE + COMMON + dep + ["-c", "-x", "hip", src, "-o", obj]
    else:
        cmd = [HIPCC] + COMMON + dep + ["-x", "hip", "--offload-arch=" + ARCH, "--offload-compress", "-c", src, "-o", obj]
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    log = "\n".join(l for l in p.stdout.splitlines() if "packed-fp32-ops' is not a recognized feature" not in l)
    return obj, log, p.returncode


def drop_stale_objects(srcs):
    """Objects (and their dependency lists) whose source file no longer exists."""
    keep = {os.path.basename(s) + ".o" for s in srcs}
    for name in os.listdir(OBJ):
        base = name[:-2] if name.endswith(".d") else name
        if base.endswith(".o") and base not in keep:
            os.remove(os.path.join(OBJ, name))


def build(jobs=None, force=False, verbose=True):
    os.makedirs(OBJ, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)
    srcs = sources()
    drop_stale_objects(srcs)
    objs = []
    failed = False
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        futs = {ex.submit(compile_one, s, force): s for s in srcs}
        for f in concurrent.futures.as_completed(futs):
            obj, log, rc = f.result()
            if verbose and (log.strip() or rc):
                print("== %s (rc=%d)\n%s" % (os.path.basename(futs[f]), rc, log), flush=True)
            if rc:
                failed = True
            objs.append(obj)
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=" + ARCH, "--offload-compress", "-Wl,--version-script=" + os.path.join(CSRC, "exports.map"),
           "-o", LIB] + sorted(objs)
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if p.returncode:
        print(p.stdout)
        raise RuntimeError("link failed")
    build_host_cost_tool()
    return LIB


def build_host_cost_tool():
    """bench_host_cost.cpp (repository root) -> cumo_amd/bench_host_cost, linked against the library."""
    src = os.path.join(ROOT, "bench_host_cost.cpp")
    if not os.path.exists(src):
        return
    cmd = [HIPCC, "-O2", "-std=c++17", "--offload-arch=" + ARCH, "-x", "hip", "-I" + os.path.join(ROOT, "include"), src,
           "-o", HOST_COST_TOOL, "-L" + HERE, "-lcumo_hip", "-Wl,-rpath,$ORIGIN"]
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if p.returncode:
        print(p.stdout)
        raise RuntimeError("bench_host_cost: hipcc failed")


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("-j", type=int, default=None)
    ap.add_argument("--force", action="store_true")
    a = ap.parse_args()
    print(build(a.j, a.force))
