"""Builds libckopt.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

Usage: python build.py [--jobs N] [--force]
Every translation unit under csrc/ is compiled to build/<name>.o (in parallel) and linked into lib/libckopt.so
next to this file; measure/ (the bare inner-loop probe bench.py reports a ceiling from) becomes the separate
lib/libckmeasure.so, which the product library does not contain. hipcc cross-compiles gfx950 code objects without a GPU.
"""
import argparse
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
MEASURE = os.path.join(HERE, "measure")
BUILD = os.path.join(HERE, "build")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libckopt.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
DEVICE_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed fp32 VALU forms are kept out of all device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-x", "c++"]


def sources(root=CSRC):
    out = []
    for name in sorted(os.listdir(root)):
        if name.endswith(".hip") or name.endswith(".cpp"):
            out.append(os.path.join(root, name))
    return out


def headers_mtime():
    m = 0.0
    for root in (CSRC, MEASURE, os.path.join(HERE, "..", "include")):
        for name in os.listdir(root):
            if name.endswith((".h", ".inc")):
                m = max(m, os.path.getmtime(os.path.join(root, name)))
    return m


def compile_one(src, force, build_dir=None, extra=()):
    obj = os.path.join(build_dir or BUILD, os.path.basename(src) + ".o")
    if not force and os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(src), headers_mtime()):
        return obj, "up to date"
    flags = (DEVICE_FLAGS if src.endswith(".hip") else HOST_FLAGS) + list(extra)
    cmd = [HIPCC] + flags + ["-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("compile failed: %s\n%s\n%s" % (" ".join(cmd), r.stdout, r.stderr))
    return obj, "compiled"


def build(jobs=8, force=False, verbose=True, out_dir=None, extra=()):
    """out_dir/extra: build a variant (extra compiler flags, e.g. a -D define) into another directory."""
    build_dir = os.path.join(out_dir, "build") if out_dir else BUILD
    lib_dir = out_dir if out_dir else LIBDIR
    lib = os.path.join(lib_dir, "libckopt.so")
    os.makedirs(build_dir, exist_ok=True)
    os.makedirs(lib_dir, exist_ok=True)
    srcs = sources()
    msrcs = sources(MEASURE)
    objs, mobjs = [], []
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        for src, (obj, what) in zip(srcs + msrcs, ex.map(lambda s: compile_one(s, force, build_dir, extra), srcs + msrcs)):
            if verbose:
                print("[build] %-40s %s" % (os.path.basename(obj), what), flush=True)
            (mobjs if src in msrcs else objs).append(obj)
    for target, members in ((lib, objs), (os.path.join(lib_dir, "libckmeasure.so"), mobjs)):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", target] + members
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed: %s\n%s\n%s" % (" ".join(cmd), r.stdout, r.stderr))
        if verbose:
            print("[build] linked %s" % target, flush=True)
    return lib


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--jobs", type=int, default=min(8, os.cpu_count() or 1))
    ap.add_argument("--force", action="store_true")
    ap.add_argument("--out-dir", default=None)
    ap.add_argument("--define", action="append", default=[])
    a = ap.parse_args()
    build(a.jobs, a.force, out_dir=a.out_dir, extra=["-D" + d for d in a.define])
    sys.exit(0)
