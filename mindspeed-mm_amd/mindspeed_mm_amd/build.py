"""Builds lib/libgdn_mi355x.so: the hand-written HIP kernels and their C-ABI, for gfx950 only.

hipcc cross-compiles without a GPU, so this runs anywhere ROCm is installed.  The library is kept
in-tree (git-ignored) next to the Python package that loads it."""
import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(PKG), "csrc")
LIBDIR = os.path.join(PKG, "lib")
LIB = os.path.join(LIBDIR, "libgdn_mi355x.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# -packed-fp32-ops is switched off on purpose: the compiler must not form v_pk_*_f32 on this target.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wno-unused-value", "-I", CSRC]


def _stale(src, obj, deps):
    if not os.path.exists(obj):
        return True
    t = os.path.getmtime(obj)
    return any(os.path.getmtime(d) > t for d in [src] + deps)


def build(force=True, verbose=False, jobs=6):
    """Compile every csrc/*.hip and link the shared library.  force=False only rebuilds stale objects."""
    os.makedirs(os.path.join(LIBDIR, "obj"), exist_ok=True)
    deps = glob.glob(os.path.join(CSRC, "*.h"))
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    if not srcs:
        raise RuntimeError("no HIP sources under " + CSRC)
    objs, cmds = [], []
    for s in srcs:
        o = os.path.join(LIBDIR, "obj", os.path.basename(s)[:-4] + ".o")
        objs.append(o)
        if force or _stale(s, o, deps):
            cmds.append([HIPCC, *FLAGS, "-c", s, "-o", o])

    def run(cmd):
        if verbose:
            print(" ".join(cmd), flush=True)
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("HIP build failed:\n" + " ".join(cmd) + "\n" + r.stdout + r.stderr)
        return r

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(run, cmds))
    if cmds or not os.path.exists(LIB):
        run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs])
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv, verbose=True))
