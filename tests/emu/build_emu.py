"""Builds tests/emu/libgdn_emu.so: the UNMODIFIED kernel sources of the package compiled for the host
with the fiber-based stand-in for the HIP runtime in this folder.  Test infrastructure only -- the
shipped library (mindspeed_mm_amd/lib/libgdn_mi355x.so) is built by hipcc and never links this."""
import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
CSRC = os.path.join(ROOT, "mindspeed-mm_amd", "csrc")
OUT = os.path.join(HERE, "libgdn_emu.so")
CLANG = os.environ.get("GDN_EMU_CXX", "/opt/rocm/llvm/bin/clang++")
FLAGS = ["-std=c++17", "-O2", "-g", "-fPIC", "-fno-strict-aliasing", "-Wno-unused-value", "-Wno-unknown-attributes",
         "-I", HERE, "-I", CSRC]


def _newer(src, dst, deps):
    if not os.path.exists(dst):
        return True
    t = os.path.getmtime(dst)
    return any(os.path.getmtime(d) > t for d in [src] + deps)


def build(force=False, verbose=False):
    os.makedirs(os.path.join(HERE, "obj"), exist_ok=True)
    deps = glob.glob(os.path.join(CSRC, "*.h")) + glob.glob(os.path.join(HERE, "hip", "*.h"))
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip"))) + [os.path.join(HERE, "emu_runtime.cpp")]
    objs, jobs = [], []
    for s in srcs:
        o = os.path.join(HERE, "obj", os.path.basename(s) + ".o")
        objs.append(o)
        if force or _newer(s, o, deps):
            jobs.append([CLANG, "-x", "c++", *FLAGS, "-c", s, "-o", o])

    def run(cmd):
        if verbose:
            print(" ".join(cmd), flush=True)
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("emu build failed:\n" + " ".join(cmd) + "\n" + r.stdout + r.stderr)

    with ThreadPoolExecutor(max_workers=6) as ex:
        list(ex.map(run, jobs))
    if jobs or not os.path.exists(OUT):
        run([CLANG, "-shared", "-o", OUT, *objs, "-lpthread"])
    return OUT


if __name__ == "__main__":
    print(build(force="--force" in sys.argv, verbose=True))
