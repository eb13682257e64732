"""Builds the gfx950 kernel library ``libxpu_graph_amd.so`` in-tree with hipcc.

    python -m xpu_graph_amd.build            # compile every csrc/*.hip and link

hipcc cross-compiles for gfx950 without a GPU.  Objects go to ``csrc/_obj``; the
shared library lands beside this file so that it travels with the source tree.
"""
import concurrent.futures
import os
import shutil
import subprocess
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
OBJ_DIR = os.path.join(CSRC, "_obj")
LIB_PATH = os.path.join(_HERE, "libxpu_graph_amd.so")

ARCH = "gfx950"
# Packed fp32 instructions are switched off for every device compile: the
# compiler otherwise forms them on its own from plain float code.
HIPCC_FLAGS = [
    "-O3",
    "-std=c++17",
    "-fPIC",
    f"--offload-arch={ARCH}",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def hipcc_path():
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found: the mi355x target needs the ROCm toolchain to build its kernels")


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile_one(src):
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
    cmd = [hipcc_path(), *HIPCC_FLAGS, "-c", src, "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{proc.stderr}")
    return obj


def build_library(verbose=True, jobs=None):
    """Compile every kernel source for gfx950 and link the C-ABI shared library."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = sources()
    wanted = {os.path.basename(s)[:-4] + ".o" for s in srcs}
    for stale in set(os.listdir(OBJ_DIR)) - wanted:
        os.remove(os.path.join(OBJ_DIR, stale))
    jobs = jobs or min(len(srcs), max(1, (os.cpu_count() or 2) - 1), 8)
    if verbose:
        print(f"[xpu_graph_amd.build] hipcc {ARCH}: {len(srcs)} sources, {jobs} jobs", flush=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(_compile_one, srcs))
    tmp = LIB_PATH + ".tmp"
    cmd = [hipcc_path(), "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", tmp, *objs]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"[xpu_graph_amd.build] wrote {LIB_PATH}", flush=True)
    return LIB_PATH


if __name__ == "__main__":
    build_library()
    sys.exit(0)
