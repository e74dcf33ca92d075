"""Builds libgptmi.so (the gfx950 kernels + C ABI) in-tree with hipcc.

    python -m gpt_triton_amd.build

hipcc cross-compiles for gfx950 without a GPU present.  The packed-fp32 VALU
instructions are disabled for all device code (-target-feature -packed-fp32-ops).
"""
import os
import shutil
import subprocess
import sys
import time
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "libgptmi.so")
SOURCES = ["rowops.hip", "gemm.hip", "flash_attn.hip", "capi.cpp"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-inline-asm",
]


def _hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found (looked on PATH and in /opt/rocm/bin)")
    return exe


def _compile(src, obj):
    cmd = [_hipcc(), *FLAGS, "-I", CSRC, "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{r.stderr[-4000:]}")
    return obj


def build(verbose=True):
    """Compiles every source and links libgptmi.so next to this file."""
    t0 = time.time()
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    objs = [os.path.join(objdir, s.rsplit(".", 1)[0] + ".o") for s in SOURCES]
    with ThreadPoolExecutor(max_workers=5) as ex:
        list(ex.map(_compile, SOURCES, objs))
    tmp = LIB_PATH + ".tmp"
    r = subprocess.run([_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs],
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr[-4000:]}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH} in {time.time() - t0:.1f}s", file=sys.stderr)
    return LIB_PATH


if __name__ == "__main__":
    build()
