"""Build libgalvatron_moe.so (the HIP kernels + C ABI) for gfx950 with hipcc.

Usage: `python hetu-galvatron_amd/build.py` or `build_library()` from Python.  The library is
written next to this file under `_lib/` so that it travels with the source tree.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "_lib")
LIB_PATH = os.path.join(LIB_DIR, "libgalvatron_moe.so")
SOURCES = ["route.hip", "losses.hip", "capacity.hip", "permute.hip", "glu.hip", "bias.hip", "gmm.hip", "gmm_dtl.hip", "gmm_fp8s.hip", "quant.hip", "norm.hip", "gate.hip", "abi.hip"]

# packed-fp32 instructions are switched off for every device compilation of this library
HIPCC_FLAGS = [
    "-O3",
    "--offload-arch=gfx950",
    "-fPIC",
    "-std=c++17",
    "-Wall",
    "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]

# loop headers of the GEMM kernels on 64-byte boundaries: the Mixtral-shape step 0.4 % faster in the
# same runs (the dW launches 0.9 %), the other shapes unchanged
SOURCE_FLAGS = {"gmm.hip": ["-falign-loops=64"], "gmm_dtl.hip": ["-falign-loops=64"]}


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the MoE kernels need the ROCm toolchain to build")
    return exe


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass warns that it does not know the packed-fp32 feature; drop that line only
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build_library(verbose: bool = False, extra_flags=()) -> str:
    """Compile every source under csrc/ and link the shared library.  Always recompiles."""
    hipcc = _hipcc()
    obj_dir = os.path.join(LIB_DIR, "obj")
    os.makedirs(obj_dir, exist_ok=True)
    objs = [os.path.join(obj_dir, s.replace(".hip", ".o")) for s in SOURCES]

    def compile_one(pair):
        src, obj = pair
        out = _run([hipcc, *HIPCC_FLAGS, *SOURCE_FLAGS.get(src, ()), *extra_flags, "-c", os.path.join(CSRC, src), "-o", obj])
        return src, out

    with ThreadPoolExecutor(max_workers=min(4, len(SOURCES))) as pool:
        for src, out in pool.map(compile_one, zip(SOURCES, objs)):
            if verbose and out.strip():
                print("[%s]\n%s" % (src, out))
    tmp = LIB_PATH + ".tmp"
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs])
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    path = build_library(verbose=True)
    print("built", path)
    sys.exit(0)
