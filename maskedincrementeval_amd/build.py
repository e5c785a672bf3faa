"""Build libmie_hip.so (hand-written HIP kernels for gfx950) in-tree with hipcc.

Usage: python -m maskedincrementeval_amd.build
The library is a plain C-ABI shared object (no torch / pybind headers); the
Python side loads it with ctypes (see _lib.py).
"""
import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_DIR = os.path.join(PKG_DIR, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libmie_hip.so")
SOURCES = ["mie_mask.hip", "mie_pointwise.hip", "mie_conv.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-fvisibility=hidden", "-fno-gpu-rdc",
    # keep the compiler from forming packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def find_hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", shutil.which("hipcc")):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, /opt/rocm/bin/hipcc, PATH)")


def build_library(verbose=True):
    """Compile every HIP source into lib/libmie_hip.so; returns its path."""
    os.makedirs(LIB_DIR, exist_ok=True)
    srcs = [os.path.join(CSRC, s) for s in SOURCES]
    tmp = LIB_PATH + ".tmp"
    cmd = [find_hipcc()] + HIPCC_FLAGS + srcs + ["-o", tmp]
    if verbose:
        print("[build]", " ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines()
                    if "packed-fp32-ops' is not a recognized feature" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out, flush=True)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library())
    sys.exit(0)
