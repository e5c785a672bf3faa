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
SOURCES = ["mie_mask.hip", "mie_pointwise.hip", "mie_conv.hip", "mie_conv_mfma_f32.hip",
           "mie_conv_mfma_bf16.hip", "mie_upconv_persist.hip", "mie_conv_fewcin.hip", "mie_events.hip", "mie_tail.hip", "mie_refresh.hip", "mie_tconv_mfma.hip"]

# Per-source additions.  The fp32 matrix-core kernels unroll their unit loops completely (up to 196 positions);
# without the higher threshold the compiler gives up on the longest ones (the 128-column 5x5 / 7x7 kernels), their
# operand ring is then indexed at run time and ends up in scratch memory (measured: 5.7 instead of 2.0 ms on the
# 8x120x160 5x5 conv).  The other sources are faster with the default.
EXTRA_FLAGS = {"mie_conv_mfma_f32.hip": ["-mllvm", "-pragma-unroll-threshold=65536"]}

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


def _run(cmd, verbose):
    if verbose:
        print("[build]", " ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines()
                    if "packed-fp32-ops' is not a recognized feature" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out, flush=True)


def build_library(verbose=True, incremental=False):
    """Compile every HIP source (one hipcc process per file, in parallel) and link
    lib/libmie_hip.so; returns its path.  incremental=True (`--incremental` on the command line)
    skips sources whose object file is newer than the source and every header."""
    from concurrent.futures import ThreadPoolExecutor
    os.makedirs(LIB_DIR, exist_ok=True)
    obj_dir = os.path.join(LIB_DIR, "obj")
    os.makedirs(obj_dir, exist_ok=True)
    hipcc = find_hipcc()
    compile_flags = [f for f in HIPCC_FLAGS if f != "-shared"]
    jobs = []
    headers = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    headers.append(os.path.join(os.path.dirname(PKG_DIR), "include", "mie.h"))
    newest_header = max(os.path.getmtime(h) for h in headers)
    for s in SOURCES:
        obj = os.path.join(obj_dir, s.replace(".hip", ".o"))
        src = os.path.join(CSRC, s)
        fresh = (incremental and os.path.exists(obj)
                 and os.path.getmtime(obj) > max(os.path.getmtime(src), newest_header))
        jobs.append(([hipcc] + compile_flags + EXTRA_FLAGS.get(s, []) + ["-c", src, "-o", obj], obj, fresh))
    with ThreadPoolExecutor(max_workers=min(len(jobs), 8)) as pool:
        list(pool.map(lambda j: None if j[2] else _run(j[0], verbose), jobs))
    tmp = LIB_PATH + ".tmp"
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc"] + [j[1] for j in jobs] + ["-o", tmp],
         verbose)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(incremental="--incremental" in sys.argv[1:]))
    sys.exit(0)
