"""Build the C-ABI library ``csrc/libflashomni_hip.so`` for gfx950 with hipcc.

Usage: ``python -m flashomni_amd.build``.  hipcc cross-compiles without a GPU.
"""
import concurrent.futures
import os
import subprocess
import sys

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
LIB_PATH = os.path.join(CSRC, "libflashomni_hip.so")
SOURCES = ["fo_error.cpp", "planner.cpp", "packbits.hip", "decode.hip", "sparse_fa.hip", "gemm.hip",
           "quant_fp8.hip", "symbols.hip"]
# -packed-fp32-ops off: the compiler must not form packed fp32 VALU instructions on this target
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-x", "hip",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument"]


def _compile(src, verbose):
    obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
    cmd = ["hipcc"] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (src, res.stderr))
    if verbose and res.stderr.strip():
        lines = [l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l]
        if lines:
            sys.stderr.write("\n".join(lines) + "\n")
    return obj


def build(verbose=False):
    """Compile every source (in parallel) and link the shared library.  Returns its path."""
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(lambda s: _compile(s, verbose), SOURCES))
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n%s" % res.stderr)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
