"""Ahead-of-time build of libhtr_gfx950.so with hipcc (gfx950 only).

The reference JIT-builds its extension on first use (htr/ops.py:11-21 of the reference); here the
library is compiled explicitly and kept in-tree next to its source, and importing the package never
compiles anything.  Run `python -m htr_amd.build`.
"""
import os
import subprocess
import sys

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
LIB = os.path.join(CSRC, "libhtr_gfx950.so")
SOURCES = [os.path.join(CSRC, "htr_gfx950.hip")]          # one translation unit; the kernels live in the parts it includes
PARTS = [os.path.join(CSRC, f) for f in ("decode.hpp", "linear.hpp", "linear_batch.hpp", "linear_gemm.hpp", "dequant.hpp",
                                         "viterbi.hpp", "anchors.hpp", "plan.hpp")]
HEADER = os.path.join(os.path.dirname(CSRC), os.pardir, "include", "htr_gfx950.h")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-shared", "-fPIC",
    # keep the compiler from forming packed-FP32 VALU instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def hipcc():
    return os.environ.get("HIPCC") or os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "bin", "hipcc")


def build(verbose=False, extra=()):
    cmd = [hipcc()] + HIPCC_FLAGS + list(extra) + ["-o", LIB] + SOURCES
    if verbose:
        print(" ".join(cmd), flush=True)
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in p.stdout.splitlines() if "not a recognized feature" not in l)
    if p.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return LIB


def is_stale():
    if not os.path.exists(LIB):
        return True
    t = os.path.getmtime(LIB)
    return any(os.path.getmtime(s) > t for s in SOURCES + PARTS + [HEADER])


if __name__ == "__main__":
    print(build(verbose=True, extra=sys.argv[1:]))
