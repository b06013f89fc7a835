"""Build recipe of the HIP library (``libegs_hip.so``) for gfx950.

``python -m expertscattergather_amd.build`` compiles ``csrc/egs_lib.hip`` in-tree with hipcc.
The library has no torch dependency; the Python side loads it with ctypes.
"""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "libegs_hip.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)
SOURCES = ["egs_lib.hip"]
HEADERS = ["egs_device.h", "egs_rows_gemm.h", "egs_dw.h", "egs_scatter_aux.h"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-munsafe-fp-atomics",                      # fp32 atomic add as one hardware instruction
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",   # no packed-fp32 VALU ops
    "-Wall", "-Wno-unused-function",
]


def hipcc() -> str:
    return os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def build(verbose: bool = False, extra_flags=()) -> str:
    """Compile the library (always recompiles) and return its path."""
    cmd = [hipcc(), *HIPCC_FLAGS, *extra_flags, "-I", os.path.join(os.path.dirname(HERE), "include"),
           *[os.path.join(CSRC, s) for s in SOURCES], "-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    noise = "is not a recognized feature for this target"
    out = "\n".join(l for l in res.stdout.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True, extra_flags=sys.argv[1:]))
