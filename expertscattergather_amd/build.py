"""Build recipe of the HIP library (``libegs_hip.so``) for gfx950.

``python -m expertscattergather_amd.build`` compiles the ``csrc/*.hip`` translation units in-tree with hipcc.
The library has no torch dependency; the Python side loads it with ctypes.  A small CPython module
(``csrc/egs_pycall.c``, built with the host C compiler against the same library) lets the four launchers be
called with plain integers, which costs a fraction of a ctypes call; without it the Python side uses ctypes.
"""
from __future__ import annotations

import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "libegs_hip.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)
SOURCES = ["egs_lib.hip", "egs_rows_launch.hip", "egs_dw_launch.hip", "egs_f8_launch.hip", "egs_mlp_launch.hip", "egs_pass_launch.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-munsafe-fp-atomics",                      # fp32 atomic add as one hardware instruction
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",   # no packed-fp32 VALU ops
    "-Wall", "-Wno-unused-function",
    # the direct-to-LDS loads are inline assembly that sets M0 (the LDS base of the load) and names it as
    # clobbered; the compiler warns once per instantiation that M0 is a reserved register
    "-Wno-inline-asm",
]
NOISE = "is not a recognized feature for this target"


def hipcc() -> str:
    return os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if NOISE not in l)
    if res.returncode != 0:
        raise RuntimeError(os.path.basename(cmd[0]) + " failed:\n" + out)
    if verbose and out.strip():
        print(out)


def build(verbose: bool = False, extra_flags=()) -> str:
    """Compile the library (always recompiles) and return its path.

    The translation units are compiled side by side (object files under ``csrc/_obj``), then linked."""
    from concurrent.futures import ThreadPoolExecutor
    obj_dir = os.path.join(CSRC, "_obj")
    os.makedirs(obj_dir, exist_ok=True)
    inc = ["-I", os.path.join(os.path.dirname(HERE), "include")]
    objs = [os.path.join(obj_dir, s.replace(".hip", ".o")) for s in SOURCES]
    cmds = [[hipcc(), *HIPCC_FLAGS, *extra_flags, *inc, "-c", os.path.join(CSRC, s), "-o", o] for s, o in zip(SOURCES, objs)]
    with ThreadPoolExecutor(max_workers=len(cmds)) as pool:
        list(pool.map(lambda c: _run(c, verbose), cmds))
    _run([hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB_PATH], verbose)
    build_pycall(verbose)
    return LIB_PATH


PYCALL_PATH = os.path.join(HERE, "_egs_pycall" + (sysconfig.get_config_var("EXT_SUFFIX") or ".so"))


def build_pycall(verbose: bool = False) -> str:
    """Compile the CPython module that calls the launchers with integer arguments; it finds libegs_hip.so next to itself."""
    cc = os.environ.get("CC", "gcc")
    cmd = [cc, "-O2", "-fPIC", "-shared", "-Wall", "-I", sysconfig.get_paths()["include"],
           "-I", os.path.join(os.path.dirname(HERE), "include"), os.path.join(CSRC, "egs_pycall.c"),
           "-L", HERE, "-legs_hip", "-Wl,-rpath,$ORIGIN", "-o", PYCALL_PATH]
    _run(cmd, verbose)
    return PYCALL_PATH


if __name__ == "__main__":
    print(build(verbose=True, extra_flags=sys.argv[1:]))
