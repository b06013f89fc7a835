"""ctypes binding of the C ABI in ``include/egs_hip.h`` (``libegs_hip.so``).

There is no CPU fallback: if the library has not been built, or a tensor is not on a HIP
device, the callers raise.
"""
from __future__ import annotations

import ctypes
import os
import threading

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libegs_hip.so")

# enums of include/egs_hip.h
EGS_OK = 0
EGS_ERR_BAD_DTYPE = -3
EGS_ERR_WORKSPACE = -6
EGS_ERR_HIP = -8
EGS_ERR_SCRATCH_LIMIT = -11
BUILTIN_SCRATCH_BYTES = 16 << 20
F32, F16, BF16, FP8_E4M3 = 0, 1, 2, 3
IND_I16, IND_I32, IND_I64, IND_U8 = 0, 1, 2, 3
W_EIJ, W_EJI = 0, 1
SCATTER_DETERMINISTIC, SCATTER_ATOMIC, SCATTER_COMPACT = 0, 1, 2
OP_GATHER_GEMM, OP_GEMM_SCATTER, OP_DW, OP_GATHER_BACKWARD, OP_SCATTER_BACKWARD = 0, 1, 2, 3, 4
ACT_NONE, ACT_RELU, ACT_GELU, ACT_SILU, ACT_GELU_TANH = 0, 1, 2, 3, 4
EGS_ERR_UNSUPPORTED = -9
ABI_VERSION = 1


class Dims(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in ("B", "T", "E", "K", "I", "J")]


_vp, _i, _i64, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_size_t
_dp = ctypes.POINTER(Dims)

# name -> (restype, argtypes); mirrors include/egs_hip.h declaration by declaration
SIGNATURES = {
    "egs_abi_version": (_i, []),
    "egs_status_string": (ctypes.c_char_p, [_i]),
    "egs_last_hip_error": (ctypes.c_char_p, []),
    "egs_testing_force_generic": (None, [_i]),       # include/egs_hip_testing.h
    "egs_testing_launch_log_begin": (None, []),
    "egs_testing_launch_log_end": (_sz, [ctypes.c_char_p, _sz]),
    "egs_workspace_bytes": (_sz, [_i, _i, _dp, _i]),
    "egs_gather_gemm": (_i, [_vp, _vp, _vp, _vp, _vp, _dp, _i64, _i64, _i, _i, _i, _i, _vp]),
    "egs_gemm_scatter": (_i, [_vp, _vp, _vp, _vp, _vp, _sz, _dp, _i, _i, _i, _i, _vp]),
    "egs_dw": (_i, [_vp, _vp, _vp, _vp, _vp, _sz, _dp, _i64, _i64, _i, _i, _i, _i, _vp]),
    "egs_dw_builtin_scratch": (_i, [_vp, _vp, _vp, _vp, _dp, _i64, _i64, _i, _i, _i, _i, _vp]),
    "egs_gather_gemm_fp8act_workspace_bytes": (_sz, [_dp]),
    "egs_gather_gemm_fp8act": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _dp, _i64, _i64, _i, _vp]),
    "egs_expert_gather_forward": (_i, [_vp, _vp, _vp, _vp, _dp, _i64, _i64, _i, _i, _vp]),
    "egs_expert_gather_backward": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _dp, _i64, _i64, _i, _i, _i, _vp]),
    "egs_expert_scatter_forward": (_i, [_vp, _vp, _vp, _vp, _vp, _sz, _dp, _i, _i, _i, _vp]),
    "egs_expert_scatter_backward": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _dp, _i64, _i64, _i, _i, _vp]),
    "egs_validate_indices": (_i, [_vp, _i, _i64, ctypes.c_int32, _vp, _vp]),
    "egs_routing_table_bytes": (_sz, [_dp, _i]),
    "egs_stream_capture_id": (_i, [_vp, ctypes.POINTER(ctypes.c_ulonglong)]),
    "egs_expert_gather_forward_table": (_i, [_vp, _vp, _vp, _vp, _vp, _sz, _dp, _i64, _i64, _i, _i, _vp]),
    "egs_expert_scatter_forward_table": (_i, [_vp, _vp, _vp, _vp, _sz, _vp, _vp, _sz, _dp, _i, _i, _i, _vp]),
    "egs_expert_gather_backward_table": (_i, [_vp, _vp, _vp, _vp, _sz, _vp, _vp, _vp, _vp, _sz, _dp, _i64, _i64, _i, _i, _i, _vp]),
    "egs_expert_mlp_supported": (_i, [_dp, _i]),
    "egs_expert_mlp_forward": (_i, [_vp, _vp, _vp, _vp, _vp, _dp, _i64, _i64, _i, _i, _i, _vp]),
}

_lib = None
_lock = threading.Lock()


def is_built() -> bool:
    return os.path.exists(LIB_PATH)


def lib() -> ctypes.CDLL:
    """Load the HIP library once (thread-safe)."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            if not is_built():
                raise RuntimeError(
                    f"{LIB_PATH} is missing: build the HIP library first "
                    "(python -m expertscattergather_amd.build); there is no CPU fallback")
            handle = ctypes.CDLL(LIB_PATH)
            for name, (res, args) in SIGNATURES.items():
                fn = getattr(handle, name)
                fn.restype, fn.argtypes = res, args
            got = handle.egs_abi_version()
            if got != ABI_VERSION:
                raise RuntimeError(f"libegs_hip.so has ABI version {got}, expected {ABI_VERSION}; rebuild it")
            _lib = handle
    return _lib


_pycall = False          # False: not looked for yet; None: not available


def pycall():
    """The CPython module that calls the four launchers of the same library with plain integers (a fraction of the
    cost of a ctypes call), or None when it has not been built: callers then use ctypes.  Loads the library first,
    so a missing library is reported the same way on both routes."""
    global _pycall
    if _pycall is False:
        lib()
        with _lock:
            if _pycall is False:
                try:
                    from . import _egs_pycall as mod
                    _pycall = mod if mod.abi_version() == ABI_VERSION else None
                except ImportError:
                    _pycall = None
    return _pycall


class launch_log:
    """``with launch_log() as log: ...`` - afterwards ``log.kernels`` lists the kernels the calls of this thread
    launched inside the block (include/egs_hip_testing.h)."""

    def __enter__(self):
        self.kernels = []
        lib().egs_testing_launch_log_begin()
        return self

    def __exit__(self, *exc):
        buf = ctypes.create_string_buffer(1024)
        lib().egs_testing_launch_log_end(buf, len(buf))
        self.kernels = [k for k in buf.value.decode().split(",") if k]
        return False


def status_string(status: int) -> str:
    return lib().egs_status_string(status).decode()


def check(status: int, what: str) -> None:
    """Turn a negative egs_status into the exception the reference would raise."""
    if status == EGS_OK:
        return
    msg = status_string(status)
    if status == EGS_ERR_BAD_DTYPE:
        raise ValueError(msg)                      # reference: ValueError("Unknown dtype")
    if status == EGS_ERR_HIP:
        msg += ": " + lib().egs_last_hip_error().decode()
    raise RuntimeError(f"{what}: {msg} (egs_status {status})")
