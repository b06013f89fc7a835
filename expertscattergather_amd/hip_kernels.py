"""Launchers and autograd Functions of the fused expert gather / scatter-with-linear path.

Same surface as the reference's ``egs/triton_kernels.py``: ``create_kernels()`` binds the four
module-level callables

    expert_gather_forward_call  (X[B,T,I], W[E,I,J], Ind[B,E,K], out_dtype)          -> Y[B,E,K,J]
    expert_gather_backward_call (X, W, Ind, grad_output[B,E,K,J], dtype)             -> (grad_X, grad_W)
    expert_scatter_forward_call (Y[B,E,K,J], W[E,J,I], Ind[B,E,K], T, out_dtype)     -> X[B,T,I]
    expert_scatter_backward_call(Y, W, Ind, grad_X[B,T,I], dtype)                    -> (grad_Y, grad_W)

(reference egs/triton_kernels.py:26-29, :361-578) and ``ExpertGatherFunction`` /
``ExpertScatterFunction`` (reference :581-639) call them.  Here the callables allocate the
outputs with torch and hand raw device pointers to the HIP library through its C ABI on the
current stream; they are registered as ``torch.library`` custom ops with fake implementations
so that ``torch.compile`` can trace through them.
"""
from __future__ import annotations

import ctypes
import os
import threading

import torch

from . import _abi

__all__ = [
    "create_kernels", "dtype_to_type_id", "ExpertGatherFunction", "ExpertScatterFunction",
    "set_scatter_mode", "get_scatter_mode", "scatter_mode_scope", "expert_gather_fp8w_forward", "expert_gather_fp8_forward", "validate_indices",
    "register_reference_namespace", "release_workspaces", "expert_mlp_forward", "expert_mlp", "ExpertMLPFunction",
    "set_routing_table_cache", "invalidate_routing_table",
]

OP_NAMESPACE = "egs_amd"


def dtype_to_type_id(dtype: torch.dtype) -> int:
    """float32 -> 0, float16 -> 1, bfloat16 -> 2 (reference egs/triton_kernels.py:15-23)."""
    if dtype == torch.float32:
        return _abi.F32
    if dtype == torch.float16:
        return _abi.F16
    if dtype == torch.bfloat16:
        return _abi.BF16
    raise ValueError("Unknown dtype")


_IND_IDS = {torch.int16: _abi.IND_I16, torch.int32: _abi.IND_I32, torch.int64: _abi.IND_I64, torch.uint8: _abi.IND_U8}


def _ind_type_id(Ind: torch.Tensor) -> int:
    try:
        return _IND_IDS[Ind.dtype]
    except KeyError:
        raise ValueError(f"Ind must be uint8, int16, int32 or int64, got {Ind.dtype}") from None


# ------------------------------------------------------------------------------ scatter mode
_MODES = {"deterministic": _abi.SCATTER_DETERMINISTIC, "atomic": _abi.SCATTER_ATOMIC, "compact": _abi.SCATTER_COMPACT}
_scatter_mode = os.environ.get("EGS_SCATTER_MODE", "deterministic").lower()
if _scatter_mode not in _MODES:
    raise ValueError(f"EGS_SCATTER_MODE must be one of {sorted(_MODES)}, got {_scatter_mode!r}")
_mode_local = threading.local()         # .override: the mode of the innermost scatter_mode_scope of this thread


def _check_mode(mode: str) -> str:
    mode = mode.lower()
    if mode not in _MODES:
        raise ValueError(f"scatter mode must be one of {sorted(_MODES)}, got {mode!r}")
    return mode


def set_scatter_mode(mode: str) -> None:
    """Process-wide default: 'deterministic' (fixed summation order, bitwise reproducible), 'atomic' (fp32
    atomics; 16-bit types: product rows kept in the element type) or 'compact' (deterministic without
    scratch memory: where the sizes allow, product rows never leave the compute unit and the picks are sorted there
    too - 0 bytes instead of 270 MB at B16 T1024 E64 K128 I512 J128 - slower per launch at large shapes with even
    routing).  A module's ``scatter_mode`` attribute and
    ``scatter_mode_scope`` take precedence.  A forward call binds the mode in force to its autograd node: the
    backward of that call runs in the same mode whatever is set by then."""
    global _scatter_mode
    _scatter_mode = _check_mode(mode)


def get_scatter_mode() -> str:
    """The mode a scatter issued now by this thread would run in."""
    return getattr(_mode_local, "override", None) or _scatter_mode


class scatter_mode_scope:
    """``with scatter_mode_scope("atomic"): ...`` - the calls this thread makes inside run in that mode
    (``None``: whatever is in force outside)."""

    def __init__(self, mode):
        self.mode = None if mode is None else _check_mode(mode)

    def __enter__(self):
        self.outer = getattr(_mode_local, "override", None)
        if self.mode is not None:
            _mode_local.override = self.mode
        return self

    def __exit__(self, *exc):
        _mode_local.override = self.outer
        return False


# ------------------------------------------------------------------------------ plumbing
def _require_gpu(*tensors: torch.Tensor) -> torch.device:
    dev = tensors[0].device
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError(
                "the egs HIP kernels need tensors on an AMD GPU (HIP device), got a tensor on "
                f"'{t.device}'; there is no CPU fallback")
        if t.device != dev:
            raise RuntimeError(f"all tensors must be on the same device, got {dev} and {t.device}")
    return dev


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream_ptr(dev: torch.device) -> int:
    if _raw_stream is not None:
        return _raw_stream(dev.index)
    return torch.cuda.current_stream(dev).cuda_stream


class _NoSwitch:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def _on_device(dev: torch.device):
    """Context that makes `dev` the current HIP device (the library launches on the current device);
    nothing to do, and nothing paid, when it already is."""
    if dev.index == torch.cuda.current_device():
        return _NO_SWITCH
    return torch.cuda.device(dev)


def _workspace(dev: torch.device, nbytes: int):
    """Scratch for one call: (tensor that owns it or None, pointer, nbytes).

    Allocated per call through torch's caching allocator, which is stream-ordered and aware of graph
    capture: a buffer handed out during capture belongs to the graph's pool and stays valid for every
    replay, and a buffer of an eager call is not reused by another stream before the call's kernels have
    run.  (A buffer cached across calls would have its address baked into captured graphs and could be
    freed or regrown underneath them.)  The caller keeps the tensor alive until the launch is enqueued."""
    if nbytes == 0:
        return None, None, 0
    buf = torch.empty(int(nbytes), dtype=torch.uint8, device=dev)
    return buf, buf.data_ptr(), int(nbytes)


def release_workspaces() -> None:
    """Kept for callers of earlier versions, which cached one scratch buffer per stream; scratch is now
    allocated per call, so there is nothing to release."""


def _dense16(t: torch.Tensor, ct: torch.dtype) -> torch.Tensor:
    """`t` in the compute dtype, contiguous and starting on a 16-byte boundary (nothing is done, and nothing paid, when
    it already is).  egs_workspace_bytes() sizes the scratch for operands like that (they take the specialised
    kernels); a view that starts at an odd element offset is copied rather than sent down the general kernels with
    a workspace sized for the others."""
    if t.dtype is ct and t.is_contiguous() and t.data_ptr() % 16 == 0:
        return t
    t = t.to(ct).contiguous()
    return t.clone() if t.data_ptr() % 16 else t


_ws_sizes: dict = {}
_dims_structs: dict = {}
_cache_lock = threading.Lock()          # the caches are filled without it (a lost insert costs one recomputation); emptying is exclusive


def _dims_struct(dims: tuple):
    """The egs_dims structure of a problem, built once per problem (the library only reads it)."""
    d = _dims_structs.get(dims)
    if d is None:
        d = _abi.Dims(*dims)
        with _cache_lock:
            if len(_dims_structs) > 4096:
                _dims_structs.clear()
            _dims_structs[dims] = d
    return d


def _workspace_bytes(op: int, mode: int, dims: tuple, dt: int) -> int:
    """egs_workspace_bytes(), remembered per problem: a pure function of its arguments, except for the test-suite's
    switch egs_testing_force_generic, after which `_ws_sizes` has to be cleared."""
    key = (op, mode, dims, dt)
    n = _ws_sizes.get(key)
    if n is None:
        n = int(_abi.lib().egs_workspace_bytes(op, mode, _abi.Dims(*dims), dt))
        with _cache_lock:
            if len(_ws_sizes) > 4096:
                _ws_sizes.clear()
            _ws_sizes[key] = n
    return n


def _rows_source(X: torch.Tensor, ct: torch.dtype):
    """[B,T,I] tensor -> (tensor in the compute dtype with unit inner stride, batch stride, token stride)."""
    if X.dtype is ct and X.is_contiguous() and X.data_ptr() % 16 == 0:
        return X, X.shape[1] * X.shape[2], X.shape[2]
    X = X.to(ct)
    if X.stride(2) != 1 and X.shape[2] > 1:
        X = X.contiguous()
    B, T, I = X.shape
    ld_t = X.stride(1) if T > 1 else max(I, 1)
    ld_b = X.stride(0) if B > 1 else ld_t * max(T, 1)
    es = X.element_size()
    if ld_t < I or ld_b < 0 or ((I * es) % 16 == 0 and ((ld_t * es) % 16 or (ld_b * es) % 16)):
        # overlapping rows, or strides that would take rows off the 16-byte grid their width allows
        X = X.contiguous()
        ld_t, ld_b = I, T * I
    if X.data_ptr() % 16:
        X = X.contiguous().clone() if not X.is_contiguous() else X.clone()
        ld_t, ld_b = I, T * I
    return X, ld_b, ld_t


def _check_shapes(X3, W, Ind, Y4, w_is_eij: bool):
    """Common shape checks; X3 is the [B,T,I] side, Y4 the [B,E,K,J] side (either may be None)."""
    if W.dim() != 3 or Ind.dim() != 3:
        raise ValueError("W must be 3-D and Ind must be [B,E,K]")
    E = W.shape[0]
    I, J = (W.shape[1], W.shape[2]) if w_is_eij else (W.shape[2], W.shape[1])
    B, E2, K = Ind.shape
    if E2 != E:
        raise ValueError(f"Ind has {E2} experts but W has {E}")
    if X3 is not None:
        if X3.dim() != 3 or X3.shape[0] != B or X3.shape[2] != I:
            raise ValueError(f"expected a [B={B},T,I={I}] tensor, got {tuple(X3.shape)}")
    if Y4 is not None:
        if Y4.dim() != 4 or tuple(Y4.shape) != (B, E, K, J):
            raise ValueError(f"expected a [B={B},E={E},K={K},J={J}] tensor, got {tuple(Y4.shape)}")
    return B, E, K, I, J


_FLOATS = (torch.float32, torch.float16, torch.bfloat16)


def _compute_dtype(out_dtype: torch.dtype, *tensors: torch.Tensor) -> torch.dtype:
    """The element type the kernels multiply in, following the reference's kernels (egs/triton_kernels.py:122-127,
    :131-136): ``out_dtype`` float16 / bfloat16 casts both operands to it; float32 leaves them as they are, i.e.
    operands that already share a 16-bit type are multiplied in that type (fp32 accumulation either way), and
    operands of different types meet in float32.  Results are returned in the dtype of the tensor they are the
    gradient of / the activation they continue (:375, :408-409, :457, :491-492)."""
    first = tensors[0].dtype
    same = True
    for t in tensors:
        if t.dtype not in _FLOATS:
            raise ValueError("Unknown dtype")
        same = same and t.dtype is first
    if out_dtype is torch.float32:
        return first if same else torch.float32
    dtype_to_type_id(out_dtype)
    return out_dtype


# ------------------------------------------------------------------------------ routing table kept with Ind
# The one-kernel scatter of small experts sorts the picks of a batch element by token before it adds product rows in a
# fixed order.  That order is a function of Ind alone, so the gather forward - the first call of a layer that sees Ind -
# builds it in its own launch (a few extra workgroups) and leaves it with the Ind tensor OBJECT; the scatter forward and
# the gather's backward that are handed the same object, unchanged, read it instead of sorting again.  The entry is
# tied to the object's data pointer, shape, dtype, version counter, T and stream, so it dies with the tensor and
# is ignored after any in-place write that autograd can see.  A write that bypasses the version counter (a custom
# kernel through data_ptr, `Ind.data`'s own counter) is not seen - the same blind spot autograd's saved-tensor check has;
# call invalidate_routing_table(Ind) after such a write, or set_routing_table_cache(False).  A table filled by a launch
# that is being captured into a graph holds nothing until the graph is replayed, and lives in the graph's memory pool: the
# entry carries the capture's identifier and serves only calls recorded into the same capture (replays rebuild it from
# whatever Ind then holds, because the launch that fills it is part of the graph).
_TABLE_ATTR = "_egs_routing_table"
_table_cache = os.environ.get("EGS_ROUTING_TABLE_CACHE", "1") != "0"
_table_sizes: dict = {}


def set_routing_table_cache(enabled: bool) -> None:
    """Switch the reuse of routing tables between calls that share an Ind tensor on or off (default on,
    EGS_ROUTING_TABLE_CACHE=0 turns it off); results are bit-identical either way."""
    global _table_cache
    _table_cache = bool(enabled)


def invalidate_routing_table(Ind: torch.Tensor) -> None:
    """Forget the routing table kept with `Ind` (after writing into it through a channel its version counter does not see)."""
    Ind.__dict__.pop(_TABLE_ATTR, None)


def _capture_id(stream: int) -> int:
    """0 outside graph capture, the capture's identifier inside one, -1 if it cannot be told (then: no table)."""
    if not torch.cuda.is_current_stream_capturing():
        return 0
    cid = ctypes.c_ulonglong(0)
    if _abi.lib().egs_stream_capture_id(stream, ctypes.byref(cid)) != 0 or cid.value == 0:
        return -1
    return int(cid.value)


def _table_key(Ind: torch.Tensor, dims: tuple, dt: int, stream: int, capture: int):
    return (Ind.data_ptr(), Ind._version, Ind.dtype, dims, dt, stream, capture)


def _table_nbytes(dims: tuple, dt: int) -> int:
    key = (dims, dt)
    n = _table_sizes.get(key)
    if n is None:
        n = _table_sizes[key] = int(_abi.lib().egs_routing_table_bytes(_abi.Dims(*dims), dt))
    return n


def _table_state(Ind: torch.Tensor, dims: tuple, dt: int, stream: int):
    """(bytes of the table these sizes can use - 0: build and read none now -, capture identifier, the table kept with
    `Ind` if it is valid for this call else None)."""
    # a tensor made under torch.inference_mode() has no version counter (reading it raises, and writes to it are
    # not recorded): no table is kept with it or read from it
    if not _table_cache or type(Ind) is not torch.Tensor or Ind.is_inference():
        return 0, 0, None
    nb = _table_nbytes(dims, dt)
    if nb == 0:
        return 0, 0, None
    capture = _capture_id(stream)
    if capture < 0:
        return 0, 0, None
    ent = Ind.__dict__.get(_TABLE_ATTR)
    if ent is not None and ent[0] == (Ind.data_ptr(), Ind._version, Ind.dtype, dims, dt, stream, capture):
        return nb, capture, ent[1]
    return nb, capture, None


def _table_lookup(Ind: torch.Tensor, dims: tuple, dt: int, stream: int):
    return _table_state(Ind, dims, dt, stream)[2]


# ------------------------------------------------------------------------------ the four launchers
def _gather_forward_impl(X: torch.Tensor, W: torch.Tensor, Ind: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    ct = _compute_dtype(out_dtype, X, W)
    dev = _require_gpu(X, W, Ind)
    B, E, K, I, J = _check_shapes(X, W, Ind, None, True)
    res_dtype = X.dtype
    X, ld_b, ld_t = _rows_source(X, ct)
    W = _dense16(W, ct)
    ind_given, Ind = Ind, Ind.contiguous()
    Y = torch.empty((B, E, K, J), device=dev, dtype=ct)
    T = X.shape[1]
    dims = (B, T, E, K, I, J)
    d = _dims_struct(dims)
    dt = dtype_to_type_id(ct)
    with _on_device(dev):
        stream = _stream_ptr(dev)
        nb, capture, table = _table_state(Ind, dims, dt, stream)
        build = None
        if nb and table is None and Ind is ind_given:      # a contiguous copy made here is gone after this call: nothing to keep a table with
            # first sight of these indices: the routing table of the scatters to come is built in this launch
            build = torch.empty(nb, dtype=torch.uint8, device=dev)
        fast = _abi.pycall()
        if fast is not None:
            rc = fast.gather_forward(X.data_ptr(), W.data_ptr(), Ind.data_ptr(), Y.data_ptr(),
                                     0 if build is None else build.data_ptr(), 0 if build is None else nb,
                                     B, T, E, K, I, J, ld_b, ld_t, dt, _ind_type_id(Ind), stream or 0)
        elif build is not None:
            rc = _abi.lib().egs_expert_gather_forward_table(X.data_ptr(), W.data_ptr(), Ind.data_ptr(), Y.data_ptr(),
                                                            build.data_ptr(), nb, d, ld_b, ld_t, dt, _ind_type_id(Ind), stream)
        else:
            rc = _abi.lib().egs_expert_gather_forward(X.data_ptr(), W.data_ptr(), Ind.data_ptr(), Y.data_ptr(), d,
                                                      ld_b, ld_t, dt, _ind_type_id(Ind), stream)
        if build is not None and rc == 0:
            Ind.__dict__[_TABLE_ATTR] = (_table_key(Ind, dims, dt, stream, capture), build)
    if rc:
        _abi.check(rc, "expert_gather_forward_call")
    return Y if res_dtype is ct else Y.to(res_dtype)


def _gather_backward_impl(X, W, Ind, grad_output, dtype):
    ct = _compute_dtype(dtype, X, W, grad_output)
    dev = _require_gpu(X, W, Ind, grad_output)
    B, E, K, I, J = _check_shapes(X, W, Ind, grad_output, True)
    x_dtype, w_dtype = X.dtype, W.dtype
    X, ld_b, ld_t = _rows_source(X, ct)
    W = _dense16(W, ct); Ind = Ind.contiguous(); grad_output = _dense16(grad_output, ct)
    T = X.shape[1]
    grad_X = torch.empty((B, T, I), device=dev, dtype=ct)
    grad_W = torch.empty((E, I, J), device=dev, dtype=ct)
    dims = (B, T, E, K, I, J)
    d = _dims_struct(dims)
    mode = _MODES[get_scatter_mode()]
    dt = dtype_to_type_id(ct)
    with _on_device(dev):
        keep, ws, ws_bytes = _workspace(dev, _workspace_bytes(_abi.OP_GATHER_BACKWARD, mode, dims, dt))
        stream = _stream_ptr(dev)
        table = _table_state(Ind, dims, dt, stream)[2]
        fast = _abi.pycall()
        if fast is not None:
            rc = fast.gather_backward(X.data_ptr(), W.data_ptr(), Ind.data_ptr(), 0 if table is None else table.data_ptr(),
                                      0 if table is None else table.numel(), grad_output.data_ptr(), grad_X.data_ptr(),
                                      grad_W.data_ptr(), ws or 0, ws_bytes, B, T, E, K, I, J, ld_b, ld_t, dt,
                                      _ind_type_id(Ind), mode, stream or 0)
        elif table is not None:
            rc = _abi.lib().egs_expert_gather_backward_table(X.data_ptr(), W.data_ptr(), Ind.data_ptr(), table.data_ptr(),
                                                             table.numel(), grad_output.data_ptr(), grad_X.data_ptr(),
                                                             grad_W.data_ptr(), ws, ws_bytes, d, ld_b, ld_t, dt,
                                                             _ind_type_id(Ind), mode, stream)
        else:
            rc = _abi.lib().egs_expert_gather_backward(X.data_ptr(), W.data_ptr(), Ind.data_ptr(), grad_output.data_ptr(),
                                                       grad_X.data_ptr(), grad_W.data_ptr(), ws, ws_bytes, d, ld_b, ld_t,
                                                       dt, _ind_type_id(Ind), mode, stream)
    del keep
    if rc == _abi.EGS_ERR_WORKSPACE and not X.is_contiguous():
        # the scratch is sized for dense operands; a strided view can select kernels that need more: run on a dense copy
        grad_X, grad_W = _gather_backward_impl(X.contiguous(), W, Ind, grad_output, dtype)
    elif rc:
        _abi.check(rc, "expert_gather_backward_call")
    return (grad_X if x_dtype is ct else grad_X.to(x_dtype)), (grad_W if w_dtype is ct else grad_W.to(w_dtype))


def _scatter_forward_impl(Y, W, Ind, T, out_dtype):
    ct = _compute_dtype(out_dtype, Y, W)
    dev = _require_gpu(Y, W, Ind)
    B, E, K, I, J = _check_shapes(None, W, Ind, Y, False)
    T = int(T)
    if T < 0:
        raise ValueError("T must be non-negative")
    res_dtype = Y.dtype
    Y = _dense16(Y, ct); W = _dense16(W, ct); Ind = Ind.contiguous()
    out = torch.empty((B, T, I), device=dev, dtype=ct)
    dims = (B, T, E, K, I, J)
    d = _dims_struct(dims)
    mode = _MODES[get_scatter_mode()]
    dt = dtype_to_type_id(ct)
    with _on_device(dev):
        keep, ws, ws_bytes = _workspace(dev, _workspace_bytes(_abi.OP_GEMM_SCATTER, mode, dims, dt))
        stream = _stream_ptr(dev)
        table = _table_state(Ind, dims, dt, stream)[2]
        fast = _abi.pycall()
        if fast is not None:
            rc = fast.scatter_forward(Y.data_ptr(), W.data_ptr(), Ind.data_ptr(), 0 if table is None else table.data_ptr(),
                                      0 if table is None else table.numel(), out.data_ptr(), ws or 0, ws_bytes,
                                      B, T, E, K, I, J, dt, _ind_type_id(Ind), mode, stream or 0)
        elif table is not None:
            rc = _abi.lib().egs_expert_scatter_forward_table(Y.data_ptr(), W.data_ptr(), Ind.data_ptr(), table.data_ptr(),
                                                             table.numel(), out.data_ptr(), ws, ws_bytes, d, dt,
                                                             _ind_type_id(Ind), mode, stream)
        else:
            rc = _abi.lib().egs_expert_scatter_forward(Y.data_ptr(), W.data_ptr(), Ind.data_ptr(), out.data_ptr(),
                                                       ws, ws_bytes, d, dt, _ind_type_id(Ind), mode, stream)
    del keep
    if rc:
        _abi.check(rc, "expert_scatter_forward_call")
    return out if res_dtype is ct else out.to(res_dtype)


def _scatter_backward_impl(Y, W, Ind, grad_X, dtype):
    ct = _compute_dtype(dtype, Y, W, grad_X)
    dev = _require_gpu(Y, W, Ind, grad_X)
    B, E, K, I, J = _check_shapes(grad_X, W, Ind, Y, False)
    y_dtype, w_dtype = Y.dtype, W.dtype
    grad_X, ld_b, ld_t = _rows_source(grad_X, ct)
    Y = _dense16(Y, ct); W = _dense16(W, ct); Ind = Ind.contiguous()
    T = grad_X.shape[1]
    grad_Y = torch.empty((B, E, K, J), device=dev, dtype=ct)
    grad_W = torch.empty((E, J, I), device=dev, dtype=ct)
    dims = (B, T, E, K, I, J)
    d = _dims_struct(dims)
    dt = dtype_to_type_id(ct)
    with _on_device(dev):
        keep, ws, ws_bytes = _workspace(dev, _workspace_bytes(_abi.OP_SCATTER_BACKWARD, 0, dims, dt))
        fast = _abi.pycall()
        if fast is not None:
            rc = fast.scatter_backward(Y.data_ptr(), W.data_ptr(), Ind.data_ptr(), grad_X.data_ptr(), grad_Y.data_ptr(),
                                       grad_W.data_ptr(), ws or 0, ws_bytes, B, T, E, K, I, J, ld_b, ld_t, dt,
                                       _ind_type_id(Ind), _stream_ptr(dev) or 0)
        else:
            rc = _abi.lib().egs_expert_scatter_backward(Y.data_ptr(), W.data_ptr(), Ind.data_ptr(), grad_X.data_ptr(),
                                                        grad_Y.data_ptr(), grad_W.data_ptr(), ws, ws_bytes, d, ld_b, ld_t,
                                                        dt, _ind_type_id(Ind), _stream_ptr(dev))
    del keep
    if rc == _abi.EGS_ERR_WORKSPACE and not grad_X.is_contiguous():
        grad_Y, grad_W = _scatter_backward_impl(Y, W, Ind, grad_X.contiguous(), dtype)    # see _gather_backward_impl
    elif rc:
        _abi.check(rc, "expert_scatter_backward_call")
    return (grad_Y if y_dtype is ct else grad_Y.to(y_dtype)), (grad_W if w_dtype is ct else grad_W.to(w_dtype))


# module globals, bound by create_kernels() (reference egs/triton_kernels.py:26-29)
expert_gather_forward_call = None
expert_gather_backward_call = None
expert_scatter_forward_call = None
expert_scatter_backward_call = None
_create_lock = threading.Lock()


_libraries: dict = {}


def _register_ops(ns: str) -> None:
    """Define the four ops in namespace `ns` (schemas of reference egs/triton_kernels.py:362, :395, :444, :478), with
    fake implementations for tracing and autograd formulas, so that the ops can also be called directly on tensors
    that require grad and traced by torch.compile."""
    lib = torch.library.Library(ns, "DEF")
    lib.define("expert_gather_forward_call_fn(Tensor X, Tensor W, Tensor Ind, ScalarType out_dtype) -> Tensor")
    lib.define("expert_gather_backward_call_fn(Tensor X, Tensor W, Tensor Ind, Tensor grad_output, "
               "ScalarType out_dtype) -> (Tensor, Tensor)")
    lib.define("expert_scatter_forward_call_fn(Tensor Y, Tensor W, Tensor Ind, int T, ScalarType out_dtype) -> Tensor")
    lib.define("expert_scatter_backward_call_fn(Tensor Y, Tensor W, Tensor Ind, Tensor grad_X, "
               "ScalarType out_dtype) -> (Tensor, Tensor)")
    if ns == OP_NAMESPACE:      # the inference block has no counterpart among the reference's ops
        lib.define("expert_mlp_forward_fn(Tensor X, Tensor W_gather, Tensor W_scatter, Tensor Ind, str activation, "
                   "bool force_block=False) -> Tensor")
        lib.impl("expert_mlp_forward_fn", _mlp_forward_impl, "CompositeExplicitAutograd")

        @torch.library.register_fake(f"{ns}::expert_mlp_forward_fn", lib=lib)
        def _(X, W_gather, W_scatter, Ind, activation, force_block=False):
            return X.new_empty(tuple(X.shape))
    lib.impl("expert_gather_forward_call_fn", _gather_forward_impl, "CompositeExplicitAutograd")
    lib.impl("expert_gather_backward_call_fn", _gather_backward_impl, "CompositeExplicitAutograd")
    lib.impl("expert_scatter_forward_call_fn", _scatter_forward_impl, "CompositeExplicitAutograd")
    lib.impl("expert_scatter_backward_call_fn", _scatter_backward_impl, "CompositeExplicitAutograd")

    @torch.library.register_fake(f"{ns}::expert_gather_forward_call_fn", lib=lib)
    def _(X, W, Ind, out_dtype):
        return X.new_empty((X.shape[0], W.shape[0], Ind.shape[2], W.shape[2]))

    @torch.library.register_fake(f"{ns}::expert_gather_backward_call_fn", lib=lib)
    def _(X, W, Ind, grad_output, out_dtype):
        return torch.empty_like(X, memory_format=torch.contiguous_format), torch.empty_like(
            W, memory_format=torch.contiguous_format)

    @torch.library.register_fake(f"{ns}::expert_scatter_forward_call_fn", lib=lib)
    def _(Y, W, Ind, T, out_dtype):
        return Y.new_empty((Y.shape[0], T, W.shape[2]))

    @torch.library.register_fake(f"{ns}::expert_scatter_backward_call_fn", lib=lib)
    def _(Y, W, Ind, grad_X, out_dtype):
        return torch.empty_like(Y, memory_format=torch.contiguous_format), torch.empty_like(
            W, memory_format=torch.contiguous_format)

    ops = getattr(torch.ops, ns)

    def gather_setup(ctx, inputs, output):
        X, W, Ind, out_dtype = inputs
        ctx.save_for_backward(X, W, Ind)
        ctx.out_dtype = out_dtype
        ctx.scatter_mode = _mode_to_bind()

    def gather_backward(ctx, grad_output):
        X, W, Ind = ctx.saved_tensors
        with scatter_mode_scope(ctx.scatter_mode):      # grad_X is a scatter: in the mode the forward was called in
            grad_X, grad_W = ops.expert_gather_backward_call_fn(X, W, Ind, grad_output, ctx.out_dtype)
        return grad_X, grad_W, None, None

    def scatter_setup(ctx, inputs, output):
        Y, W, Ind, T, out_dtype = inputs
        ctx.save_for_backward(Y, W, Ind)
        ctx.out_dtype = out_dtype

    def scatter_backward(ctx, grad_X):
        Y, W, Ind = ctx.saved_tensors
        grad_Y, grad_W = ops.expert_scatter_backward_call_fn(Y, W, Ind, grad_X, ctx.out_dtype)
        return grad_Y, grad_W, None, None, None

    torch.library.register_autograd(f"{ns}::expert_gather_forward_call_fn", gather_backward, setup_context=gather_setup, lib=lib)
    torch.library.register_autograd(f"{ns}::expert_scatter_forward_call_fn", scatter_backward, setup_context=scatter_setup, lib=lib)
    _libraries[ns] = lib            # keeps the registration alive


def create_kernels() -> None:
    """Register the four ops once per process and bind the module-level callables.

    Counterpart of reference egs/triton_kernels.py:32-578; here it only defines the
    ``torch.library`` ops (nothing is compiled at run time) and is safe to call from several
    threads."""
    global expert_gather_forward_call, expert_gather_backward_call
    global expert_scatter_forward_call, expert_scatter_backward_call
    if expert_scatter_backward_call is not None:
        return
    with _create_lock:
        if expert_scatter_backward_call is not None:
            return
        _register_ops(OP_NAMESPACE)
        ops = getattr(torch.ops, OP_NAMESPACE)
        compiling = torch.compiler.is_compiling
        plain = (torch.Tensor, torch.nn.Parameter)       # not a fake / functional / subclass tensor of some tracer

        # The callables the Functions use.  Like the reference's (plain Python functions, egs/triton_kernels.py:569-578)
        # they run the launcher directly for tensors on the GPU in eager mode, which saves the dispatcher's
        # round trip per call (several microseconds, more than some of the kernels take); while torch.compile is
        # tracing, and for meta / fake tensors, they go through the registered ops, whose fake implementations
        # describe the outputs.
        def gather_forward_call(X, W, Ind, out_dtype):
            if type(X) in plain and X.is_cuda and not compiling():
                return _gather_forward_impl(X, W, Ind, out_dtype)
            return ops.expert_gather_forward_call_fn(X, W, Ind, out_dtype)

        def gather_backward_call(X, W, Ind, grad_output, out_dtype):
            if type(X) in plain and X.is_cuda and not compiling():
                return _gather_backward_impl(X, W, Ind, grad_output, out_dtype)
            return ops.expert_gather_backward_call_fn(X, W, Ind, grad_output, out_dtype)

        def scatter_forward_call(Y, W, Ind, T, out_dtype):
            if type(Y) in plain and Y.is_cuda and not compiling():
                return _scatter_forward_impl(Y, W, Ind, T, out_dtype)
            return ops.expert_scatter_forward_call_fn(Y, W, Ind, T, out_dtype)

        def scatter_backward_call(Y, W, Ind, grad_X, out_dtype):
            if type(Y) in plain and Y.is_cuda and not compiling():
                return _scatter_backward_impl(Y, W, Ind, grad_X, out_dtype)
            return ops.expert_scatter_backward_call_fn(Y, W, Ind, grad_X, out_dtype)

        expert_gather_forward_call = gather_forward_call
        expert_gather_backward_call = gather_backward_call
        expert_scatter_forward_call = scatter_forward_call
        expert_scatter_backward_call = scatter_backward_call


def register_reference_namespace(ns: str = "mylib") -> None:
    """Also expose the four ops as ``torch.ops.mylib.*``, the namespace the reference registers them under
    (egs/triton_kernels.py:362), for code that addresses the ops by name instead of through the module-level
    callables.  Optional and explicit because an op name can be defined only once per process: it raises if the
    reference package (or anything else) has already defined these names."""
    create_kernels()
    with _create_lock:
        if ns not in _libraries:
            _register_ops(ns)


# ------------------------------------------------------------------------------ autograd Functions
def _mode_to_bind():
    """The scatter mode a forward call hands to its backward; None while torch.compile is tracing (thread-local state
    is not traced: the compiled backward then runs in the mode in force when it is called)."""
    return None if torch.compiler.is_compiling() else get_scatter_mode()


class ExpertGatherFunction(torch.autograd.Function):
    """Y[b,e,k,j] = sum_i X[b, Ind[b,e,k], i] * W[e,i,j]   (reference egs/triton_kernels.py:581-608)."""

    @staticmethod
    def forward(ctx, X: torch.Tensor, W: torch.Tensor, Ind: torch.Tensor, out_type=torch.float32):
        create_kernels()
        ctx.save_for_backward(X, W, Ind)
        ctx.dtype = out_type
        ctx.scatter_mode = _mode_to_bind()
        return expert_gather_forward_call(X, W, Ind, out_type)

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        X, W, Ind = ctx.saved_tensors
        if ctx.scatter_mode is None:
            grad_X, grad_W = expert_gather_backward_call(X, W, Ind, grad_output, ctx.dtype)
        else:
            with scatter_mode_scope(ctx.scatter_mode):      # grad_X is a scatter: in the mode the forward was called in
                grad_X, grad_W = expert_gather_backward_call(X, W, Ind, grad_output, ctx.dtype)
        return grad_X, grad_W, None, None


class ExpertScatterFunction(torch.autograd.Function):
    """X[b,t,i] = sum_{e,k: Ind[b,e,k]=t} sum_j Y[b,e,k,j] * W[e,j,i]   (reference egs/triton_kernels.py:610-639)."""

    @staticmethod
    def forward(ctx, Y: torch.Tensor, W: torch.Tensor, Ind: torch.Tensor, T: int, out_type=torch.float32):
        create_kernels()
        ctx.save_for_backward(Y, W, Ind)
        ctx.dtype = out_type
        return expert_scatter_forward_call(Y, W, Ind, T, out_type)

    @staticmethod
    def backward(ctx, grad_X: torch.Tensor):
        Y, W, Ind = ctx.saved_tensors
        grad_Y, grad_W = expert_scatter_backward_call(Y, W, Ind, grad_X, ctx.dtype)
        # one gradient per forward input: (Y, W, Ind, T) or (Y, W, Ind, T, out_type).  The reference returns four
        # (egs/triton_kernels.py:639), which autograd rejects when out_type is passed explicitly.
        return (grad_Y, grad_W) + (None,) * (len(ctx.needs_input_grad) - 2)


# ------------------------------------------------------------------------------ extras (not in the reference)
def expert_gather_fp8w_forward(X: torch.Tensor, Wq: torch.Tensor, scale: torch.Tensor, Ind: torch.Tensor) -> torch.Tensor:
    """Inference-only gather with fp8 weights: Y = X[b,Ind] . (Wq[e] * scale[e, None, :]).

    X is bfloat16 [B,T,I]; Wq is float8_e4m3fn [E,I,J]; scale is float32 [E,J]."""
    dev = _require_gpu(X, Wq, scale, Ind)
    if X.dtype != torch.bfloat16 or Wq.dtype != torch.float8_e4m3fn or scale.dtype != torch.float32:
        raise ValueError("fp8-weight gather needs bfloat16 X, float8_e4m3fn W and float32 scale")
    B, E, K, I, J = _check_shapes(X, Wq, Ind, None, True)
    if tuple(scale.shape) != (E, J):
        raise ValueError(f"scale must be [E={E},J={J}], got {tuple(scale.shape)}")
    X, ld_b, ld_t = _rows_source(X, torch.bfloat16)
    Wq = Wq.contiguous(); scale = scale.contiguous(); Ind = Ind.contiguous()
    Y = torch.empty((B, E, K, J), device=dev, dtype=X.dtype)
    d = _abi.Dims(B, X.shape[1], E, K, I, J)
    with _on_device(dev):
        rc = _abi.lib().egs_gather_gemm(X.data_ptr(), Wq.data_ptr(), Ind.data_ptr(), Y.data_ptr(), scale.data_ptr(), d,
                                        ld_b, ld_t, _abi.BF16, _abi.FP8_E4M3, _ind_type_id(Ind), _abi.W_EIJ,
                                        _stream_ptr(dev))
    _abi.check(rc, "expert_gather_fp8w_forward")
    return Y


def expert_gather_fp8_forward(X: torch.Tensor, Wq: torch.Tensor, scale: torch.Tensor, Ind: torch.Tensor,
                              return_quantised: bool = False):
    """Inference-only gather with fp8 weights and fp8 activations on the fp8 matrix instruction.

    Every row X[b,t,:] is quantised once to float8_e4m3fn with its own scale xs[b,t] = max|X[b,t,:]| / 448, then
    Y[b,e,k,:] = xs[b,t] * scale[e,:] * (Xq[b,t,:] . Wq[e]) with fp32 accumulation, t = Ind[b,e,k].
    X is bfloat16 [B,T,I] (I a multiple of 128); Wq is float8_e4m3fn [E,I,J] (J a multiple of 16); scale is
    float32 [E,J].  With ``return_quantised`` the quantised rows [B,T,I] and their scales [B,T] are returned too."""
    dev = _require_gpu(X, Wq, scale, Ind)
    if X.dtype != torch.bfloat16 or Wq.dtype != torch.float8_e4m3fn or scale.dtype != torch.float32:
        raise ValueError("fp8 gather needs bfloat16 X, float8_e4m3fn W and float32 scale")
    B, E, K, I, J = _check_shapes(X, Wq, Ind, None, True)
    if tuple(scale.shape) != (E, J):
        raise ValueError(f"scale must be [E={E},J={J}], got {tuple(scale.shape)}")
    X, ld_b, ld_t = _rows_source(X, torch.bfloat16)
    T = X.shape[1]
    Wq = Wq.contiguous(); scale = scale.contiguous(); Ind = Ind.contiguous()
    Y = torch.empty((B, E, K, J), device=dev, dtype=X.dtype)
    d = _abi.Dims(B, T, E, K, I, J)
    nbytes = _abi.lib().egs_gather_gemm_fp8act_workspace_bytes(d)
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=dev)
    ws_ptr = ws.data_ptr()
    with _on_device(dev):
        rc = _abi.lib().egs_gather_gemm_fp8act(X.data_ptr(), Wq.data_ptr(), scale.data_ptr(), Ind.data_ptr(), Y.data_ptr(),
                                               ws_ptr, nbytes, d, ld_b, ld_t, _ind_type_id(Ind), _stream_ptr(dev))
    _abi.check(rc, "expert_gather_fp8_forward")
    if not return_quantised:
        return Y
    xq_bytes = (B * T * I + 255) // 256 * 256
    Xq = ws[:B * T * I].view(torch.float8_e4m3fn).view(B, T, I)
    xs = ws[xq_bytes:xq_bytes + B * T * 4].view(torch.float32).view(B, T)
    return Y, Xq, xs


_ACTIVATIONS = {None: _abi.ACT_NONE, "none": _abi.ACT_NONE, "identity": _abi.ACT_NONE, "relu": _abi.ACT_RELU,
                "gelu": _abi.ACT_GELU, "silu": _abi.ACT_SILU, "swish": _abi.ACT_SILU, "gelu_tanh": _abi.ACT_GELU_TANH}
_TORCH_ACT = {
    _abi.ACT_NONE: lambda y: y,
    _abi.ACT_RELU: torch.relu,
    _abi.ACT_GELU: torch.nn.functional.gelu,
    _abi.ACT_SILU: torch.nn.functional.silu,
    _abi.ACT_GELU_TANH: lambda y: torch.nn.functional.gelu(y, approximate="tanh"),
}

# derivative of the activation applied to an incoming gradient: (grad, input) -> grad * act'(input), torch's own kernels
_TORCH_ACT_BACKWARD = {
    _abi.ACT_RELU: lambda g, y: torch.ops.aten.threshold_backward(g, y, 0),
    _abi.ACT_GELU: lambda g, y: torch.ops.aten.gelu_backward(g, y, approximate="none"),
    _abi.ACT_SILU: lambda g, y: torch.ops.aten.silu_backward(g, y),
    _abi.ACT_GELU_TANH: lambda g, y: torch.ops.aten.gelu_backward(g, y, approximate="tanh"),
}


def _mlp_block_pays(B: int, E: int, K: int, I: int, J: int, act: int) -> bool:
    """Measured on MI355X (bf16, one graph replay per call): the one kernel wins while its workgroups fit one round of the
    device (256), the batch is large enough (its time hardly depends on the batch: every workgroup walks all E*K picks of
    its batch element, while the separate launches shrink with it) and the activation is cheap or the (expert, 32-pick)
    units few - its four slice workgroups per batch element each repeat the activation, and exponentials run at a quarter
    of the vector rate.  B64 T256 E32 K32 I128 J64, block / separate launches: relu 27.5 / 30.5 us, silu 31.0 / 31.6, gelu
    33.9 / 31.6; E16: 19.0 / 22.1, 21.4 / 22.2, 23.7 / 22.7; I64 J32: relu 21.3 / 22.9; B32: relu 25.3 / 24.1;
    B128 relu: 43.3 / 41.6 us."""
    blocks = 8 * ((B + 7) // 8) * (I // 32)
    cheap = act in (_abi.ACT_NONE, _abi.ACT_RELU)
    return blocks <= 256 and B >= 48 and (cheap or E * ((K + 31) // 32) <= 16)


def expert_mlp_forward(X: torch.Tensor, W_gather: torch.Tensor, W_scatter: torch.Tensor, Ind: torch.Tensor,
                       activation="relu", force_block: bool = False) -> torch.Tensor:
    """See `_mlp_forward_impl`.  In eager mode on GPU tensors this runs the launcher directly; while torch.compile
    is tracing (and for fake / meta tensors) it goes through the op ``egs_amd::expert_mlp_forward_fn``, whose fake
    implementation describes the output."""
    if type(X) in (torch.Tensor, torch.nn.Parameter) and X.is_cuda and not torch.compiler.is_compiling():
        return _mlp_forward_impl(X, W_gather, W_scatter, Ind, activation, force_block)
    create_kernels()
    return getattr(torch.ops, OP_NAMESPACE).expert_mlp_forward_fn(X, W_gather, W_scatter, Ind,
                                                                  "none" if activation is None else activation, force_block)


def _mlp_forward_impl(X: torch.Tensor, W_gather: torch.Tensor, W_scatter: torch.Tensor, Ind: torch.Tensor,
                      activation="relu", force_block: bool = False) -> torch.Tensor:
    """Inference block ``scatter(act(gather(X, W_gather, Ind)), W_scatter, Ind, T)`` - the call pattern of the
    reference's layers (test_speed.ipynb:73-75 on egs/triton_kernels.py:49-143, :156-247) - without autograd.

    X [B,T,I], W_gather [E,I,J], W_scatter [E,J,I], Ind [B,E,K] -> [B,T,I].  For small experts in a 16-bit type
    (I in {32, 64, 128}, J in {32, 64}, at most 1024 picks per batch element) this is ONE kernel and the rows
    Y [B,E,K,J] between the two products never exist in memory; every other case, and every case where the one
    kernel is known to lose (more workgroups than one round of the device, or an expensive activation on many
    experts: its four slice workgroups per batch element each repeat the gather product), runs the two forward
    launchers with torch's activation in between (on the GPU all the same).  ``force_block=True`` takes the one
    kernel whenever it can run.  ``activation``: "none", "relu",
    "gelu", "gelu_tanh", "silu".  The activation is applied to the fp32 product and rounded to the element
    type once, exactly where a stored Y would have been rounded."""
    if activation not in _ACTIVATIONS:
        raise ValueError(f"activation must be one of {sorted(k for k in _ACTIVATIONS if k)}, got {activation!r}")
    act = _ACTIVATIONS[activation]
    dev = _require_gpu(X, W_gather, W_scatter, Ind)
    B, E, K, I, J = _check_shapes(X, W_gather, Ind, None, True)
    if W_scatter.dim() != 3 or tuple(W_scatter.shape) != (E, J, I):
        raise ValueError(f"W_scatter must be [E,J,I] = {(E, J, I)}, got {tuple(W_scatter.shape)}")
    ct = _compute_dtype(torch.float32, X, W_gather, W_scatter)
    T = X.shape[1]
    d = _abi.Dims(B, T, E, K, I, J)
    lib = _abi.lib()
    if ct is not torch.float32 and (force_block or _mlp_block_pays(B, E, K, I, J, act)) \
            and lib.egs_expert_mlp_supported(d, dtype_to_type_id(ct)):
        res_dtype = X.dtype
        Xs, ld_b, ld_t = _rows_source(X, ct)
        Wg = _dense16(W_gather, ct); Ws = _dense16(W_scatter, ct); Indc = Ind.contiguous()
        out = torch.empty((B, T, I), device=dev, dtype=ct)
        with _on_device(dev):
            rc = lib.egs_expert_mlp_forward(Xs.data_ptr(), Wg.data_ptr(), Ws.data_ptr(), Indc.data_ptr(), out.data_ptr(), d,
                                            ld_b, ld_t, dtype_to_type_id(ct), _ind_type_id(Indc), act, _stream_ptr(dev))
        if rc == 0:
            return out if res_dtype is ct else out.to(res_dtype)
        if rc != _abi.EGS_ERR_UNSUPPORTED:
            _abi.check(rc, "expert_mlp_forward")
    with torch.no_grad():
        Y = _TORCH_ACT[act](_gather_forward_impl(X, W_gather, Ind, torch.float32))
        return _scatter_forward_impl(Y, W_scatter, Ind, T, torch.float32)


class ExpertMLPFunction(torch.autograd.Function):
    """Trainable ``scatter(act(gather(X, W_gather, Ind)), W_scatter, Ind, T)`` that keeps no ``Y[B,E,K,J]`` between
    forward and backward (the layer pattern of the reference, test_speed.ipynb:73-75, as one autograd node).

    Forward: `expert_mlp_forward` (one kernel for small experts, the rows between the two products never in memory).
    Saved for backward: ``X``, the two weights and ``Ind`` only - none of the ``B*E*K*J`` activations the two separate
    Functions save (``Y`` for the activation, ``act(Y)`` for the scatter).  Backward recomputes the gather product
    (one more launch) and then runs what the separate Functions would: the scatter's backward on ``act(Y)``, the
    activation's derivative (torch), the gather's backward.  The recomputed rows are rounded to the element type before
    the activation (the one-kernel forward rounds after it), so for activations other than relu/none the ``act(Y)`` the weight
    gradient sees can differ from the forward's in the last bit."""

    @staticmethod
    def forward(ctx, X: torch.Tensor, W_gather: torch.Tensor, W_scatter: torch.Tensor, Ind: torch.Tensor, activation="relu"):
        create_kernels()
        if activation not in _ACTIVATIONS:
            raise ValueError(f"activation must be one of {sorted(k for k in _ACTIVATIONS if k)}, got {activation!r}")
        ctx.save_for_backward(X, W_gather, W_scatter, Ind)
        ctx.act = _ACTIVATIONS[activation]
        ctx.scatter_mode = _mode_to_bind()
        return expert_mlp_forward(X, W_gather, W_scatter, Ind, activation)

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad_out: torch.Tensor):
        X, Wg, Ws, Ind = ctx.saved_tensors
        Y = expert_gather_forward_call(X, Wg, Ind, torch.float32)
        A = Y.relu_() if ctx.act == _abi.ACT_RELU else _TORCH_ACT[ctx.act](Y)    # relu's derivative can be read off its result
        grad_Y, grad_Ws = expert_scatter_backward_call(A, Ws, Ind, grad_out, torch.float32)
        del A
        if ctx.act != _abi.ACT_NONE:
            grad_Y = _TORCH_ACT_BACKWARD[ctx.act](grad_Y, Y)
        del Y
        if ctx.scatter_mode is None:
            grad_X, grad_Wg = expert_gather_backward_call(X, Wg, Ind, grad_Y, torch.float32)
        else:
            with scatter_mode_scope(ctx.scatter_mode):
                grad_X, grad_Wg = expert_gather_backward_call(X, Wg, Ind, grad_Y, torch.float32)
        return grad_X, grad_Wg, grad_Ws, None, None


def expert_mlp(X: torch.Tensor, W_gather: torch.Tensor, W_scatter: torch.Tensor, Ind: torch.Tensor, activation="relu") -> torch.Tensor:
    """Differentiable block, see `ExpertMLPFunction`.  X [B,T,I], W_gather [E,I,J], W_scatter [E,J,I], Ind [B,E,K] -> [B,T,I]."""
    return ExpertMLPFunction.apply(X, W_gather, W_scatter, Ind, activation)


def validate_indices(Ind: torch.Tensor, T: int) -> int:
    """Number of entries of Ind outside [0, T) (synchronises; debugging aid)."""
    dev = _require_gpu(Ind)
    Ind = Ind.contiguous()
    bad = torch.zeros(1, dtype=torch.int32, device=dev)
    with _on_device(dev):
        rc = _abi.lib().egs_validate_indices(Ind.data_ptr(), _ind_type_id(Ind), Ind.numel(), int(T), bad.data_ptr(),
                                             _stream_ptr(dev))
    _abi.check(rc, "validate_indices")
    return int(bad.item())
