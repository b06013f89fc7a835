"""CPU oracle for the fused expert gather / scatter-with-linear path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``expertscattergather_amd/`` may import this
module; it is the checker for ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py``.

It restates, in numpy (float64 accumulation unless told otherwise), the algorithm the
reference defines in plain torch:

* gather forward   -- reference ``egs/baselines.py:69-76`` (``TorchReshapedGatherEinsum``),
                      same definition in ``README.md:15-22`` and the kernel docstring
                      ``egs/triton_kernels.py:589``.
* scatter forward  -- reference ``egs/baselines.py:174-184`` (``TorchEinsumScatter``),
                      ``README.md:23-32``, ``egs/triton_kernels.py:618``.
* gather backward  -- closed forms of reference ``egs/baselines.py:126-149``
                      (``FusedGatherEinsumFunction.backward``); kernel docstrings
                      ``egs/triton_kernels.py:177-178`` (dX) and ``:283`` (dW).
* scatter backward -- the transposed identities the reference realises by swapping W
                      strides at ``egs/triton_kernels.py:504`` (dY) and ``:521`` (dW).

* inference block   -- the two forwards chained through an elementwise activation, the way the
                      reference's notebook calls its layers (``test_speed.ipynb:73-75``).

How each function is pinned (the reference ships no golden vectors for this path, its
tests are unseeded random GPU comparisons, ``test_all.py:97-101``):

* ``brute_*`` below are index-by-index Python loops written straight from the summation
  formulas; the vectorised functions are checked against them on tiny shapes.
* ``Ind = arange`` with ``E = 1, K = T`` collapses gather to a plain ``X @ W`` and scatter
  to ``Y @ W`` (library matmul).
* gather and scatter with the same ``Ind`` are exact adjoints of each other for a fixed
  ``W``; dX/dY/dW are checked against torch autograd through an independent torch
  restatement of the forward (``oracle/torch_port.py``) and by finite differences.
* the C restatement ``oracle/egs_oracle.c`` is a second, loop-level implementation.

fp8 weights (not in the reference; defined by the benchmark configuration that stores W as
e4m3 with one fp32 scale per expert and output column): the oracle dequantises
``W[e,i,j] = fp8_to_float(Wq[e,i,j]) * scale[e,j]`` and runs the ordinary gather.  The
decode table is checked against ``torch.float8_e4m3fn`` in the tests.

fp8 activations (not in the reference either): every source row is quantised to e4m3 with its
own scale ``max|row| / 448`` (``quantize_rows_e4m3``: float32 arithmetic, round to nearest even
by search over the 256-entry decode table, checked against ``torch.float8_e4m3fn``), then the
oracle dequantises rows and weights and runs the ordinary gather (``gather_forward_fp8``).
"""
from __future__ import annotations

import numpy as np

__all__ = [
    "gather_forward", "scatter_forward", "gather_backward", "scatter_backward",
    "brute_gather_forward", "brute_scatter_forward", "brute_gather_backward",
    "brute_scatter_backward", "fp8_e4m3fn_to_float", "dequant_fp8_weights",
    "gather_forward_fp8w", "float_to_fp8_e4m3fn", "quantize_rows_e4m3", "gather_forward_fp8",
    "round_to_bf16", "round_to_f16",
]


# ----------------------------------------------------------------------------- helpers
def _as_index(Ind: np.ndarray) -> np.ndarray:
    Ind = np.asarray(Ind)
    if not np.issubdtype(Ind.dtype, np.integer):
        raise TypeError("Ind must be an integer array")
    return Ind.astype(np.int64)


def round_to_bf16(a: np.ndarray) -> np.ndarray:
    """Round float32 values to the nearest bfloat16 (ties to even), returned as float32."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    u = a.view(np.uint32).astype(np.uint64)
    nan = np.isnan(a)
    rounded = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    out = rounded.astype(np.uint32).view(np.float32).copy()
    out[nan] = np.nan
    return out


def round_to_f16(a: np.ndarray) -> np.ndarray:
    return np.asarray(a, dtype=np.float32).astype(np.float16).astype(np.float32)


# ----------------------------------------------------------------------------- forward
def gather_forward(X, W, Ind, acc=np.float64):
    """Y[b,e,k,j] = sum_i X[b, Ind[b,e,k], i] * W[e,i,j].

    Follows reference egs/baselines.py:69-76: gather rows of X along T with the index
    reshaped to [B, E*K], view as [B,E,K,I], contract with W over i.
    """
    X = np.asarray(X, dtype=acc)
    W = np.asarray(W, dtype=acc)
    Ind = _as_index(Ind)
    B, T, I = X.shape
    E, I2, J = W.shape
    assert I2 == I and Ind.shape[0] == B and Ind.shape[1] == E
    K = Ind.shape[2]
    flat = Ind.reshape(B, E * K)
    Xg = np.take_along_axis(X, flat[:, :, None], axis=1).reshape(B, E, K, I)
    # per-expert dense contraction [B*K, I] @ [I, J]
    Y = np.empty((B, E, K, J), dtype=acc)
    for e in range(E):
        Y[:, e] = (Xg[:, e].reshape(B * K, I) @ W[e]).reshape(B, K, J)
    return Y


def scatter_forward(Y, W, Ind, T, acc=np.float64):
    """out[b,t,i] = sum_{e,k: Ind[b,e,k]=t} sum_j Y[b,e,k,j] * W[e,j,i].

    Follows reference egs/baselines.py:174-184: contract first, then scatter_add the
    [B, E*K, I] rows into a zero [B,T,I] tensor along T.
    """
    Y = np.asarray(Y, dtype=acc)
    W = np.asarray(W, dtype=acc)
    Ind = _as_index(Ind)
    B, E, K, J = Y.shape
    E2, J2, I = W.shape
    assert E2 == E and J2 == J and Ind.shape == (B, E, K)
    pre = np.empty((B, E, K, I), dtype=acc)
    for e in range(E):
        pre[:, e] = (Y[:, e].reshape(B * K, J) @ W[e]).reshape(B, K, I)
    out = np.zeros((B, T, I), dtype=acc)
    bidx = np.broadcast_to(np.arange(B)[:, None], (B, E * K))
    np.add.at(out, (bidx, Ind.reshape(B, E * K)), pre.reshape(B, E * K, I))
    return out


# ----------------------------------------------------------------------------- backward
def gather_backward(X, W, Ind, dY, acc=np.float64):
    """Gradients of gather_forward.  Reference egs/baselines.py:136-146.

    dX[b,t,i]   = sum_{e,k: Ind=t} sum_j dY[b,e,k,j] * W[e,i,j]
    dW[e,i,j]   = sum_{b,k} X[b,Ind[b,e,k],i] * dY[b,e,k,j]
    """
    X = np.asarray(X, dtype=acc)
    W = np.asarray(W, dtype=acc)
    dY = np.asarray(dY, dtype=acc)
    Ind = _as_index(Ind)
    B, T, I = X.shape
    E, _, J = W.shape
    K = Ind.shape[2]
    # dX is a scatter with the transposed weight [E,J,I]
    dX = scatter_forward(dY, np.swapaxes(W, 1, 2), Ind, T, acc=acc)
    flat = Ind.reshape(B, E * K)
    Xg = np.take_along_axis(X, flat[:, :, None], axis=1).reshape(B, E, K, I)
    dW = np.empty((E, I, J), dtype=acc)
    for e in range(E):
        dW[e] = Xg[:, e].reshape(B * K, I).T @ dY[:, e].reshape(B * K, J)
    return dX, dW


def scatter_backward(Y, W, Ind, dOut, acc=np.float64):
    """Gradients of scatter_forward (W is [E,J,I]).

    dY[b,e,k,j] = sum_i dOut[b,Ind[b,e,k],i] * W[e,j,i]    (reference egs/triton_kernels.py:500-508)
    dW[e,j,i]   = sum_{b,k} Y[b,e,k,j] * dOut[b,Ind[b,e,k],i]   (reference :515-523)
    """
    Y = np.asarray(Y, dtype=acc)
    W = np.asarray(W, dtype=acc)
    dOut = np.asarray(dOut, dtype=acc)
    Ind = _as_index(Ind)
    B, E, K, J = Y.shape
    I = W.shape[2]
    dY = gather_forward(dOut, np.swapaxes(W, 1, 2), Ind, acc=acc)
    flat = Ind.reshape(B, E * K)
    Gg = np.take_along_axis(dOut, flat[:, :, None], axis=1).reshape(B, E, K, I)
    dW = np.empty((E, J, I), dtype=acc)
    for e in range(E):
        dW[e] = Y[:, e].reshape(B * K, J).T @ Gg[:, e].reshape(B * K, I)
    return dY, dW


# ----------------------------------------------------------------------------- brute force
# ---------------------------------------------------------------------------------------------------------
# Inference block: the reference's layers chained the way its notebook calls them, out = scatter(act(gather(x, Ind)), Ind, T)
# (test_speed.ipynb:73-75 with gather = egs/baselines.py:69-76 and scatter = egs/baselines.py:174-184).
def activation(y, name):
    """Elementwise activations by their textbook closed forms (float64): relu, gelu (erf form, the default of
    torch.nn.functional.gelu), gelu_tanh (its tanh approximation), silu, none.  Pinned in tests/test_oracle.py against
    torch.nn.functional on the CPU and against special values."""
    y = np.asarray(y, dtype=np.float64)
    if name in (None, "none", "identity"):
        return y
    if name == "relu":
        return np.maximum(y, 0.0)
    if name == "gelu":
        from math import erf
        return 0.5 * y * (1.0 + np.vectorize(erf, otypes=[np.float64])(y / np.sqrt(2.0)))
    if name == "gelu_tanh":
        return 0.5 * y * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (y + 0.044715 * y ** 3)))
    if name == "silu":
        return y / (1.0 + np.exp(-y))
    raise ValueError(f"unknown activation {name!r}")


def mlp_forward(X, Wg, Ws, Ind, T, act="relu", round_y=None, round_before_act=False):
    """out = scatter_forward(act(gather_forward(X, Wg, Ind)), Ws, Ind, T), picks outside [0, T) contributing nothing.

    `round_y`: function that rounds the activated rows to the element type a stored Y would have (e.g. round_to_bf16), or
    None.  `round_before_act`: also round before the activation, as separate launches that store Y do."""
    Ind = _as_index(np.asarray(Ind))
    bad = (Ind < 0) | (Ind >= T)
    safe = np.where(bad, 0, Ind)
    Y = gather_forward(X, Wg, safe)
    if round_y is not None and round_before_act:
        Y = round_y(Y.astype(np.float32)).astype(np.float64)
    Y = activation(Y, act) * (~bad)[..., None]
    if round_y is not None:
        Y = round_y(Y.astype(np.float32)).astype(np.float64)
    return scatter_forward(Y, Ws, safe, T)


def brute_gather_forward(X, W, Ind):
    """Index-by-index restatement of the summation formula (tiny shapes only)."""
    B, T, I = X.shape
    E, _, J = W.shape
    K = Ind.shape[2]
    Y = np.zeros((B, E, K, J), dtype=np.float64)
    for b in range(B):
        for e in range(E):
            for k in range(K):
                t = int(Ind[b, e, k])
                for j in range(J):
                    s = 0.0
                    for i in range(I):
                        s += float(X[b, t, i]) * float(W[e, i, j])
                    Y[b, e, k, j] = s
    return Y


def brute_scatter_forward(Y, W, Ind, T):
    B, E, K, J = Y.shape
    I = W.shape[2]
    out = np.zeros((B, T, I), dtype=np.float64)
    for b in range(B):
        for e in range(E):
            for k in range(K):
                t = int(Ind[b, e, k])
                for i in range(I):
                    s = 0.0
                    for j in range(J):
                        s += float(Y[b, e, k, j]) * float(W[e, j, i])
                    out[b, t, i] += s
    return out


def brute_gather_backward(X, W, Ind, dY):
    B, T, I = X.shape
    E, _, J = W.shape
    K = Ind.shape[2]
    dX = np.zeros((B, T, I), dtype=np.float64)
    dW = np.zeros((E, I, J), dtype=np.float64)
    for b in range(B):
        for e in range(E):
            for k in range(K):
                t = int(Ind[b, e, k])
                for i in range(I):
                    for j in range(J):
                        g = float(dY[b, e, k, j])
                        dX[b, t, i] += g * float(W[e, i, j])
                        dW[e, i, j] += float(X[b, t, i]) * g
    return dX, dW


def brute_scatter_backward(Y, W, Ind, dOut):
    B, E, K, J = Y.shape
    I = W.shape[2]
    dY = np.zeros((B, E, K, J), dtype=np.float64)
    dW = np.zeros((E, J, I), dtype=np.float64)
    for b in range(B):
        for e in range(E):
            for k in range(K):
                t = int(Ind[b, e, k])
                for j in range(J):
                    for i in range(I):
                        g = float(dOut[b, t, i])
                        dY[b, e, k, j] += g * float(W[e, j, i])
                        dW[e, j, i] += float(Y[b, e, k, j]) * g
    return dY, dW


# ----------------------------------------------------------------------------- fp8 weights
def fp8_e4m3fn_to_float(bits) -> np.ndarray:
    """Decode OCP e4m3fn bytes (1 sign, 4 exponent bias 7, 3 mantissa; no inf, 0x7f/0xff NaN)."""
    b = np.asarray(bits, dtype=np.uint8).astype(np.int32)
    sign = np.where(b & 0x80, -1.0, 1.0)
    exp = (b >> 3) & 0xF
    man = b & 0x7
    normal = np.ldexp(1.0 + man / 8.0, exp - 7)
    sub = np.ldexp(man / 8.0, -6)
    val = np.where(exp == 0, sub, normal)
    val = np.where((exp == 0xF) & (man == 0x7), np.nan, val)
    return (sign * val).astype(np.float64)


def dequant_fp8_weights(Wq_bits, scale) -> np.ndarray:
    """W[e,i,j] = decode(Wq[e,i,j]) * scale[e,j]  (per expert, per output column)."""
    Wf = fp8_e4m3fn_to_float(Wq_bits)
    scale = np.asarray(scale, dtype=np.float64)
    return Wf * scale[:, None, :]


def gather_forward_fp8w(X, Wq_bits, scale, Ind, acc=np.float64):
    """Dequantise-then-einsum reference for the fp8-weight gather."""
    return gather_forward(X, dequant_fp8_weights(Wq_bits, scale), Ind, acc=acc)


# ----------------------------------------------------------------------------- fp8 activations
def float_to_fp8_e4m3fn(x) -> np.ndarray:
    """Encode finite values of magnitude <= 448 as OCP e4m3fn bytes, round to nearest, ties to even.

    Works on the decode table: the two neighbouring codes of |x| are found by search, the nearer one
    wins and a tie goes to the code with an even mantissa (even byte value: consecutive codes
    alternate parity)."""
    x = np.asarray(x, dtype=np.float64)
    mags = fp8_e4m3fn_to_float(np.arange(0x7F, dtype=np.uint8))        # codes 0x00..0x7e, increasing, 0x7e = 448
    a = np.abs(x)
    if a.size and a.max() > 448.0:
        raise ValueError("magnitude above the e4m3 maximum")
    hi = np.clip(np.searchsorted(mags, a, side="left"), 0, 0x7E)      # first code >= |x|
    lo = np.maximum(hi - 1, 0)
    d_hi, d_lo = mags[hi] - a, a - mags[lo]
    pick_lo = (d_lo < d_hi) | ((d_lo == d_hi) & (lo % 2 == 0))
    code = np.where(pick_lo, lo, hi).astype(np.uint8)
    return np.where(np.signbit(x), code | 0x80, code).astype(np.uint8)


def quantize_rows_e4m3(X):
    """Per-row e4m3 quantisation of X[..., I] in float32 arithmetic: scale = max|row| / 448 (1 for a zero
    row, NaN for a row with a non-finite element), q = encode(clamp(x * (1 / scale), -448, 448)).
    Returns (bytes [..., I], scale [...])."""
    X = np.asarray(X, dtype=np.float32)
    finite = np.isfinite(X).all(axis=-1)
    Xf = np.where(finite[..., None], X, np.float32(0.0))
    amax = np.abs(Xf).max(axis=-1)
    scale = np.where(amax > 0, amax / np.float32(448.0), np.float32(1.0)).astype(np.float32)
    inv = (np.float32(1.0) / scale).astype(np.float32)
    y = np.clip((Xf * inv[..., None]).astype(np.float32), np.float32(-448.0), np.float32(448.0))
    # a row that holds a NaN or an infinity cannot be represented: its scale is NaN, so that every product
    # using the row is NaN as in unquantised arithmetic; its bytes are unspecified (zeros here)
    scale = np.where(finite, scale, np.float32(np.nan)).astype(np.float32)
    return float_to_fp8_e4m3fn(y), scale


def gather_forward_fp8(X, Wq_bits, scale, Ind, acc=np.float64):
    """fp8-activation, fp8-weight gather: rows quantised per row, both sides dequantised exactly, ordinary gather."""
    q, xs = quantize_rows_e4m3(X)
    Xd = fp8_e4m3fn_to_float(q) * xs[..., None].astype(np.float64)
    return gather_forward(Xd, dequant_fp8_weights(Wq_bits, scale), Ind, acc=acc)
