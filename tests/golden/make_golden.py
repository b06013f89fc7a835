"""Writes the golden fixtures ``egs_golden.npz`` next to this file.

The reference ships no vectors for this path (its tests are unseeded random comparisons,
test_all.py:97-101), so the fixtures are produced by this repository's own CPU oracle
(oracle/egs_oracle.py, pinned by tests/test_oracle.py).  They freeze the oracle's answers on a
few tiny seeded cases so that a later change to the oracle or to the kernels shows up as a diff
against committed data.  Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import egs_oracle as O  # noqa: E402

# name: (B, T, E, K, I, J, input rounding, index dtype, with replacement)
CASES = {
    "odd_f32": (2, 7, 3, 5, 6, 4, "f32", np.int64, True),
    "dup_heavy_f32": (1, 3, 2, 8, 5, 3, "f32", np.int16, True),
    "aligned_bf16": (2, 16, 4, 8, 32, 16, "bf16", np.int64, False),
    "ragged_bf16": (3, 9, 2, 4, 24, 8, "bf16", np.int32, True),
    "f16_small": (1, 5, 3, 2, 8, 8, "f16", np.uint8, True),
}


def build_case(seed, B, T, E, K, I, J, rounding, ind_dtype, replace):
    g = np.random.default_rng(seed)
    rnd = {"f32": lambda a: a.astype(np.float32), "bf16": O.round_to_bf16, "f16": O.round_to_f16}[rounding]
    X = rnd(g.standard_normal((B, T, I)).astype(np.float32))
    Wg = rnd((g.standard_normal((E, I, J)) / np.sqrt(I)).astype(np.float32))
    Ws = rnd((g.standard_normal((E, J, I)) / np.sqrt(J)).astype(np.float32))
    Y = rnd(g.standard_normal((B, E, K, J)).astype(np.float32))
    dOut = rnd(g.standard_normal((B, T, I)).astype(np.float32))
    if replace:
        Ind = g.integers(0, T, size=(B, E, K))
    else:
        Ind = np.stack([np.stack([g.permutation(T)[:K] for _ in range(E)]) for _ in range(B)])
    Ind = Ind.astype(ind_dtype)
    out = {"X": X, "Wg": Wg, "Ws": Ws, "Y": Y, "dOut": dOut, "Ind": Ind}
    out["gather_Y"] = O.gather_forward(X, Wg, Ind)
    out["scatter_out"] = O.scatter_forward(Y, Ws, Ind, T)
    out["gather_dX"], out["gather_dW"] = O.gather_backward(X, Wg, Ind, Y)
    out["scatter_dY"], out["scatter_dW"] = O.scatter_backward(Y, Ws, Ind, dOut)
    return out


def main():
    blob = {}
    for i, (name, spec) in enumerate(CASES.items()):
        for key, val in build_case(500 + i, *spec).items():
            blob[f"{name}/{key}"] = val
    # fp8 weights: bits, scales and the dequantise-then-einsum answer
    g = np.random.default_rng(77)
    X = O.round_to_bf16(g.standard_normal((2, 6, 16)).astype(np.float32))
    bits = g.integers(0, 256, size=(3, 16, 8)).astype(np.uint8)
    bits[(bits & 0x7F) == 0x7F] = 0x3A                         # no NaN encodings
    scale = (g.random((3, 8)) * 0.01 + 0.001).astype(np.float32)
    Ind = g.integers(0, 6, size=(2, 3, 4)).astype(np.int64)
    blob.update({"fp8/X": X, "fp8/Wq_bits": bits, "fp8/scale": scale, "fp8/Ind": Ind,
                 "fp8/gather_Y": O.gather_forward_fp8w(X, bits, scale, Ind)})
    # inference block (gather -> activation -> scatter), bf16 inputs, rows rounded to bf16 after the activation; one
    # rejected pick; a shape the one-kernel form takes (8 batch elements, I = J = 32)
    g = np.random.default_rng(91)
    B, T, E, K, I, J = 8, 12, 4, 6, 32, 32
    X = O.round_to_bf16(g.standard_normal((B, T, I)).astype(np.float32))
    Wg = O.round_to_bf16((g.standard_normal((E, I, J)) / np.sqrt(I)).astype(np.float32))
    Ws = O.round_to_bf16((g.standard_normal((E, J, I)) / np.sqrt(J)).astype(np.float32))
    Ind = g.integers(0, T, size=(B, E, K)).astype(np.int32)
    Ind[3, 2, 1] = T + 1
    blob.update({"mlp/X": X, "mlp/Wg": Wg, "mlp/Ws": Ws, "mlp/Ind": Ind})
    for act in ("relu", "silu", "gelu"):
        blob[f"mlp/out_{act}"] = O.mlp_forward(X, Wg, Ws, Ind, T, act, round_y=O.round_to_bf16)
    path = os.path.join(HERE, "egs_golden.npz")
    np.savez_compressed(path, **blob)
    print(path, os.path.getsize(path), "bytes,", len(blob), "arrays")


if __name__ == "__main__":
    main()
