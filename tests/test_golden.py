"""Committed golden fixtures (tests/golden/egs_golden.npz, written by tests/golden/make_golden.py
from the CPU oracle): the oracle must still reproduce them exactly, the C restatement must agree
with them, and on the GPU the HIP path must match them within the dtype's tolerance."""
import os

import numpy as np
import pytest
import torch

from oracle import egs_oracle as O
from oracle import c_oracle as C
from tests._util import assert_close

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "egs_golden.npz")
GOLD = np.load(PATH)
CASES = sorted({k.split("/")[0] for k in GOLD.files} - {"fp8", "mlp"})
DTYPE = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}


def case(name):
    return {k.split("/", 1)[1]: GOLD[k] for k in GOLD.files if k.startswith(name + "/")}


@pytest.mark.parametrize("name", CASES)
def test_oracle_reproduces_the_fixtures(name):
    c = case(name)
    T = c["X"].shape[1]
    np.testing.assert_array_equal(O.gather_forward(c["X"], c["Wg"], c["Ind"]), c["gather_Y"])
    np.testing.assert_array_equal(O.scatter_forward(c["Y"], c["Ws"], c["Ind"], T), c["scatter_out"])
    dX, dW = O.gather_backward(c["X"], c["Wg"], c["Ind"], c["Y"])
    np.testing.assert_array_equal(dX, c["gather_dX"]); np.testing.assert_array_equal(dW, c["gather_dW"])
    dY, dWs = O.scatter_backward(c["Y"], c["Ws"], c["Ind"], c["dOut"])
    np.testing.assert_array_equal(dY, c["scatter_dY"]); np.testing.assert_array_equal(dWs, c["scatter_dW"])
    # second, loop-level implementation
    np.testing.assert_allclose(C.gather(c["X"], c["Wg"], c["Ind"]), c["gather_Y"], rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(C.scatter(c["Y"], c["Ws"], c["Ind"], T), c["scatter_out"], rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(C.dw(c["X"], c["Y"], c["Ind"]), c["gather_dW"], rtol=1e-12, atol=1e-12)


def test_fp8_fixture():
    c = case("fp8")
    np.testing.assert_array_equal(O.gather_forward_fp8w(c["X"], c["Wq_bits"], c["scale"], c["Ind"]), c["gather_Y"])
    W = torch.from_numpy(c["Wq_bits"]).view(torch.float8_e4m3fn).double().numpy() * c["scale"].astype(np.float64)[:, None, :]
    np.testing.assert_allclose(O.gather_forward(c["X"], W, c["Ind"]), c["gather_Y"], rtol=1e-12, atol=1e-15)


def test_inference_block_fixture():
    c = case("mlp")
    T = c["X"].shape[1]
    for act in ("relu", "silu", "gelu"):
        np.testing.assert_array_equal(O.mlp_forward(c["X"], c["Wg"], c["Ws"], c["Ind"], T, act, round_y=O.round_to_bf16),
                                      c[f"out_{act}"])


@pytest.mark.gpu
def test_hip_inference_block_matches_the_fixture():
    from expertscattergather_amd import hip_kernels as hk
    c = case("mlp")
    dev = "cuda"
    t = lambda a: torch.from_numpy(a).to(dev, torch.bfloat16)
    Ind = torch.from_numpy(c["Ind"]).to(dev)
    for act in ("relu", "silu", "gelu"):
        got = hk.expert_mlp_forward(t(c["X"]), t(c["Wg"]), t(c["Ws"]), Ind, act, force_block=True)
        assert_close(got, c[f"out_{act}"], torch.bfloat16, f"inference block {act}")


@pytest.mark.gpu
@pytest.mark.parametrize("name", CASES)
def test_hip_path_matches_the_fixtures(name):
    from expertscattergather_amd import hip_kernels as hk
    hk.create_kernels()
    c = case(name)
    dt = DTYPE[name.split("_")[-1]] if name.split("_")[-1] in DTYPE else DTYPE[name.split("_")[0]]
    dev = "cuda"
    t = lambda a: torch.from_numpy(a).to(dev, dt)
    Ind = torch.from_numpy(c["Ind"]).to(dev)
    T = c["X"].shape[1]
    assert_close(hk.expert_gather_forward_call(t(c["X"]), t(c["Wg"]), Ind, torch.float32), c["gather_Y"], dt, "gather_Y")
    assert_close(hk.expert_scatter_forward_call(t(c["Y"]), t(c["Ws"]), Ind, T, torch.float32), c["scatter_out"], dt, "scatter_out")
    dX, dW = hk.expert_gather_backward_call(t(c["X"]), t(c["Wg"]), Ind, t(c["Y"]), torch.float32)
    assert_close(dX, c["gather_dX"], dt, "gather_dX"); assert_close(dW, c["gather_dW"], dt, "gather_dW")
    dY, dWs = hk.expert_scatter_backward_call(t(c["Y"]), t(c["Ws"]), Ind, t(c["dOut"]), torch.float32)
    assert_close(dY, c["scatter_dY"], dt, "scatter_dY"); assert_close(dWs, c["scatter_dW"], dt, "scatter_dW")


@pytest.mark.gpu
def test_hip_fp8_weight_gather_matches_the_fixture():
    from expertscattergather_amd import hip_kernels as hk
    c = case("fp8")
    dev = "cuda"
    Y = hk.expert_gather_fp8w_forward(torch.from_numpy(c["X"]).to(dev, torch.bfloat16),
                                      torch.from_numpy(c["Wq_bits"]).to(dev).view(torch.float8_e4m3fn),
                                      torch.from_numpy(c["scale"]).to(dev), torch.from_numpy(c["Ind"]).to(dev))
    assert_close(Y, c["gather_Y"], torch.bfloat16, "fp8 gather_Y")
