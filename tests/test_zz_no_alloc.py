"""The entry point that allocates nothing (egs_dw_builtin_scratch) against the entry point it is a variant of
(egs_dw with a caller-provided workspace), through the C ABI: same bits, and within the stated tolerance of the
CPU oracle, on two calls in a row of which the second is smaller (the built-in buffer then still holds the first
call's partial sums)."""
import numpy as np
import pytest
import torch

from oracle import egs_oracle as O
from tests._util import assert_close, make_case, np64

pytestmark = pytest.mark.gpu

from expertscattergather_amd import _abi
from expertscattergather_amd import hip_kernels as hk

DEV = "cuda"


def _dw_both(case, shape, dtype, layout):
    """(result of egs_dw_builtin_scratch, result of egs_dw, oracle) for one weight-gradient problem."""
    B, T, E, K, I, J = shape
    lib = _abi.lib()
    d = _abi.Dims(B, T, E, K, I, J)
    dt = hk.dtype_to_type_id(dtype)
    X, Y, Ind = case["X"].to(DEV), case["Y"].to(DEV), case["Ind"].to(DEV)
    shape_w = (E, I, J) if layout == _abi.W_EIJ else (E, J, I)
    stream = torch.cuda.current_stream().cuda_stream
    need = lib.egs_workspace_bytes(_abi.OP_DW, 0, d, dt)
    assert 0 < need <= _abi.BUILTIN_SCRATCH_BYTES, "the case must exercise the scratch buffer"
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    ref = torch.full(shape_w, float("nan"), dtype=dtype, device=DEV)
    got = torch.full(shape_w, float("nan"), dtype=dtype, device=DEV)
    print(f"egs_dw_builtin_scratch case shape={shape} dtype={dtype} layout={layout} scratch={need}", flush=True)
    rc = lib.egs_dw(X.data_ptr(), Y.data_ptr(), Ind.data_ptr(), ref.data_ptr(), ws.data_ptr(), need, d, T * I, I,
                    dt, dt, _abi.IND_I64, layout, stream)
    assert rc == 0, _abi.status_string(rc)
    rc = lib.egs_dw_builtin_scratch(X.data_ptr(), Y.data_ptr(), Ind.data_ptr(), got.data_ptr(), d, T * I, I,
                                    dt, dt, _abi.IND_I64, layout, stream)
    assert rc == 0, _abi.status_string(rc)
    torch.cuda.synchronize()
    Xn, Yn, Indn = np64(case["X"]), np64(case["Y"]), case["Ind"].numpy()
    if layout == _abi.W_EIJ:
        oracle = O.gather_backward(Xn, np.zeros((E, I, J)), Indn, Yn)[1]
    else:
        oracle = O.scatter_backward(Yn, np.zeros((E, J, I)), Indn, Xn)[1]
    return got, ref, oracle


@pytest.mark.parametrize("dtype,first,second", [
    (torch.bfloat16, (16, 128, 8, 32, 128, 64), (8, 64, 8, 32, 128, 64)),      # small-expert kernel, splits over the picks
    (torch.float32, (5, 127, 2, 126, 100, 72), (3, 37, 5, 11, 29, 13)),        # general tiled kernel, ragged tiles
], ids=["bf16-small-experts", "fp32-general"])
@pytest.mark.parametrize("layout", [_abi.W_EIJ, _abi.W_EJI], ids=["EIJ", "EJI"])
def test_builtin_scratch_matches_workspace_entry_point(dtype, first, second, layout):
    for n, shape in enumerate((first, second)):
        case = make_case(77 + n, *shape, dtype)
        got, ref, oracle = _dw_both(case, shape, dtype, layout)
        assert torch.equal(got, ref), f"call {n} {shape}: differs from egs_dw"
        assert_close(got, oracle, dtype, f"call {n} {shape}")


def test_builtin_scratch_rejects_sizes_beyond_its_buffer():
    lib = _abi.lib()
    d = _abi.Dims(16, 512, 4, 256, 1024, 1024)
    assert lib.egs_workspace_bytes(_abi.OP_DW, 0, d, _abi.BF16) > _abi.BUILTIN_SCRATCH_BYTES
    p = 0x1000          # never dereferenced: the size check comes first
    rc = lib.egs_dw_builtin_scratch(p, p, p, p, d, 512 * 1024, 1024, _abi.BF16, _abi.BF16, _abi.IND_I64, _abi.W_EIJ, None)
    assert rc == _abi.EGS_ERR_SCRATCH_LIMIT
    assert b"built-in" in lib.egs_status_string(rc)


def test_builtin_scratch_allocates_nothing_and_can_be_captured():
    """The call leaves the device's free memory and torch's allocator untouched, and - made once eagerly, so that the
    buffer's address is known - it can be recorded into a HIP graph (where hipMalloc is not allowed); every replay
    gives the bits of egs_dw, with the program's own eager work between the replays."""
    shape, dtype, layout = (16, 128, 8, 32, 128, 64), torch.bfloat16, _abi.W_EIJ
    B, T, E, K, I, J = shape
    lib = _abi.lib()
    d = _abi.Dims(*shape)
    dt = hk.dtype_to_type_id(dtype)
    case = make_case(83, *shape, dtype)
    X, Y, Ind = case["X"].to(DEV), case["Y"].to(DEV), case["Ind"].to(DEV)
    need = lib.egs_workspace_bytes(_abi.OP_DW, 0, d, dt)
    assert 0 < need <= _abi.BUILTIN_SCRATCH_BYTES
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    ref = torch.empty(E, I, J, dtype=dtype, device=DEV)
    got = torch.full((E, I, J), float("nan"), dtype=dtype, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.egs_dw(X.data_ptr(), Y.data_ptr(), Ind.data_ptr(), ref.data_ptr(), ws.data_ptr(), need, d, T * I, I, dt, dt,
                      _abi.IND_I64, layout, stream) == 0

    def call(s):
        return lib.egs_dw_builtin_scratch(X.data_ptr(), Y.data_ptr(), Ind.data_ptr(), got.data_ptr(), d, T * I, I, dt, dt,
                                          _abi.IND_I64, layout, s)

    assert call(stream) == 0                     # first call on the device: looks the buffer's address up
    torch.cuda.synchronize()
    free0, alloc0, reserved0 = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    for _ in range(3):
        assert call(stream) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0
    assert (torch.cuda.memory_allocated(), torch.cuda.memory_reserved()) == (alloc0, reserved0)
    assert torch.equal(got, ref)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        assert call(torch.cuda.current_stream().cuda_stream) == 0
    for n in range(3):
        got.fill_(float("nan"))
        X.mul_(-1.0)                             # eager work between the replays; the graph reads X in place
        assert lib.egs_dw(X.data_ptr(), Y.data_ptr(), Ind.data_ptr(), ref.data_ptr(), ws.data_ptr(), need, d, T * I, I, dt, dt,
                          _abi.IND_I64, layout, stream) == 0
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got, ref), f"replay {n}"
