"""GPU parity: the HIP path (through the C ABI) against the CPU oracle on the same seeded
inputs.  Covers the four launchers, both weight layouts, fp32/bf16/fp16, all index widths,
ragged shapes (the reference draws every dimension from 1..127, test_all.py:97-99),
duplicate-heavy routing, both scatter modes and the module/autograd surface."""
import numpy as np
import pytest
import torch

from oracle import egs_oracle as O
from oracle import torch_port as P
from tests._util import assert_close, make_case, np64

pytestmark = pytest.mark.gpu

import expertscattergather_amd as egs
from expertscattergather_amd import hip_kernels as hk

hk.create_kernels()
DEV = "cuda"

# (B, T, E, K, I, J)
SHAPES = [
    (2, 16, 3, 8, 32, 16),        # small aligned
    (4, 64, 8, 16, 128, 64),      # default-like, scaled down
    (3, 37, 5, 11, 29, 13),       # everything odd, unaligned rows
    (1, 1, 1, 1, 1, 1),
    (5, 127, 2, 126, 100, 72),    # tails in every tile dimension
    (2, 50, 9, 40, 136, 200),     # N > 128: two column tiles; E not a multiple of 8
    (7, 9, 17, 3, 8, 4),
    (2, 300, 4, 130, 260, 96),    # several reduction slabs and row tiles
    (3, 300, 5, 200, 192, 256),   # large products: 256 x 256 tiles, ragged last row tile, 192 of 256 columns
    (2, 128, 9, 260, 128, 200),   # large gather with half a 16-column tile at the edge
    (2, 200, 3, 128, 256, 72),    # large weight gradient without splits, 72 of 128 columns
    (3, 100, 5, 200, 256, 128),   # large scatter products with a short reduction (128), ragged last row tile
    (2, 80, 3, 260, 512, 256),    # the same with reduction 256 and two column tiles
    (3, 100, 5, 200, 128, 256),   # large dY with 128 output columns (256 x 128 tiles, weight stored [column][reduction])
    (2, 150, 3, 300, 128, 136),   # large gather with 136 output columns: two 128-column tiles, the second nearly empty
    (2, 150, 3, 300, 136, 128),   # the same for dY
    (2, 200, 3, 150, 256, 128),   # 300 rows per expert: the smallest products the 256-row tiles are used for
]
DTYPES = [torch.float32, torch.bfloat16, torch.float16]


def dev(t):
    return t.to(DEV)


def run_all(case, T, mode="deterministic"):
    hk.set_scatter_mode(mode)
    X, Wg, Ws, Y, dOut, Ind = (dev(case[k]) for k in ("X", "Wg", "Ws", "Y", "dOut", "Ind"))
    out = {}
    out["Y"] = hk.expert_gather_forward_call(X, Wg, Ind, torch.float32)
    out["out"] = hk.expert_scatter_forward_call(Y, Ws, Ind, T, torch.float32)
    out["dX"], out["dWg"] = hk.expert_gather_backward_call(X, Wg, Ind, Y, torch.float32)
    out["dY"], out["dWs"] = hk.expert_scatter_backward_call(Y, Ws, Ind, dOut, torch.float32)
    torch.cuda.synchronize()
    hk.set_scatter_mode("deterministic")
    return out


def oracle_all(case, T):
    X, Wg, Ws, Y, dOut = (np64(case[k]) for k in ("X", "Wg", "Ws", "Y", "dOut"))
    Ind = case["Ind"].to(torch.int64).numpy()
    ref = {}
    ref["Y"] = O.gather_forward(X, Wg, Ind)
    ref["out"] = O.scatter_forward(Y, Ws, Ind, T)
    ref["dX"], ref["dWg"] = O.gather_backward(X, Wg, Ind, Y)
    ref["dY"], ref["dWs"] = O.scatter_backward(Y, Ws, Ind, dOut)
    return ref


# shapes that qualify for the small-expert kernels (16-bit, reduction length 32/64/128, output
# width a multiple of 8 and <= 64 for the gather, K <= 64 for the scatter), with ragged K, T, E
SMALL_SHAPES = [
    (3, 50, 9, 11, 64, 32),       # ragged K, T, E; expert groups of unequal size
    (2, 33, 5, 64, 128, 64),      # K = 64: four row tiles, E < 8: one expert group
    (5, 20, 3, 7, 32, 8),
    (2, 256, 32, 32, 128, 64),    # two batch elements of the default shape
    (9, 40, 12, 33, 128, 32),     # K = 33
    (2, 700, 8, 20, 32, 64),      # long T: accumulators of one expert group fill the LDS
    (3, 64, 16, 16, 64, 56),      # J not a multiple of 16 (gather columns), scatter takes the general path
    (8, 60, 6, 20, 64, 128),      # reduction 128 on the one-kernel scatter, ragged 16-pick tiles
    (4, 300, 40, 25, 96, 32),     # 1000 picks per batch element, three 32-column slices
    (2, 48, 40, 9, 72, 40),       # one-pass weight gradient with ragged 32 x 32 / 32 x 64 tiles (72 = 2 x 32 + 8, 40 = 32 + 8)
    (1, 16, 64, 3, 40, 104),      # ... with fewer picks per expert (3) than one 32-pick step, many experts
    # one-kernel scatter in passes over groups of experts (more picks per batch element than LDS holds product rows for)
    (2, 256, 48, 32, 128, 64),    # 1536 picks: two passes of 24 experts
    (4, 100, 20, 100, 64, 32),    # 2000 picks, K = 100 (ragged 32-pick units): two passes of 10 experts
    (8, 500, 33, 64, 32, 64),     # 2112 picks, T near the limit of 512, uneven last group (11 + 11 + 11 / 17 + 16)
    (8, 64, 64, 64, 32, 32),      # 4096 picks: four passes of 16 experts
]

# sizes beyond the one-kernel scatters above that the compact mode's one-kernel scatter in passes takes (16-bit types,
# reduction 32 / 64 / 128, T <= 1024): 32-pick units, the sums of up to 1024 tokens in registers
PASS_SHAPES = [
    (8, 700, 20, 100, 320, 64),   # 2000 picks, ragged units (K = 100), three passes, T > 512
    (3, 1000, 33, 150, 1024, 32), # 4950 picks, reduction 32, 32 slices
    (10, 1024, 40, 128, 256, 128),# 5120 picks, reduction 128, T at the limit, five passes of whole experts
    (2, 600, 7, 300, 128, 128),   # few workgroups (8), one expert spans ten units: a wavefront's units change expert mid-pass
]


@pytest.fixture(params=[False, True], ids=["fastpaths", "generic"])
def force_generic(request):
    from expertscattergather_amd import _abi
    _abi.lib().egs_testing_force_generic(1 if request.param else 0)
    hk._ws_sizes.clear()                    # remembered workspace and table sizes belong to the other kernel family
    hk._table_sizes.clear()
    yield request.param
    _abi.lib().egs_testing_force_generic(0)
    hk._ws_sizes.clear()
    hk._table_sizes.clear()


@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("shape", SHAPES + SMALL_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_four_launchers_match_oracle(shape, dtype, force_generic):
    B, T, E, K, I, J = shape
    case = make_case(100 + sum(shape), *shape, dtype)
    got = run_all(case, T)
    ref = oracle_all(case, T)
    for name in ("Y", "out", "dX", "dWg", "dY", "dWs"):
        assert got[name].dtype == dtype
        assert_close(got[name], ref[name], dtype, f"{name} {shape} {dtype}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [SHAPES[1], SHAPES[2], SHAPES[5]], ids=lambda s: "x".join(map(str, s)))
def test_atomic_mode_matches_oracle(shape, dtype):
    B, T, E, K, I, J = shape
    case = make_case(7 + sum(shape), *shape, dtype)
    got = run_all(case, T, mode="atomic")
    ref = oracle_all(case, T)
    for name in ("out", "dX"):
        assert_close(got[name], ref[name], dtype, f"atomic {name} {shape} {dtype}")


@pytest.mark.parametrize("ind_dtype", [torch.uint8, torch.int16, torch.int32, torch.int64])
def test_index_widths_pass_through(ind_dtype):
    shape = (3, 100, 4, 12, 48, 24)
    case = make_case(5, *shape, torch.float32, ind_dtype=ind_dtype)
    before = case["Ind"].clone()
    got = run_all(case, shape[1])
    ref = oracle_all(case, shape[1])
    for name in ("Y", "out", "dX", "dWg", "dY", "dWs"):
        assert_close(got[name], ref[name], torch.float32, f"{name} {ind_dtype}")
    assert torch.equal(case["Ind"], before)


def test_ind_is_never_written():
    case = make_case(6, 4, 40, 6, 10, 64, 32, torch.bfloat16)
    Ind = dev(case["Ind"]); keep = Ind.clone()
    hk.expert_scatter_forward_call(dev(case["Y"]), dev(case["Ws"]), Ind, 40, torch.float32)
    hk.expert_gather_backward_call(dev(case["X"]), dev(case["Wg"]), Ind, dev(case["Y"]), torch.float32)
    torch.cuda.synchronize()
    assert torch.equal(Ind, keep)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bfloat16", "float16"])
@pytest.mark.parametrize("shape", PASS_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_compact_mode_matches_oracle(shape, dtype):
    from expertscattergather_amd import _abi
    B, T, E, K, I, J = shape
    case = make_case(300 + sum(shape), *shape, dtype)
    with _abi.launch_log() as log:
        got = run_all(case, T, mode="compact")
    assert log.kernels.count("scatter_pass_kernel") == 2, log.kernels          # the scatter forward, and dX
    ref = oracle_all(case, T)
    for name in ("Y", "out", "dX", "dWg", "dY", "dWs"):
        assert_close(got[name], ref[name], dtype, f"compact {name} {shape} {dtype}")
    d = _abi.Dims(*shape)
    dt = hk.dtype_to_type_id(dtype)
    lib = _abi.lib()
    assert lib.egs_workspace_bytes(_abi.OP_GEMM_SCATTER, _abi.SCATTER_COMPACT, d, dt) < \
        lib.egs_workspace_bytes(_abi.OP_GEMM_SCATTER, _abi.SCATTER_DETERMINISTIC, d, dt) // 8


def test_deterministic_mode_is_bitwise_reproducible_with_hot_tokens():
    # all picks of every expert land on 3 tokens: long same-token chains
    B, T, E, K, I, J = 4, 64, 8, 48, 96, 40
    case = make_case(9, B, T, E, K, I, J, torch.float32)
    case["Ind"] = torch.randint(0, 3, (B, E, K), generator=torch.Generator().manual_seed(1))
    Y, Ws, Ind = dev(case["Y"]), dev(case["Ws"]), dev(case["Ind"])
    hk.set_scatter_mode("deterministic")
    first = hk.expert_scatter_forward_call(Y, Ws, Ind, T, torch.float32)
    junk = torch.randn(1 << 20, device=DEV)          # disturb the allocator between runs
    for _ in range(3):
        again = hk.expert_scatter_forward_call(Y, Ws, Ind, T, torch.float32)
        assert torch.equal(first, again)
    assert_close(first, O.scatter_forward(np64(case["Y"]), np64(case["Ws"]), case["Ind"].numpy(), T), torch.float32, "hot tokens")
    dW1 = hk.expert_gather_backward_call(dev(case["X"]), dev(case["Wg"]), Ind, Y, torch.float32)[1]
    dW2 = hk.expert_gather_backward_call(dev(case["X"]), dev(case["Wg"]), Ind, Y, torch.float32)[1]
    assert torch.equal(dW1, dW2)
    hk.set_scatter_mode("atomic")
    atomic = hk.expert_scatter_forward_call(Y, Ws, Ind, T, torch.float32)
    hk.set_scatter_mode("deterministic")
    assert_close(atomic, np64(first), torch.float32, "atomic vs deterministic")
    del junk


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bfloat16", "float16"])
def test_pass_scatter_with_long_segments_is_ordered(dtype):
    """The one-kernel scatter in passes (compact mode) under skew: a quarter of a batch element's picks on one token (its
    16-token block's list holds a quarter of every pass), a few tokens with 65 .. 500 picks, many with 5 .. 64, rejected
    picks, tokens nobody picks; both weight layouts; bitwise repeatable; the kernel is the one asserted."""
    from expertscattergather_amd import _abi
    B, T, E, K, I, J = 8, 900, 50, 120, 320, 64
    case = make_case(23, B, T, E, K, I, J, dtype)
    g = torch.Generator().manual_seed(4)
    p = torch.arange(1, T + 1, dtype=torch.float64).pow(-1.2)
    Ind = torch.multinomial(p.expand(B * E, T), K, replacement=True, generator=g).reshape(B, E, K)
    Ind = torch.randperm(T, generator=g)[Ind]
    Ind[Ind == 17] = 18                                     # a token nobody picks
    Ind[0, 0, 0] = -1; Ind[B - 1, E - 1, K - 1] = T; Ind[3, 7, 50] = 30000
    counts = torch.bincount(Ind[1][(Ind[1] >= 0) & (Ind[1] < T)].reshape(-1), minlength=T)
    assert counts.max() > 0.2 * E * K and ((counts > 64) & (counts < 400)).sum() >= 3 and ((counts > 4) & (counts <= 64)).sum() > 20
    bad = (Ind < 0) | (Ind >= T)
    safe = Ind.clone(); safe[bad] = 0
    mask = (~bad).numpy()[..., None]
    Y, Ws, Wg, Indg = dev(case["Y"]), dev(case["Ws"]), dev(case["Wg"]), dev(Ind)
    with hk.scatter_mode_scope("compact"):
        with _abi.launch_log() as log:
            out = hk.expert_scatter_forward_call(Y, Ws, Indg, T, torch.float32)
        assert "scatter_pass_kernel" in log.kernels, log.kernels
        for _ in range(3):
            assert torch.equal(out, hk.expert_scatter_forward_call(Y, Ws, Indg, T, torch.float32))
        assert_close(out, O.scatter_forward(np64(case["Y"]) * mask, np64(case["Ws"]), safe.numpy(), T), dtype, "pass scatter, skewed")
        assert out[:, 17].abs().max().item() == 0.0
        with _abi.launch_log() as log:
            dX, _ = hk.expert_gather_backward_call(dev(case["X"]), Wg, Indg, Y, torch.float32)
        assert "scatter_pass_kernel" in log.kernels, log.kernels
        assert torch.equal(dX, hk.expert_gather_backward_call(dev(case["X"]), Wg, Indg, Y, torch.float32)[0])
        assert_close(dX, O.gather_backward(np64(case["X"]), np64(case["Wg"]), safe.numpy(), np64(case["Y"]) * mask)[0], dtype,
                     "pass scatter as dX, skewed")


def test_pass_scatter_with_more_long_tokens_than_slots():
    """Seventy tokens of a batch element with more than 64 picks each, spread over the token blocks of all wavefronts:
    repeatable and within tolerance."""
    B, T, E, K, I, J = 10, 600, 64, 100, 256, 32
    dtype = torch.bfloat16
    case = make_case(29, B, T, E, K, I, J, dtype)
    g = torch.Generator().manual_seed(6)
    hot = torch.randperm(T, generator=g)[:70]
    Ind = hot[torch.randint(0, 70, (B, E, K), generator=g)]          # 6400 picks on 70 tokens: ~91 each
    counts = torch.bincount(Ind[0].reshape(-1), minlength=T)
    assert (counts > 64).sum() > 64
    Y, Ws, Indg = dev(case["Y"]), dev(case["Ws"]), dev(Ind)
    with hk.scatter_mode_scope("compact"):
        out = hk.expert_scatter_forward_call(Y, Ws, Indg, T, torch.float32)
        assert torch.equal(out, hk.expert_scatter_forward_call(Y, Ws, Indg, T, torch.float32))
    assert_close(out, O.scatter_forward(np64(case["Y"]), np64(case["Ws"]), Ind.numpy(), T), dtype, "pass scatter, 70 long tokens")


def test_pass_scatter_keeps_a_value_that_is_not_finite_to_its_token():
    """Compact mode adds with matrix instructions whose selector is 0 or 1; 0 x inf would be NaN for the other tokens of a
    16-token block, so a pass with a product that is not finite takes its sums without multiplications: the value reaches
    the token that picked it and nobody else, and every other row is what it is without that pick."""
    from expertscattergather_amd import _abi
    B, T, E, K, I, J = 8, 600, 20, 100, 64, 64           # T > 512: beyond the one-kernel scatter of small experts
    dtype = torch.bfloat16
    case = make_case(41, B, T, E, K, I, J, dtype)
    Ind = case["Ind"].clone()
    Yc = case["Y"].clone()
    b, e, k = 2, 7, 33
    t_bad = int(Ind[b, e, k])
    Yc[b, e, k, :] = float("inf")
    Yc[b + 1, e, k, 3] = float("nan")
    t_nan = int(Ind[b + 1, e, k])
    Y, Ws, Indg = dev(Yc), dev(case["Ws"]), dev(Ind)
    with hk.scatter_mode_scope("compact"), _abi.launch_log() as log:
        out = hk.expert_scatter_forward_call(Y, Ws, Indg, T, torch.float32)
        again = hk.expert_scatter_forward_call(Y, Ws, Indg, T, torch.float32)
    assert log.kernels.count("scatter_pass_kernel") == 2, log.kernels
    finite = torch.isfinite(out.float())
    assert not finite[b, t_bad].any() and not finite[b + 1, t_nan].any()       # inf . W has both signs in every column: inf or nan
    finite[b, t_bad] = True; finite[b + 1, t_nan] = True
    assert finite.all(), "a value that is not finite leaked to another token"
    assert torch.equal(torch.nan_to_num(out.float(), 0.0, 0.0, 0.0), torch.nan_to_num(again.float(), 0.0, 0.0, 0.0))
    Yz = Yc.clone(); Yz[b, e, k, :] = 0; Yz[b + 1, e, k, :] = 0
    ref = O.scatter_forward(np64(Yz), np64(case["Ws"]), Ind.numpy(), T)
    got = out.clone(); got[b, t_bad] = 0; got[b + 1, t_nan] = 0
    ref[b, t_bad] = 0; ref[b + 1, t_nan] = 0
    assert_close(got, ref, dtype, "pass scatter beside a value that is not finite")


@pytest.mark.parametrize("ind_dtype", [torch.int32, torch.int16], ids=["int32", "int16"])
def test_pass_scatter_reads_narrow_indices(ind_dtype):
    """The compact mode sorts each pass's picks from Ind itself (no routing table in memory): every index width, ragged
    K (units of 32 picks with a short last one), T not a multiple of 16."""
    from expertscattergather_amd import _abi
    B, T, E, K, I, J = 9, 777, 37, 45, 96, 32
    dtype = torch.float16
    case = make_case(43, B, T, E, K, I, J, dtype)
    Ind = case["Ind"].clone()
    Ind[0, 0, 0] = -1; Ind[4, 5, 6] = T
    bad = (Ind < 0) | (Ind >= T)
    safe = Ind.clone(); safe[bad] = 0
    mask = (~bad).numpy()[..., None]
    with hk.scatter_mode_scope("compact"), _abi.launch_log() as log:
        out = hk.expert_scatter_forward_call(dev(case["Y"]), dev(case["Ws"]), dev(Ind.to(ind_dtype)), T, torch.float32)
    assert "scatter_pass_kernel" in log.kernels, log.kernels
    assert_close(out, O.scatter_forward(np64(case["Y"]) * mask, np64(case["Ws"]), safe.numpy(), T), dtype, f"pass scatter, {ind_dtype}")


def test_multi_pass_scatter_is_bitwise_reproducible_with_hot_tokens():
    # 1536 picks per batch element on 5 tokens: every segment spans both passes of the one-kernel scatter
    B, T, E, K, I, J = 4, 64, 48, 32, 64, 32
    case = make_case(21, B, T, E, K, I, J, torch.bfloat16)
    case["Ind"] = torch.randint(0, 5, (B, E, K), generator=torch.Generator().manual_seed(2))
    Y, Ws, Ind = dev(case["Y"]), dev(case["Ws"]), dev(case["Ind"])
    hk.set_scatter_mode("deterministic")
    first = hk.expert_scatter_forward_call(Y, Ws, Ind, T, torch.float32)
    for _ in range(3):
        assert torch.equal(first, hk.expert_scatter_forward_call(Y, Ws, Ind, T, torch.float32))
    assert_close(first, O.scatter_forward(np64(case["Y"]), np64(case["Ws"]), case["Ind"].numpy(), T), torch.bfloat16, "hot tokens, two passes")
    assert first[:, 5:].abs().max().item() == 0.0      # tokens nobody picked


@pytest.mark.parametrize("shape,dtype", [((3, 40, 6, 100, 24, 16), torch.float32),      # small-expert rows, table built by the general sorter
                                         ((2, 64, 8, 64, 128, 64), torch.bfloat16),     # small-expert rows, table rides along
                                         ((2, 50, 4, 300, 30, 24), torch.float16),      # I not a multiple of 4: scalar columns
                                         ((2, 300, 4, 200, 256, 192), torch.bfloat16)], # 256 x 256 tile rows
                         ids=lambda v: "x".join(map(str, v)) if isinstance(v, tuple) else str(v).split(".")[-1])
@pytest.mark.parametrize("mode", ["deterministic", "atomic"])
def test_long_segments_are_reduced_in_chunks(shape, dtype, mode):
    # tokens picked far more often than one thread group reduces in one go: segment lengths around the
    # chunk size and its double (63, 64, 65, 127, 128, 129), many chunks, one token taking most picks, and empty tokens
    B, T, E, K, I, J = shape
    case = make_case(21, B, T, E, K, I, J, dtype)
    N = E * K
    gen = torch.Generator().manual_seed(5)
    Ind = torch.empty(B, N, dtype=torch.int64)
    for b in range(B):
        lens = [63, 64, 65, 127, 128, 129] if b == 0 else [N // 2 + 3, 193]
        lens = [n for n in lens if n > 0]
        while sum(lens) > N:
            lens.pop()
        toks = torch.randperm(T, generator=gen)
        flat = torch.cat([torch.full((n,), int(toks[i])) for i, n in enumerate(lens)] +
                         [toks[len(lens) + torch.randint(0, max(1, T // 2 - len(lens)), (N - sum(lens),), generator=gen)]])
        Ind[b] = flat[torch.randperm(N, generator=gen)]
    Ind = Ind.reshape(B, E, K)
    hk.set_scatter_mode(mode)
    Y, Ws = dev(case["Y"]), dev(case["Ws"])
    got = hk.expert_scatter_forward_call(Y, Ws, dev(Ind), T, torch.float32)
    ref = O.scatter_forward(np64(case["Y"]), np64(case["Ws"]), Ind.numpy(), T)
    hk.set_scatter_mode("deterministic")
    assert_close(got, ref, dtype, "long segments")
    if mode == "deterministic":
        hk.set_scatter_mode(mode)
        for _ in range(3):
            assert torch.equal(got, hk.expert_scatter_forward_call(Y, Ws, dev(Ind), T, torch.float32))
    # the same table drives dX
    dX = hk.expert_gather_backward_call(dev(case["X"]), dev(case["Wg"]), dev(Ind), Y, torch.float32)[0]
    assert_close(dX, O.gather_backward(np64(case["X"]), np64(case["Wg"]), Ind.numpy(), np64(case["Y"]))[0], dtype, "dX long segments")


@pytest.mark.parametrize("mode", ["deterministic", "atomic"])
def test_scatter_output_does_not_depend_on_stale_memory(mode):
    # the reference allocates the scatter output with torch.empty and only adds into it
    # (egs/triton_kernels.py:457); here unpicked tokens must read exactly zero on every call
    B, T, E, K, I, J = 2, 200, 2, 5, 64, 16
    case = make_case(11, B, T, E, K, I, J, torch.bfloat16)
    hk.set_scatter_mode(mode)
    Y, Ws, Ind = dev(case["Y"]), dev(case["Ws"]), dev(case["Ind"])
    outs = []
    for _ in range(3):
        dirty = torch.full((B, T, I), 7.0, device=DEV, dtype=torch.bfloat16)
        del dirty                                        # freed block is handed to the next empty()
        outs.append(hk.expert_scatter_forward_call(Y, Ws, Ind, T, torch.float32).clone())
    hk.set_scatter_mode("deterministic")
    picked = torch.zeros(B, T, dtype=torch.bool)
    picked.scatter_(1, case["Ind"].reshape(B, -1), True)
    for o in outs:
        assert (o.cpu()[~picked] == 0).all()
        assert_close(o, O.scatter_forward(np64(case["Y"]), np64(case["Ws"]), case["Ind"].numpy(), T), torch.bfloat16, "stale")


@pytest.mark.parametrize("shape,dtype", [((2, 20, 3, 6, 32, 16), torch.float32),
                                         ((2, 300, 3, 260, 192, 256), torch.bfloat16),      # 256 x 256 tile kernels
                                         # small-expert kernels (register-resident gather, one-kernel scatter, split weight
                                         # gradient); a rejected pick reads row 0 / a clamped address there and is masked
                                         ((2, 64, 8, 16, 128, 64), torch.bfloat16),
                                         # the same with enough experts for the one-pass weight gradient (its rejected picks
                                         # get a buffer offset outside the descriptor) and its shared launch with the gather
                                         ((8, 64, 32, 16, 128, 64), torch.float16),
                                         ((8, 64, 32, 16, 128, 64), torch.float32),         # fp32 form of the same kernels
                                         # one-kernel scatter in two passes: a rejected pick has no place in the table
                                         ((4, 64, 48, 32, 64, 32), torch.bfloat16)],
                         ids=["small-f32", "large-bf16", "small-experts-bf16", "one-pass-dw-f16", "one-pass-dw-f32", "two-pass-scatter-bf16"])
def test_out_of_range_picks_contribute_nothing(shape, dtype):
    B, T, E, K, I, J = shape
    case = make_case(13, B, T, E, K, I, J, dtype)
    Ind = case["Ind"].clone()
    Ind[0, 0, 0] = T; Ind[1, 2, 3] = -1; Ind[1, 1, 1] = 10 ** 9
    bad = (Ind < 0) | (Ind >= T)
    assert hk.validate_indices(dev(Ind), T) == int(bad.sum())
    assert hk.validate_indices(dev(case["Ind"]), T) == 0
    case2 = dict(case, Ind=Ind)
    got = run_all(case2, T)
    # oracle with the bad picks removed: zero their Y rows / route them to a spare token
    X, Wg, Ws, Y, dOut = (np64(case[k]) for k in ("X", "Wg", "Ws", "Y", "dOut"))
    safe = Ind.clone(); safe[bad] = 0
    mask = (~bad).numpy()[..., None]
    refY = O.gather_forward(X, Wg, safe.numpy()) * mask
    assert_close(got["Y"], refY, dtype, "Y with bad picks")
    assert_close(got["out"], O.scatter_forward(Y * mask, Ws, safe.numpy(), T), dtype, "out with bad picks")
    dX, dWg = O.gather_backward(X, Wg, safe.numpy(), Y * mask)
    assert_close(got["dX"], dX, dtype, "dX with bad picks")
    assert_close(got["dWg"], dWg, dtype, "dWg with bad picks")
    dYo, dWso = O.scatter_backward(Y * mask, Ws, safe.numpy(), dOut)
    assert_close(got["dY"], dYo * mask, dtype, "dY with bad picks")
    assert_close(got["dWs"], dWso, dtype, "dWs with bad picks")


def test_strided_source_rows():
    B, T, E, K, I, J = 3, 30, 4, 7, 64, 32
    case = make_case(17, B, T, E, K, I, J, torch.float32)
    big = torch.randn(B, T, 2 * I + 8)
    big[:, :, 8:8 + I] = case["X"]
    Xs = dev(big)[:, :, 8:8 + I]                      # token stride 2I+8, inner stride 1
    assert not Xs.is_contiguous()
    Y = hk.expert_gather_forward_call(Xs, dev(case["Wg"]), dev(case["Ind"]), torch.float32)
    assert_close(Y, O.gather_forward(np64(case["X"]), np64(case["Wg"]), case["Ind"].numpy()), torch.float32, "strided X")
    Xt = dev(case["X"].transpose(1, 2).contiguous()).transpose(1, 2)   # inner stride != 1 -> copied
    Y2 = hk.expert_gather_forward_call(Xt, dev(case["Wg"]), dev(case["Ind"]), torch.float32)
    assert torch.equal(Y, Y2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bfloat16", "float32"])
def test_strided_source_rows_on_the_small_expert_kernels(dtype):
    # rows of X and of the scatter's incoming gradient taken out of wider tensors (token stride 2I + 8 elements, 16-byte
    # aligned): register-resident gather, one-pass weight gradient in both backward calls, inference block
    B, T, E, K, I, J = 8, 64, 32, 16, 128, 64
    case = make_case(19, B, T, E, K, I, J, dtype)
    def widen(t):
        big = torch.randn(B, T, 2 * I + 8).to(dtype)
        big[:, :, 8:8 + I] = t
        v = dev(big)[:, :, 8:8 + I]
        assert not v.is_contiguous()
        return v
    Xs, dOs = widen(case["X"]), widen(case["dOut"])
    Wg, Ws, Y, Ind = (dev(case[k]) for k in ("Wg", "Ws", "Y", "Ind"))
    Xn, Wgn, Wsn, Yn, dOn = (np64(case[k]) for k in ("X", "Wg", "Ws", "Y", "dOut"))
    Indn = case["Ind"].numpy()
    assert_close(hk.expert_gather_forward_call(Xs, Wg, Ind, torch.float32), O.gather_forward(Xn, Wgn, Indn), dtype, "strided X")
    dX, dWg = hk.expert_gather_backward_call(Xs, Wg, Ind, Y, torch.float32)
    rX, rWg = O.gather_backward(Xn, Wgn, Indn, Yn)
    assert_close(dX, rX, dtype, "dX, strided X"); assert_close(dWg, rWg, dtype, "dWg, strided X")
    dY, dWs = hk.expert_scatter_backward_call(Y, Ws, Ind, dOs, torch.float32)
    rY, rWs = O.scatter_backward(Yn, Wsn, Indn, dOn)
    assert_close(dY, rY, dtype, "dY, strided gradient"); assert_close(dWs, rWs, dtype, "dWs, strided gradient")
    if dtype is torch.bfloat16:
        got = hk.expert_mlp_forward(Xs, Wg, Ws, Ind, "relu", force_block=True)
        assert_close(got, _mlp_oracle(case, T, "relu", dtype), dtype, "inference block, strided X")


def test_empty_inputs():
    Wg = torch.zeros(3, 8, 4, device=DEV); Ws = torch.zeros(3, 4, 8, device=DEV)
    X = torch.zeros(2, 5, 8, device=DEV)
    Ind0 = torch.zeros(2, 3, 0, dtype=torch.int64, device=DEV)
    assert hk.expert_gather_forward_call(X, Wg, Ind0, torch.float32).shape == (2, 3, 0, 4)
    out = hk.expert_scatter_forward_call(torch.zeros(2, 3, 0, 4, device=DEV), Ws, Ind0, 5, torch.float32)
    assert out.shape == (2, 5, 8) and (out == 0).all()
    dX, dW = hk.expert_gather_backward_call(X, Wg, Ind0, torch.zeros(2, 3, 0, 4, device=DEV), torch.float32)
    assert (dX == 0).all() and (dW == 0).all()


def test_errors_are_python_exceptions():
    X = torch.zeros(2, 5, 8, device=DEV); W = torch.zeros(3, 8, 4, device=DEV)
    Ind = torch.zeros(2, 3, 2, dtype=torch.int64, device=DEV)
    with pytest.raises(ValueError, match="Unknown dtype"):
        hk.expert_gather_forward_call(X.double(), W.double(), Ind, torch.float32)
    with pytest.raises(ValueError, match="Unknown dtype"):
        hk.expert_gather_forward_call(X, W, Ind, torch.int32)
    # mixed activation / weight dtypes are not an error (the reference casts inside its kernels): they meet in float32
    assert hk.expert_gather_forward_call(X, W.half(), Ind, torch.float32).dtype == torch.float32
    with pytest.raises(ValueError):
        hk.expert_gather_forward_call(X, W, Ind.float(), torch.float32)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        hk.expert_gather_forward_call(X.cpu(), W.cpu(), Ind.cpu(), torch.float32)


# ------------------------------------------------------------------ module / autograd surface
@pytest.mark.parametrize("seed", range(5))
def test_modules_like_the_reference_tests(seed):
    """Counterpart of the reference's test_all.py: random dims in [1,128), fp32, int16 Ind with
    replacement, loss = sum, compare forward and both gradients with the torch baseline at
    atol=1e-3 (test_all.py:9-11)."""
    g = torch.Generator().manual_seed(seed)
    B, T, K, E, I, J = torch.randint(1, 128, (6,), generator=g).tolist()
    torch.manual_seed(seed)
    X = torch.randn(B, T, I, device=DEV, requires_grad=True)
    Yin = torch.randn(B, E, K, J, device=DEV, requires_grad=True)
    Ind = torch.randint(0, T, (B, E, K), generator=g).to(torch.int16).to(DEV)
    gather = egs.ExpertGather(E, I, J).to(DEV)
    scatter = egs.ExpertScatter(E, J, I).to(DEV)

    def compare(mine, theirs, name):
        # the reference's check (test_all.py:9-11): isclose(atol=1e-3), default rtol=1e-5;
        # the baseline runs in float64 so that only this library's rounding is measured.
        # W_grad of a sum-loss is a length B*K sum with values in the hundreds, where fp32
        # accumulation alone costs ~sqrt(B*K)*2^-24 relative: it is held to the fp32 bound
        # 1e-4 * max|ref| instead of the absolute 1e-3.
        diff = (mine.detach().cpu().double() - theirs).abs()
        if name == "W_grad":
            ok = diff.max().item() <= 1e-4 * theirs.abs().max().item()
        else:
            ok = bool((diff <= 1e-3 + 1e-5 * theirs.abs()).all())
        if not ok:
            raise AssertionError(f"{name}: max diff {diff.max().item():.3e} dims {(B, T, K, E, I, J)}")

    Y = gather(X, Ind); Y.sum().backward()
    Xc = X.detach().cpu().double().requires_grad_(True); Wc = gather.W.detach().cpu().double().requires_grad_(True)
    Yr = P.gather(Xc, Wc, Ind.cpu()); Yr.sum().backward()
    compare(Y, Yr.detach(), "Y"); compare(X.grad, Xc.grad, "X_grad"); compare(gather.W.grad, Wc.grad, "W_grad")

    out = scatter(Yin, Ind, T); out.sum().backward()
    Yc = Yin.detach().cpu().double().requires_grad_(True); Wsc = scatter.W.detach().cpu().double().requires_grad_(True)
    outr = P.scatter(Yc, Wsc, Ind.cpu(), T); outr.sum().backward()
    compare(out, outr.detach(), "X"); compare(Yin.grad, Yc.grad, "Y_grad"); compare(scatter.W.grad, Wsc.grad, "W_grad")


def test_chain_bf16_fwd_bwd_scaled_default_shape():
    """gather -> scatter -> backward in bf16 through the modules (benchmark step, reduced B)."""
    from expertscattergather_amd import workloads as wl
    cfg = wl.CONFIGS["C2"]
    dims = (8, cfg.T, cfg.E, cfg.K, cfg.I, cfg.J)
    inp = wl.make_inputs(cfg, dims=dims)
    B, T, E, K, I, J = dims
    gather = egs.ExpertGather(E, I, J).to(DEV, torch.bfloat16); scatter = egs.ExpertScatter(E, J, I).to(DEV, torch.bfloat16)
    with torch.no_grad():
        gather.W.copy_(inp["Wg"]); scatter.W.copy_(inp["Ws"])
    X = dev(inp["X"]).requires_grad_(True); Ind = dev(inp["Ind"])
    Y = gather(X, Ind); out = scatter(Y, Ind, T); out.backward(dev(inp["dOut"]))
    Xn, Wgn, Wsn, dOn = (np64(inp[k]) for k in ("X", "Wg", "Ws", "dOut")); Indn = inp["Ind"].numpy()
    Yo = O.gather_forward(Xn, Wgn, Indn)
    assert_close(Y, Yo, torch.bfloat16, "Y")
    Yb = np64(Y)                                       # downstream oracles start from the rounded Y
    assert_close(out, O.scatter_forward(Yb, Wsn, Indn, T), torch.bfloat16, "out")
    dYo, dWso = O.scatter_backward(Yb, Wsn, Indn, dOn)
    assert_close(scatter.W.grad, dWso, torch.bfloat16, "dWs")
    dYb = np64(torch.from_numpy(dYo).to(torch.bfloat16))
    dXo, dWgo = O.gather_backward(Xn, Wgn, Indn, dYb)
    assert_close(X.grad, dXo, torch.bfloat16, "dX")
    assert_close(gather.W.grad, dWgo, torch.bfloat16, "dWg")


def test_gather_bias_and_scatter_bias():
    B, T, E, K, I, J = 2, 12, 3, 5, 16, 8
    case = make_case(23, B, T, E, K, I, J, torch.float32)
    gather = egs.ExpertGather(E, I, J, bias=True).to(DEV); scatter = egs.ExpertScatter(E, J, I, bias=True).to(DEV)
    Ind = dev(case["Ind"])
    Y = gather(dev(case["X"]), Ind)
    ref = O.gather_forward(np64(case["X"]), np64(gather.W), case["Ind"].numpy()) + np64(gather.bias)[None]
    assert_close(Y, ref, torch.float32, "gather bias")
    out = scatter(dev(case["Y"]), Ind, T)
    ref = O.scatter_forward(np64(case["Y"]), np64(scatter.W), case["Ind"].numpy(), T)
    bias = np64(scatter.bias)
    for b in range(B):
        for e in range(E):
            for k in range(K):
                ref[b, int(case["Ind"][b, e, k])] += bias[e, 0]
    assert_close(out, ref, torch.float32, "scatter bias")
    # a pick outside [0,T) adds neither its product row nor its expert's bias (and does not trip an index assert)
    bad = case["Ind"].clone(); bad[0, 1, 2] = T + 5; bad[1, 0, 0] = -3
    out2 = scatter(dev(case["Y"]), dev(bad), T)
    live = ((bad >= 0) & (bad < T)).numpy()
    safe = torch.where(torch.from_numpy(live), bad, torch.zeros_like(bad)).numpy()
    ref2 = O.scatter_forward(np64(case["Y"]) * live[..., None], np64(scatter.W), safe, T)
    for b in range(B):
        for e in range(E):
            for k in range(K):
                if live[b, e, k]:
                    ref2[b, int(bad[b, e, k])] += bias[e, 0]
    assert_close(out2, ref2, torch.float32, "scatter bias with rejected picks")


def test_fp8_weight_gather_matches_dequantised_oracle():
    from expertscattergather_amd import workloads as wl
    B, T, E, K, I, J = 3, 64, 5, 16, 128, 96
    case = make_case(29, B, T, E, K, I, J, torch.bfloat16, replace=False)
    Wq, scale = wl.quantize_fp8_weights(case["Wg"].float())
    Y = hk.expert_gather_fp8w_forward(dev(case["X"]), dev(Wq), dev(scale), dev(case["Ind"]))
    bits = Wq.view(torch.uint8).numpy()
    ref = O.gather_forward_fp8w(np64(case["X"]), bits, scale.numpy(), case["Ind"].numpy())
    assert_close(Y, ref, torch.bfloat16, "fp8 weights")
    # odd sizes take the unaligned byte path
    B, T, E, K, I, J = 2, 9, 3, 4, 19, 11
    case = make_case(31, B, T, E, K, I, J, torch.bfloat16)
    Wq, scale = wl.quantize_fp8_weights(case["Wg"].float())
    Y = hk.expert_gather_fp8w_forward(dev(case["X"]), dev(Wq), dev(scale), dev(case["Ind"]))
    ref = O.gather_forward_fp8w(np64(case["X"]), Wq.view(torch.uint8).numpy(), scale.numpy(), case["Ind"].numpy())
    assert_close(Y, ref, torch.bfloat16, "fp8 weights odd")
    # large product: 256 x 256 tiles, weight bytes staged in LDS as they are and widened after the transpose read
    B, T, E, K, I, J = 3, 300, 5, 200, 192, 208
    case = make_case(33, B, T, E, K, I, J, torch.bfloat16, replace=False)
    Wq, scale = wl.quantize_fp8_weights(case["Wg"].float())
    Y = hk.expert_gather_fp8w_forward(dev(case["X"]), dev(Wq), dev(scale), dev(case["Ind"]))
    ref = O.gather_forward_fp8w(np64(case["X"]), Wq.view(torch.uint8).numpy(), scale.numpy(), case["Ind"].numpy())
    assert_close(Y, ref, torch.bfloat16, "fp8 weights large")


@pytest.mark.parametrize("shape,ind_dtype,oob", [((2, 40, 3, 50, 128, 64), torch.int64, False),
                                                  ((3, 300, 9, 100, 256, 272), torch.int32, True),
                                                  ((2, 64, 8, 256, 384, 512), torch.int16, False)],
                         ids=["one-slab", "ragged-tiles", "full-tiles"])
def test_fp8_activation_gather_matches_quantised_oracle(shape, ind_dtype, oob):
    """fp8 x fp8 gather: the row quantiser is bit-exact against the oracle's, the product matches the oracle
    on the quantised operands to bf16 output accuracy, and stays within 5e-2 relative RMS (the stated bound of
    per-row e4m3 activations) of the fp8-weight gather that keeps bf16 activations."""
    from expertscattergather_amd import workloads as wl
    B, T, E, K, I, J = shape
    case = make_case(41, B, T, E, K, I, J, torch.bfloat16, ind_dtype=ind_dtype)
    case["X"][0, 0] = 0                                      # an all-zero row: scale 1
    if oob:
        case["Ind"][0, 0, 0] = T + 3                         # contributes a zero row
        case["Ind"][1, 2, 5] = -1
    Wq, scale = wl.quantize_fp8_weights(case["Wg"].float())
    Y, Xq, xs = hk.expert_gather_fp8_forward(dev(case["X"]), dev(Wq), dev(scale), dev(case["Ind"]), return_quantised=True)
    q_o, xs_o = O.quantize_rows_e4m3(case["X"].float().numpy())
    assert np.array_equal(xs.cpu().numpy(), xs_o)
    assert np.array_equal(Xq.cpu().view(torch.uint8).numpy(), q_o)
    bits = Wq.view(torch.uint8).numpy()
    ind = case["Ind"].numpy().astype(np.int64)
    live = (ind >= 0) & (ind < T)
    safe = np.where(live, ind, 0)
    ref = O.gather_forward_fp8(case["X"].float().numpy(), bits, scale.numpy(), safe) * live[..., None]
    assert_close(Y, ref, torch.bfloat16, "fp8 activations")
    assert torch.equal(Y, hk.expert_gather_fp8_forward(dev(case["X"]), dev(Wq), dev(scale), dev(case["Ind"])))
    ref_bf16_act = O.gather_forward_fp8w(np64(case["X"]), bits, scale.numpy(), safe) * live[..., None]
    rel_rms = np.sqrt(((np64(Y) - ref_bf16_act) ** 2).mean() / (ref_bf16_act ** 2).mean())
    assert rel_rms <= 5e-2, rel_rms


def test_fp8_activation_gather_rejects_shapes_outside_its_tile_layout():
    from expertscattergather_amd import workloads as wl
    case = make_case(43, 2, 16, 2, 4, 96, 32, torch.bfloat16)   # I not a multiple of 128
    Wq, scale = wl.quantize_fp8_weights(case["Wg"].float())
    with pytest.raises(RuntimeError, match="unsupported"):
        hk.expert_gather_fp8_forward(dev(case["X"]), dev(Wq), dev(scale), dev(case["Ind"]))


def test_ops_pass_opcheck_and_router_output_feeds_the_kernels():
    # registration of the four ops (schema, fake implementations, no hidden mutation), the counterpart of the
    # reference's ~220 lines of torch.library glue (egs/triton_kernels.py:361-578)
    from expertscattergather_amd.router import expert_choice_router
    hk.create_kernels()
    B, T, E, K, I, J = 2, 24, 3, 5, 32, 16
    case = make_case(41, B, T, E, K, I, J, torch.float32)
    logits = torch.randn(B, T, E, generator=torch.Generator().manual_seed(1))
    Ind, _ = expert_choice_router(dev(logits), K, torch.int32)
    X, Wg, Ws, Y, dOut = (dev(case[k]) for k in ("X", "Wg", "Ws", "Y", "dOut"))
    ops = torch.ops.egs_amd
    tests = ("test_schema", "test_faketensor", "test_autograd_registration", "test_aot_dispatch_dynamic")
    torch.library.opcheck(ops.expert_gather_forward_call_fn.default, (X, Wg, Ind, torch.float32), test_utils=tests)
    torch.library.opcheck(ops.expert_scatter_forward_call_fn.default, (Y, Ws, Ind, T, torch.float32), test_utils=tests)
    torch.library.opcheck(ops.expert_gather_backward_call_fn.default, (X, Wg, Ind, Y, torch.float32), test_utils=tests)
    torch.library.opcheck(ops.expert_scatter_backward_call_fn.default, (Y, Ws, Ind, dOut, torch.float32), test_utils=tests)
    got = hk.expert_gather_forward_call(X, Wg, Ind, torch.float32)
    assert_close(got, O.gather_forward(np64(case["X"]), np64(case["Wg"]), Ind.cpu().numpy().astype("int64")), torch.float32, "router picks")


@pytest.mark.parametrize("shape", [(8, 64, 8, 16, 128, 64), (2, 300, 4, 200, 256, 192)], ids=["small-experts", "large-tiles"])
def test_graph_replays_match_eager_results(shape):
    # the whole forward+backward sequence captured once and replayed with other work in between: every replay
    # must reproduce the eager results bit for bit (scratch is cleared by kernels, nothing depends on capture-time state)
    B, T, E, K, I, J = shape
    case = make_case(51, B, T, E, K, I, J, torch.bfloat16)
    X, Wg, Ws, dOut, Ind = (dev(case[k]) for k in ("X", "Wg", "Ws", "dOut", "Ind"))
    hk.set_scatter_mode("deterministic")

    def step():
        Y = hk.expert_gather_forward_call(X, Wg, Ind, torch.float32)
        out = hk.expert_scatter_forward_call(Y, Ws, Ind, T, torch.float32)
        dY, dWs = hk.expert_scatter_backward_call(Y, Ws, Ind, dOut, torch.float32)
        dX, dWg = hk.expert_gather_backward_call(X, Wg, Ind, dY, torch.float32)
        return Y, out, dX, dWg, dWs

    eager = [t.clone() for t in step()]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        outs = step()
    for rep in range(4):
        for t in outs:
            t.fill_(float("nan"))                   # stale results must not survive a replay
        junk = torch.randn(1 << 18, device=DEV).sum()      # unrelated eager work between replays
        graph.replay()
        torch.cuda.synchronize()
        for name, got, ref in zip(("Y", "out", "dX", "dWg", "dWs"), outs, eager):
            assert torch.equal(got, ref), f"replay {rep}: {name} differs from the eager result"
        del junk


@pytest.mark.parametrize("out_type", [torch.bfloat16, torch.float32], ids=["out-bf16", "out-f32"])
def test_mixed_precision_follows_the_reference_kernels(out_type):
    """bf16 activations with fp32 parameters.  out_type bfloat16: the weights are rounded to bf16 and the products run in
    bf16 (reference egs/triton_kernels.py:122-127); out_type float32: the operands meet in fp32.  Results come back in the
    activation's dtype, weight gradients in the parameter's (:375, :408-409, :457, :491-492)."""
    B, T, E, K, I, J = 3, 40, 6, 9, 64, 32
    case = make_case(61, B, T, E, K, I, J, torch.bfloat16)
    g = torch.Generator().manual_seed(3)
    Wg32 = torch.randn(E, I, J, generator=g) / I ** 0.5
    Ws32 = torch.randn(E, J, I, generator=g) / J ** 0.5
    X = dev(case["X"]).requires_grad_(True); Wg = dev(Wg32).requires_grad_(True); Ws = dev(Ws32).requires_grad_(True)
    Ind = dev(case["Ind"])
    Y = hk.ExpertGatherFunction.apply(X, Wg, Ind, out_type)
    out = hk.ExpertScatterFunction.apply(Y, Ws, Ind, T, out_type)
    assert Y.dtype == torch.bfloat16 and out.dtype == torch.bfloat16
    out.backward(dev(case["dOut"]))
    assert X.grad.dtype == torch.bfloat16 and Wg.grad.dtype == torch.float32 and Ws.grad.dtype == torch.float32
    rnd = (lambda w: w.to(torch.bfloat16)) if out_type == torch.bfloat16 else (lambda w: w)
    Wgn, Wsn = np64(rnd(Wg32)), np64(rnd(Ws32))
    Indn = case["Ind"].numpy()
    assert_close(Y, O.gather_forward(np64(case["X"]), Wgn, Indn), torch.bfloat16, "Y mixed")
    assert_close(out, O.scatter_forward(np64(Y), Wsn, Indn, T), torch.bfloat16, "out mixed")
    dYo, dWso = O.scatter_backward(np64(Y), Wsn, Indn, np64(case["dOut"]))
    wtol = torch.bfloat16 if out_type == torch.bfloat16 else torch.float32
    assert_close(Ws.grad, dWso, wtol, "dWs mixed")
    dY = torch.from_numpy(dYo).to(torch.bfloat16)
    dXo, dWgo = O.gather_backward(np64(case["X"]), Wgn, Indn, np64(dY))
    assert_close(X.grad, dXo, torch.bfloat16, "dX mixed")
    # dW_gather sees dY rounded to the compute type before it is used; the fp32 path keeps dY in fp32
    if out_type == torch.bfloat16:
        assert_close(Wg.grad, dWgo, torch.bfloat16, "dWg mixed")


def test_modules_trace_through_torch_compile():
    """gather -> scatter forward and backward through the modules under torch.compile (aot_eager, one graph): the custom ops
    carry fake implementations and autograd formulas, so nothing falls back to eager or breaks the graph; results equal the
    eager ones bit for bit.  Counterpart of the reference's registration glue (egs/triton_kernels.py:527-567)."""
    B, T, E, K, I, J = 4, 64, 8, 16, 128, 64
    case = make_case(71, B, T, E, K, I, J, torch.bfloat16)
    gather = egs.ExpertGather(E, I, J).to(DEV, torch.bfloat16); scatter = egs.ExpertScatter(E, J, I).to(DEV, torch.bfloat16)
    with torch.no_grad():
        gather.W.copy_(case["Wg"]); scatter.W.copy_(case["Ws"])
    Ind = dev(case["Ind"]); dOut = dev(case["dOut"])

    def block(x):
        return scatter(gather(x, Ind), Ind, T)

    def run(fn):
        for m in (gather, scatter):
            m.W.grad = None
        x = dev(case["X"]).requires_grad_(True)
        out = fn(x)
        out.backward(dOut)
        return out.detach(), x.grad, gather.W.grad.clone(), scatter.W.grad.clone()

    eager = run(block)
    torch._dynamo.reset()
    compiled = run(torch.compile(block, backend="aot_eager", fullgraph=True))
    for name, a, b in zip(("out", "dX", "dWg", "dWs"), eager, compiled):
        assert torch.equal(a, b), f"{name}: compiled differs from eager"
    assert_close(eager[0], O.scatter_forward(np64(gather(dev(case["X"]), Ind)), np64(case["Ws"]), case["Ind"].numpy(), T),
                 torch.bfloat16, "compiled block")


# ---------------------------------------------------------------------------------------------------------
# inference block: scatter(act(gather(x, Ind)), Ind, T) in one kernel (reference call pattern test_speed.ipynb:73-75)
def _mlp_oracle(case, T, act, dtype, stored_y=False):
    """oracle/egs_oracle.py mlp_forward with the rows rounded to the element type where a stored Y would be rounded
    (`stored_y`: also before the activation, as the separate launches do)."""
    rnd = lambda v: torch.from_numpy(v).to(dtype).to(torch.float32).numpy()
    X, Wg, Ws = (np64(case[k]) for k in ("X", "Wg", "Ws"))
    return O.mlp_forward(X, Wg, Ws, case["Ind"].numpy(), T, act, round_y=rnd, round_before_act=stored_y)


MLP_SHAPES = [
    (4, 64, 8, 16, 128, 64),      # default-like, scaled down
    (2, 256, 32, 32, 128, 64),    # two batch elements of the default shape
    (4, 50, 9, 11, 64, 32),       # J = 32: half of the lanes of the second product carry nothing; ragged K, E
    (5, 40, 12, 33, 128, 64),     # K = 33: a second, nearly empty unit per expert
    (8, 33, 5, 64, 32, 64),       # I = 32: one output slice, one step of the first product
    (4, 700, 8, 20, 64, 32),      # long T
]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bfloat16", "float16"])
@pytest.mark.parametrize("shape", MLP_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_inference_block_matches_oracle(shape, dtype):
    from expertscattergather_amd import _abi
    B, T, E, K, I, J = shape
    assert _abi.lib().egs_expert_mlp_supported(_abi.Dims(*shape), hk.dtype_to_type_id(dtype)) == 1
    case = make_case(31, B, T, E, K, I, J, dtype)
    X, Wg, Ws, Ind = (dev(case[k]) for k in ("X", "Wg", "Ws", "Ind"))
    got = hk.expert_mlp_forward(X, Wg, Ws, Ind, "relu", force_block=True)
    assert got.dtype == dtype and tuple(got.shape) == (B, T, I)
    assert_close(got, _mlp_oracle(case, T, "relu", dtype), dtype, "inference block")
    assert torch.equal(got, hk.expert_mlp_forward(X, Wg, Ws, Ind, "relu", force_block=True))     # fixed order of additions


@pytest.mark.gpu
@pytest.mark.parametrize("act", ["none", "relu", "gelu", "gelu_tanh", "silu"])
def test_inference_block_activations_and_rejected_picks(act):
    B, T, E, K, I, J = 8, 96, 16, 24, 128, 64
    dtype = torch.bfloat16
    case = make_case(37, B, T, E, K, I, J, dtype, ind_dtype=torch.int16)
    case["Ind"][0, 0, 0] = T; case["Ind"][1, 2, 3] = -1; case["Ind"][7, 15, 23] = 30000
    X, Wg, Ws, Ind = (dev(case[k]) for k in ("X", "Wg", "Ws", "Ind"))
    got = hk.expert_mlp_forward(X, Wg, Ws, Ind, act, force_block=True)
    assert_close(got, _mlp_oracle(case, T, act, dtype), dtype, f"inference block, {act}")
    # the same through the two forward launchers with torch's activation in between
    y = hk.expert_gather_forward_call(X, Wg, Ind, torch.float32)
    y = {"none": lambda v: v, "relu": torch.relu, "gelu": torch.nn.functional.gelu, "silu": torch.nn.functional.silu,
         "gelu_tanh": lambda v: torch.nn.functional.gelu(v, approximate="tanh")}[act](y)
    two = np64(hk.expert_scatter_forward_call(y, Ws, Ind, T, torch.float32))
    # the separate launches round Y to bf16 before AND after the activation, the block once; and the block feeds the
    # reduction elements of the second product to the matrix instruction in another order (fp32 sums differ in the last bit)
    g64 = np64(got)
    if act in ("none", "relu"):
        assert_close(got, two, dtype, f"inference block vs separate launches, {act}")
    else:
        assert np.abs(g64 - two).max() <= 4 * 2.0 ** -8 * np.abs(two).max()
        assert np.sqrt(((g64 - two) ** 2).mean()) <= 8e-3 * np.sqrt((two ** 2).mean())


@pytest.mark.gpu
def test_inference_block_composes_what_the_kernel_does_not_take():
    # fp32, a 16-bit shape with 2048 picks per batch element, J = 128: same result through the separate launchers
    for shape, dtype in (((2, 40, 6, 9, 64, 32), torch.float32), ((2, 64, 32, 64, 128, 64), torch.bfloat16),
                         ((5, 40, 12, 33, 128, 128), torch.float16)):
        B, T, E, K, I, J = shape
        case = make_case(41, B, T, E, K, I, J, dtype)
        X, Wg, Ws, Ind = (dev(case[k]) for k in ("X", "Wg", "Ws", "Ind"))
        got = hk.expert_mlp_forward(X, Wg, Ws, Ind, "silu")
        assert_close(got, _mlp_oracle(case, T, "silu", dtype, stored_y=True), dtype, "composed inference block")
    with pytest.raises(ValueError):
        hk.expert_mlp_forward(X, Wg, Ws, Ind, "softmax")


@pytest.mark.gpu
@pytest.mark.parametrize("act", ["relu", "silu", "none"])
@pytest.mark.parametrize("shape,dtype", [((48, 96, 16, 24, 128, 64), torch.bfloat16),    # the one-kernel forward
                                         ((3, 40, 6, 9, 64, 96), torch.float16),          # J = 96: composed forward
                                         ((2, 33, 5, 7, 24, 40), torch.float32)],
                         ids=["block-bf16", "composed-f16", "composed-f32"])
def test_trainable_block_keeps_no_rows_and_matches_the_chain_rule(shape, dtype, act):
    """hip_kernels.expert_mlp: output and the three gradients against the oracle's chain with every stored stage
    rounded to the element type (the activation and its derivative from torch in float64 on the CPU), and nothing of
    size B*E*K*J saved for backward."""
    B, T, E, K, I, J = shape
    case = make_case(47, B, T, E, K, I, J, dtype)
    X, Wg, Ws = (dev(case[k]).requires_grad_(True) for k in ("X", "Wg", "Ws"))
    Ind = dev(case["Ind"])
    out = hk.expert_mlp(X, Wg, Ws, Ind, act)
    assert {t.data_ptr() for t in out.grad_fn.saved_tensors} <= {t.data_ptr() for t in (X, Wg, Ws, Ind)}
    out.backward(dev(case["dOut"]))

    rnd = lambda v: torch.from_numpy(np.asarray(v)).to(dtype).to(torch.float64).numpy()
    Xn, Wgn, Wsn, dOn = (np64(case[k]) for k in ("X", "Wg", "Ws", "dOut")); Indn = case["Ind"].numpy()
    fn = {"none": lambda v: v, "relu": torch.relu, "silu": torch.nn.functional.silu}[act]
    Yo = torch.from_numpy(rnd(O.gather_forward(Xn, Wgn, Indn))).requires_grad_(True)
    Ao = fn(Yo)
    An = rnd(Ao.detach().numpy())
    one_kernel = dtype is not torch.float32 and J in (32, 64) and hk._mlp_block_pays(B, E, K, I, J, hk._ACTIVATIONS[act])
    assert_close(out, _mlp_oracle(case, T, act, dtype, stored_y=not one_kernel), dtype, "trainable block, out")
    dAo, dWso = O.scatter_backward(An, Wsn, Indn, dOn)
    assert_close(Ws.grad, dWso, dtype, "trainable block, dWs")
    dYo = rnd(torch.autograd.grad(Ao, Yo, torch.from_numpy(rnd(dAo)))[0].numpy()) if act != "none" else rnd(dAo)
    dXo, dWgo = O.gather_backward(Xn, Wgn, Indn, dYo)
    assert_close(X.grad, dXo, dtype, "trainable block, dX")
    assert_close(Wg.grad, dWgo, dtype, "trainable block, dWg")


def test_inference_block_is_a_traceable_op():
    hk.create_kernels()
    B, T, E, K, I, J = 8, 48, 8, 16, 64, 32
    dtype = torch.bfloat16
    case = make_case(43, B, T, E, K, I, J, dtype)
    X, Wg, Ws, Ind = (dev(case[k]) for k in ("X", "Wg", "Ws", "Ind"))
    torch.library.opcheck(torch.ops.egs_amd.expert_mlp_forward_fn.default, (X, Wg, Ws, Ind, "relu"),
                          test_utils=("test_schema", "test_faketensor"))
    eager = hk.expert_mlp_forward(X, Wg, Ws, Ind, "relu")

    @torch.compile(backend="aot_eager", fullgraph=True)
    def f(x, wg, ws, ind):
        return hk.expert_mlp_forward(x, wg, ws, ind, "relu") * 2.0

    assert torch.equal(f(X, Wg, Ws, Ind), eager * 2.0)


def test_concurrent_callers_on_their_own_streams():
    # the library keeps no per-call state: two host threads, each on a stream of its own, run different shapes
    # (different kernels, different LDS grants) at the same time and both get the oracle's answer
    import threading
    jobs = [((4, 64, 8, 16, 128, 64), torch.bfloat16), ((2, 256, 48, 32, 128, 64), torch.float16)]
    cases = [make_case(51 + n, *shape, dtype) for n, (shape, dtype) in enumerate(jobs)]
    results, errors = [None, None], []

    def worker(n):
        try:
            shape, dtype = jobs[n]
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for _ in range(5):
                    results[n] = run_all(cases[n], shape[1])
            stream.synchronize()
        except Exception as exc:            # surfaced in the main thread below
            errors.append(exc)

    threads = [threading.Thread(target=worker, args=(n,)) for n in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for n, (shape, dtype) in enumerate(jobs):
        ref = oracle_all(cases[n], shape[1])
        for name in ("Y", "out", "dX", "dWg", "dY", "dWs"):
            assert_close(results[n][name], ref[name], dtype, f"thread {n} {name}")


@pytest.mark.parametrize("shape,dtype", [((4, 64, 8, 16, 128, 64), torch.bfloat16), ((2, 300, 4, 200, 256, 192), torch.bfloat16),
                                         ((3, 40, 6, 100, 24, 16), torch.float32)], ids=["small-bf16", "large-bf16", "general-f32"])
def test_ctypes_and_integer_call_routes_agree(shape, dtype, monkeypatch):
    """The launchers reach the library through the integer-call module when it is built and through ctypes otherwise."""
    from expertscattergather_amd import _abi
    assert _abi.pycall() is not None
    case = make_case(77, *shape, dtype)
    fast = run_all(case, shape[1])
    monkeypatch.setattr(_abi, "_pycall", None)
    assert _abi.pycall() is None
    slow = run_all(case, shape[1])
    for name in fast:
        assert torch.equal(fast[name], slow[name]), name



@pytest.mark.parametrize("shape", [(3, 300, 5, 200, 192, 256),    # 128 x 128 tiles, rows of several batch elements in one tile
                                   (2, 90, 4, 128, 48, 24),       # 128 x 64 tiles, a tile is exactly the picks of one (b, e)
                                   (2, 64, 3, 300, 520, 72)],     # more distinct repeated tokens per tile than partial-sum slots
                         ids=lambda s: "x".join(map(str, s)))
def test_fp32_atomic_mode_adds_up_repeated_tokens_inside_a_tile(shape):
    """Skewed routing in the fp32 atomic mode: most picks of an expert land on a handful of tokens, some are rejected."""
    B, T, E, K, I, J = shape
    case = make_case(91 + sum(shape), *shape, torch.float32)
    g = torch.Generator().manual_seed(5)
    hot = torch.randint(0, T, (B, E, K), generator=g)
    Ind = case["Ind"].clone()
    pick_hot = torch.rand(B, E, K, generator=g) < 0.7
    Ind[pick_hot] = (hot[pick_hot] % 3) * 7 % T             # three hot tokens take 70 % of the picks
    pairs = torch.rand(B, E, K, generator=g) < 0.5
    Ind[~pick_hot & pairs] = Ind[~pick_hot & pairs] // 2 * 2 % T   # and many tokens are picked twice or more
    Ind[0, 0, 0] = -1; Ind[B - 1, E - 1, K - 1] = T
    bad = (Ind < 0) | (Ind >= T)
    safe = Ind.clone(); safe[bad] = 0
    mask = (~bad).numpy()[..., None]
    got = run_all(dict(case, Ind=Ind), T, mode="atomic")
    X, Wg, Ws, Y = (np64(case[k]) for k in ("X", "Wg", "Ws", "Y"))
    assert_close(got["out"], O.scatter_forward(Y * mask, Ws, safe.numpy(), T), torch.float32, "out, skewed atomic")
    dX, _ = O.gather_backward(X, Wg, safe.numpy(), Y * mask)
    assert_close(got["dX"], dX, torch.float32, "dX, skewed atomic")


def test_tensors_made_under_inference_mode():
    """Tensors created under torch.inference_mode() carry no version counter: the forward launchers and the inference
    block must neither read one nor keep a routing table with such an Ind."""
    B, T, E, K, I, J = 8, 256, 32, 32, 128, 64          # the default shape's kernels (its routing table applies)
    dtype = torch.bfloat16
    case = make_case(53, B, T, E, K, I, J, dtype)
    with torch.inference_mode():
        X, Wg, Ws, Ind = (dev(case[k]) for k in ("X", "Wg", "Ws", "Ind"))
        assert Ind.is_inference()
        Y = hk.expert_gather_forward_call(X, Wg, Ind, torch.float32)
        out = hk.expert_scatter_forward_call(Y, Ws, Ind, T, torch.float32)
        blk = hk.expert_mlp_forward(X, Wg, Ws, Ind, "relu")
        composed = hk.expert_mlp_forward(X, Wg, Ws, Ind, "gelu")        # E * K / 32 > 16: the two launchers with torch's gelu
        mods = egs.ExpertScatter(E, J, I).to(DEV, dtype)(egs.ExpertGather(E, I, J).to(DEV, dtype)(X, Ind), Ind, T)
        torch.cuda.synchronize()
    assert hk._TABLE_ATTR not in Ind.__dict__
    assert mods.shape == (B, T, I)
    Xn, Wgn, Wsn, Indn = np64(case["X"]), np64(case["Wg"]), np64(case["Ws"]), case["Ind"].numpy()
    assert_close(Y, O.gather_forward(Xn, Wgn, Indn), dtype, "Y under inference_mode")
    assert_close(out, O.scatter_forward(np64(Y), Wsn, Indn, T), dtype, "out under inference_mode")
    assert_close(blk, _mlp_oracle(case, T, "relu", dtype), dtype, "inference block under inference_mode")
    assert_close(composed, _mlp_oracle(case, T, "gelu", dtype, stored_y=True), dtype, "composed block under inference_mode")


def test_inference_block_takes_the_views_the_gather_takes():
    """A batch/token-transposed X and a batch-expanded X (batch stride 0) go through the block like through the gather."""
    B, T, E, K, I, J = 8, 64, 8, 16, 128, 64
    dtype = torch.bfloat16
    case = make_case(59, B, T, E, K, I, J, dtype)
    Wg, Ws, Ind = (dev(case[k]) for k in ("Wg", "Ws", "Ind"))
    Xt = dev(case["X"]).transpose(0, 1).contiguous().transpose(0, 1)      # [B,T,I] view with strides (I, B*I, 1)
    assert not Xt.is_contiguous() and Xt.stride(0) < Xt.stride(1)
    ref = _mlp_oracle(case, T, "relu", dtype)
    assert_close(hk.expert_mlp_forward(Xt, Wg, Ws, Ind, "relu", force_block=True), ref, dtype, "block, transposed X")
    x0 = dev(case["X"][:1])
    Xe = x0.expand(B, T, I)                                               # batch stride 0
    assert Xe.stride(0) == 0
    case_e = dict(case, X=case["X"][:1].expand(B, T, I).contiguous())
    assert_close(hk.expert_mlp_forward(Xe, Wg, Ws, Ind, "relu", force_block=True), _mlp_oracle(case_e, T, "relu", dtype), dtype,
                 "block, expanded X")
    assert_close(hk.expert_gather_forward_call(Xe, Wg, Ind, torch.float32),
                 O.gather_forward(np64(case_e["X"]), np64(case["Wg"]), case["Ind"].numpy()), dtype, "gather, expanded X")


def test_module_scatter_mode_overrides_the_global_and_is_bound_at_forward():
    """`module.scatter_mode` wins over the process-wide mode, and a backward issued after the process-wide mode has been
    switched still runs in the mode its forward was called in (16-bit types beyond the one-kernel scatter: the two modes
    differ in the precision of the product rows, so their results differ in a few last bits)."""
    B, T, E, K, I, J = 2, 300, 4, 200, 256, 192
    dtype = torch.bfloat16
    case = make_case(61, B, T, E, K, I, J, dtype)
    Y, Ws, Ind, dOut, X, Wg = (dev(case[k]) for k in ("Y", "Ws", "Ind", "dOut", "X", "Wg"))
    ref = {}
    for mode in ("deterministic", "atomic"):
        hk.set_scatter_mode(mode)
        try:
            ref[mode] = (hk.expert_scatter_forward_call(Y, Ws, Ind, T, torch.float32),
                         hk.expert_gather_backward_call(X, Wg, Ind, Y, torch.float32)[0])
        finally:
            hk.set_scatter_mode("deterministic")
    assert not torch.equal(ref["deterministic"][0], ref["atomic"][0])   # otherwise the test below proves nothing
    smod = egs.ExpertScatter(E, J, I).to(DEV, dtype)
    gmod = egs.ExpertGather(E, I, J).to(DEV, dtype)
    with torch.no_grad():
        smod.W.copy_(Ws); gmod.W.copy_(Wg)
    smod.scatter_mode = "atomic"
    assert torch.equal(smod(Y, Ind, T), ref["atomic"][0])
    smod.scatter_mode = None
    assert torch.equal(smod(Y, Ind, T), ref["deterministic"][0])
    # the gather's backward scatters: mode bound when the forward ran
    gmod.scatter_mode = "atomic"
    x = X.clone().requires_grad_(True)
    y = gmod(x, Ind)
    gmod.scatter_mode = None
    y.backward(Y)
    assert torch.equal(x.grad, ref["atomic"][1])
    x = X.clone().requires_grad_(True)
    y = gmod(x, Ind)                       # deterministic now
    hk.set_scatter_mode("atomic")
    try:
        y.backward(Y)
    finally:
        hk.set_scatter_mode("deterministic")
    assert torch.equal(x.grad, ref["deterministic"][1])


def test_fp32_atomic_mode_at_zipf_sizes():
    """fp32 atomic mode at the sizes of the Zipf-routed configuration (two batch elements): a quarter of the picks on one
    token, far more distinct repeated tokens per 128-row tile than the in-tile pre-reduction has slots for."""
    from expertscattergather_amd import workloads as wl
    cfg = wl.CONFIGS["C4"]
    B, T, E, K, I, J = 2, cfg.T, cfg.E, cfg.K, cfg.I, cfg.J
    inp = wl.make_inputs(cfg, dims=(B, T, E, K, I, J))
    Y = torch.randn(B, E, K, J, generator=torch.Generator().manual_seed(7))
    Ws = inp["Ws"].float()
    Ind = inp["Ind"]
    counts = torch.bincount(Ind[0].reshape(-1), minlength=T)
    assert counts.max() > 0.15 * E * K
    hk.set_scatter_mode("atomic")
    try:
        out = hk.expert_scatter_forward_call(dev(Y), dev(Ws), dev(Ind), T, torch.float32)
        torch.cuda.synchronize()
    finally:
        hk.set_scatter_mode("deterministic")
    assert_close(out, O.scatter_forward(np64(Y), np64(Ws), Ind.numpy(), T), torch.float32, "fp32 atomic, Zipf sizes")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bfloat16", "float16"])
@pytest.mark.parametrize("shape", [(3, 450, 256, 400, 136, 72),      # one split of 1200 rows per expert: a chunk of 1024 and a ragged one
                                   (5, 500, 128, 450, 264, 128),     # two splits of 1152 rows, two 256-row tiles of I, the second nearly empty
                                   (5, 600, 40, 420, 264, 200)],     # 256-column tiles in four stages of 32 rows: 2100 rows, one split
                         ids=lambda s: "x".join(map(str, s)))
def test_large_weight_gradient_over_several_row_chunks(shape, dtype):
    """The weight gradient of large shapes stages the row offsets of 1024 reduction rows at a time and keeps two or
    three slabs in flight (reference kernel: egs/triton_kernels.py:261-356); more rows than one chunk,
    a ragged last chunk and both layouts, against the oracle."""
    B, T, E, K, I, J = shape
    case = make_case(4242 + sum(shape), *shape, dtype)
    X, Wg, Ws, Y, dOut, Ind = (dev(case[k]) for k in ("X", "Wg", "Ws", "Y", "dOut", "Ind"))
    _, dWg = hk.expert_gather_backward_call(X, Wg, Ind, Y, torch.float32)
    _, dWs = hk.expert_scatter_backward_call(Y, Ws, Ind, dOut, torch.float32)
    torch.cuda.synchronize()
    Indn = case["Ind"].to(torch.int64).numpy()
    ref_g = O.gather_backward(np64(case["X"]), np64(case["Wg"]), Indn, np64(case["Y"]))[1]
    ref_s = O.scatter_backward(np64(case["Y"]), np64(case["Ws"]), Indn, np64(case["dOut"]))[1]
    assert_close(dWg, ref_g, dtype, f"dWg {shape} {dtype}")
    assert_close(dWs, ref_s, dtype, f"dWs {shape} {dtype}")


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["deterministic", "atomic"])
@pytest.mark.parametrize("shape", [(2, 777, 37, 130, 256, 128),      # 4810 picks per batch element: two table workgroups, ragged shares
                                   (3, 1500, 70, 129, 192, 128),     # 9030 picks: three
                                   (2, 3000, 140, 150, 192, 128)],   # 21000 picks and 3000 tokens: six, and wavefront slices of 512
                         ids=lambda s: "x".join(map(str, s)))
def test_routing_table_built_by_several_workgroups(shape, mode):
    """Batch elements with more than 4096 picks have their routing table built by several workgroups, each ranking a share
    of the picks and counting the rest (the reference's scatter, egs/triton_kernels.py:156-247, has no table: it adds with
    atomics).  Hot tokens, rejected picks and odd sizes, against the oracle, and the same bits on a second call."""
    B, T, E, K, I, J = shape
    dtype = torch.bfloat16
    case = make_case(977 + sum(shape), *shape, dtype)
    Ind = case["Ind"].clone()
    g = torch.Generator().manual_seed(5)
    hot = torch.rand(B, E, K, generator=g) < 0.2
    Ind[hot] = 7                                           # a fifth of all picks on one token: segments cut into chunks
    Ind[0, 0, 0] = T; Ind[-1, E // 2, 3] = -1; Ind[-1, E - 1, K - 1] = 10 ** 9
    bad = (Ind < 0) | (Ind >= T)
    Y, Ws = dev(case["Y"]), dev(case["Ws"])
    from expertscattergather_amd import _abi
    hk.set_scatter_mode(mode)
    try:
        with _abi.launch_log() as log:
            out = hk.expert_scatter_forward_call(Y, Ws, dev(Ind), T, torch.float32)
        again = hk.expert_scatter_forward_call(Y, Ws, dev(Ind), T, torch.float32)
        torch.cuda.synchronize()
    finally:
        hk.set_scatter_mode("deterministic")
    # the table rides in the product launch (no table kernel of its own), which is where it is built in parts
    assert "rows_gemm_dl_kernel" in log.kernels and not any(k.startswith("csr_") for k in log.kernels), log.kernels
    safe = Ind.clone(); safe[bad] = 0
    mask = (~bad).numpy()[..., None]
    ref = O.scatter_forward(np64(case["Y"]) * mask, np64(case["Ws"]), safe.numpy(), T)
    # the hot token sums a few thousand products: its row sets the scale of the comparison
    assert_close(out, ref, dtype, f"out {shape} {mode}")
    if mode == "deterministic":
        assert torch.equal(out, again)
