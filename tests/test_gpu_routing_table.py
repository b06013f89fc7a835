"""The routing table that the gather forward leaves with an Ind tensor for the scatter forward and the gather's backward:
results are the same bit for bit with and without it, the table is the stable sort of the picks by token, and it is never
used for indices other than the ones it was built from."""
import numpy as np
import pytest
import torch

from oracle import egs_oracle as O
from tests._util import assert_close, make_case, np64

pytestmark = pytest.mark.gpu

from expertscattergather_amd import _abi
from expertscattergather_amd import hip_kernels as hk

hk.create_kernels()
DEV = "cuda"
ATTR = hk._TABLE_ATTR

# shapes the one-kernel scatter takes in a single pass (the only consumer of a table) in every element type, and whose
# gather forward runs on a small-expert kernel (the launch that builds it)
TABLE_SHAPES = [
    (2, 256, 32, 32, 128, 64),      # two batch elements of the default shape
    (5, 50, 9, 11, 64, 32),         # ragged K, T, E
    (2, 33, 5, 64, 128, 64),
    (4, 300, 40, 25, 64, 32),       # 1000 picks per batch element
    (8, 700, 8, 20, 32, 64),        # long T
    (9, 20, 3, 7, 32, 32),
    (2, 256, 48, 32, 128, 64),      # 1536 picks: the scatter runs in two passes over groups of experts
    (4, 100, 20, 100, 64, 32),      # 2000 picks, ragged 32-pick units
]


@pytest.fixture(autouse=True)
def cache_on():
    hk.set_routing_table_cache(True)
    yield
    hk.set_routing_table_cache(True)


def chain(case, T, ind=None):
    """gather forward -> scatter forward -> gather backward, the three calls that share a table."""
    X, Wg, Ws, Y = (case[k].to(DEV) for k in ("X", "Wg", "Ws", "Y"))
    Ind = case["Ind"].to(DEV) if ind is None else ind
    y = hk.expert_gather_forward_call(X, Wg, Ind, torch.float32)
    out = hk.expert_scatter_forward_call(Y, Ws, Ind, T, torch.float32)
    dX, dWg = hk.expert_gather_backward_call(X, Wg, Ind, Y, torch.float32)
    torch.cuda.synchronize()
    return Ind, (y, out, dX, dWg)


@pytest.mark.parametrize("ind_dtype", [torch.int64, torch.int16], ids=["i64", "i16"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=["bfloat16", "float16", "float32"])
@pytest.mark.parametrize("shape", TABLE_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_results_do_not_depend_on_the_table(shape, dtype, ind_dtype):
    B, T, E, K, I, J = shape
    case = make_case(31 + sum(shape), *shape, dtype, ind_dtype=ind_dtype)
    hk.set_routing_table_cache(False)
    ind0, plain = chain(case, T)
    assert ATTR not in ind0.__dict__
    hk.set_routing_table_cache(True)
    ind1, tabled = chain(case, T)
    if dtype is torch.float32 and E * K > 1024:
        assert ATTR not in ind1.__dict__        # fp32 scatter in passes sorts for itself (measured faster)
    else:
        assert ATTR in ind1.__dict__, "these sizes have a table: the gather forward must have left one"
    for a, b, name in zip(plain, tabled, ("Y", "out", "dX", "dWg")):
        assert torch.equal(a, b), f"{name} differs with the table {shape} {dtype}"
    assert_close(tabled[1], O.scatter_forward(np64(case["Y"]), np64(case["Ws"]), case["Ind"].to(torch.int64).numpy(), T), dtype, "out")


@pytest.mark.parametrize("shape", [(5, 50, 9, 11, 64, 32),        # 99 picks: one workgroup per batch element builds the table
                                   (4, 300, 40, 25, 64, 32),      # 1000 picks: two workgroups, 512 + 488 picks (csr_count_half_body)
                                   (3, 77, 13, 31, 128, 64)],     # 403 picks: two workgroups, 256 + 147 picks
                         ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("dtype,type_id", [(torch.bfloat16, _abi.BF16), (torch.float32, _abi.F32)], ids=["bfloat16", "float32"])
def test_table_is_the_stable_sort_of_the_picks_by_token(dtype, type_id, shape):
    B, T, E, K, I, J = shape
    case = make_case(3, B, T, E, K, I, J, dtype)
    Ind = case["Ind"].clone()
    Ind[1, 2, 3] = T; Ind[2, 0, 0] = -5         # rejected picks have no place in any token's list
    Ind[0, E - 1, K - 1] = -1; Ind[0, E // 2, :] = 7       # ... in either half; a token that a whole expert picks K times
    X, Wg, IndD = case["X"].to(DEV), case["Wg"].to(DEV), Ind.to(DEV)
    d = _abi.Dims(B, T, E, K, I, J)
    nb = _abi.lib().egs_routing_table_bytes(d, type_id)
    assert nb > 0
    table = torch.full((nb,), 0xEE, dtype=torch.uint8, device=DEV)
    Y = torch.empty(B, E, K, J, dtype=dtype, device=DEV)
    rc = _abi.lib().egs_expert_gather_forward_table(X.data_ptr(), Wg.data_ptr(), IndD.data_ptr(), Y.data_ptr(), table.data_ptr(), nb,
                                                    d, T * I, I, type_id, _abi.IND_I64, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    safe = Ind.clone(); safe[(Ind < 0) | (Ind >= T)] = 0
    mask = ((Ind >= 0) & (Ind < T)).numpy()[..., None]
    assert_close(Y, O.gather_forward(np64(case["X"]), np64(case["Wg"]), safe.numpy()) * mask, dtype, "Y of the launch that builds the table")
    words = table.cpu().numpy().view(np.int32)
    perm_at = -(-(B * (T + 1) * 4) // 256) * 256 // 4
    seg = words[:B * (T + 1)].reshape(B, T + 1)
    perm = words[perm_at:perm_at + B * E * K].reshape(B, E * K)
    flat = Ind.numpy().reshape(B, E * K)
    for b in range(B):
        valid = (flat[b] >= 0) & (flat[b] < T)
        counts = np.bincount(flat[b][valid], minlength=T)
        assert (seg[b] == np.concatenate([[0], np.cumsum(counts)])).all()
        order = np.argsort(np.where(valid, flat[b], T), kind="stable")[:valid.sum()]
        assert (perm[b, :valid.sum()] == order).all()


def test_in_place_writes_to_ind_retire_the_table():
    shape = (2, 64, 8, 16, 128, 64)
    B, T, E, K, I, J = shape
    case = make_case(41, *shape, torch.bfloat16)
    other = make_case(42, *shape, torch.bfloat16)["Ind"]
    assert not torch.equal(other, case["Ind"])
    hk.set_routing_table_cache(False)
    _, want = chain(dict(case, Ind=other), T)
    hk.set_routing_table_cache(True)
    Ind, _ = chain(case, T)
    assert ATTR in Ind.__dict__
    Ind.copy_(other.to(DEV))            # same object, same address, new contents: the version counter moves
    Y, Ws, X, Wg = (case[k].to(DEV) for k in ("Y", "Ws", "X", "Wg"))
    out = hk.expert_scatter_forward_call(Y, Ws, Ind, T, torch.float32)
    dX, dWg = hk.expert_gather_backward_call(X, Wg, Ind, Y, torch.float32)
    assert torch.equal(out, want[1]) and torch.equal(dX, want[2]) and torch.equal(dWg, want[3])
    # the next gather forward builds the table of the new contents
    _, again = chain(case, T, ind=Ind)
    for a, b in zip(again, want):
        assert torch.equal(a, b)
    # single elements too
    Ind[0, 0, 0] = (int(Ind[0, 0, 0]) + 1) % T
    hk.set_routing_table_cache(False)
    _, want2 = chain(case, T, ind=Ind.clone())
    hk.set_routing_table_cache(True)
    out2 = hk.expert_scatter_forward_call(Y, Ws, Ind, T, torch.float32)
    assert torch.equal(out2, want2[1])


def test_a_table_serves_only_the_sizes_and_stream_it_was_built_for():
    shape = (2, 64, 8, 16, 128, 64)
    B, T, E, K, I, J = shape
    case = make_case(43, *shape, torch.bfloat16)
    Ind, _ = chain(case, T)
    Y, Ws = case["Y"].to(DEV), case["Ws"].to(DEV)
    # a scatter into more tokens than the gather read from: other sizes, no table
    T2 = T + 16
    out = hk.expert_scatter_forward_call(Y, Ws, Ind, T2, torch.float32)
    assert_close(out, O.scatter_forward(np64(case["Y"]), np64(case["Ws"]), case["Ind"].numpy(), T2), torch.bfloat16, "other T")
    # another stream: its launches are not ordered after the launch that builds the table
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        assert hk._table_lookup(Ind, shape, _abi.BF16, hk._stream_ptr(Ind.device)) is None
        out_side = hk.expert_scatter_forward_call(Y, Ws, Ind, T, torch.float32)
    side.synchronize()
    hk.set_routing_table_cache(False)
    want = hk.expert_scatter_forward_call(Y, Ws, Ind, T, torch.float32)
    assert torch.equal(out_side, want)
    # explicit invalidation
    hk.set_routing_table_cache(True)
    assert ATTR in Ind.__dict__
    hk.invalidate_routing_table(Ind)
    assert ATTR not in Ind.__dict__


def test_no_table_for_fp32_multi_pass_or_a_gather_that_cannot_carry_it():
    for shape, dtype in [((4, 64, 8, 16, 128, 128), torch.float32),      # fp32 scatter with a reduction of 128: general path
                         ((2, 256, 96, 32, 128, 64), torch.bfloat16),    # scatter in passes over more than 2048 picks
                         ((4, 300, 40, 25, 96, 32), torch.bfloat16)]:    # gather forward on the tiled kernel: nothing to ride in
        case = make_case(44, *shape, dtype)
        Ind, _ = chain(case, shape[1])
        assert ATTR not in Ind.__dict__


def test_a_table_of_a_captured_launch_serves_that_capture_only():
    shape = (8, 64, 8, 16, 128, 64)
    B, T, E, K, I, J = shape
    case = make_case(45, *shape, torch.bfloat16)
    others = [make_case(46 + i, *shape, torch.bfloat16)["Ind"].to(DEV) for i in range(3)]
    X, Wg, Ws, Y, Ind = (case[k].to(DEV) for k in ("X", "Wg", "Ws", "Y", "Ind"))

    def eager(ind):
        hk.set_routing_table_cache(False)
        r = (hk.expert_gather_forward_call(X, Wg, ind, torch.float32), hk.expert_scatter_forward_call(Y, Ws, ind, T, torch.float32),
             *hk.expert_gather_backward_call(X, Wg, ind, Y, torch.float32))
        hk.set_routing_table_cache(True)
        return r

    hk.expert_gather_forward_call(X, Wg, Ind, torch.float32)       # an eager table exists before the capture starts
    eager_entry = Ind.__dict__[ATTR]
    assert eager_entry[0][-1] == 0
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        # the eager table is for another stream and no capture: the captured gather builds its own, the two captured
        # scatters read it
        gy = hk.expert_gather_forward_call(X, Wg, Ind, torch.float32)
        captured_entry = Ind.__dict__[ATTR]
        assert captured_entry is not eager_entry and captured_entry[0][-1] > 0
        assert hk._table_lookup(Ind, shape, _abi.BF16, hk._stream_ptr(Ind.device)) is captured_entry[1]
        gout = hk.expert_scatter_forward_call(Y, Ws, Ind, T, torch.float32)
        gdx, gdw = hk.expert_gather_backward_call(X, Wg, Ind, Y, torch.float32)
    # after the capture the entry is not used by eager calls (its contents exist only after a replay)
    assert hk._table_lookup(Ind, shape, _abi.BF16, hk._stream_ptr(Ind.device)) is None
    for other in [Ind.clone()] + others:
        Ind.copy_(other)                    # the graph's static input changes between replays
        want = eager(other)
        graph.replay()
        torch.cuda.synchronize()
        for got, ref in zip((gy, gout, gdx, gdw), want):
            assert torch.equal(got, ref)
        # eager calls on the same Ind between replays build and use their own table
        _, mine = chain(case, T, ind=Ind)
        for got, ref in zip(mine, want):
            assert torch.equal(got, ref)


def test_autograd_chain_uses_and_survives_the_table():
    import expertscattergather_amd as egs
    B, T, E, K, I, J = 4, 64, 8, 16, 128, 64
    torch.manual_seed(0)
    g = egs.ExpertGather(E, I, J).to(DEV).bfloat16()
    s = egs.ExpertScatter(E, J, I).to(DEV).bfloat16()
    x = torch.randn(B, T, I, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    Ind = torch.randint(0, T, (B, E, K), device=DEV)

    def run():
        for p in (x, g.W, s.W):
            p.grad = None
        out = s(torch.relu(g(x, Ind)), Ind, T)
        out.float().square().sum().backward()
        return out.detach().clone(), x.grad.clone(), g.W.grad.clone(), s.W.grad.clone()

    hk.set_routing_table_cache(False)
    want = run()
    hk.set_routing_table_cache(True)
    got = run()
    assert ATTR in Ind.__dict__
    again = run()                   # second step with the same Ind object: the table is found, not rebuilt
    for a, b, c in zip(want, got, again):
        assert torch.equal(a, b) and torch.equal(a, c)


def test_a_strided_ind_gets_no_table_and_the_same_results():
    shape = (4, 64, 8, 16, 128, 64)
    case = make_case(61, *shape, torch.bfloat16)
    strided = case["Ind"].to(DEV).transpose(1, 2).contiguous().transpose(1, 2)      # [B,E,K] values, K-major memory
    assert not strided.is_contiguous() and torch.equal(strided.cpu(), case["Ind"])
    _, got = chain(case, shape[1], ind=strided)
    assert ATTR not in strided.__dict__, "the launchers work on a contiguous copy that does not outlive the call"
    hk.set_routing_table_cache(False)
    _, want = chain(case, shape[1])
    for a, b in zip(got, want):
        assert torch.equal(a, b)


def test_a_table_of_garbage_gives_wrong_sums_but_ends():
    """The C entry points cannot know whose table they are handed; they must stay inside the workgroup's rows and finish."""
    for shape in [(4, 64, 8, 16, 128, 64), (2, 256, 48, 32, 128, 64)]:      # one pass, and passes over groups of experts
        B, T, E, K, I, J = shape
        case = make_case(71, *shape, torch.bfloat16)
        Y, Ws, Ind = (case[k].to(DEV) for k in ("Y", "Ws", "Ind"))
        d = _abi.Dims(*shape)
        nb = _abi.lib().egs_routing_table_bytes(d, _abi.BF16)
        assert nb > 0
        out = torch.empty(B, T, I, dtype=torch.bfloat16, device=DEV)
        gen = torch.Generator(device="cpu").manual_seed(1)
        for table in (torch.randint(-2 ** 31, 2 ** 31 - 1, (nb // 4,), generator=gen, dtype=torch.int64).to(torch.int32).to(DEV),
                      torch.full((nb // 4,), 2 ** 31 - 1, dtype=torch.int32, device=DEV),
                      torch.zeros(nb // 4, dtype=torch.int32, device=DEV)):
            rc = _abi.lib().egs_expert_scatter_forward_table(Y.data_ptr(), Ws.data_ptr(), Ind.data_ptr(), table.data_ptr(), nb,
                                                             out.data_ptr(), None, 0, d, _abi.BF16, _abi.IND_I64, 0,
                                                             torch.cuda.current_stream().cuda_stream)
            assert rc == 0
            torch.cuda.synchronize()
            assert torch.isfinite(out.float()).all()
