"""Pins the CPU oracle (numpy, C, torch port) without the reference code:
brute-force loops on tiny shapes, closed-form special cases, adjointness, linearity,
autograd through an independent forward, finite differences and the fp8 decode table."""
import numpy as np
import pytest
import torch

from oracle import egs_oracle as O
from oracle import c_oracle as C
from oracle import torch_port as P


def rand_case(seed, B, T, E, K, I, J, replace=True):
    g = np.random.default_rng(seed)
    X = g.standard_normal((B, T, I))
    Wg = g.standard_normal((E, I, J)) / np.sqrt(I)
    Ws = g.standard_normal((E, J, I)) / np.sqrt(J)
    if replace:
        Ind = g.integers(0, T, size=(B, E, K))
    else:
        Ind = np.stack([np.stack([g.permutation(T)[:K] for _ in range(E)]) for _ in range(B)])
    Y = g.standard_normal((B, E, K, J))
    dOut = g.standard_normal((B, T, I))
    return X, Wg, Ws, Ind.astype(np.int64), Y, dOut


TINY = [(1, 1, 1, 1, 1, 1), (2, 3, 2, 4, 3, 2), (3, 4, 3, 2, 4, 3), (2, 5, 1, 7, 2, 5), (1, 2, 4, 3, 5, 1)]


@pytest.mark.parametrize("shape", TINY)
def test_vectorised_matches_brute_force(shape):
    X, Wg, Ws, Ind, Y, dOut = rand_case(7, *shape)
    T = shape[1]
    np.testing.assert_allclose(O.gather_forward(X, Wg, Ind), O.brute_gather_forward(X, Wg, Ind), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(O.scatter_forward(Y, Ws, Ind, T), O.brute_scatter_forward(Y, Ws, Ind, T), rtol=1e-12, atol=1e-12)
    dX, dW = O.gather_backward(X, Wg, Ind, Y)
    bX, bW = O.brute_gather_backward(X, Wg, Ind, Y)
    np.testing.assert_allclose(dX, bX, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(dW, bW, rtol=1e-12, atol=1e-12)
    dY, dWs = O.scatter_backward(Y, Ws, Ind, dOut)
    bY, bWs = O.brute_scatter_backward(Y, Ws, Ind, dOut)
    np.testing.assert_allclose(dY, bY, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(dWs, bWs, rtol=1e-12, atol=1e-12)


def test_hand_computed_known_answer():
    # one batch, two tokens, one expert picking token 1 twice and token 0 once
    X = np.array([[[1.0, 2.0], [3.0, 4.0]]])                 # [1,2,2]
    W = np.array([[[1.0, 0.0, 2.0], [0.0, 1.0, -1.0]]])      # [1,2,3]
    Ind = np.array([[[1, 1, 0]]])
    Y = O.gather_forward(X, W, Ind)
    expect = np.array([[[[3.0, 4.0, 2.0], [3.0, 4.0, 2.0], [1.0, 2.0, 0.0]]]])
    np.testing.assert_array_equal(Y, expect)
    Ws = np.array([[[1.0, 1.0], [0.0, 2.0], [1.0, 0.0]]])    # [1,3,2]
    out = O.scatter_forward(Y, Ws, Ind, 2)
    # row picks: [3,4,2]@Ws = [5, 11]; twice into token 1; [1,2,0]@Ws=[1,5] into token 0
    np.testing.assert_array_equal(out, np.array([[[1.0, 5.0], [10.0, 22.0]]]))


def test_identity_routing_reduces_to_matmul():
    g = np.random.default_rng(3)
    B, T, I, J = 3, 9, 5, 4
    X = g.standard_normal((B, T, I)); W = g.standard_normal((1, I, J))
    Ind = np.broadcast_to(np.arange(T)[None, None, :], (B, 1, T)).copy()
    np.testing.assert_allclose(O.gather_forward(X, W, Ind)[:, 0], X @ W[0], rtol=1e-13, atol=1e-13)
    Y = g.standard_normal((B, 1, T, J)); Ws = g.standard_normal((1, J, I))
    np.testing.assert_allclose(O.scatter_forward(Y, Ws, Ind, T), Y[:, 0] @ Ws[0], rtol=1e-13, atol=1e-13)


def test_scatter_of_gather_counts_picks():
    # W_g @ W_s = identity and every token picked c(t) times => out = c(t) * X
    g = np.random.default_rng(5)
    B, T, E, K, I = 2, 6, 3, 4, 5
    X = g.standard_normal((B, T, I))
    Q = np.linalg.qr(g.standard_normal((I, I)))[0]
    Wg = np.broadcast_to(Q, (E, I, I)).copy(); Ws = np.broadcast_to(Q.T, (E, I, I)).copy()
    Ind = g.integers(0, T, size=(B, E, K))
    out = O.scatter_forward(O.gather_forward(X, Wg, Ind), Ws, Ind, T)
    cnt = np.zeros((B, T))
    for b in range(B):
        np.add.at(cnt[b], Ind[b].ravel(), 1)
    np.testing.assert_allclose(out, cnt[..., None] * X, rtol=1e-12, atol=1e-12)
    assert (out[cnt == 0] == 0).all()


def test_adjointness_and_linearity():
    X, Wg, Ws, Ind, Y, dOut = rand_case(11, 3, 7, 4, 5, 6, 3)
    T = 7
    G = Y
    lhs = (O.gather_forward(X, Wg, Ind) * G).sum()
    rhs = (X * O.scatter_forward(G, np.swapaxes(Wg, 1, 2), Ind, T)).sum()
    assert abs(lhs - rhs) <= 1e-10 * abs(lhs)
    X2 = rand_case(12, 3, 7, 4, 5, 6, 3)[0]
    np.testing.assert_allclose(O.gather_forward(2 * X - 3 * X2, Wg, Ind),
                               2 * O.gather_forward(X, Wg, Ind) - 3 * O.gather_forward(X2, Wg, Ind), atol=1e-12)
    # permuting k inside (b,e) leaves the scatter output unchanged
    perm = np.random.default_rng(1).permutation(5)
    np.testing.assert_allclose(O.scatter_forward(Y[:, :, perm], Ws, Ind[:, :, perm], T),
                               O.scatter_forward(Y, Ws, Ind, T), atol=1e-12)


@pytest.mark.parametrize("shape", [(2, 5, 3, 4, 6, 3), (3, 17, 5, 9, 13, 7), (4, 33, 2, 40, 8, 19)])
def test_c_restatement_matches_numpy(shape):
    X, Wg, Ws, Ind, Y, dOut = rand_case(21, *shape)
    T = shape[1]
    f = lambda a: a.astype(np.float32)
    X, Wg, Ws, Y, dOut = map(f, (X, Wg, Ws, Y, dOut))
    np.testing.assert_allclose(C.gather(X, Wg, Ind), O.gather_forward(X, Wg, Ind), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(C.scatter(Y, Ws, Ind, T), O.scatter_forward(Y, Ws, Ind, T), rtol=1e-12, atol=1e-12)
    dX, dW = O.gather_backward(X, Wg, Ind, Y)
    np.testing.assert_allclose(C.scatter(Y, Wg, Ind, T, C.W_EIJ), dX, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(C.dw(X, Y, Ind, C.W_EIJ), dW, rtol=1e-12, atol=1e-12)
    dY, dWs = O.scatter_backward(Y, Ws, Ind, dOut)
    np.testing.assert_allclose(C.gather(dOut, Ws, Ind, C.W_EJI), dY, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(C.dw(dOut, Y, Ind, C.W_EJI), dWs, rtol=1e-12, atol=1e-12)
    with pytest.raises(IndexError):
        bad = Ind.copy(); bad[0, 0, 0] = T
        C.gather(X, Wg, bad)


def test_torch_port_and_autograd_match_closed_forms():
    X, Wg, Ws, Ind, Y, dOut = rand_case(31, 3, 11, 4, 6, 7, 5)
    T = 11
    t = lambda a: torch.from_numpy(a)
    np.testing.assert_allclose(P.gather(t(X), t(Wg), t(Ind)).numpy(), O.gather_forward(X, Wg, Ind), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(P.scatter(t(Y), t(Ws), t(Ind), T).numpy(), O.scatter_forward(Y, Ws, Ind, T), rtol=1e-12, atol=1e-12)
    # autograd through the torch forward vs the oracle's closed-form backward
    Xt = t(X).requires_grad_(True); Wt = t(Wg).requires_grad_(True)
    P.gather(Xt, Wt, t(Ind)).backward(t(Y))
    dX, dW = O.gather_backward(X, Wg, Ind, Y)
    np.testing.assert_allclose(Xt.grad.numpy(), dX, rtol=1e-11, atol=1e-11)
    np.testing.assert_allclose(Wt.grad.numpy(), dW, rtol=1e-11, atol=1e-11)
    Yt = t(Y).requires_grad_(True); Wst = t(Ws).requires_grad_(True)
    P.scatter(Yt, Wst, t(Ind), T).backward(t(dOut))
    dY, dWs = O.scatter_backward(Y, Ws, Ind, dOut)
    np.testing.assert_allclose(Yt.grad.numpy(), dY, rtol=1e-11, atol=1e-11)
    np.testing.assert_allclose(Wst.grad.numpy(), dWs, rtol=1e-11, atol=1e-11)
    # whole chain
    Yc, outc, dXc, dWgc, dWsc = P.chain_fwd_bwd(t(X), t(Wg), t(Ws), t(Ind), t(dOut))
    Yo = O.gather_forward(X, Wg, Ind); outo = O.scatter_forward(Yo, Ws, Ind, T)
    dYo, dWso = O.scatter_backward(Yo, Ws, Ind, dOut); dXo, dWgo = O.gather_backward(X, Wg, Ind, dYo)
    for a, b in ((Yc, Yo), (outc, outo), (dXc, dXo), (dWgc, dWgo), (dWsc, dWso)):
        np.testing.assert_allclose(a.numpy(), b, rtol=1e-10, atol=1e-10)


def test_finite_difference_of_loss():
    X, Wg, Ws, Ind, Y, dOut = rand_case(41, 2, 5, 3, 4, 3, 2)
    G = Y
    loss = lambda X_, W_: (O.gather_forward(X_, W_, Ind) * G).sum()
    dX, dW = O.gather_backward(X, Wg, Ind, G)
    eps = 1e-6
    for idx in [(0, 1, 2), (1, 4, 0)]:
        Xp = X.copy(); Xp[idx] += eps; Xm = X.copy(); Xm[idx] -= eps
        assert abs((loss(Xp, Wg) - loss(Xm, Wg)) / (2 * eps) - dX[idx]) < 1e-6
    for idx in [(0, 0, 1), (2, 2, 0)]:
        Wp = Wg.copy(); Wp[idx] += eps; Wm = Wg.copy(); Wm[idx] -= eps
        assert abs((loss(X, Wp) - loss(X, Wm)) / (2 * eps) - dW[idx]) < 1e-6


def test_fp8_decode_table_matches_torch():
    bits = np.arange(256, dtype=np.uint8)
    ours = O.fp8_e4m3fn_to_float(bits)
    theirs = torch.from_numpy(bits).view(torch.float8_e4m3fn).to(torch.float32).numpy().astype(np.float64)
    nan = np.isnan(theirs)
    assert (np.isnan(ours) == nan).all()
    np.testing.assert_array_equal(ours[~nan], theirs[~nan])
    assert ours[0x7E] == 448.0 and ours[0x08] == 2.0 ** -6 and ours[0x01] == 2.0 ** -9


def test_bf16_rounding_matches_torch():
    a = np.random.default_rng(0).standard_normal(4096).astype(np.float32) * 37
    np.testing.assert_array_equal(O.round_to_bf16(a), torch.from_numpy(a).to(torch.bfloat16).to(torch.float32).numpy())


def test_fp8_encoder_and_row_quantiser_match_torch():
    """Pins float_to_fp8_e4m3fn / quantize_rows_e4m3 against torch's float8_e4m3fn cast (round to nearest even),
    including every code, every midpoint between codes, subnormals and the zero row."""
    codes = torch.arange(256, dtype=torch.uint8)
    vals = codes.view(torch.float8_e4m3fn).float()
    finite = ~torch.isnan(vals)
    assert np.array_equal(O.float_to_fp8_e4m3fn(vals[finite].numpy())[vals[finite] != 0], codes[finite][vals[finite] != 0].numpy())
    mags = vals[:0x7F]
    mids = (mags[:-1] + mags[1:]) / 2                        # exact in float32: ties
    g = torch.Generator().manual_seed(5)
    x = torch.cat([mids, -mids, torch.rand(20000, generator=g) * 896 - 448, torch.randn(20000, generator=g) * 0.02,
                   torch.tensor([0.0, -0.0, 448.0, -448.0, 2.0 ** -9, 2.0 ** -10, 3 * 2.0 ** -11])])
    ours = O.float_to_fp8_e4m3fn(x.numpy())
    theirs = x.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(ours, theirs)
    X = torch.randn(7, 5, 64, generator=g).to(torch.bfloat16)
    X[2, 3] = 0
    X[1, 1] *= 1e-3
    q, xs = O.quantize_rows_e4m3(X.float().numpy())
    amax = X.float().abs().amax(dim=-1)
    xs_t = torch.where(amax > 0, amax / 448.0, torch.ones_like(amax))
    q_t = (X.float() * (1.0 / xs_t)[..., None]).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8)
    assert np.array_equal(xs, xs_t.numpy()) and np.array_equal(q, q_t.numpy())
    # a quantised row reproduces the row to e4m3 accuracy: |x - dequant| <= 2^-4 |x| + half a subnormal step
    deq = O.fp8_e4m3fn_to_float(q) * xs[..., None]
    assert (np.abs(deq - X.float().numpy()) <= 2.0 ** -4 * np.abs(X.float().numpy()) + xs[..., None] * 2.0 ** -10).all()
    # rows with a NaN or an infinity: NaN scale (every product of the row is NaN, as in unquantised arithmetic);
    # the other rows are untouched
    Xn = X.float().numpy().copy()
    Xn[0, 0, 5] = np.nan; Xn[3, 2, 0] = np.inf; Xn[6, 4, 63] = -np.inf
    q2, xs2 = O.quantize_rows_e4m3(Xn)
    bad = np.zeros(xs.shape, dtype=bool); bad[0, 0] = bad[3, 2] = bad[6, 4] = True
    assert np.isnan(xs2[bad]).all() and np.array_equal(xs2[~bad], xs[~bad]) and np.array_equal(q2[~bad], q[~bad])


# ---------------------------------------------------------------------------------------------------------
# inference block: activation closed forms and the chained forward
def test_activations_against_torch_and_special_values():
    y = np.linspace(-9.0, 9.0, 721)
    t = torch.from_numpy(y)
    F = torch.nn.functional
    for name, fn in (("relu", torch.relu), ("gelu", F.gelu), ("silu", F.silu),
                     ("gelu_tanh", lambda v: F.gelu(v, approximate="tanh")), ("none", lambda v: v)):
        np.testing.assert_allclose(O.activation(y, name), fn(t).numpy(), rtol=1e-12, atol=1e-14, err_msg=name)
    # what the mathematics fixes: zero at zero, identity far to the right, zero (relu) or vanishing far to the left,
    # gelu(x) - gelu(-x) = x and silu(x) - silu(-x) = x (the even parts cancel)
    for name in ("relu", "gelu", "gelu_tanh", "silu"):
        assert O.activation(np.array([0.0]), name)[0] == 0.0
        assert abs(O.activation(np.array([30.0]), name)[0] - 30.0) < 1e-9
        assert abs(O.activation(np.array([-30.0]), name)[0]) < 1e-9
    for name in ("gelu", "gelu_tanh", "silu"):
        np.testing.assert_allclose(O.activation(y, name) - O.activation(-y, name), y, rtol=0, atol=1e-12)
    assert abs(O.activation(np.array([1.0]), "gelu")[0] - 0.8413447460685429) < 1e-15      # Phi(1)
    assert abs(O.activation(np.array([1.0]), "silu")[0] - 0.7310585786300049) < 1e-15      # 1 / (1 + 1/e)
    with pytest.raises(ValueError):
        O.activation(y, "softmax")


def test_inference_block_is_the_chain_of_the_two_forwards():
    rng = np.random.default_rng(5)
    B, T, E, K, I, J = 2, 7, 3, 4, 5, 6
    X = rng.standard_normal((B, T, I)); Wg = rng.standard_normal((E, I, J)); Ws = rng.standard_normal((E, J, I))
    Ind = rng.integers(0, T, (B, E, K))
    Ind[0, 1, 2] = T + 3; Ind[1, 0, 0] = -1                              # rejected picks contribute nothing
    bad = (Ind < 0) | (Ind >= T)
    for act in ("none", "relu", "gelu", "silu"):
        # index-by-index: rows of Y for the valid picks only, activated, multiplied and added where they belong
        out = np.zeros((B, T, I))
        for b in range(B):
            for e in range(E):
                for k in range(K):
                    if bad[b, e, k]:
                        continue
                    y = O.activation(X[b, Ind[b, e, k]] @ Wg[e], act)
                    out[b, Ind[b, e, k]] += y @ Ws[e]
        np.testing.assert_allclose(O.mlp_forward(X, Wg, Ws, Ind, T, act), out, rtol=1e-12, atol=1e-12)
    # without an activation the block is linear in X; with rounding hooks the rows pass through them
    a = O.mlp_forward(X, Wg, Ws, Ind, T, "none"); b2 = O.mlp_forward(2.5 * X, Wg, Ws, Ind, T, "none")
    np.testing.assert_allclose(b2, 2.5 * a, rtol=1e-12, atol=1e-12)
    calls = []
    def spy(v):
        calls.append(v.shape); return v
    O.mlp_forward(X, Wg, Ws, Ind, T, "relu", round_y=spy, round_before_act=True)
    assert calls == [(B, E, K, J), (B, E, K, J)]
