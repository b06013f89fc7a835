"""Torch-CPU port of the reference's pure-torch baselines (the arithmetic the reference tests
compare its kernels with).  TEST INFRASTRUCTURE ONLY, like everything under ``oracle/``.

* ``gather``  restates reference egs/baselines.py:69-76  (torch.gather along T + einsum 'beki,eij->bekj')
* ``scatter`` restates reference egs/baselines.py:174-184 (einsum 'bekj,eji->beki' + zeros.scatter_add_)

Both are differentiable, so torch autograd through them gives dX/dW/dY independently of the
closed forms in ``egs_oracle.py``.  ``bench.py`` times ``chain_fwd_bwd`` on the host cores as
its ``cpu_baseline`` ("port").
"""
from __future__ import annotations

import torch


def gather(X: torch.Tensor, W: torch.Tensor, Ind: torch.Tensor) -> torch.Tensor:
    B, T, I = X.shape
    _, E, K = Ind.shape
    index = Ind.to(torch.int64).reshape(B, E * K)[..., None].expand(-1, -1, I)
    Xg = torch.gather(X, dim=1, index=index).reshape(B, E, K, I)
    return torch.einsum('beki,eij->bekj', Xg, W)


def scatter(Y: torch.Tensor, W: torch.Tensor, Ind: torch.Tensor, T: int) -> torch.Tensor:
    B, E, K, J = Y.shape
    pre = torch.einsum('bekj,eji->beki', Y, W)
    I = pre.shape[-1]
    out = torch.zeros(B, T, I, device=Y.device, dtype=Y.dtype)
    index = Ind.to(torch.int64)[..., None].expand(-1, -1, -1, I).reshape(B, E * K, I)
    out.scatter_add_(1, index, pre.reshape(B, E * K, I))
    return out


def chain_fwd_bwd(X, Wg, Ws, Ind, dOut):
    """gather -> scatter -> backward with upstream gradient dOut (the benchmark's step).

    Returns (Y, out, dX, dWg, dWs)."""
    X = X.detach().clone().requires_grad_(True)
    Wg = Wg.detach().clone().requires_grad_(True)
    Ws = Ws.detach().clone().requires_grad_(True)
    Y = gather(X, Wg, Ind)
    out = scatter(Y, Ws, Ind, X.shape[1])
    out.backward(dOut)
    return Y.detach(), out.detach(), X.grad, Wg.grad, Ws.grad
