"""``nn.Module`` wrappers that own the expert weights (API of the reference's
``egs/torch_interface.py``: same class names, constructor arguments, parameter names and
shapes, ``reset_parameters``, ``forward`` and ``to``)."""
from __future__ import annotations

import math

import torch
from torch import nn

from .hip_kernels import ExpertGatherFunction, ExpertScatterFunction, create_kernels, scatter_mode_scope


class ExpertGather(nn.Module):
    """Gathers K tokens per (batch, expert) and applies that expert's [I,J] weight.

    Reference: egs/torch_interface.py:11-63.  ``W`` is [E,I,J]; the optional ``bias`` is
    [E,1,J] and is added to every picked row of its expert.

    ``scatter_mode`` (attribute, default ``None`` = the process-wide setting of ``hip_kernels.set_scatter_mode`` /
    ``EGS_SCATTER_MODE``): "deterministic" or "atomic" for the scatter in this module's backward (grad of ``x``)."""

    scatter_mode = None

    def __init__(self, E: int, I: int, J: int, bias: bool = False):
        super().__init__()
        self.E, self.I, self.J = E, I, J
        self.W = nn.Parameter(torch.empty(E, I, J))
        if bias:
            self.bias = nn.Parameter(torch.empty(E, 1, J))
        else:
            self.register_parameter('bias', None)
        self.reset_parameters()
        create_kernels()

    def reset_parameters(self):
        bound = 1 / math.sqrt(self.I)                    # reference egs/torch_interface.py:37-42
        nn.init.uniform_(self.W, -bound, bound)
        if self.bias is not None:
            nn.init.uniform_(self.bias, -bound, bound)

    def forward(self, x: torch.Tensor, Ind: torch.Tensor):
        """x: [B,T,I];  Ind: integers in [0,T) of shape [B,E,K]  ->  [B,E,K,J]."""
        if self.scatter_mode is None:
            y = ExpertGatherFunction.apply(x, self.W, Ind)
        else:
            with scatter_mode_scope(self.scatter_mode):     # bound to the autograd node: the backward runs in it too
                y = ExpertGatherFunction.apply(x, self.W, Ind)
        if self.bias is not None:
            y = y + self.bias
        return y

    def to(self, *args, **kwargs):
        return super().to(*args, **kwargs)


class ExpertScatter(nn.Module):
    """Applies each expert's [J,I] weight to its K rows and adds them back onto their tokens.

    Reference: egs/torch_interface.py:66-119.  ``W`` is [E,J,I]; the optional ``bias`` is
    [E,1,I] and every pick of expert e adds bias[e] to the token it lands on.

    ``scatter_mode`` (attribute, default ``None`` = the process-wide setting of ``hip_kernels.set_scatter_mode`` /
    ``EGS_SCATTER_MODE``): "deterministic" or "atomic" for this module's forward."""

    scatter_mode = None

    def __init__(self, E: int, J: int, I: int, bias: bool = False):
        super().__init__()
        self.E, self.J, self.I = E, J, I
        self.W = nn.Parameter(torch.empty(E, J, I))
        if bias:
            self.bias = nn.Parameter(torch.empty(E, 1, I))
        else:
            self.register_parameter('bias', None)
        self.reset_parameters()
        create_kernels()

    def reset_parameters(self):
        bound = 1 / math.sqrt(self.I)                    # reference egs/torch_interface.py:92-97
        nn.init.uniform_(self.W, -bound, bound)
        if self.bias is not None:
            nn.init.uniform_(self.bias, -bound, bound)

    def forward(self, Y: torch.Tensor, Ind: torch.Tensor, T: int):
        """Y: [B,E,K,J];  Ind: [B,E,K] in [0,T);  T: output sequence length  ->  [B,T,I]."""
        if self.scatter_mode is None:
            y = ExpertScatterFunction.apply(Y, self.W, Ind, T)
        else:
            with scatter_mode_scope(self.scatter_mode):
                y = ExpertScatterFunction.apply(Y, self.W, Ind, T)
        if self.bias is not None and T > 0 and Ind.numel() > 0:
            # picks[b,t,e] = how many times expert e selected token t; each adds bias[e]
            # (a pick outside [0,T) contributes nothing, as in the kernels: it is routed to slot 0 with weight 0)
            B, E, K = Ind.shape
            picks = torch.zeros(B, T, E, device=y.device, dtype=torch.float32)
            e_ids = torch.arange(E, device=y.device).view(1, E, 1).expand(B, E, K).reshape(B, E * K)
            ind = Ind.to(torch.int64).reshape(B, E * K)
            valid = (ind >= 0) & (ind < T)
            flat = torch.where(valid, ind * E + e_ids, torch.zeros_like(ind))
            picks.view(B, T * E).scatter_add_(1, flat, valid.to(torch.float32))
            y = y + (picks @ self.bias[:, 0, :].float()).to(y.dtype)
        return y

    def to(self, *args, **kwargs):
        return super().to(*args, **kwargs)
