"""Seeded synthetic inputs of the five benchmark configurations (host-side helper for the
tests and ``bench.py``).  Everything is generated on the CPU with a ``torch.Generator`` so
that the CPU baseline and the GPU path see the same bits."""
from __future__ import annotations

from dataclasses import dataclass

import torch


@dataclass(frozen=True)
class Config:
    name: str
    B: int
    T: int
    E: int
    K: int
    I: int
    J: int
    dtype: torch.dtype
    routing: str          # "uniform" (without replacement per (b,e)) or "zipf" (with replacement)
    seed: int
    what: str

    @property
    def dims(self):
        return self.B, self.T, self.E, self.K, self.I, self.J


CONFIGS = {
    "C1": Config("C1", 64, 256, 32, 32, 128, 64, torch.float32, "uniform", 1001, "default shape, fp32, forward only"),
    "C2": Config("C2", 64, 256, 32, 32, 128, 64, torch.bfloat16, "uniform", 1002, "default shape, bf16, fwd+bwd chain"),
    "C3": Config("C3", 8, 4096, 128, 256, 1024, 256, torch.bfloat16, "uniform", 1003, "long sequence, fine-grained experts"),
    "C4": Config("C4", 16, 1024, 64, 128, 512, 128, torch.bfloat16, "zipf", 1004, "Zipf(1.2) routing with replacement"),
    "C5": Config("C5", 32, 2048, 256, 64, 2048, 512, torch.bfloat16, "uniform", 1005, "fp8 e4m3 weights, forward only"),
}


def uniform_routing(B, T, E, K, gen, dtype=torch.int64):
    """K distinct token ids per (b,e): the first K entries of a random permutation of T."""
    assert K <= T
    out = torch.empty(B, E, K, dtype=torch.int64)
    for b in range(B):          # chunked so that the [E,T] sort keys stay small
        out[b] = torch.argsort(torch.rand(E, T, generator=gen), dim=-1)[:, :K]
    return out.to(dtype)


def zipf_routing(B, T, E, K, gen, s=1.2, dtype=torch.int64):
    """K draws with replacement per (b,e) from p(r) ~ r^-s over a seeded permutation of T."""
    p = torch.arange(1, T + 1, dtype=torch.float64).pow(-s)
    perm = torch.randperm(T, generator=gen)
    ranks = torch.multinomial(p.expand(B * E, T), K, replacement=True, generator=gen)
    return perm[ranks].reshape(B, E, K).to(dtype)


def make_inputs(cfg: Config, dims=None, ind_dtype=torch.int64):
    """Returns dict with X, Wg [E,I,J], Ws [E,J,I], Ind, dOut (CPU tensors in cfg.dtype)."""
    B, T, E, K, I, J = dims or cfg.dims
    gen = torch.Generator().manual_seed(cfg.seed)
    X = torch.randn(B, T, I, generator=gen)
    Wg = torch.randn(E, I, J, generator=gen) / (I ** 0.5)
    Ws = torch.randn(E, J, I, generator=gen) / (J ** 0.5)
    dOut = torch.randn(B, T, I, generator=gen)
    if cfg.routing == "zipf":
        Ind = zipf_routing(B, T, E, K, gen, dtype=ind_dtype)
    else:
        Ind = uniform_routing(B, T, E, K, gen, dtype=ind_dtype)
    dt = cfg.dtype
    return {"X": X.to(dt), "Wg": Wg.to(dt), "Ws": Ws.to(dt), "dOut": dOut.to(dt), "Ind": Ind}


def quantize_fp8_weights(W: torch.Tensor):
    """W [E,I,J] float -> (Wq float8_e4m3fn [E,I,J], scale float32 [E,J]) with
    scale[e,j] = max_i |W[e,i,j]| / 448."""
    W = W.float()
    scale = (W.abs().amax(dim=1) / 448.0).clamp_min(1e-12)
    Wq = (W / scale[:, None, :]).to(torch.float8_e4m3fn)
    return Wq, scale


def algorithmic_bytes(dims, act_bytes, w_bytes=None, ind_bytes=8, fp8_scales=False, dw=False, out_bytes=None):
    """HBM bytes one kernel call must move at the very least (every tensor touched once)."""
    B, T, E, K, I, J = dims
    w_bytes = act_bytes if w_bytes is None else w_bytes
    rows = min(B * T, B * E * K) * I * act_bytes
    picks = B * E * K
    if dw:
        out_bytes = act_bytes if out_bytes is None else out_bytes
        return rows + picks * J * act_bytes + picks * ind_bytes + E * I * J * out_bytes
    return rows + E * I * J * w_bytes + (E * J * 4 if fp8_scales else 0) + picks * ind_bytes + picks * J * act_bytes


def flops(dims):
    B, T, E, K, I, J = dims
    return 2 * B * E * K * I * J
