"""Shared helpers of the parity tests: exact numpy views of torch tensors, seeded cases and
the stated tolerances."""
import numpy as np
import torch

# Tolerances (vs the float64 oracle evaluated on the same, already rounded, inputs).
#   fp32 : max|a-o| <= 1e-4 * max|o|   and elementwise |a-o| <= 1e-4*|o| + 1e-4*rms(o)
#   bf16 : fp32 accumulation, one final rounding: max|a-o| <= 2*2^-8 * max|o|, rel-RMS <= 3e-3
#   fp16 : same with 2^-11:                        max|a-o| <= 2*2^-11 * max|o|, rel-RMS <= 4e-4
TOL = {
    torch.float32: dict(max_rel=1e-4, rms_rel=1e-5),
    torch.bfloat16: dict(max_rel=2 * 2.0 ** -8, rms_rel=3e-3),
    torch.float16: dict(max_rel=2 * 2.0 ** -11, rms_rel=4e-4),
}


def np64(t: torch.Tensor) -> np.ndarray:
    return t.detach().to("cpu", torch.float64).numpy()


def assert_close(actual: torch.Tensor, oracle: np.ndarray, dtype, what=""):
    a = np64(actual)
    assert a.shape == oracle.shape, f"{what}: shape {a.shape} vs {oracle.shape}"
    assert np.isfinite(a).all(), f"{what}: non-finite values"
    tol = TOL[dtype]
    scale = np.abs(oracle).max() if oracle.size else 0.0
    err = np.abs(a - oracle).max() if oracle.size else 0.0
    assert err <= tol["max_rel"] * scale + 1e-30, f"{what}: max err {err:.3e} vs scale {scale:.3e} (limit {tol['max_rel']:.1e})"
    rms_o = np.sqrt((oracle ** 2).mean()) if oracle.size else 0.0
    rms_e = np.sqrt(((a - oracle) ** 2).mean()) if oracle.size else 0.0
    assert rms_e <= tol["rms_rel"] * rms_o + 1e-30, f"{what}: rms err {rms_e:.3e} vs rms {rms_o:.3e}"
    if dtype == torch.float32 and oracle.size:
        ok = np.abs(a - oracle) <= 1e-4 * np.abs(oracle) + 1e-4 * rms_o
        assert ok.all(), f"{what}: {int((~ok).sum())} elements outside rtol=1e-4"


def make_case(seed, B, T, E, K, I, J, dtype, ind_dtype=torch.int64, replace=True):
    """Random tensors rounded to `dtype` (CPU).  Ind drawn with replacement like the reference's
    tests (test_all.py:16) or without."""
    g = torch.Generator().manual_seed(seed)
    X = torch.randn(B, T, I, generator=g).to(dtype)
    Wg = (torch.randn(E, I, J, generator=g) / max(I, 1) ** 0.5).to(dtype)
    Ws = (torch.randn(E, J, I, generator=g) / max(J, 1) ** 0.5).to(dtype)
    Y = torch.randn(B, E, K, J, generator=g).to(dtype)
    dOut = torch.randn(B, T, I, generator=g).to(dtype)
    if replace or K > T:
        Ind = torch.randint(0, max(T, 1), (B, E, K), generator=g)
    else:
        Ind = torch.stack([torch.stack([torch.randperm(T, generator=g)[:K] for _ in range(E)]) for _ in range(B)])
    return dict(X=X, Wg=Wg, Ws=Ws, Y=Y, dOut=dOut, Ind=Ind.to(ind_dtype))
