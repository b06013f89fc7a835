"""Expert-choice router: the step in front of the gather/scatter path.

The reference draws ``Ind`` at random in its tests and benchmark (test_all.py:16, test_speed.ipynb:62)
and ships no router; in a model ``Ind[b, e, :]`` is what expert ``e`` picks from batch element ``b``.
This is the usual expert-choice rule: every expert takes the K tokens with the highest affinity, so
tokens are distinct within one ``(b, e)`` and may repeat across experts — the ``configs[0..2]`` input
distribution of the benchmark.  Plain torch (``topk`` runs on the GPU); the scores come back with the
indices so that a caller can weight the gathered rows.
"""
from __future__ import annotations

import torch


def expert_choice_router(logits: torch.Tensor, K: int, ind_dtype: torch.dtype = torch.int64):
    """logits [B, T, E] -> (Ind [B, E, K] token ids, scores [B, E, K] softmax-over-experts affinity).

    Picks are ordered by decreasing affinity; ``ind_dtype`` may be any integer type the kernels read
    (int16 as in the reference's benchmark, int32, int64, uint8) that can hold ``T - 1``."""
    if logits.dim() != 3:
        raise ValueError("logits must be [B, T, E]")
    B, T, E = logits.shape
    if not 0 < K <= T:
        raise ValueError("K must be in 1..T")
    if ind_dtype not in (torch.int16, torch.int32, torch.int64, torch.uint8):
        raise ValueError("Unknown dtype")
    if T - 1 > torch.iinfo(ind_dtype).max:
        raise ValueError(f"{ind_dtype} cannot hold token ids up to {T - 1}")
    affinity = torch.softmax(logits.float(), dim=-1).transpose(1, 2)      # [B, E, T]
    scores, ind = torch.topk(affinity, K, dim=-1)
    return ind.to(ind_dtype), scores
