"""Materialising implementation of the column reduction, in plain torch ops.

Same signature and semantics as the reference's `naive_colreduce`
(flash_colreduce/naive.py:8-40): the whole [B,H,M,N] probability matrix is built in the input
dtype on the input's device, then reduced over the query axis.  It exists for users who want the
simple form on small problems; `flash_colreduce` never calls it.
"""
from __future__ import annotations

import math
from typing import Optional

import torch

__all__ = ["naive_colreduce"]


def _visible_queries_per_key(m: int, n: int, is_causal: bool, device) -> torch.Tensor:
    """Divisor of reduction='mean' (naive.py:29-35): M, or N-j from the right-alignment offset on."""
    cnt = torch.full((n,), m, device=device, dtype=torch.int64)
    if is_causal:
        c = max(n - m, 0)
        cnt[c:] = torch.arange(n - c, 0, -1, device=device)
    return cnt


def naive_colreduce(query: torch.Tensor, key: torch.Tensor, reduction: str, is_causal: bool = False,
                    scale: Optional[float] = None) -> torch.Tensor:
    if reduction not in ("sum", "mean", "max"):
        raise ValueError(f"Invalid reduction: {reduction}. Must be 'sum', 'mean', or 'max'.")
    m, n = query.shape[2], key.shape[2]
    if scale is None:
        scale = 1 / math.sqrt(query.shape[-1])
    logits = torch.einsum("bhmd,bhnd->bhmn", query, key) * scale
    if is_causal:
        rows = torch.arange(m, device=query.device)[:, None]
        cols = torch.arange(n, device=query.device)[None, :]
        hidden = cols > rows + max(n - m, 0)
        logits = logits.masked_fill(hidden, float("-inf"))
    probs = logits.softmax(dim=-1)
    if reduction == "max":
        return probs.amax(dim=2).to(query.dtype)
    col = probs.sum(dim=2)
    if reduction == "mean":
        col = col / _visible_queries_per_key(m, n, is_causal, query.device)
    return col.to(query.dtype)
