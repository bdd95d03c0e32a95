"""CPU oracle for the attention column reduction.  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this module, and only as the checker.  The shipped operator
(flash_colreduce_amd.flash_colreduce) never routes through it.

It restates, independently and in fp32/fp64 on the host, what the reference
computes (citations are paths inside the reference tree):

  scores  S[i,j] = scale * <q_i, k_j>                flash_colreduce/naive.py:19
  default scale  = 1/sqrt(D)                         flash_colreduce/naive.py:16-17
  causal  mask   : key j hidden from query i iff i + max(N-M,0) < j
                                                     flash_colreduce/naive.py:20-24
                                                     flash_colreduce/flash.py:22-27
  P = softmax over keys                              flash_colreduce/naive.py:25
  sum[j]  = sum_i P[i,j]                             flash_colreduce/naive.py:27-28
  max[j]  = max_i P[i,j]                             flash_colreduce/naive.py:36-37
  mean[j] = sum[j] / cnt[j], cnt = M (non-causal, or j < c), N-j (j >= c)
                                                     flash_colreduce/naive.py:29-35
                                                     flash_colreduce/flash.py:377-384

How each function is pinned (none needs the reference to be imported):

  mean_divisor         closed form above; brute-force count of visible queries
                       for M <= N, and the as-written N-j rule for M > N
                       (tests/test_oracle.py::test_mean_divisor_*).
  visible              brute-force enumeration on tiny M,N incl. M > N
                       (test_mask_enumeration).
  colreduce_bruteforce float64 scalar loops; pinned by closed forms: q = 0 gives
                       harmonic-number column sums (golden rationals in
                       tests/golden/closed_forms.json), M = 1 gives the softmax
                       row itself, row sums add to M, torch.softmax/sum/max.
  colreduce_ref        the fast, chunked fp32 oracle used at full sizes; pinned
                       against colreduce_bruteforce, the closed forms, the
                       invariants (key-shift, permutation, D zero padding,
                       scale == prescaled q) and against an unchunked run.
  row_lse2_ref         base-2 log-sum-exp per query row; pinned by
                       2**lse == sum(2**s) and by brute force.

The reference stores no golden vectors for this path (its only test draws from
the CUDA generator and compares two implementations), so there are none to
replay; the closed forms above are what the mathematics fixes.
"""
from __future__ import annotations

import math
from typing import Optional

import numpy as np
import torch

__all__ = [
    "mean_divisor",
    "visible",
    "colreduce_bruteforce",
    "colreduce_ref",
    "row_lse2_ref",
    "topk_mask_ref",
]


def causal_offset(m: int, n: int) -> int:
    """Right-alignment offset, clamped at zero (naive.py:21, flash.py:24,202)."""
    return max(n - m, 0)


def visible(i: int, j: int, m: int, n: int, is_causal: bool) -> bool:
    """True iff key j takes part in query i's softmax (naive.py:24)."""
    if not is_causal:
        return True
    return not (i + causal_offset(m, n) < j)


def mean_divisor(m: int, n: int, is_causal: bool) -> np.ndarray:
    """Divisor the reference applies per key column for reduction='mean'.

    naive.py:29-35 / flash.py:377-384: M everywhere when not causal; when causal
    M for j < c and N-j (M, M-1, ..., 1 when M <= N) for j >= c.  For M > N the
    reference still divides by N-j; that is reproduced as written.
    """
    if not is_causal:
        return np.full(n, m, dtype=np.float64)
    c = causal_offset(m, n)
    div = np.empty(n, dtype=np.float64)
    div[:c] = m
    div[c:] = np.arange(n - c, 0, -1, dtype=np.float64)
    return div


def colreduce_bruteforce(q, k, reduction: str, is_causal: bool = False,
                         scale: Optional[float] = None) -> np.ndarray:
    """Scalar float64 loops over [B,H,M,N]; for tiny shapes only."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    b_, h_, m, d = q.shape
    n = k.shape[2]
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    if reduction not in ("sum", "mean", "max"):
        raise ValueError(f"Invalid reduction: {reduction}. Must be 'sum', 'mean', or 'max'.")
    out = np.zeros((b_, h_, n), dtype=np.float64)
    div = mean_divisor(m, n, is_causal)
    for b in range(b_):
        for h in range(h_):
            for i in range(m):
                s = [scale * float(np.dot(q[b, h, i], k[b, h, j])) if visible(i, j, m, n, is_causal)
                     else -math.inf for j in range(n)]
                top = max(s)
                e = [math.exp(x - top) if x != -math.inf else 0.0 for x in s]
                z = math.fsum(e)
                for j in range(n):
                    p = e[j] / z
                    if reduction == "max":
                        out[b, h, j] = max(out[b, h, j], p)
                    else:
                        out[b, h, j] += p
            if reduction == "mean":
                out[b, h] /= div
    return out


def _head_block(qh: torch.Tensor, kh: torch.Tensor, row0: int, m: int, n: int,
                scale: float, is_causal: bool):
    """softmax rows [row0, row0+R) of one head against the keys they can see."""
    r = qh.shape[0]
    c = causal_offset(m, n)
    nvis = min(n, row0 + r + c) if is_causal else n
    s = (qh @ kh[:nvis].T) * scale
    if is_causal:
        rows = torch.arange(row0, row0 + r).view(-1, 1)
        cols = torch.arange(nvis).view(1, -1)
        s = torch.where(cols <= rows + c, s, torch.full_like(s, -math.inf))
    return torch.softmax(s, dim=-1), nvis


def colreduce_ref(q: torch.Tensor, k: torch.Tensor, reduction: str, is_causal: bool = False,
                  scale: Optional[float] = None, chunk_rows: int = 4096,
                  compute_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """fp32 (or fp64) softmax-then-reduce on the upcast inputs, [B,H,N] in compute_dtype.

    Walks heads and blocks of query rows with *global* row indices, so the
    M x N matrix of a long head is never held at once; blocks combine by + (sum,
    mean) or max (max) and the mean divisor is applied once at the end.
    """
    if reduction not in ("sum", "mean", "max"):
        raise ValueError(f"Invalid reduction: {reduction}. Must be 'sum', 'mean', or 'max'.")
    b_, h_, m, d = q.shape
    n = k.shape[2]
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    out = torch.zeros((b_, h_, n), dtype=compute_dtype)
    for b in range(b_):
        for h in range(h_):
            qh = q[b, h].to(device="cpu", dtype=compute_dtype)
            kh = k[b, h].to(device="cpu", dtype=compute_dtype)
            col = out[b, h]
            for row0 in range(0, m, chunk_rows):
                p, nvis = _head_block(qh[row0:row0 + chunk_rows], kh, row0, m, n, scale, is_causal)
                if reduction == "max":
                    torch.maximum(col[:nvis], p.amax(dim=0), out=col[:nvis])
                else:
                    col[:nvis] += p.sum(dim=0)
    if reduction == "mean":
        out /= torch.from_numpy(mean_divisor(m, n, is_causal)).to(compute_dtype)
    return out


def row_lse2_ref(q: torch.Tensor, k: torch.Tensor, is_causal: bool = False,
                 scale: Optional[float] = None, chunk_rows: int = 4096) -> torch.Tensor:
    """Base-2 log-sum-exp of every query row: log2 sum_j 2**(scale*log2(e)*<q_i,k_j>).

    This is the quantity the device's first pass hands to its second pass
    (the reference keeps it in registers: flash.py:242, scale folded at flash.py:291).
    Returned as float64 [B,H,M].
    """
    b_, h_, m, d = q.shape
    n = k.shape[2]
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    c = causal_offset(m, n)
    out = torch.empty((b_, h_, m), dtype=torch.float64)
    for b in range(b_):
        for h in range(h_):
            qh = q[b, h].to(device="cpu", dtype=torch.float64)
            kh = k[b, h].to(device="cpu", dtype=torch.float64)
            for row0 in range(0, m, chunk_rows):
                qb = qh[row0:row0 + chunk_rows]
                s = (qb @ kh.T) * (scale * math.log2(math.e))
                if is_causal:
                    rows = torch.arange(row0, row0 + qb.shape[0]).view(-1, 1)
                    cols = torch.arange(n).view(1, -1)
                    s = s.masked_fill(cols > rows + c, -math.inf)
                out[b, h, row0:row0 + qb.shape[0]] = torch.logsumexp(s * math.log(2.0), dim=-1) / math.log(2.0)
    return out


def topk_mask_ref(scores, k: int) -> np.ndarray:
    """Keep-mask of the k largest entries of every row of a 2-D array; among equal values the lower
    column wins; a NaN ranks above +inf and NaNs tie with each other (the order torch.topk uses).
    Pinned by its defining properties (tests/test_oracle.py::test_topk_mask_ref): exactly
    min(max(k,0),N) kept, every kept value >= every dropped one, kept ties precede dropped ties; and
    against torch.topk on rows with NaNs.
    The reference has no such function; its callers do this step themselves (README.md:9)."""
    a = np.asarray(scores)
    rows, n = a.shape
    kk = min(max(int(k), 0), n)
    mask = np.zeros((rows, n), dtype=bool)
    cols = np.arange(n)
    for r in range(rows):
        v = a[r].astype(np.float64)
        nan = np.isnan(v)
        # NaNs first, then by value descending, then column ascending
        order = np.lexsort((cols, np.where(nan, 0.0, -v), ~nan))
        mask[r, order[:kk]] = True
    return mask
