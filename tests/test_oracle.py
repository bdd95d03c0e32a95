"""Pins the CPU oracle without importing the reference: golden closed forms,
brute force, library routines and invariants.  Each check is chosen so that a
plausible slip (wrong mask alignment, wrong divisor, transposed operand, missing
scale) fails it."""
import json
import math
import os
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle.colreduce_oracle import (colreduce_bruteforce, colreduce_ref, mean_divisor,
                                     row_lse2_ref, visible)

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "closed_forms.json")
REDUCTIONS = ["sum", "mean", "max"]


def _golden_cases():
    with open(GOLDEN) as f:
        return json.load(f)["cases"]


def _materialise(case):
    m, n, d = case["m"], case["n"], case["d"]
    g = torch.Generator().manual_seed(7)
    if case["q"] == "zeros":
        q = torch.zeros(1, 1, m, d)
    else:
        q = torch.tensor(case["q"], dtype=torch.float64).view(1, 1, m, d)
    if case["k"] == "any":
        k = torch.randn(1, 1, n, d, generator=g)
    else:
        rows = [[math.log(3.0) if v == "ln3" else v for v in row] for row in case["k"]]
        k = torch.tensor(rows, dtype=torch.float64).view(1, 1, n, d)
    return q, k


@pytest.mark.parametrize("case", _golden_cases(), ids=lambda c: c["name"])
@pytest.mark.parametrize("reduction", REDUCTIONS)
def test_golden_closed_forms(case, reduction):
    q, k = _materialise(case)
    want = np.array([float(Fraction(x)) for x in case[reduction]])
    kw = dict(is_causal=case["is_causal"], scale=case.get("scale"))
    got_bf = colreduce_bruteforce(q.numpy(), k.numpy(), reduction, **kw)[0, 0]
    np.testing.assert_allclose(got_bf, want, rtol=1e-13, atol=0)
    got64 = colreduce_ref(q, k, reduction, compute_dtype=torch.float64, **kw)[0, 0].numpy()
    np.testing.assert_allclose(got64, want, rtol=1e-13, atol=0)
    got32 = colreduce_ref(q, k, reduction, chunk_rows=2, **kw)[0, 0].numpy()
    np.testing.assert_allclose(got32, want, rtol=2e-6, atol=0)


@pytest.mark.parametrize("m,n", [(1, 1), (3, 5), (5, 5), (5, 3), (4, 9), (7, 2)])
def test_mask_enumeration(m, n):
    c = n - m if n > m else 0
    for i in range(m):
        for j in range(n):
            assert visible(i, j, m, n, False)
            assert visible(i, j, m, n, True) == (j <= i + c)
    if m <= n:  # right aligned: last query sees all keys, first sees c+1
        assert sum(visible(0, j, m, n, True) for j in range(n)) == n - m + 1
        assert all(visible(m - 1, j, m, n, True) for j in range(n))
    else:  # top-left aligned once the offset clamps
        assert sum(visible(0, j, m, n, True) for j in range(n)) == 1
        assert all(visible(i, j, m, n, True) for i in range(n - 1, m) for j in range(n))


@pytest.mark.parametrize("m,n", [(3, 5), (5, 5), (1, 4), (128, 1024)])
def test_mean_divisor_counts_visible_queries(m, n):
    cnt = [sum(visible(i, j, m, n, True) for i in range(m)) for j in range(n)]
    np.testing.assert_array_equal(mean_divisor(m, n, True), cnt)
    np.testing.assert_array_equal(mean_divisor(m, n, False), [m] * n)


def test_mean_divisor_more_queries_than_keys_is_as_written():
    # the reference divides by N-j even though M-j queries see key j
    np.testing.assert_array_equal(mean_divisor(5, 3, True), [3, 2, 1])


def _rand(b, h, m, n, d, seed=0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(b, h, m, d, generator=g).to(dtype),
            torch.randn(b, h, n, d, generator=g).to(dtype))


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("reduction", REDUCTIONS)
@pytest.mark.parametrize("m,n,d", [(5, 5, 4), (3, 9, 8), (9, 4, 3), (1, 6, 2), (6, 1, 2)])
def test_ref_matches_bruteforce(m, n, d, reduction, causal):
    q, k = _rand(2, 2, m, n, d, seed=m * 100 + n)
    want = colreduce_bruteforce(q.numpy(), k.numpy(), reduction, causal)
    got = colreduce_ref(q, k, reduction, causal, chunk_rows=4, compute_dtype=torch.float64)
    np.testing.assert_allclose(got.numpy(), want, rtol=1e-12, atol=1e-300)
    got32 = colreduce_ref(q, k, reduction, causal, chunk_rows=2)
    np.testing.assert_allclose(got32.numpy(), want, rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("reduction", REDUCTIONS)
def test_bruteforce_matches_library_softmax(reduction, causal):
    """Reduces to torch.softmax + sum/max on a materialised matrix."""
    m, n, d = 6, 10, 8
    q, k = _rand(1, 3, m, n, d, seed=3, dtype=torch.float64)
    s = torch.einsum("bhmd,bhnd->bhmn", q, k) / math.sqrt(d)
    keep = torch.tensor([[(not causal) or j <= i + (n - m) for j in range(n)] for i in range(m)])
    s = s.masked_fill(~keep, -math.inf)
    p = torch.softmax(s, -1)
    want = {"sum": p.sum(2), "max": p.amax(2), "mean": p.sum(2) / keep.sum(0)}[reduction]
    got = colreduce_bruteforce(q.numpy(), k.numpy(), reduction, causal)
    np.testing.assert_allclose(got, want.numpy(), rtol=1e-12)


@pytest.mark.parametrize("causal", [False, True])
def test_single_query_is_the_softmax_row(causal):
    q, k = _rand(1, 2, 1, 33, 16, seed=5)
    row = torch.softmax((q.double() @ k.double().transpose(-1, -2)) / 4.0, -1)[:, :, 0]
    for red in REDUCTIONS:
        got = colreduce_ref(q, k, red, causal, compute_dtype=torch.float64)
        np.testing.assert_allclose(got.numpy(), row.numpy(), rtol=1e-12)


@pytest.mark.parametrize("causal", [False, True])
def test_invariants(causal):
    b, h, m, n, d = 2, 3, 40, 56, 24
    q, k = _rand(b, h, m, n, d, seed=11)
    s = colreduce_ref(q, k, "sum", causal)
    mx = colreduce_ref(q, k, "max", causal)
    mean = colreduce_ref(q, k, "mean", causal)
    # every softmax row adds to one
    np.testing.assert_allclose(s.sum(-1).numpy(), np.full((b, h), m), rtol=1e-5)
    assert (mx > 0).all() and (mx <= 1).all()
    assert (mean <= mx * (1 + 1e-6)).all() and (mx <= s * (1 + 1e-6)).all()
    # adding one vector to every key of a head shifts each row's scores by a constant
    shift = torch.randn(b, h, 1, d, generator=torch.Generator().manual_seed(1))
    np.testing.assert_allclose(colreduce_ref(q, k + shift, "sum", causal).numpy(), s.numpy(),
                               rtol=2e-4, atol=1e-6)
    # zero padding of the head dimension changes nothing when scale is given
    qp = torch.nn.functional.pad(q, (0, 8))
    kp = torch.nn.functional.pad(k, (0, 8))
    np.testing.assert_allclose(
        colreduce_ref(qp, kp, "max", causal, scale=1 / math.sqrt(d)).numpy(), mx.numpy(), rtol=1e-6)
    # explicit scale == pre-scaled queries
    np.testing.assert_allclose(
        colreduce_ref(q * 0.25, k, "sum", causal, scale=1.0).numpy(),
        colreduce_ref(q, k, "sum", causal, scale=0.25).numpy(), rtol=1e-5, atol=1e-7)
    # (b,h) slices are independent
    np.testing.assert_array_equal(colreduce_ref(q[1:2, 2:3], k[1:2, 2:3], "sum", causal).numpy(),
                                  s[1:2, 2:3].numpy())
    if not causal:
        pk = torch.randperm(n, generator=torch.Generator().manual_seed(2))
        pq = torch.randperm(m, generator=torch.Generator().manual_seed(3))
        np.testing.assert_allclose(colreduce_ref(q[:, :, pq], k[:, :, pk], "sum").numpy(),
                                   s[:, :, pk].numpy(), rtol=1e-5, atol=1e-7)
    else:
        # only the last query sees the last key
        sc = torch.einsum("bhd,bhnd->bhn", q[:, :, -1].double(), k.double()) / math.sqrt(d)
        np.testing.assert_allclose(s[..., -1].numpy(), torch.softmax(sc, -1)[..., -1].numpy(), rtol=1e-5)


def test_chunking_is_invisible():
    q, k = _rand(1, 2, 300, 420, 32, seed=4)
    for causal in (False, True):
        for red in REDUCTIONS:
            a = colreduce_ref(q, k, red, causal, chunk_rows=64)
            b = colreduce_ref(q, k, red, causal, chunk_rows=100000)
            np.testing.assert_allclose(a.numpy(), b.numpy(), rtol=2e-5, atol=1e-8)


@pytest.mark.parametrize("causal", [False, True])
def test_row_lse2(causal):
    m, n, d = 7, 12, 5
    q, k = _rand(1, 2, m, n, d, seed=9)
    lse = row_lse2_ref(q, k, causal, chunk_rows=3)
    sc = torch.einsum("bhmd,bhnd->bhmn", q.double(), k.double()) / math.sqrt(d) * math.log2(math.e)
    for i in range(m):
        js = [j for j in range(n) if visible(i, j, m, n, causal)]
        want = torch.log2(torch.pow(2.0, sc[:, :, i, js]).sum(-1))
        np.testing.assert_allclose(lse[:, :, i].numpy(), want.numpy(), rtol=1e-12)


def test_topk_mask_ref():
    from oracle.colreduce_oracle import topk_mask_ref
    a = np.array([[0.5, 0.25, 0.5, 0.125, 0.5], [-1.0, 3.0, 0.0, -0.0, 2.0]])
    np.testing.assert_array_equal(topk_mask_ref(a, 2), [[1, 0, 1, 0, 0], [0, 1, 0, 0, 1]])
    np.testing.assert_array_equal(topk_mask_ref(a, 4), [[1, 1, 1, 0, 1], [0, 1, 1, 1, 1]])
    assert not topk_mask_ref(a, 0).any() and topk_mask_ref(a, 9).all() and not topk_mask_ref(a, -3).any()
    rng = np.random.default_rng(0)
    b = rng.integers(0, 6, size=(7, 40)).astype(np.float32)  # many ties
    for k in (1, 5, 17, 39):
        m = topk_mask_ref(b, k)
        assert (m.sum(1) == k).all()
        for r in range(7):
            kept, dropped = b[r][m[r]], b[r][~m[r]]
            assert kept.min() >= dropped.max()
            t = kept.min()
            tie_cols = np.nonzero(b[r] == t)[0]
            kept_ties = [c for c in tie_cols if m[r, c]]
            assert kept_ties == list(tie_cols[:len(kept_ties)])


def test_topk_mask_ref_with_nans():
    """NaNs rank above +inf and tie with each other: hand cases, then torch.topk (which orders NaNs the
    same way) on rows of distinct values with NaNs of both signs."""
    import torch
    from oracle.colreduce_oracle import topk_mask_ref
    nan, inf = float("nan"), float("inf")
    a = np.array([[1.0, nan, inf, -inf, nan, 2.0]])
    np.testing.assert_array_equal(topk_mask_ref(a, 1), [[0, 1, 0, 0, 0, 0]])
    np.testing.assert_array_equal(topk_mask_ref(a, 2), [[0, 1, 0, 0, 1, 0]])
    np.testing.assert_array_equal(topk_mask_ref(a, 3), [[0, 1, 1, 0, 1, 0]])
    np.testing.assert_array_equal(topk_mask_ref(a, 5), [[1, 1, 1, 0, 1, 1]])
    g = torch.Generator().manual_seed(3)
    v = torch.randperm(300, generator=g).float().view(3, 100) - 150.0    # distinct values
    v[0, [3, 50, 77]] = nan
    v[1, 9] = -nan
    v[2, 5] = inf
    v[2, 6] = nan
    for k in (1, 2, 3, 4, 10, 99):
        want = torch.zeros(3, 100, dtype=torch.bool)
        want.scatter_(1, torch.topk(v, k, dim=1).indices, True)
        if k >= 3:    # fewer than the NaNs of row 0: torch may pick any of them, the oracle the first
            np.testing.assert_array_equal(topk_mask_ref(v.numpy(), k), want.numpy())
        else:
            np.testing.assert_array_equal(topk_mask_ref(v.numpy(), k)[1:], want.numpy()[1:])


def test_bad_reduction():
    q, k = _rand(1, 1, 2, 2, 2)
    with pytest.raises(ValueError, match="Invalid reduction"):
        colreduce_ref(q, k, "median")
    with pytest.raises(ValueError, match="Invalid reduction"):
        colreduce_bruteforce(q.numpy(), k.numpy(), "median")
