"""GPU parity: libfcr (through flash_colreduce / the C ABI) against the CPU oracle on the same
seeded inputs.  Tolerances are those of the headline metric: rtol 2e-3 / atol 1e-5 for sum and mean,
2e-3 relative for max, checked on the kernel's fp32 result."""
import math

import pytest
import torch

import flash_colreduce_amd as fca
from oracle.colreduce_oracle import colreduce_ref, row_lse2_ref
from tests import _inputs

pytestmark = pytest.mark.gpu
REDUCTIONS = ["sum", "mean", "max"]


def check(got: torch.Tensor, want: torch.Tensor, reduction: str, what=""):
    got = got.detach().float().cpu()
    want = want.float()
    assert got.shape == want.shape, (got.shape, want.shape)
    assert torch.isfinite(got).all(), what
    if reduction == "max":
        rel = ((got - want).abs() / want.abs().clamp_min(1e-30)).max().item()
        assert rel <= 2e-3, f"{what} max: relative error {rel:.3e}"
    else:
        torch.testing.assert_close(got, want, rtol=2e-3, atol=1e-5, msg=lambda m: f"{what} {reduction}: {m}")


def run_all(q, k, causal, scale=None, what="", reductions=REDUCTIONS, chunk_rows=4096):
    qd, kd = q.cuda(), k.cuda()
    for red in reductions:
        got = fca.flash_colreduce(qd, kd, red, is_causal=causal, scale=scale, out_dtype=torch.float32)
        want = colreduce_ref(q, k, red, causal, scale=scale, chunk_rows=chunk_rows)
        check(got, want, red, f"{what} causal={causal}")


# --- the reference's own grid (tests/test_correctness.py:8-13), all fp16 ----------------------
@pytest.mark.parametrize("is_causal", [False, True])
@pytest.mark.parametrize("d", [16, 32, 64, 48, 72])
@pytest.mark.parametrize("m,n", [(128, 128), (131, 131), (128, 1024), (131, 1027)])
@pytest.mark.parametrize("h", [8, 13])
@pytest.mark.parametrize("b", [1, 4, 7])
def test_reference_grid(b, h, m, n, d, is_causal):
    q, k = _inputs.randn_pair(b, h, m, n, d, seed=0)
    run_all(q, k, is_causal, what=f"b{b} h{h} m{m} n{n} d{d}")


@pytest.mark.parametrize("is_causal", [False, True])
@pytest.mark.parametrize("reduction", REDUCTIONS)
@pytest.mark.parametrize("m,n,d", [(128, 128, 64), (131, 1027, 72), (128, 1024, 48)])
def test_reference_tolerance_on_native_dtype(m, n, d, reduction, is_causal):
    """The reference's assertion as written (tests/test_correctness.py:29-32): fp16 result against
    the materialising implementation run in fp16 on the same device, atol = rtol = 1e-3."""
    q, k = _inputs.randn_pair(4, 8, m, n, d, seed=0)
    q, k = q.cuda(), k.cuda()
    output = fca.flash_colreduce(q, k, reduction=reduction, is_causal=is_causal)
    target = fca.naive_colreduce(q, k, reduction=reduction, is_causal=is_causal)
    assert output.dtype == torch.float16 and output.shape == (4, 8, n)
    torch.testing.assert_close(output, target, atol=1e-3, rtol=1e-3)


# --- the benchmark set's five configurations ---------------------------------------------------------------
def test_config1_rounded_to_fp16():
    """Config 1 is the fp32 CPU case; the device path takes 16-bit inputs, so the kernel is fed
    the fp16 rounding of the same tensors and compared with the oracle on those."""
    q, k = _inputs.config1()
    run_all(q.half(), k.half(), False, what="config1")


def test_config1_fp32():
    """Config 1 as given: fp32 operands, multiplied on the fp32 matrix instructions.  The device result
    is good far beyond the metric's tolerance; 1e-5 would fail with any 16-bit rounding of the operands."""
    q, k = _inputs.config1()
    qd, kd = q.cuda(), k.cuda()
    for red in REDUCTIONS:
        got = fca.flash_colreduce(qd, kd, red)
        assert got.dtype == torch.float32 and got.shape == (1, 2, 256)
        want = colreduce_ref(q, k, red, compute_dtype=torch.float64).float()
        check(got, want, red, "config1 fp32")
        torch.testing.assert_close(got.cpu(), want, rtol=1e-5, atol=1e-8)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("m,n,d", [(100, 260, 20), (257, 300, 80), (64, 500, 128), (300, 300, 100), (33, 700, 6),
                                   (130, 140, 200), (300, 420, 132), (64, 1000, 256), (257, 129, 252),
                                   (40, 3000, 160)])
def test_fp32_operands(m, n, d, causal):
    """fp32 inputs are multiplied in fp32 for every D up to 256: held to 1e-5, which no 16-bit rounding of
    the operands meets (D = 6 is zero padded to 8; rows of more than 512 bytes take the 1 KiB ring)."""
    q, k = _inputs.randn_pair(2, 2, m, n, d, seed=d, dtype=torch.float32)
    qd, kd = q.cuda(), k.cuda()
    for red in REDUCTIONS:
        got = fca.flash_colreduce(qd, kd, red, is_causal=causal, scale=0.11)
        want = colreduce_ref(q, k, red, causal, scale=0.11, compute_dtype=torch.float64).float()
        assert got.dtype == torch.float32
        check(got, want, red, f"fp32 d{d}")
        torch.testing.assert_close(got.cpu(), want, rtol=1e-5, atol=1e-8)


@pytest.mark.parametrize("terms,d,rtol", [(3, 80, 2e-5), (3, 20, 2e-5), (1, 200, 5e-3)])
def test_fp32_operands_packed_for_the_16_bit_matrix_instructions(terms, d, rtol):
    """fcr_pack_f32 + FCR_DTYPE_F16 through the C ABI: the faster, less exact way to feed fp32 operands
    (three fp16 segments give products to about 2^-22, one segment is a single rounding to fp16)."""
    from flash_colreduce_amd import _lib, flash as F
    b, h, m, n = 2, 2, 130, 700
    q, k = _inputs.randn_pair(b, h, m, n, d, seed=terms + d, dtype=torch.float32)
    qp, kp = F.pack_f32(q.cuda(), False, terms), F.pack_f32(k.cuda(), True, terms)
    lib = _lib.load()
    out = torch.empty(b * h, n, device="cuda")
    lse = torch.empty(lib.fcr_lse_bytes(b, h, m, n, qp.shape[3]) // 4, device="cuda")
    _lib.check(lib.fcr_colreduce(qp.data_ptr(), kp.data_ptr(), out.data_ptr(), lse.data_ptr(), _lib.DTYPE_F16, b, h, m, n,
                                 qp.shape[3], _lib.strides4(qp.stride()), _lib.strides4(kp.stride()), 0.11,
                                 _lib.REDUCE_SUM, 1, torch.cuda.current_stream().cuda_stream))
    want = colreduce_ref(q, k, "sum", True, scale=0.11, compute_dtype=torch.float64).float()
    torch.testing.assert_close(out.view(b, h, n).cpu(), want, rtol=rtol, atol=1e-7)


@pytest.mark.parametrize("d", [64, 192])
def test_fp32_operands_beyond_the_fp16_range(d):
    """fp32 keeps its range: queries of magnitude 3e5 (an fp16 rounding would give inf and NaN results)
    with a scale that brings the scores back to order one, and keys of magnitude 1e-7."""
    b, h, m, n = 1, 3, 200, 333
    q, k = _inputs.randn_pair(b, h, m, n, d, seed=77, dtype=torch.float32)
    for fq, fk in ((3e5, 1.0), (1.0, 1e-7), (2e4, 2e4)):
        qq, kk = q * fq, k * fk
        scale = 0.125 / (fq * fk)
        for red, causal in (("sum", True), ("max", False), ("mean", True)):
            got = fca.flash_colreduce(qq.cuda(), kk.cuda(), red, is_causal=causal, scale=scale)
            want = colreduce_ref(qq, kk, red, causal, scale=scale, compute_dtype=torch.float64).float()
            check(got, want, red, f"fp32 range {fq} {fk}")


def test_config2():
    q, k = _inputs.config2()
    run_all(q, k, False, what="config2")


def test_config3():
    q, k = _inputs.config3()
    run_all(q, k, True, what="config3")


def _full_size(q, k, reductions, oracle_heads, what):
    """Full-size run: every head on the GPU, the oracle on a few heads, and properties that
    hold at any size on all heads (rows of a softmax add to one; 0 < max <= 1; mean <= max)."""
    m, n = q.shape[2], k.shape[2]
    qd, kd = q.cuda(), k.cuda()
    outs = {r: fca.flash_colreduce(qd, kd, r, is_causal=True, out_dtype=torch.float32) for r in reductions}
    for r, got in outs.items():
        want = colreduce_ref(q[:, oracle_heads], k[:, oracle_heads], r, True)
        check(got[:, oracle_heads], want, r, f"{what} heads {oracle_heads}")
    if "sum" in outs or "mean" in outs:
        if "sum" in outs:
            s = outs["sum"].double()
        else:
            cnt = torch.arange(n, 0, -1, device="cuda", dtype=torch.float64) if m == n else None
            s = outs["mean"].double() * cnt
        total = s.sum(-1).cpu()
        torch.testing.assert_close(total, torch.full_like(total, float(m)), rtol=1e-4, atol=0)
    if "max" in outs:
        mx = outs["max"]
        assert (mx > 0).all() and (mx <= 1 + 1e-6).all()
        # causal, M == N: only the last query sees the last key, so max == sum == mean there
        if "mean" in outs:
            assert (outs["mean"] <= mx * (1 + 1e-5)).all()
            torch.testing.assert_close(outs["mean"][..., -1], mx[..., -1], rtol=1e-5, atol=0)


def test_config4_full_size():
    q, k = _inputs.config4()
    _full_size(q, k, ["sum"], [0, 10, 21, 31], "config4")


def test_config5_full_size():
    q, k = _inputs.config5()
    _full_size(q, k, ["mean", "max"], [0, 9, 17, 31], "config5")


def test_headline_shape_fp16():
    q, k = _inputs.headline()
    _full_size(q, k, ["sum"], [0, 5, 18, 31], "headline")


# --- beyond the reference's grid ----------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("m,n,d", [
    (1, 1, 8), (1, 77, 16), (77, 1, 24), (2, 300, 128), (300, 2, 128), (257, 255, 128),
    (64, 64, 128), (513, 513, 96), (1000, 40, 40), (40, 1000, 20), (333, 777, 104), (700, 300, 56),
])
def test_ragged_shapes(m, n, d, causal, dtype):
    """M > N (offset clamps to 0), single rows/columns, D that needs zero padding, both dtypes."""
    q, k = _inputs.randn_pair(2, 3, m, n, d, seed=m * 7 + n, dtype=dtype)
    run_all(q, k, causal, what=f"m{m} n{n} d{d} {dtype}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("m,n,d", [(300, 420, 136), (257, 129, 192), (130, 1000, 256), (64, 64, 200),
                                   (1, 700, 250), (520, 520, 144)])
def test_head_dims_above_128(m, n, d, causal, dtype):
    """D in (128, 256]: one resident 32-row block per wave, 128-row tiles."""
    q, k = _inputs.randn_pair(1, 3, m, n, d, seed=d + m, dtype=dtype)
    run_all(q, k, causal, what=f"m{m} n{n} d{d} {dtype}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("m,n,d", [(300, 420, 264), (257, 129, 320), (130, 1000, 512), (64, 64, 400),
                                   (1, 700, 500), (520, 520, 384), (40, 3000, 512), (200, 200, 257), (90, 300, 449)])
def test_head_dims_above_256(m, n, d, causal, dtype):
    """D in (256, 512] for 16-bit elements: rows of up to 1 KiB, 9 to 16 k-steps, one workgroup per CU
    (the reference pads such a D to 512 and runs it when it fits, flash.py:368-373); every k-step count,
    D that is no multiple of 8 (padded by the host), few queries against many keys (split row sweep)."""
    q, k = _inputs.randn_pair(1, 3, m, n, d, seed=d + m, dtype=dtype)
    run_all(q, k, causal, what=f"m{m} n{n} d{d} {dtype}")


def test_every_k_step_count_of_long_16_bit_rows():
    for d in range(264, 513, 32):     # 264, 296, ..: 9 to 16 k-steps of 32 elements
        q, k = _inputs.randn_pair(2, 2, 150, 333, d, seed=d)
        run_all(q.half(), k.half(), True, what=f"d{d}")


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("b,h,m,n,d", [(1, 4, 40, 5000, 64), (1, 32, 128, 4096, 128), (1, 1, 300, 3001, 128),
                                       (2, 3, 1, 2048, 32), (1, 2, 257, 1100, 72)])
def test_few_queries_many_keys(b, h, m, n, d, causal):
    """Shapes where the row kernel splits the keys of a tile over several workgroups and a second
    small kernel merges the partial log-sum-exps."""
    q, k = _inputs.randn_pair(b, h, m, n, d, seed=n + m)
    qd, kd = q.cuda(), k.cuda()
    got = fca.row_lse2(qd, kd, is_causal=causal).double().cpu()
    torch.testing.assert_close(got, row_lse2_ref(q, k, causal), rtol=0, atol=3e-4)
    run_all(q, k, causal, what=f"split b{b} h{h} m{m} n{n} d{d}")


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("b,h,m,n,d", [
    (103, 10, 32, 40, 8),      # one tile per (b,h): 1030 pairs, more than one launch group either way
    (5, 68, 700, 520, 16),     # three row tiles, 340 pairs: last group is partial
    (5, 8, 64, 4096, 32),      # split keys, 40 pairs in groups of 16 without the mask
    (3, 23, 520, 300, 8),      # 69 pairs, not a multiple of 8
])
def test_many_heads_in_launch_groups(b, h, m, n, d, causal):
    """(b,h) pairs are launched in groups; cover more pairs than one group holds, partial last groups
    and pair counts that are not multiples of 8, for both kernels and the split-key row sweep."""
    q, k = _inputs.randn_pair(b, h, m, n, d, seed=b * h + m)
    run_all(q, k, causal, what=f"groups b{b} h{h} m{m} n{n} d{d}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("m,n,d", [
    (1, 1, 8), (1, 4100, 128), (16, 64, 64), (17, 65, 72), (63, 200, 128), (64, 1100, 128), (64, 10, 32),
    (33, 4097, 96), (64, 6000, 128), (8, 2048, 16), (64, 129, 136),
])
def test_at_most_64_queries(m, n, d, causal, dtype):
    """Few query rows against few or many keys: the row sweep keeps one 32-row block per wave and the
    waves without any query only help staging; the causal diagonal is the last M keys.  Also the fused
    sum+max form."""
    q, k = _inputs.randn_pair(2, 5, m, n, d, seed=m + 3 * n + d, dtype=dtype)
    run_all(q, k, causal, what=f"small m{m} n{n} d{d} {dtype}")
    got = fca.flash_colreduce_multi(q.cuda(), k.cuda(), ("sum", "max"), is_causal=causal, out_dtype=torch.float32)
    check(got[0], colreduce_ref(q, k, "sum", causal), "sum", f"small fused m{m} n{n} d{d}")
    check(got[1], colreduce_ref(q, k, "max", causal), "max", f"small fused m{m} n{n} d{d}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("b,h,m,n,d", [
    (4, 16, 64, 4100, 128),    # 64 pairs x 4 key ranges
    (2, 130, 33, 1030, 64),    # one range per pair, a ragged last chunk, padded query groups
    (4, 40, 1, 2048, 16),      # a single query
    (6, 50, 64, 1100, 72),     # D not a multiple of 32
    (1, 8, 17, 40000, 32),     # many ranges per pair
    (4, 16, 128, 4100, 128),   # eight resident query groups
    (4, 70, 97, 1030, 48),     # eight groups, the last two partly / wholly padding
])
def test_few_queries_with_streamed_keys(b, h, m, n, d, causal, dtype):
    """At most 128 queries, D <= 128 and enough (b,h) pairs x keys to fill the chip: the column
    sweep with the queries resident in every wave and the keys streamed in ranges; sum, mean, max and
    the fused sum+max form.  With the mask the diagonal is the last M keys."""
    q, k = _inputs.randn_pair(b, h, m, n, d, seed=b * h + m + n, dtype=dtype)
    run_all(q, k, causal, what=f"streamed keys b{b} h{h} m{m} n{n} d{d} {dtype}")
    got = fca.flash_colreduce_multi(q.cuda(), k.cuda(), ("sum", "max"), is_causal=causal, out_dtype=torch.float32)
    check(got[0], colreduce_ref(q, k, "sum", causal), "sum", "streamed keys fused")
    check(got[1], colreduce_ref(q, k, "max", causal), "max", "streamed keys fused")


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("b,h,m,n,d", [
    (1, 32, 2048, 2048, 128),   # 256 workgroups of 256 rows either way: both sweeps take 128-row tiles
    (4, 16, 300, 1100, 64),     # only the column sweep is in that range
    (2, 8, 8192, 520, 32),      # only the row sweep is; M > N
    (1, 16, 8192, 8192, 16),    # exactly two per CU: finer tiles with the mask only
    (1, 32, 512, 2880, 128),    # 384 column workgroups of 256 keys: finer tiles without the mask too
])
def test_between_one_and_two_workgroups_per_cu(b, h, m, n, d, causal):
    """Launches that would put between one and two 256-row workgroups on a CU use 128-row tiles (at
    exactly one or two per CU depending on the sweep and the mask)."""
    q, k = _inputs.randn_pair(b, h, m, n, d, seed=m + n + d)
    run_all(q, k, causal, what=f"finer tiles b{b} h{h} m{m} n{n} d{d}", reductions=("sum", "max"))


@pytest.mark.parametrize("m", [100, 128, 300, 384, 600])
def test_row_sweep_block_choice(m):
    """Query counts for which the row sweep keeps one 32-row block per wave (M <= 128 and ragged M
    such as 300, 384, 600) next to ones that keep two; the last tile has waves without any query."""
    q, k = _inputs.randn_pair(1, 6, m, 1500, 128, seed=m)
    for causal in (False, True):
        got = fca.row_lse2(q.cuda(), k.cuda(), is_causal=causal).double().cpu()
        torch.testing.assert_close(got, row_lse2_ref(q, k, causal), rtol=0, atol=3e-4)
        run_all(q, k, causal, what=f"row blocks m{m}", reductions=("sum",))


def test_key_operand_beyond_4_gib():
    """One head whose keys take more than 4 GiB: row offsets inside an operand exceed 32 bits and the
    buffer views are clamped; the last columns lie past that mark.  Relative check only (the sums are
    far below the absolute tolerance)."""
    n, d = (1 << 24) + 77, 128
    g = torch.Generator(device="cuda").manual_seed(3)
    k = torch.randn(1, 1, n, d, device="cuda", dtype=torch.float16, generator=g)
    q = torch.randn(1, 1, 4, d, device="cuda", dtype=torch.float16, generator=g)
    qc, kc = q.cpu(), k.cpu()
    for causal in (False, True):
        got_s, got_m = fca.flash_colreduce_multi(q, k, ("sum", "max"), is_causal=causal, out_dtype=torch.float32)
        for got, red in ((got_s, "sum"), (got_m, "max")):
            want = colreduce_ref(qc, kc, red, causal, chunk_rows=16)
            torch.testing.assert_close(got.cpu(), want, rtol=2e-3, atol=0, msg=lambda m: f"{red} causal={causal}: {m}")


# --- the single sweep for few queries against many keys (keys read once) -------------------------------------
def _c_abi_colreduce(q, k, red, causal, scale=None):
    """fcr_colreduce through ctypes on device tensors; returns (out [B,H,N] fp32, lse [B,H,M] fp32, status)."""
    from flash_colreduce_amd import _lib
    lib = _lib.load()
    b, h, m, d = q.shape
    n = k.shape[2]
    out = torch.empty(b * h, n, device="cuda")
    lse = torch.empty(lib.fcr_lse_bytes(b, h, m, n, d) // 4, device="cuda")
    dt = {torch.float16: _lib.DTYPE_F16, torch.bfloat16: _lib.DTYPE_BF16}[q.dtype]
    _lib.check(lib.fcr_colreduce(q.data_ptr(), k.data_ptr(), out.data_ptr(), lse.data_ptr(), dt, b, h, m, n, d,
                                 _lib.strides4(q.stride()), _lib.strides4(k.stride()),
                                 float(scale if scale is not None else 1 / math.sqrt(d)),
                                 _lib.REDUCE_MAX if red == "max" else _lib.REDUCE_SUM, int(causal), None))
    status = lib.fcr_colreduce_status(lse.data_ptr(), dt, b, h, m, n, d, None)
    return out.view(b, h, n), lse[: b * h * m].view(b, h, m), status


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("b,h,m,n,d", [
    (1, 2, 64, 1024, 128),     # the smallest problem that takes the single sweep: one workgroup per pair
    (1, 3, 64, 16384, 128),    # teams of 16 workgroups
    (2, 3, 128, 4096, 128),    # two query halves, teams of 8
    (3, 5, 40, 3001, 64),      # ragged queries and keys, a partial last chunk
    (1, 2, 100, 5000, 72),     # two halves, the second ragged; D not a multiple of 32
    (2, 7, 17, 2100, 16),      # rows of 32 bytes
    (1, 1, 1, 70000, 128),     # one query, 69 workgroups on one pair
    (40, 16, 64, 2048, 32),    # 640 pairs for 128 teams: five rounds per workgroup
    (40, 16, 16, 8192, 64),    # at most 32 queries: two groups of queries per wave, 2048 keys per workgroup and pair
    (8, 32, 32, 8192, 128),    # the same with all 32 rows
    (64, 8, 7, 4100, 128),     # a ragged third workgroup
    (300, 4, 9, 1500, 32),     # a single workgroup per pair sweeping less than its share
    (3, 5, 20, 9000, 72),      # ragged everything
])
def test_single_sweep(b, h, m, n, d, causal, dtype):
    """At most 128 queries against at least 1024 keys: one sweep over the keys computes the row statistics
    and the columns (col_fused_kernel).  Sum, mean and max against the oracle through the operator; the
    row statistics and the status word through the C ABI; and the two-kernel path on the same inputs."""
    from flash_colreduce_amd import _lib
    q, k = _inputs.randn_pair(b, h, m, n, d, seed=b + h + m + n, dtype=dtype)
    qd, kd = q.cuda(), k.cuda()
    what = f"single sweep b{b} h{h} m{m} n{n} d{d} {dtype}"
    run_all(q, k, causal, what=what)
    got, lse, status = _c_abi_colreduce(qd, kd, "sum", causal)
    assert status == 0
    torch.testing.assert_close(lse.double().cpu(), row_lse2_ref(q, k, causal), rtol=0, atol=3e-4)
    lib = _lib.load()
    lib.fcr_set_option(_lib.OPT_SINGLE_SWEEP, 0)
    try:
        two, lse2, _ = _c_abi_colreduce(qd, kd, "sum", causal)
    finally:
        lib.fcr_set_option(_lib.OPT_SINGLE_SWEEP, 1)
    torch.testing.assert_close(got, two, rtol=2e-5, atol=1e-7)
    torch.testing.assert_close(lse, lse2, rtol=0, atol=2e-5)
    assert torch.equal(got, _c_abi_colreduce(qd, kd, "sum", causal)[0])   # no atomic adds: repeatable bit for bit
    # sums and maxima from the same single sweep (fcr_colreduce_sum_max)
    both_sum, both_max = fca.flash_colreduce_multi(qd, kd, ["sum", "max"], is_causal=causal, out_dtype=torch.float32)
    check(both_sum.cpu(), colreduce_ref(q, k, "sum", causal), "sum", what + " both")
    check(both_max.cpu(), colreduce_ref(q, k, "max", causal), "max", what + " both")
    torch.testing.assert_close(both_sum, got, rtol=2e-5, atol=1e-7)
    # (the team's partial values are merged by half as many waves, in another order: equal to rounding)
    torch.testing.assert_close(both_max.view(b, h, n), _c_abi_colreduce(qd, kd, "max", causal)[0], rtol=2e-5, atol=0)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("m", [64, 128])
def test_single_sweep_scores_far_from_zero(m, causal):
    """Row sums of 2^score that overflow or vanish in fp32 (an enormous aligned key late in the sweep, rows
    whose scores are all around -190, unscaled scores): the workgroup sweeps its keys a second time keeping
    the scores and reduces them maximum first."""
    b, h, n, d = 1, 3, 4096, 64
    q, k = _inputs.randn_pair(b, h, m, n, d, seed=9)
    q, k = q.float(), k.float()
    k[:, 0, 3000] = 40.0 * q[:, 0, 50]
    k[:, 0, 3001] = -40.0 * q[:, 0, 50]
    k[:, 1] = -3.0 * q[:, 1, :1] + 0.1 * k[:, 1]
    k[:, 1, 3500:] *= 0.0
    for scale in (None, 1.0):
        run_all(q.half(), k.half(), causal, scale=scale, what=f"single sweep, far scores, m{m} scale={scale}")


@pytest.mark.parametrize("causal", [False, True])
def test_single_sweep_nan_and_inf_inputs(causal):
    """As test_nan_and_inf_inputs, on a shape that takes the single sweep: NaN rows make the columns they
    see NaN and leave the others alone; the maxima are compared where no NaN row looks."""
    b, h, m, n, d = 1, 4, 100, 2600, 64
    q, k = _inputs.randn_pair(b, h, m, n, d, seed=56)
    q, k = q.clone(), k.clone()
    q[0, 0, 70, 5] = float("nan")
    q[0, 1, 20, 3] = float("inf")
    k[0, 2, 1000, 7] = float("-inf")
    c = max(n - m, 0)
    scores = torch.einsum("bhmd,bhnd->bhmn", q.float(), k.float())
    vis = (torch.arange(m)[:, None] + c >= torch.arange(n)[None, :]) if causal else torch.ones(m, n, dtype=torch.bool)
    bad = ((torch.isnan(scores) | (scores == float("inf"))) & vis).any(-1)
    assert bad[0, 0].sum() == 1 and bad[0, 1].sum() == 1 and bad[0, 2].sum() > 10 and not bad[0, 3].any()
    nan_cols = (bad[..., None] & vis).any(-2)
    q_clean = torch.where(bad[..., None], torch.zeros_like(q), q)
    k_clean = torch.nan_to_num(k, neginf=0.0)
    qd, kd = q.cuda(), k.cuda()
    for red in REDUCTIONS:
        got = fca.flash_colreduce(qd, kd, red, is_causal=causal, out_dtype=torch.float32).cpu()
        want = colreduce_ref(q_clean, k_clean, red, causal)
        if red != "max":
            assert torch.equal(torch.isnan(got), nan_cols), red
        ok = ~nan_cols
        ok[0, 2] = False
        if causal:
            assert ok[0, 0].any() and ok[0, 1].any()
        check(got[ok], want[ok], red, f"single sweep, columns no NaN row sees, causal={causal}")


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("m", [3, 20, 40, 100])
def test_single_sweep_rows_of_padding_meet_a_non_finite_key(m, causal):
    """Fewer queries than a workgroup holds rows for: the rows of padding are rows of zeros, which the fast form
    of the sweep leaves in place.  A key with an infinite element turns their scores into NaN (0 * inf); the
    sweep notices and hides them the slow way.  Here every real query is positive where the key is -inf, so
    the key's scores are -inf, its column is exactly 0 and every other column is untouched."""
    b, h, n, d = 2, 3, 3000, 64
    q, k = _inputs.randn_pair(b, h, m, n, d, seed=91 + m)
    q, k = q.half().clone(), k.half().clone()
    q[..., 7] = q[..., 7].abs() + 0.5
    k[0, 1, 1234, 7] = float("-inf")
    k[1, 2, n - 1, 7] = float("-inf")
    for red in REDUCTIONS:
        got = fca.flash_colreduce(q.cuda(), k.cuda(), red, is_causal=causal, out_dtype=torch.float32).cpu()
        assert not torch.isnan(got).any(), red
        assert got[0, 1, 1234] == 0 and got[1, 2, n - 1] == 0
        check(got, colreduce_ref(q, k, red, causal), red, f"padding rows m{m} {red}")


def test_single_sweep_bounded_wait():
    """The wait for the team is bounded from the host: with a limit of zero polls a workgroup whose partners
    have not all published gives up at once, stores NaN for its columns of that pair, sets the status word
    and goes on; every workgroup ends normally.  What is not NaN is right, the status says whether anything
    is, and the next call with the usual limit is clean."""
    from flash_colreduce_amd import _lib
    lib = _lib.load()
    b, h, m, n, d = 4, 16, 64, 8192, 64
    q, k = _inputs.randn_pair(b, h, m, n, d, seed=5)
    qd, kd = q.cuda(), k.cuda()
    want = colreduce_ref(q, k, "sum", True)
    assert lib.fcr_set_option(_lib.OPT_WAIT_POLLS, 0) == 0
    try:
        got, _, status = _c_abi_colreduce(qd, kd, "sum", True)
    finally:
        assert lib.fcr_set_option(_lib.OPT_WAIT_POLLS, 1 << 20) == 0
    got = got.cpu()
    gave_up = torch.isnan(got)
    assert status == (_lib.E_WAIT if gave_up.any() else 0), (status, int(gave_up.sum()))
    if status:
        assert b"gave up waiting" in lib.fcr_last_error()
    torch.testing.assert_close(got[~gave_up], want[~gave_up], rtol=2e-3, atol=1e-5)
    got, _, status = _c_abi_colreduce(qd, kd, "sum", True)
    assert status == 0
    check(got, want, "sum", "after the limit is restored")
    assert lib.fcr_set_option(7, 1) == -3 and lib.fcr_set_option(_lib.OPT_WAIT_POLLS, -1) == -3


def test_single_sweeps_on_two_streams_are_chained():
    """A single sweep expects the whole chip (its workgroups wait for each other), so the library chains the
    single sweeps that a process issues on different streams with an event: calls issued alternately on two
    streams, with no host synchronisation between them, all give the results of the calls made alone."""
    qa, ka = _inputs.randn_pair(2, 8, 64, 8192, 128, seed=5, dtype=torch.float16)
    qb, kb = _inputs.randn_pair(1, 16, 128, 4096, 64, seed=6, dtype=torch.bfloat16)
    qa, ka, qb, kb = qa.cuda(), ka.cuda(), qb.cuda(), kb.cuda()
    want_a = fca.flash_colreduce(qa, ka, "sum", is_causal=True)
    want_b = fca.flash_colreduce(qb, kb, "max", is_causal=False)
    check(want_a.float().cpu(), colreduce_ref(qa.cpu(), ka.cpu(), "sum", True), "sum", "alone")
    sa, sb = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    got = []
    for _ in range(25):
        with torch.cuda.stream(sa):
            got.append((want_a, fca.flash_colreduce(qa, ka, "sum", is_causal=True)))
        with torch.cuda.stream(sb):
            got.append((want_b, fca.flash_colreduce(qb, kb, "max", is_causal=False)))
    torch.cuda.synchronize()
    for want, out in got:
        assert torch.equal(out, want)


def test_single_sweep_under_graph_capture():
    """The single sweep (a small kernel that clears the slots, then the sweep) captured and replayed."""
    b, h, m, n, d = 2, 8, 64, 4096, 128
    qs = torch.zeros(b, h, m, d, device="cuda", dtype=torch.float16)
    ks = torch.zeros(b, h, n, d, device="cuda", dtype=torch.float16)
    q0, k0 = _inputs.randn_pair(b, h, m, n, d, seed=31)
    qs.copy_(q0)
    ks.copy_(k0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fca.flash_colreduce(qs, ks, "mean", True, out_dtype=torch.float32)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = fca.flash_colreduce(qs, ks, "mean", True, out_dtype=torch.float32)
    for seed in (32, 33, 34):
        q1, k1 = _inputs.randn_pair(b, h, m, n, d, seed=seed)
        qs.copy_(q1)
        ks.copy_(k1)
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        eager = fca.flash_colreduce(qs, ks, "mean", True, out_dtype=torch.float32)
        torch.cuda.synchronize()
        assert torch.equal(got, eager), seed
        check(got, colreduce_ref(q1, k1, "mean", True), "mean", f"single sweep, graph replay seed {seed}")


@pytest.mark.parametrize("causal", [False, True])
def test_explicit_and_negative_scale(causal):
    q, k = _inputs.randn_pair(1, 4, 200, 333, 64, seed=21)
    for scale in (0.05, 1.0 / 3.0, -0.125, 0.0):
        run_all(q, k, causal, scale=scale, what=f"scale={scale}")


@pytest.mark.parametrize("causal", [False, True])
def test_strided_inputs(causal):
    """[B,M,H,D] storage viewed as [B,H,M,D], a slice with a storage offset, and a layout that
    forces a copy (d stride 2)."""
    g = torch.Generator().manual_seed(5)
    b, h, m, n, d = 2, 5, 150, 290, 64
    q_store = torch.randn(b, m, h, d, generator=g).half()
    k_store = torch.randn(b, n + 16, h, 2 * d, generator=g).half()
    q = q_store.permute(0, 2, 1, 3)
    k = k_store.permute(0, 2, 1, 3)[:, :, 8:8 + n, d:]
    assert not q.is_contiguous() and not k.is_contiguous()
    run_all(q, k, causal, what="permuted+sliced")
    k2 = torch.randn(b, h, n, 2 * d, generator=g).half()[..., ::2]
    assert k2.stride(3) == 2
    run_all(q, k2, causal, what="d-stride 2")
    # contiguous but starting 2 bytes off a 16-byte boundary
    flat = torch.randn(b * h * n * d + 1, generator=g).half().cuda()
    k3 = flat[1:].view(b, h, n, d)
    assert k3.is_contiguous() and k3.data_ptr() % 16 != 0
    got = fca.flash_colreduce(q.cuda(), k3, "sum", is_causal=causal, out_dtype=torch.float32)
    check(got, colreduce_ref(q, k3.cpu(), "sum", causal), "sum", "misaligned base")


@pytest.mark.parametrize("causal", [False, True])
def test_expanded_operands(causal):
    """Operands whose rows overlap in memory (expand() gives a row stride of 0): the library's buffer
    views cannot describe them, so the host copies; one query repeated M times, one key repeated N
    times, and a batch/head broadcast (stride 0 on those dimensions is addressed directly)."""
    b, h, m, n, d = 2, 3, 70, 200, 64
    q, k = _inputs.randn_pair(b, h, m, n, d, seed=61)
    qd, kd = q.cuda(), k.cuda()

    def run(qx, kx, what):  # expanded on the device: a host-to-device copy would make them dense
        assert qx.is_cuda and kx.is_cuda
        for red in REDUCTIONS:
            got = fca.flash_colreduce(qx, kx, red, is_causal=causal, out_dtype=torch.float32)
            check(got, colreduce_ref(qx.cpu(), kx.cpu(), red, causal), red, what)

    q1 = qd[:, :, :1].expand(b, h, m, d)
    assert q1.stride(2) == 0
    run(q1, kd, "expanded query rows")
    k1 = kd[:, :, 3:4].expand(b, h, n, d)
    run(qd, k1, "expanded key rows")
    kb = kd[:1, :1].expand(b, h, n, d)
    assert kb.stride(0) == 0 and kb.stride(1) == 0
    run(qd, kb, "key broadcast over batch and heads")
    # through the C ABI the overlapping rows are rejected, not misread
    from flash_colreduce_amd import _lib
    lib = _lib.load()
    out = torch.empty(b * h, n, device="cuda")
    lse = torch.empty(lib.fcr_lse_bytes(b, h, m, n, d) // 4, device="cuda")
    rc = lib.fcr_colreduce(q1.data_ptr(), kd.data_ptr(), out.data_ptr(), lse.data_ptr(), _lib.DTYPE_F16, b, h, m, n, d,
                           _lib.strides4(q1.stride()), _lib.strides4(kd.stride()), 0.125, 0, int(causal), None)
    assert rc == -4 and b"row stride" in lib.fcr_last_error()


@pytest.mark.parametrize("causal", [False, True])
def test_single_row_with_any_row_stride(causal):
    """One query row or one key row whose row stride is smaller than D (a slice of an expanded tensor keeps
    stride 0; torch reports arbitrary strides for dimensions of size one): the stride of a single row is
    never used, through the operator and through the C ABI alike."""
    from flash_colreduce_amd import _lib
    b, h, d = 2, 3, 64
    q, k = _inputs.randn_pair(b, h, 40, 700, d, seed=77)
    qd, kd = q.cuda(), k.cuda()
    q1 = qd[:, :, 7:8].expand(b, h, 5, d)[:, :, :1]       # M = 1, row stride 0
    k1 = kd[:, :, 9:10].expand(b, h, 6, d)[:, :, :1]      # N = 1, row stride 0
    assert q1.stride(2) == 0 and k1.stride(2) == 0
    lib = _lib.load()
    for qx, kx in ((q1, kd), (qd, k1), (q1, k1)):
        m, n = qx.shape[2], kx.shape[2]
        for red in REDUCTIONS:
            got = fca.flash_colreduce(qx, kx, red, is_causal=causal, out_dtype=torch.float32)
            check(got, colreduce_ref(qx.cpu(), kx.cpu(), red, causal), red, f"m{m} n{n}")
        out = torch.empty(b * h, n, device="cuda")
        lse = torch.empty(lib.fcr_lse_bytes(b, h, m, n, d) // 4, device="cuda")
        _lib.check(lib.fcr_colreduce(qx.data_ptr(), kx.data_ptr(), out.data_ptr(), lse.data_ptr(), _lib.DTYPE_F16, b, h,
                                     m, n, d, _lib.strides4(qx.stride()), _lib.strides4(kx.stride()), 0.125, 0,
                                     int(causal), None))
        check(out.view(b, h, n), colreduce_ref(qx.cpu(), kx.cpu(), "sum", causal), "sum", f"C ABI m{m} n{n}")


@pytest.mark.parametrize("causal", [False, True])
def test_score_jumps_renormalise(causal):
    """Scores that jump by far more than 64 binades in the middle of the sweep, and rows whose
    scores are all hugely negative: exercises the renormalisation of the running row sum."""
    b, h, m, n, d = 1, 2, 96, 640, 64
    q, k = _inputs.randn_pair(b, h, m, n, d, seed=9)
    q = q.float()
    k = k.float()
    k[:, 0, 300] = 40.0 * q[:, 0, 50]          # one enormous aligned key, late
    k[:, 0, 301] = -40.0 * q[:, 0, 50]         # and an enormously negative one
    k[:, 1, :, :] = -3.0 * q[:, 1, :1, :] + 0.1 * k[:, 1]   # all scores of row 0 around -190
    k[:, 1, 500:] *= 0.0
    run_all(q.half(), k.half(), causal, what="jumps")
    run_all(q.half(), k.half(), causal, scale=1.0, what="jumps scale 1")


@pytest.mark.parametrize("causal", [False, True])
def test_nan_and_inf_inputs(causal):
    """Non-finite inputs.  A row of scores with a NaN or a +inf (inf - inf in the softmax) is a NaN row:
    every column it may see gets a NaN sum and mean, as in the materialising reference (naive.py:19-28).
    Columns hidden from every such row are untouched (the reference's materialised softmax makes the
    hidden entries of a NaN row NaN as well, naive.py:24-25; its kernel, like this one, never visits
    them, flash.py:198-207), as are rows and (b,h) pairs without one.  The column maximum follows IEEE
    maxNum (a NaN operand is dropped, like the Triton max at flash.py:123-124), so 'max' is compared on
    the columns no NaN row sees (test_max_leaves_nan_rows_out checks it on the others)."""
    b, h, m, n, d = 1, 4, 150, 260, 64
    q, k = _inputs.randn_pair(b, h, m, n, d, seed=55)
    q = q.clone()
    k = k.clone()
    q[0, 0, 70, 5] = float("nan")          # head 0: a NaN in query 70
    q[0, 1, 20, 3] = float("inf")          # head 1: an infinity in query 20 (scores +inf and -inf)
    k[0, 2, 100, 7] = float("-inf")        # head 2: an infinity in key 100: +inf scores for queries with q[7] < 0
    c = max(n - m, 0)
    scores = torch.einsum("bhmd,bhnd->bhmn", q.float(), k.float())
    vis = (torch.arange(m)[:, None] + c >= torch.arange(n)[None, :]) if causal else torch.ones(m, n, dtype=torch.bool)
    bad = ((torch.isnan(scores) | (scores == float("inf"))) & vis).any(-1)          # [b, h, m]: NaN rows
    assert bad[0, 0].sum() == 1 and bad[0, 1].sum() == 1 and bad[0, 2].sum() > 10 and not bad[0, 3].any()
    nan_cols = (bad[..., None] & vis).any(-2)                                          # [b, h, n]
    q_clean = torch.where(bad[..., None], torch.zeros_like(q), q)   # a zero row adds nothing to columns it cannot see
    k_clean = torch.nan_to_num(k, neginf=0.0)
    qd, kd = q.cuda(), k.cuda()
    for red in REDUCTIONS:
        got = fca.flash_colreduce(qd, kd, red, is_causal=causal, out_dtype=torch.float32).cpu()
        want = colreduce_ref(q_clean, k_clean, red, causal)
        if red != "max":
            assert torch.equal(torch.isnan(got), nan_cols), red
        ok = ~nan_cols
        ok[0, 2] = False     # head 2: the key with the infinity changes every row that sees it
        if causal:
            assert ok[0, 0].any() and ok[0, 1].any()
        check(got[ok], want[ok], red, f"columns no NaN row sees, causal={causal}")


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("m,n", [(150, 260), (300, 3000), (64, 700), (100, 900), (64, 2048), (128, 4096)])
def test_max_leaves_nan_rows_out(m, n, causal):
    """The column maximum of a column that a NaN row sees is the maximum over the other rows that see it,
    and 0 when there is none: a NaN is dropped by the maximum (IEEE maxNum), as in the reference's kernel
    (tl.max and tl.atomic_max, flash.py:123-124,262-273), not propagated as by the materialising reference
    (naive.py:36-37).  Every column kernel (resident keys, streamed keys, single sweep, sum and max from
    one sweep), checked ON the columns the NaN rows see, against a float64 softmax written out here."""
    b, h, d = 1, 3, 64
    q, k = _inputs.randn_pair(b, h, m, n, d, seed=77 + m)
    q, k = q.half().clone(), k.half().clone()
    q[0, 0, m // 2, 5] = float("nan")       # head 0: one NaN row in the middle
    q[0, 1, m - 1, 0] = float("nan")        # head 1: the last row, the only one that sees the last column when causal
    q[0, 1, 3, 1] = float("inf")            #         and a row with +inf and -inf scores
    k[0, 2, n - 5, 7] = float("-inf")       # head 2: a key that gives +inf, -inf scores
    c = max(n - m, 0)
    vis = (torch.arange(m)[:, None] + c >= torch.arange(n)[None, :]) if causal else torch.ones(m, n, dtype=torch.bool)
    s = torch.einsum("bhmd,bhnd->bhmn", q.double(), k.double()) / math.sqrt(d)
    s = torch.where(vis, s, torch.full_like(s, float("-inf")))
    bad = (torch.isnan(s) | (s == float("inf"))).any(-1)                     # [b, h, m]
    p = torch.softmax(torch.where(bad[..., None], torch.zeros_like(s), s), dim=-1)
    p = torch.where(vis, p, torch.zeros_like(p))
    want_max = torch.where(bad[..., None], torch.zeros_like(p), p).amax(-2)
    nan_cols = (bad[..., None] & vis).any(-2)
    want_sum = torch.where(nan_cols, torch.full_like(want_max, float("nan")),
                           torch.where(bad[..., None], torch.zeros_like(p), p).sum(-2))
    assert bad[0, 0].sum() == 1 and bad[0, 1].sum() == 2 and bad[0, 2].sum() >= 1
    if causal:
        assert want_max[0, 1, -1] == 0    # no row left for the last column
    qd, kd = q.cuda(), k.cuda()
    got = fca.flash_colreduce(qd, kd, "max", is_causal=causal, out_dtype=torch.float32).cpu()
    assert not torch.isnan(got).any()
    torch.testing.assert_close(got.double(), want_max, rtol=2e-3, atol=1e-30)
    both_sum, both_max = fca.flash_colreduce_multi(qd, kd, ["sum", "max"], is_causal=causal, out_dtype=torch.float32)
    torch.testing.assert_close(both_max.cpu().double(), want_max, rtol=2e-3, atol=1e-30)
    torch.testing.assert_close(both_sum.cpu().double(), want_sum, rtol=2e-3, atol=1e-5, equal_nan=True)


def test_heavy_hitter_columns_small():
    q, k = _inputs.config4(heads=2, n=1024)
    run_all(q, k, True, what="config4-small")
    q, k = _inputs.config5(heads=2, n=1536)
    run_all(q, k, True, what="config5-small")


@pytest.mark.parametrize("causal", [False, True])
def test_row_lse2(causal):
    q, k = _inputs.randn_pair(2, 3, 300, 520, 80, seed=13)
    got = fca.row_lse2(q.cuda(), k.cuda(), is_causal=causal).double().cpu()
    want = row_lse2_ref(q, k, causal)
    assert got.shape == (2, 3, 300)
    torch.testing.assert_close(got, want, rtol=0, atol=2e-5 * 12)


def test_key_shift_invariance_bf16_inputs():
    """Adding one vector to every key of a head only shifts each row's scores (config 5's
    perturbation); exact in real arithmetic, so checked in fp16 where the shift is representable."""
    q, k = _inputs.randn_pair(1, 2, 256, 384, 64, seed=31)
    k = (k.float() * 4).round() / 4
    shift = torch.tensor([0.5, -0.25] * 32).view(1, 1, 1, 64)
    a = fca.flash_colreduce(q.cuda(), k.half().cuda(), "sum", True, out_dtype=torch.float32)
    b = fca.flash_colreduce(q.cuda(), (k + shift).half().cuda(), "sum", True, out_dtype=torch.float32)
    torch.testing.assert_close(a, b, rtol=2e-3, atol=1e-5)


def test_deterministic_and_stream_safe():
    """No atomics: results are bitwise repeatable, also on a side stream."""
    q, k = _inputs.randn_pair(2, 4, 700, 900, 128, seed=17)
    q, k = q.cuda(), k.cuda()
    ref = {r: fca.flash_colreduce(q, k, r, True, out_dtype=torch.float32) for r in REDUCTIONS}
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        again = {r: fca.flash_colreduce(q, k, r, True, out_dtype=torch.float32) for r in REDUCTIONS}
    s.synchronize()
    for r in REDUCTIONS:
        assert torch.equal(ref[r], again[r]), r


def test_output_dtype_and_mean_epilogue():
    q, k = _inputs.randn_pair(1, 2, 64, 200, 32, seed=3, dtype=torch.bfloat16)
    q, k = q.cuda(), k.cuda()
    out = fca.flash_colreduce(q, k, "mean", True)
    assert out.dtype == torch.bfloat16 and out.shape == (1, 2, 200)
    s = fca.flash_colreduce(q, k, "sum", True)
    div = torch.cat([torch.full((136,), 64.0), torch.arange(64, 0, -1).float()]).cuda()
    torch.testing.assert_close(out, (s / div.to(torch.bfloat16)), rtol=0, atol=0)


@pytest.mark.parametrize("res_dtype", [None, torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("m,n,d,dtype", [(300, 5000, 64, torch.bfloat16),     # counts that bf16 and fp16 round
                                         (700, 300, 128, torch.float16),     # more queries than keys
                                         (40, 9000, 128, torch.float16),     # the few-queries column sweep
                                         (1, 77, 32, torch.bfloat16), (513, 513, 72, torch.float16)])
def test_cast_and_mean_in_the_kernel_repeat_the_torch_steps(m, n, d, dtype, causal, res_dtype):
    """The column kernel's typed store against the reference's own sequence of torch operations
    (flash.py:308 cast, 377-384 in-place divisions) applied to the fp32 result of the C ABI: bit for bit."""
    from flash_colreduce_amd import flash as F
    q, k = _inputs.randn_pair(2, 3, m, n, d, seed=m + n, dtype=dtype)
    q, k = q.cuda(), k.cuda()
    want_dtype = dtype if res_dtype is None else res_dtype
    for red in REDUCTIONS:
        got = fca.flash_colreduce(q, k, red, is_causal=causal, out_dtype=res_dtype)
        (acc,), _ = F._launch(q, k, ["max" if red == "max" else "sum"], causal, None)
        scores = acc.view(2, 3, n).to(want_dtype)
        if red == "mean":
            if causal:
                c = max(n - m, 0)
                scores[..., :c] /= m
                scores[..., c:] /= torch.arange(n - c, 0, -1, device=q.device)
            else:
                scores /= m
        assert got.dtype == want_dtype and got.shape == (2, 3, n)
        assert torch.equal(got, scores), (red, (got.float() - scores.float()).abs().max().item())


@pytest.mark.parametrize("causal", [False, True])
def test_multi_reduction_shares_the_row_pass(causal):
    q, k = _inputs.randn_pair(2, 3, 300, 450, 64, seed=8, dtype=torch.bfloat16)
    qd, kd = q.cuda(), k.cuda()
    outs = fca.flash_colreduce_multi(qd, kd, ["mean", "max", "sum", "mean"], is_causal=causal,
                                     out_dtype=torch.float32)
    assert len(outs) == 4
    for red, got in zip(["mean", "max", "sum", "mean"], outs):
        one = fca.flash_colreduce(qd, kd, red, is_causal=causal, out_dtype=torch.float32)
        if red == "max":
            assert torch.equal(got, one)  # a maximum does not depend on the tiling
        else:
            torch.testing.assert_close(got, one, rtol=1e-5, atol=1e-7)
        check(got, colreduce_ref(q, k, red, causal), red, "multi")
    only_sums = fca.flash_colreduce_multi(qd, kd, ["sum", "mean"], is_causal=causal, out_dtype=torch.float32)
    assert torch.equal(only_sums[0], fca.flash_colreduce(qd, kd, "sum", is_causal=causal, out_dtype=torch.float32))
    with pytest.raises(ValueError, match="Invalid reduction: median"):
        fca.flash_colreduce_multi(qd, kd, ["sum", "median"])
    with pytest.raises(ValueError, match="at least one"):
        fca.flash_colreduce_multi(qd, kd, [])


@pytest.mark.parametrize("res_dtype", [None, torch.float32])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("m,n,d,dtype", [(300, 5000, 64, torch.bfloat16), (64, 4096, 128, torch.float16),
                                         (100, 2000, 32, torch.bfloat16), (700, 300, 128, torch.float16)])
def test_sum_or_mean_with_max_finished_in_the_kernel(m, n, d, dtype, causal, res_dtype):
    """'sum' or 'mean' together with 'max' is one call of fcr_colreduce_sum_max_to (two kernels, or the single
    sweep): both results leave it in the result type, the means divided as flash.py:377-384 does.  Held to
    the torch sequence on the same call's fp32 sums bit for bit, and to the one-reduction calls."""
    q, k = _inputs.randn_pair(2, 3, m, n, d, seed=m + n, dtype=dtype)
    qd, kd = q.cuda(), k.cuda()
    rt = dtype if res_dtype is None else res_dtype
    s32, x32 = fca.flash_colreduce_multi(qd, kd, ["sum", "max"], is_causal=causal, out_dtype=torch.float32)
    check(s32.cpu(), colreduce_ref(q, k, "sum", causal), "sum", "pair")
    check(x32.cpu(), colreduce_ref(q, k, "max", causal), "max", "pair")
    for red in ("sum", "mean"):
        got, mx = fca.flash_colreduce_multi(qd, kd, [red, "max"], is_causal=causal, out_dtype=res_dtype)
        assert got.dtype == rt and mx.dtype == rt and got.shape == (2, 3, n) and mx.shape == (2, 3, n)
        want = s32.to(rt)
        if red == "mean":
            c = max(n - m, 0) if causal else n
            want[..., :c] /= m
            if c < n:
                want[..., c:] /= torch.arange(n - c, 0, -1, device="cuda")
        assert torch.equal(got, want), red
        assert torch.equal(mx, x32.to(rt))
        one = fca.flash_colreduce(qd, kd, red, is_causal=causal, out_dtype=res_dtype)
        torch.testing.assert_close(got.float(), one.float(), rtol=2e-5 if rt == torch.float32 else 1e-2, atol=1e-7)
    twice = fca.flash_colreduce_multi(qd, kd, ["max", "mean", "max"], is_causal=causal)
    assert torch.equal(twice[0], twice[2]) and twice[0].data_ptr() != twice[2].data_ptr()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("m,n,d", [(1, 1, 8), (131, 1027, 72), (700, 300, 128), (40, 1000, 24), (300, 420, 200),
                                   (1024, 1024, 128)])
def test_sum_and_max_from_one_sweep(m, n, d, causal, dtype):
    q, k = _inputs.randn_pair(2, 2, m, n, d, seed=m + n + d, dtype=dtype)
    s, mx, mean = fca.flash_colreduce_multi(q.cuda(), k.cuda(), ["sum", "max", "mean"], is_causal=causal,
                                            out_dtype=torch.float32)
    check(s, colreduce_ref(q, k, "sum", causal), "sum", "fused")
    check(mx, colreduce_ref(q, k, "max", causal), "max", "fused")
    check(mean, colreduce_ref(q, k, "mean", causal), "mean", "fused")


@pytest.mark.parametrize("n,k", [(1, 1), (5, 2), (256, 100), (257, 256), (1000, 0), (1000, 1000), (1000, 1500),
                                 (4099, 1024), (8192, 2048), (8200, 8199), (32768, 8192), (32769, 1), (40000, 5000),
                                 (70001, 0), (70001, 69000), (131072, 200)])
def test_topk_keep_mask(n, k):
    from oracle.colreduce_oracle import topk_mask_ref
    g = torch.Generator().manual_seed(n + k)
    vals = torch.rand(6, n, generator=g)
    vals[1] = (vals[1] * 8).floor() / 8          # heavy ties
    vals[2] = 0.25                                # all equal
    vals[3] = -vals[3]                            # negatives
    vals[4, ::3] = 0.0
    vals[4, 1::3] = -0.0
    mask, thr = fca.topk_keep_mask(vals.cuda().view(2, 3, n), k, return_threshold=True)
    assert mask.dtype == torch.bool and mask.shape == (2, 3, n) and thr.shape == (2, 3)
    want = topk_mask_ref(vals.numpy(), k)
    assert (mask.view(6, n).cpu().numpy() == want).all()
    if 0 < k <= n:
        kth = torch.sort(vals, dim=1, descending=True).values[:, k - 1]
        assert torch.equal(thr.view(6).cpu(), kth)


@pytest.mark.parametrize("rows,n,k", [(5, 32769, 5), (5, 40000, 39999), (5, 70001, 1234), (5, 262144, 65536),
                                      (5, 300007, 100000),
                                      (128, 65537, 3000), (64, 131072, 131000)])   # 32 keys per thread
def test_topk_long_rows_with_and_without_scratch(rows, n, k):
    """Rows of more than 32768 columns: spread over workgroups when the caller brings scratch
    (fcr_topk_mask_ws), one workgroup per row otherwise (fcr_topk_mask); both against the oracle."""
    from flash_colreduce_amd import _lib
    from oracle.colreduce_oracle import topk_mask_ref
    g = torch.Generator().manual_seed(n)
    vals = torch.randn(rows, n, generator=g)
    vals[1] = (vals[1] * 4).round() / 4           # heavy ties, both signs
    vals[2] = 1.5                                 # all equal: the lowest k columns win
    vals[3, : n // 2] = vals[3, n // 2: n // 2 * 2]   # every value of the first half twice
    want = topk_mask_ref(vals.numpy(), k)
    kth = torch.sort(vals, dim=1, descending=True).values[:, k - 1]
    lib = _lib.load()
    dev = vals.cuda()
    stream = torch.cuda.current_stream().cuda_stream
    nbytes = lib.fcr_topk_bytes(rows, n)
    assert nbytes > 0 and lib.fcr_topk_bytes(rows, 32768) == 0
    ws = torch.full((nbytes,), 0xAB, device="cuda", dtype=torch.uint8)   # the scratch need not be cleared
    for use_ws in (True, False):
        mask = torch.full((rows, n), 7, device="cuda", dtype=torch.uint8)
        thr = torch.empty(rows, device="cuda")
        if use_ws:
            _lib.check(lib.fcr_topk_mask_ws(dev.data_ptr(), mask.data_ptr(), thr.data_ptr(), rows, n, k, ws.data_ptr(),
                                            nbytes, stream))
        else:
            _lib.check(lib.fcr_topk_mask(dev.data_ptr(), mask.data_ptr(), thr.data_ptr(), rows, n, k, stream))
        assert (mask.cpu().numpy() == want).all(), use_ws
        assert torch.equal(thr.cpu(), kth), use_ws


def test_topk_takes_the_operator_result_as_it_comes():
    """fp16 / bf16 scores, as flash_colreduce returns them for 16-bit operands: same mask as for their fp32 values."""
    from oracle.colreduce_oracle import topk_mask_ref
    q, k = _inputs.randn_pair(1, 3, 200, 3000, 64, seed=21, dtype=torch.bfloat16)
    scores = fca.flash_colreduce(q.cuda(), k.cuda(), "sum", is_causal=True)
    assert scores.dtype == torch.bfloat16
    mask = fca.topk_keep_mask(scores, 500)
    want = topk_mask_ref(scores.float().cpu().view(3, 3000).numpy(), 500)
    assert (mask.view(3, 3000).cpu().numpy() == want).all()
    with pytest.raises(ValueError):
        fca.topk_keep_mask(scores.to(torch.float64), 5)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("n,k", [(1, 1), (7, 3), (1000, 100), (1027, 1000), (8192, 2048), (8190, 17), (32768, 5000),
                                 (32770, 300), (70001, 20000), (300004, 1000)])
def test_topk_reads_16_bit_rows(n, k, dtype):
    """16-bit score rows are read by the kernels themselves (every kernel of the selection, rows that do and
    do not start on 8-byte boundaries): heavy ties, as 16-bit values have them, against the oracle on the
    widened values; the threshold is the k-th largest value, widened."""
    from oracle.colreduce_oracle import topk_mask_ref
    g = torch.Generator().manual_seed(7 * n + k)
    vals = torch.randn(5, n, generator=g).to(dtype)
    vals[1] = (torch.rand(n, generator=g) * 4).to(dtype)          # a few hundred distinct values
    vals[2] = 0.5
    vals[3, ::2] = -0.0
    vals[3, 1::2] = 0.0
    mask, thr = fca.topk_keep_mask(vals.cuda(), k, return_threshold=True)
    want = topk_mask_ref(vals.float().numpy(), k)
    assert (mask.cpu().numpy() == want).all()
    kth = torch.sort(vals.float(), dim=1, descending=True).values[:, k - 1]
    assert thr.dtype == torch.float32 and torch.equal(thr.cpu() + 0.0, kth + 0.0)   # + 0.0: -0 and +0 are one value


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("n", [100, 5000, 20000, 40000, 70001])
def test_topk_orders_nans_above_everything(n, dtype):
    """A NaN of either sign ranks above +inf, NaNs tie (lower column first): every kernel of the selection
    against the oracle; the threshold is a NaN exactly when the k-th largest entry is one."""
    from oracle.colreduce_oracle import topk_mask_ref
    g = torch.Generator().manual_seed(n)
    vals = torch.randn(4, n, generator=g).to(dtype)
    nan = float("nan")
    vals[0, [3, n // 2, n - 1]] = nan
    vals[0, 7] = float("inf")
    vals[1, 5] = -nan
    vals[1, 50] = nan
    vals[2, ::3] = nan                                   # a third of the row
    vals[3] = nan                                        # the whole row
    vals[3, 10] = 1.0
    lib_rows = vals.cuda()
    for k in (1, 2, 3, 4, 5, n // 3, n // 2, n - 1, n):
        mask, thr = fca.topk_keep_mask(lib_rows, k, return_threshold=True)
        want = topk_mask_ref(vals.float().numpy(), k)
        assert (mask.cpu().numpy() == want).all(), k
        nans = torch.isnan(vals.float()).sum(1)
        assert torch.equal(torch.isnan(thr.cpu()), nans >= k), k


def test_topk_on_reduced_columns():
    from oracle.colreduce_oracle import topk_mask_ref
    q, k = _inputs.config4(heads=4, n=2048)
    s = fca.flash_colreduce(q.cuda(), k.cuda(), "sum", is_causal=True, out_dtype=torch.float32)
    mask = fca.topk_keep_mask(s, 512)
    assert (mask.sum(-1) == 512).all()
    assert (mask.view(4, 2048).cpu().numpy() == topk_mask_ref(s.view(4, 2048).cpu().numpy(), 512)).all()
    assert mask[..., 0].all()   # the sink column is always kept


def test_random_shapes_against_oracle():
    """Seeded sweep over shapes, dtypes, masks, scales and layouts that no other test names."""
    import random
    rng = random.Random(20240607)
    for case in range(60):
        b, h = rng.randint(1, 3), rng.randint(1, 5)
        m = rng.choice([1, 2, 15, 16, 17, 31, 33, 63, 64, 65, 100, 127, 129, 255, 257, 400, 513, 700])
        n = rng.choice([1, 3, 16, 17, 32, 63, 65, 128, 130, 255, 256, 257, 300, 511, 640, 1025, 2100])
        d = rng.choice([8, 16, 24, 32, 40, 64, 72, 96, 100, 128, 136, 160, 192, 256])
        dtype = rng.choice([torch.float16, torch.bfloat16])
        causal = rng.random() < 0.5
        scale = rng.choice([None, None, 0.07, 0.3])
        q, k = _inputs.randn_pair(b, h, m, n, d, seed=1000 + case, dtype=dtype)
        if rng.random() < 0.3:  # [B, rows, H, D] storage
            q = q.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
            k = k.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
        reds = rng.sample(REDUCTIONS, rng.randint(1, 3))
        what = f"case {case}: b{b} h{h} m{m} n{n} d{d} {dtype} causal={causal} scale={scale} {reds}"
        outs = fca.flash_colreduce_multi(q.cuda(), k.cuda(), reds, is_causal=causal, scale=scale,
                                         out_dtype=torch.float32)
        for red, got in zip(reds, outs):
            check(got, colreduce_ref(q, k, red, causal, scale=scale), red, what)


def test_random_decode_shapes_and_fp32_against_oracle():
    """Second seeded sweep: few queries against many keys (single sweep and its neighbours on either side of
    its limits: 128 queries, 1024 keys, rows of 256 bytes) and fp32 operands of any shape."""
    import random
    rng = random.Random(977)
    for case in range(60):
        b, h = rng.randint(1, 2), rng.randint(1, 6)
        if case % 3 == 2:
            dtype = torch.float32
            m = rng.choice([1, 5, 64, 100, 129, 300])
            n = rng.choice([7, 130, 513, 1500, 2600])
            d = rng.choice([4, 12, 64, 100, 128, 200, 256])
        else:
            dtype = rng.choice([torch.float16, torch.bfloat16])
            m = rng.choice([1, 2, 16, 33, 63, 64, 65, 100, 127, 128, 129, 140])
            n = rng.choice([960, 1023, 1024, 1025, 1100, 2047, 2049, 3000, 4097, 7000, 9001])
            d = rng.choice([8, 32, 64, 72, 128, 136])
        causal = rng.random() < 0.5
        scale = rng.choice([None, None, 0.05, 0.4])
        q, k = _inputs.randn_pair(b, h, m, n, d, seed=5000 + case, dtype=dtype)
        if rng.random() < 0.3:  # [B, rows, H, D] storage
            q = q.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
            k = k.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
        reds = rng.sample(REDUCTIONS, rng.randint(1, 3))
        what = f"case {case}: b{b} h{h} m{m} n{n} d{d} {dtype} causal={causal} scale={scale} {reds}"
        for red in reds:   # one call per reduction: the calls that may take the single sweep
            got = fca.flash_colreduce(q.cuda(), k.cuda(), red, is_causal=causal, scale=scale, out_dtype=torch.float32)
            check(got, colreduce_ref(q, k, red, causal, scale=scale), red, what)


def test_hip_graph_capture_and_replay():
    """The whole call (torch allocations, both kernels, cast) captured in a graph and replayed with
    new contents in the static inputs; every replay must equal the eager result for those contents."""
    b, h, m, n, d = 1, 4, 300, 500, 64
    qs = torch.zeros(b, h, m, d, device="cuda", dtype=torch.float16)
    ks = torch.zeros(b, h, n, d, device="cuda", dtype=torch.float16)
    q0, k0 = _inputs.randn_pair(b, h, m, n, d, seed=77)
    qs.copy_(q0)
    ks.copy_(k0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm up outside the capture
        fca.flash_colreduce_multi(qs, ks, ["sum", "max"], True, out_dtype=torch.float32)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        s_out, m_out = fca.flash_colreduce_multi(qs, ks, ["sum", "max"], True, out_dtype=torch.float32)
        one = fca.flash_colreduce(qs, ks, "mean", True, out_dtype=torch.float32)
    for seed in (78, 79, 80):
        q1, k1 = _inputs.randn_pair(b, h, m, n, d, seed=seed)
        qs.copy_(q1)
        ks.copy_(k1)
        graph.replay()
        torch.cuda.synchronize()
        got = (s_out.clone(), m_out.clone(), one.clone())
        es, em = fca.flash_colreduce_multi(qs, ks, ["sum", "max"], True, out_dtype=torch.float32)
        e1 = fca.flash_colreduce(qs, ks, "mean", True, out_dtype=torch.float32)
        torch.cuda.synchronize()
        assert torch.equal(got[0], es) and torch.equal(got[1], em) and torch.equal(got[2], e1), seed
        check(got[0], colreduce_ref(q1, k1, "sum", True), "sum", f"graph replay seed {seed}")


def test_graph_capture_of_a_causal_mean_never_seen_before():
    """The causal mean divisor is built on the device by every call.  Capture a causal mean whose
    divisor length was never used in this process, call eagerly BEFORE the first replay, then capture a
    second graph with the same length and replay only that one: each result must be the oracle's."""
    b, h, m, n, d = 1, 3, 211, 347, 32      # divisor length 211, used by no other test
    qc, kc = _inputs.randn_pair(b, h, m, n, d, seed=91)
    q, k = qc.cuda(), kc.cuda()
    want = colreduce_ref(qc, kc, "mean", True)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm up the kernels, but not the mean epilogue
        fca.flash_colreduce(q, k, "sum", True, out_dtype=torch.float32)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g1 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g1):
        out1 = fca.flash_colreduce(q, k, "mean", True, out_dtype=torch.float32)
    eager = fca.flash_colreduce(q, k, "mean", True, out_dtype=torch.float32)   # before any replay
    torch.cuda.synchronize()
    check(eager, want, "mean", "eager call between capture and first replay")
    g2 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g2):
        out2 = fca.flash_colreduce(q, k, "mean", True, out_dtype=torch.float32)
    g2.replay()                                                                  # g1 never replayed so far
    torch.cuda.synchronize()
    check(out2, want, "mean", "second graph replayed alone")
    assert torch.equal(out2, eager)
    g1.replay()
    torch.cuda.synchronize()
    assert torch.equal(out1, eager)


def test_launcher_stub_of_the_integration_notes():
    """The ctypes launcher shown to maintainers (the first python block of section 2 of the integration
    notes) is executed as written, against the built library, and must reproduce flash_colreduce."""
    import os
    import re
    from flash_colreduce_amd import _lib
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    text = open(os.path.join(root, "INTEGRATION.md")).read()
    section = text[text.index("## 2."):]
    code = re.search(r"```python\n(.*?)```", section, flags=re.S).group(1)
    code = code.replace("/path/to/libfcr.so", _lib.LIB_PATH)
    scope = {}
    exec(compile(code, "INTEGRATION.md", "exec"), scope)
    for dtype in (torch.float16, torch.bfloat16, torch.float32):   # the three element types the reference's tl.dot takes
        q, k = _inputs.randn_pair(2, 3, 130, 1000, 64, seed=4, dtype=dtype)
        qd, kd = q.cuda(), k.cuda()
        for red, causal in (("sum", True), ("max", False)):
            got = scope["_flash_colreduce"](qd, kd, red, causal, 0.125)
            assert got.dtype == dtype and got.shape == (2, 3, 1000)
            assert torch.equal(got, fca.flash_colreduce(qd, kd, red, is_causal=causal, scale=0.125))


def test_plain_c_caller_of_the_c_abi():
    """tests/c_abi/check.c: hipMalloc, fcr_colreduce, closed forms; no Python or torch in that process."""
    import os
    import subprocess
    from flash_colreduce_amd import build as fcr_build
    from flash_colreduce_amd import _lib
    header = os.path.join(fcr_build.INCLUDE, "fcr.h")
    newest = max(os.path.getmtime(f) for f in (fcr_build.C_CHECK_SRC, header, _lib.LIB_PATH))
    if not os.path.exists(fcr_build.C_CHECK_BIN) or os.path.getmtime(fcr_build.C_CHECK_BIN) < newest:
        fcr_build.build_c_check(verbose=False)   # never a binary older than its source, the header or the library
    done = subprocess.run([fcr_build.C_CHECK_BIN], capture_output=True, text=True, timeout=100)
    assert done.returncode == 0 and done.stdout.strip() == "ok", (done.returncode, done.stdout, done.stderr)


def test_python_errors_on_device():
    q = torch.zeros(1, 2, 4, 8, dtype=torch.float16, device="cuda")
    k = torch.zeros(1, 2, 6, 8, dtype=torch.float16, device="cuda")
    with pytest.raises(ValueError, match="Head dimension must be <= 512"):
        fca.flash_colreduce(torch.zeros(1, 1, 4, 513, dtype=torch.float16, device="cuda"),
                            torch.zeros(1, 1, 4, 513, dtype=torch.float16, device="cuda"), "sum")
    with pytest.raises(ValueError, match="Head dimension must be <= 256"):
        fca.flash_colreduce(torch.zeros(1, 1, 4, 260, device="cuda"), torch.zeros(1, 1, 4, 260, device="cuda"), "sum")
    with pytest.raises(ValueError, match="Invalid reduction: median"):
        fca.flash_colreduce(q, k, "median")
    with pytest.raises(ValueError, match="same batch size, number of heads, and head dimension"):
        fca.flash_colreduce(q, k[:, :1], "sum")
    with pytest.raises(ValueError, match="float16, bfloat16 or float32"):
        fca.flash_colreduce(q.double(), k.double(), "sum")
    with pytest.raises(ValueError, match="float16, bfloat16 or float32"):
        fca.flash_colreduce(q.float(), k, "sum")
    # zero queries see no key: every column is 1/N
    out = fca.flash_colreduce(q, k, "max", out_dtype=torch.float32)
    torch.testing.assert_close(out, torch.full((1, 2, 6), 1 / 6, device="cuda"))
    assert fca.flash_colreduce(q[:, :, :0], k, "sum").shape == (1, 2, 6)
    assert fca.flash_colreduce(q, k[:, :, :0], "sum").shape == (1, 2, 0)
