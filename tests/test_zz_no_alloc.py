"""fcr_colreduce_static, the entry point that allocates nothing: called through the C ABI and held to
the bitwise result of fcr_colreduce (same kernels, same order of operations) and to the CPU oracle,
on calls in a row that share the built-in scratch buffer, each smaller than the one before."""
import pytest
import torch

from flash_colreduce_amd import _lib
from oracle.colreduce_oracle import colreduce_ref
from tests import _inputs

STATIC_SCRATCH_BYTES = 16 << 20


def _args(q, k, scale):
    b, h, m, d = q.shape
    return (_lib.DTYPE_F16 if q.dtype == torch.float16 else _lib.DTYPE_BF16, b, h, m, k.shape[2], d,
            _lib.strides4(q.stride()), _lib.strides4(k.stride()), scale)


@pytest.mark.gpu
def test_static_scratch_entry_matches_the_allocating_one():
    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    # (b, h, m, n, d, dtype, causal): a general shape, then smaller ones; the third splits the keys of
    # its row tiles, so the partial results behind the row statistics are in use as well
    cases = [(2, 4, 700, 900, 128, torch.float16, True),
             (1, 3, 130, 333, 64, torch.bfloat16, False),
             (1, 8, 64, 2048, 64, torch.float16, True),
             (1, 1, 1, 1, 8, torch.float16, False)]
    for seed, (b, h, m, n, d, dtype, causal) in enumerate(cases):
        qc, kc = _inputs.randn_pair(b, h, m, n, d, seed=400 + seed, dtype=dtype)
        q, k = qc.cuda(), kc.cuda()
        scale = 1.0 / d ** 0.5
        need = lib.fcr_lse_bytes(b, h, m, n, d)
        assert need <= STATIC_SCRATCH_BYTES
        for red, name in ((_lib.REDUCE_SUM, "sum"), (_lib.REDUCE_MAX, "max")):
            lse = torch.empty(need // 4, device="cuda", dtype=torch.float32)
            want = torch.empty(b * h, n, device="cuda", dtype=torch.float32)
            got = torch.full((b * h, n), float("nan"), device="cuda", dtype=torch.float32)
            _lib.check(lib.fcr_colreduce(q.data_ptr(), k.data_ptr(), want.data_ptr(), lse.data_ptr(),
                                         *_args(q, k, scale), red, int(causal), stream))
            _lib.check(lib.fcr_colreduce_static(q.data_ptr(), k.data_ptr(), got.data_ptr(),
                                                *_args(q, k, scale), red, int(causal), stream))
            torch.cuda.synchronize()
            assert torch.equal(got, want), (seed, name)
            ref = colreduce_ref(qc, kc, name, causal).view(b * h, n)
            if name == "max":
                assert ((got.cpu() - ref).abs() / ref).max().item() <= 2e-3
            else:
                torch.testing.assert_close(got.cpu(), ref, rtol=2e-3, atol=1e-5)


@pytest.mark.gpu
def test_static_scratch_entry_rejects_what_does_not_fit():
    lib = _lib.load()
    q = torch.zeros(1, 1, 8, 64, device="cuda", dtype=torch.float16)
    out = torch.zeros(1, 8, device="cuda", dtype=torch.float32)
    # 64 x 32 x 4096 rows need 32 MiB of row statistics: rejected from the sizes alone, nothing is read
    big = (_lib.DTYPE_F16, 64, 32, 4096, 4096, 64, _lib.strides4((0, 0, 64, 1)), _lib.strides4((0, 0, 64, 1)), 0.125)
    assert lib.fcr_lse_bytes(64, 32, 4096, 4096, 64) > STATIC_SCRATCH_BYTES
    rc = lib.fcr_colreduce_static(q.data_ptr(), q.data_ptr(), out.data_ptr(), *big, _lib.REDUCE_SUM, 0, None)
    assert rc == -7 and b"scratch" in lib.fcr_last_error()
    rc = lib.fcr_colreduce_static(q.data_ptr(), q.data_ptr(), None, *big, _lib.REDUCE_SUM, 0, None)
    assert rc == -1
