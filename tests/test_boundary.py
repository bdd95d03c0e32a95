"""Host-side checks that need no GPU: the C-ABI library loads, exports what include/fcr.h
declares, rejects bad arguments before touching the device, and the Python entry point mirrors
the reference's validation (flash_colreduce/flash.py:354-364)."""
import ctypes
import os
import re

import pytest
import torch

import flash_colreduce_amd as fca
from flash_colreduce_amd import _lib
from oracle.colreduce_oracle import colreduce_ref
from tests import _inputs

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "fcr.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fcr_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(_lib.LIB_PATH)
    names = _declared_symbols()
    assert {"fcr_version", "fcr_last_error", "fcr_lse_bytes", "fcr_row_lse", "fcr_col_reduce",
            "fcr_col_reduce_sum_max", "fcr_pack_f32", "fcr_colreduce", "fcr_colreduce_static",
            "fcr_colreduce_to", "fcr_topk_mask", "fcr_topk_mask_ws", "fcr_topk_mask_typed", "fcr_topk_bytes", "fcr_set_option",
            "fcr_colreduce_status", "fcr_colreduce_sum_max", "fcr_colreduce_sum_max_to"} <= set(names)
    for name in names:
        assert hasattr(lib, name), name


def test_version_and_sizes():
    lib = _lib.load()
    assert lib.fcr_version() == 320
    assert lib.fcr_lse_bytes(2, 3, 5, 7, 64) == 2 * 3 * 5 * 4
    assert lib.fcr_lse_bytes(1, 32, 8192, 8192, 128) == 32 * 8192 * 4      # enough row tiles: no scratch
    assert lib.fcr_lse_bytes(1, 32, 512, 16384, 128) == 32 * 512 * 4 * 9   # 8 key ranges + the result
    # few queries, many keys (256 CUs assumed without a device): the result, two sets of 64-bit slots for
    # one workgroup per CU of 128 rows, and the status line
    assert lib.fcr_lse_bytes(1, 32, 128, 4096, 128) == (32 * 128 + 2 * 2 * 256 * 128 + 32) * 4
    assert lib.fcr_lse_bytes(-1, 3, 5, 7, 8) == 0 and lib.fcr_lse_bytes(1, 3, 0, 7, 8) == 0


def _call(lib, fn, **over):
    a = dict(q=16, k=32, lse=48, out=64, dtype=0, B=1, H=1, M=8, N=8, D=64,
             qs=(512, 512, 64, 1), ks=(512, 512, 64, 1), scale=0.125, red=0, causal=0)
    a.update(over)
    qs = _lib.strides4(a["qs"]) if a["qs"] is not None else None
    ks = _lib.strides4(a["ks"]) if a["ks"] is not None else None
    common = (a["dtype"], a["B"], a["H"], a["M"], a["N"], a["D"], qs, ks, a["scale"])
    if fn == "row_lse":
        return lib.fcr_row_lse(a["q"], a["k"], a["lse"], *common, a["causal"], None)
    if fn == "col_reduce":
        return lib.fcr_col_reduce(a["q"], a["k"], a["lse"], a["out"], *common, a["red"], a["causal"], None)
    if fn == "colreduce_to":
        return lib.fcr_colreduce_to(a["q"], a["k"], a["out"], a.get("out_dtype", 0), a["lse"], *common, a["red"],
                                    a["causal"], None)
    if fn == "colreduce_sum_max":
        return lib.fcr_colreduce_sum_max(a["q"], a["k"], a["out"], a.get("out_max", 80), a["lse"], *common, a["causal"],
                                         None)
    return lib.fcr_colreduce(a["q"], a["k"], a["out"], a["lse"], *common, a["red"], a["causal"], None)


@pytest.mark.parametrize("fn", ["row_lse", "col_reduce", "colreduce", "colreduce_to", "colreduce_sum_max"])
def test_c_abi_rejects_bad_arguments_without_a_device(fn):
    """Every rejection happens before the first HIP call, so fake pointers are safe here."""
    lib = _lib.load()
    cases = [
        (dict(q=None), -1), (dict(k=None), -1), (dict(lse=None), -1), (dict(qs=None), -1),
        (dict(dtype=3), -2), (dict(dtype=-1), -2),
        (dict(B=0), -3), (dict(M=0), -3), (dict(N=-4), -3), (dict(D=0), -3), (dict(D=12), -3),
        (dict(D=520), -3), (dict(D=516), -3), (dict(M=(1 << 30) + 1), -3),
        (dict(dtype=2, D=260), -3), (dict(dtype=2, D=6), -3),                 # fp32: a multiple of 4, at most 256
        (dict(dtype=2, D=64, qs=(512, 512, 66, 1)), -4),                       # fp32: strides in multiples of 4
        (dict(qs=(512, 512, 64, 2)), -4), (dict(ks=(512, 512, 60, 1)), -4), (dict(q=18), -4),
        (dict(H=2, ks=(512, -512, 64, 1)), -4), (dict(B=2, qs=(-512, 512, 64, 1)), -4),
        (dict(H=2, qs=(512, 4, 64, 1)), -4),                                   # head stride not a multiple of 16 bytes
        (dict(B=1 << 12, H=1 << 12), -3),                                      # 2^24 workgroups: more threads than a launch may have
        (dict(qs=(512, 512, 0, 1)), -4), (dict(ks=(512, 512, 32, 1)), -4),   # overlapping rows
        (dict(scale=float("inf")), -6), (dict(scale=float("nan")), -6),
    ]
    if fn == "colreduce_to":   # takes the mean as a third reduction, and a result type
        cases += [(dict(out=None), -1), (dict(red=3), -5), (dict(red=-1), -5), (dict(out_dtype=3), -2),
                  (dict(out_dtype=-1), -2)]
    elif fn == "colreduce_sum_max":
        cases += [(dict(out=None), -1), (dict(out_max=None), -1)]
    elif fn != "row_lse":
        cases += [(dict(out=None), -1), (dict(red=2), -5), (dict(red=-1), -5)]
    for over, code in cases:
        assert _call(lib, fn, **over) == code, over
        assert lib.fcr_last_error() != b""
    with pytest.raises(_lib.FcrError) as e:
        _lib.check(_call(lib, fn, D=12))
    assert e.value.code == -3 and "multiple of 8" in str(e.value)


def test_options_and_status_reject_bad_arguments_without_a_device():
    lib = _lib.load()
    assert lib.fcr_set_option(99, 1) == -3
    assert lib.fcr_set_option(_lib.OPT_WAIT_POLLS, -5) == -3
    assert lib.fcr_set_option(_lib.OPT_SINGLE_SWEEP, 1) == 0 and lib.fcr_set_option(_lib.OPT_WAIT_POLLS, 1 << 20) == 0
    assert lib.fcr_colreduce_status(None, 0, 1, 1, 8, 8, 64, None) == -1
    assert lib.fcr_colreduce_status(16, 0, 1, 1, 0, 8, 64, None) == -3
    # problems that never take the single sweep have nothing to report: no device is asked
    assert lib.fcr_colreduce_status(16, 0, 1, 1, 512, 512, 64, None) == 0      # more than 128 queries
    assert lib.fcr_colreduce_status(16, 2, 1, 1, 64, 4096, 64, None) == 0      # fp32 operands
    assert lib.fcr_colreduce_status(16, 0, 1, 1, 64, 512, 64, None) == 0       # fewer than 1024 keys


def test_pack_f32_rejects_bad_arguments_without_a_device():
    lib = _lib.load()
    assert lib.fcr_pack_f32(None, 16, 4, 8, 3, 0, None) == -1
    assert lib.fcr_pack_f32(16, None, 4, 8, 3, 0, None) == -1
    assert lib.fcr_pack_f32(16, 32, 0, 8, 3, 0, None) == -3
    assert lib.fcr_pack_f32(16, 32, 4, 8, 2, 0, None) == -3      # terms must be 1 or 3
    assert lib.fcr_pack_f32(16, 32, 4, 88, 3, 0, None) == -3     # 3 * 88 > 256
    assert lib.fcr_pack_f32(16, 32, 4, 264, 1, 0, None) == -3


def test_python_entry_validation_matches_reference_messages():
    q = torch.zeros(1, 2, 4, 8, dtype=torch.float16)
    k = torch.zeros(1, 2, 6, 8, dtype=torch.float16)
    with pytest.raises(ValueError, match="must be on CUDA device"):
        fca.flash_colreduce(q, k, "sum")
    with pytest.raises(ValueError, match="must be on CUDA device"):
        fca.flash_colreduce(q, k, "bogus")  # device is checked first, as in the reference


def test_naive_colreduce_matches_oracle_on_config1():
    """Configuration 1 of the benchmark set: the CPU-runnable fp32 case, non-causal, all three reductions."""
    q, k = _inputs.config1()
    for red in ("sum", "mean", "max"):
        got = fca.naive_colreduce(q, k, red)
        assert got.shape == (1, 2, 256) and got.dtype == torch.float32
        want = colreduce_ref(q, k, red, compute_dtype=torch.float64).float()
        torch.testing.assert_close(got, want, rtol=2e-3, atol=1e-5)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("m,n", [(5, 9), (9, 5), (6, 6)])
def test_naive_colreduce_matches_oracle_small(m, n, causal):
    q, k = _inputs.randn_pair(2, 3, m, n, 12, seed=m + n, dtype=torch.float32)
    for red in ("sum", "mean", "max"):
        got = fca.naive_colreduce(q, k, red, is_causal=causal, scale=0.3)
        want = colreduce_ref(q, k, red, causal, scale=0.3, compute_dtype=torch.float64).float()
        torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-7)
    with pytest.raises(ValueError, match="Invalid reduction"):
        fca.naive_colreduce(q, k, "median")
