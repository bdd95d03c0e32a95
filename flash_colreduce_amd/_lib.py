"""ctypes binding of libfcr.so (declared in include/fcr.h).

torch must be imported before the library is opened so that both share one HIP runtime
(torch bundles libamdhip64 under the same SONAME); importing this module does that.
There is no fallback: a missing library raises.
"""
from __future__ import annotations

import ctypes
import os

import torch  # noqa: F401  (loads the HIP runtime the library binds to)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libfcr.so")

DTYPE_F16, DTYPE_BF16, DTYPE_F32 = 0, 1, 2
REDUCE_SUM, REDUCE_MAX, REDUCE_MEAN = 0, 1, 2
OPT_SINGLE_SWEEP, OPT_WAIT_POLLS = 0, 1
E_WAIT = -8

_I64x4 = ctypes.c_int64 * 4
_lib = None


class FcrError(RuntimeError):
    """Non-zero return code from libfcr (negative: rejected argument, positive: hipError_t)."""

    def __init__(self, code: int, text: str):
        super().__init__(f"libfcr error {code}: {text}")
        self.code = code


def _declare(lib):
    c = ctypes
    common = [c.c_int, c.c_int, c.c_int, c.c_int, c.c_int, c.c_int,  # dtype B H M N D
              c.POINTER(c.c_int64), c.POINTER(c.c_int64), c.c_float]
    lib.fcr_version.restype = c.c_int
    lib.fcr_version.argtypes = []
    lib.fcr_last_error.restype = c.c_char_p
    lib.fcr_last_error.argtypes = []
    lib.fcr_lse_bytes.restype = c.c_size_t
    lib.fcr_lse_bytes.argtypes = [c.c_int, c.c_int, c.c_int, c.c_int, c.c_int]
    lib.fcr_row_lse.restype = c.c_int
    lib.fcr_row_lse.argtypes = [c.c_void_p, c.c_void_p, c.c_void_p] + common + [c.c_int, c.c_void_p]
    lib.fcr_col_reduce.restype = c.c_int
    lib.fcr_col_reduce.argtypes = ([c.c_void_p, c.c_void_p, c.c_void_p, c.c_void_p] + common +
                                   [c.c_int, c.c_int, c.c_void_p])
    lib.fcr_colreduce_sum_max.restype = c.c_int
    lib.fcr_colreduce_sum_max.argtypes = ([c.c_void_p] * 5 + common + [c.c_int, c.c_void_p])
    lib.fcr_colreduce_sum_max_to.restype = c.c_int
    lib.fcr_colreduce_sum_max_to.argtypes = ([c.c_void_p] * 4 + [c.c_int, c.c_void_p] + common +
                                             [c.c_int, c.c_int, c.c_void_p])
    lib.fcr_col_reduce_sum_max.restype = c.c_int
    lib.fcr_col_reduce_sum_max.argtypes = ([c.c_void_p] * 5 + common + [c.c_int, c.c_void_p])
    lib.fcr_topk_mask.restype = c.c_int
    lib.fcr_topk_mask.argtypes = [c.c_void_p, c.c_void_p, c.c_void_p, c.c_int64, c.c_int, c.c_int, c.c_void_p]
    lib.fcr_topk_mask_typed.restype = c.c_int
    lib.fcr_topk_mask_typed.argtypes = [c.c_void_p, c.c_int, c.c_void_p, c.c_void_p, c.c_int64, c.c_int, c.c_int,
                                        c.c_void_p, c.c_size_t, c.c_void_p]
    lib.fcr_topk_bytes.restype = c.c_size_t
    lib.fcr_topk_bytes.argtypes = [c.c_int64, c.c_int]
    lib.fcr_topk_mask_ws.restype = c.c_int
    lib.fcr_topk_mask_ws.argtypes = [c.c_void_p, c.c_void_p, c.c_void_p, c.c_int64, c.c_int, c.c_int, c.c_void_p,
                                     c.c_size_t, c.c_void_p]
    lib.fcr_pack_f32.restype = c.c_int
    lib.fcr_pack_f32.argtypes = [c.c_void_p, c.c_void_p, c.c_int64, c.c_int, c.c_int, c.c_int, c.c_void_p]
    lib.fcr_colreduce.restype = c.c_int
    lib.fcr_colreduce.argtypes = ([c.c_void_p, c.c_void_p, c.c_void_p, c.c_void_p] + common +
                                  [c.c_int, c.c_int, c.c_void_p])
    lib.fcr_colreduce_to.restype = c.c_int
    lib.fcr_colreduce_to.argtypes = ([c.c_void_p, c.c_void_p, c.c_void_p, c.c_int, c.c_void_p] + common +
                                     [c.c_int, c.c_int, c.c_void_p])
    lib.fcr_colreduce_static.restype = c.c_int
    lib.fcr_colreduce_static.argtypes = ([c.c_void_p, c.c_void_p, c.c_void_p] + common +
                                         [c.c_int, c.c_int, c.c_void_p])
    lib.fcr_set_option.restype = c.c_int
    lib.fcr_set_option.argtypes = [c.c_int, c.c_longlong]
    lib.fcr_colreduce_status.restype = c.c_int
    lib.fcr_colreduce_status.argtypes = [c.c_void_p] + [c.c_int] * 6 + [c.c_void_p]
    return lib


def load():
    """Open libfcr.so once per process."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m flash_colreduce_amd.build` "
                "(there is no fallback path)")
        _lib = _declare(ctypes.CDLL(LIB_PATH))
    return _lib


def strides4(values):
    return _I64x4(*[int(v) for v in values])


def check(rc: int):
    if rc != 0:
        raise FcrError(rc, load().fcr_last_error().decode("utf-8", "replace"))
