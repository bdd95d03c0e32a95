"""`flash_colreduce`: the reference's operator interface on top of libfcr.so.

Mirrors flash_colreduce/flash.py:311-385 (signature, validation order, error messages, default
scale, mean epilogue, output dtype).  The device work is two hand-written gfx950 kernels behind
a C ABI (include/fcr.h); torch is used for device memory and the current stream only.
"""
from __future__ import annotations

import functools
import math
from typing import Optional

import torch

from . import _lib

__all__ = ["flash_colreduce", "flash_colreduce_multi", "row_lse2", "topk_keep_mask"]

_DTYPES = {torch.float16: _lib.DTYPE_F16, torch.bfloat16: _lib.DTYPE_BF16, torch.float32: _lib.DTYPE_F32}


def _validate(query: torch.Tensor, key: torch.Tensor, reduction: Optional[str]):
    # flash.py:354-364, same order and messages
    if not query.is_cuda or not key.is_cuda:
        raise ValueError("Query and key tensors must be on CUDA device.")
    if query.dim() != 4 or key.dim() != 4 or not all(query.shape[i] == key.shape[i] for i in (0, 1, 3)):
        raise ValueError(
            f"Query and key tensors must have same batch size, number of heads, and head dimension. "
            f"Got query shape: {query.shape}, key shape: {key.shape}."
        )
    if reduction is not None and reduction not in ("sum", "mean", "max"):
        raise ValueError(f"Invalid reduction: {reduction}. Must be 'sum', 'mean', or 'max'.")
    if query.dtype != key.dtype or query.dtype not in _DTYPES:
        raise ValueError(
            f"Query and key tensors must both be float16, bfloat16 or float32. "
            f"Got query dtype: {query.dtype}, key dtype: {key.dtype}."
        )
    if query.device != key.device:
        raise ValueError("Query and key tensors must be on the same device.")
    # rows of at most 1 KiB (the reference pads any D to a power of two, flash.py:368-373, and runs what fits
    # its shared memory)
    limit = 1024 // query.element_size()
    if query.shape[3] > limit:
        raise ValueError(f"Head dimension must be <= {limit} for {query.dtype}. Got {query.shape[3]}.")


def _device_layout(x: torch.Tensor) -> torch.Tensor:
    """What the C ABI needs: unit d stride, 16-byte aligned rows, rows a multiple of 16 bytes.

    The reference pads D to a power of two (flash.py:368-373); zero columns do not change <q,k>.
    Here a copy is made only when a row is not a multiple of 16 bytes or for layouts the kernels
    cannot address.
    """
    d = x.shape[3]
    al = 16 // x.element_size()   # elements per 16 bytes: 8 (fp16, bf16) or 4 (fp32)
    if (d % al == 0 and x.is_contiguous() and x.data_ptr() % 16 == 0 and x.stride(2) == d and
            x.stride(0) % al == 0 and x.stride(1) % al == 0):
        return x   # the usual case (dimensions of size one may carry any stride, hence the last three tests)
    if d % al != 0:
        return torch.nn.functional.pad(x, (0, al - d % al))  # new contiguous tensor
    ok = (x.stride(3) == 1 and x.data_ptr() % 16 == 0 and
          all(x.stride(i) % al == 0 and x.stride(i) >= 0 for i in (0, 1, 2)) and
          x.stride(2) * x.element_size() < (1 << 25) and
          (x.shape[2] <= 1 or x.stride(2) >= d))  # rows must not overlap (expand() gives stride 0)
    if ok:
        return x
    # a contiguous tensor can still start at a misaligned address: contiguous() would hand it back
    return x.clone(memory_format=torch.contiguous_format) if x.is_contiguous() else x.contiguous()


def pack_f32(x: torch.Tensor, is_key: bool, terms: int = 3) -> torch.Tensor:
    """fp32 (B,H,R,D) -> the fp16 segments of fcr_pack_f32 (include/fcr.h), for callers of the C ABI that
    want fp32 operands multiplied on the 16-bit matrix instructions (16 times the fp32 rate) and accept
    fp16's range: terms = 3 gives products to about 2^-22 and needs 3 * ceil8(D) <= 256, terms = 1 is one
    rounding to fp16.  flash_colreduce itself never comes here: it multiplies fp32 operands in fp32."""
    b, h, r, d = x.shape
    dpad = (d + 7) // 8 * 8
    src = x.contiguous()
    dst = torch.empty((b, h, r, terms * dpad), device=x.device, dtype=torch.float16)
    if dst.numel():
        with torch.cuda.device(x.device):
            _lib.check(_lib.load().fcr_pack_f32(src.data_ptr(), dst.data_ptr(), b * h * r, d, terms,
                                                int(is_key), torch.cuda.current_stream(x.device).cuda_stream))
    return dst


def _operands(query, key):
    """query and key as the C ABI takes them."""
    return _device_layout(query), _device_layout(key)


_REDUCTIONS = {"sum": _lib.REDUCE_SUM, "max": _lib.REDUCE_MAX, "mean": _lib.REDUCE_MEAN}


@functools.lru_cache(maxsize=4096)
def _lse_floats(dev_index: int, b: int, h: int, m: int, n: int, d: int) -> int:
    """Floats of the row-statistics buffer (fcr_lse_bytes depends on the device's CU count, hence dev_index)."""
    with torch.cuda.device(dev_index):
        return max(b * h * m, _lib.load().fcr_lse_bytes(b, h, m, n, d) // 4)


def _raw_stream(dev: torch.device) -> int:
    """The current stream of `dev` as a hipStream_t value."""
    try:
        return torch._C._cuda_getCurrentRawStream(dev.index if dev.index is not None else torch.cuda.current_device())
    except AttributeError:   # the private shortcut is gone: the public, slower way
        return torch.cuda.current_stream(dev).cuda_stream


def _launch_to(query, key, reduction, is_causal, scale, res_dtype):
    """One reduction, finished on the device: the column kernel stores res_dtype and divides the means
    (fcr_colreduce_to), so nothing is left for torch to do after the two launches.  Needs M, N, B*H > 0."""
    b, h, m, d = query.shape
    n = key.shape[2]
    if scale is None:
        scale = 1 / math.sqrt(d)  # the unpadded D (flash.py:366-367)
    q, k = _operands(query, key)
    lib = _lib.load()
    dev = query.device
    index = dev.index if dev.index is not None else torch.cuda.current_device()
    lse = torch.empty(_lse_floats(index, b, h, m, n, q.shape[3]), device=dev, dtype=torch.float32)
    out = torch.empty((b, h, n), device=dev, dtype=res_dtype)
    args = (q.data_ptr(), k.data_ptr(), out.data_ptr(), _DTYPES[res_dtype], lse.data_ptr(), _DTYPES[q.dtype], b, h, m, n,
            q.shape[3], _lib.strides4(q.stride()), _lib.strides4(k.stride()), float(scale), _REDUCTIONS[reduction],
            1 if is_causal else 0)
    if torch.cuda.current_device() == index:
        rc = lib.fcr_colreduce_to(*args, _raw_stream(dev))
    else:
        with torch.cuda.device(index):
            rc = lib.fcr_colreduce_to(*args, _raw_stream(dev))
    if rc:
        _lib.check(rc)
    return out


def _launch_pair_to(query, key, sum_reduction, is_causal, scale, res_dtype):
    """Sums (or means) and maxima from one call, finished on the device (fcr_colreduce_sum_max_to)."""
    b, h, m, d = query.shape
    n = key.shape[2]
    if scale is None:
        scale = 1 / math.sqrt(d)  # the unpadded D (flash.py:366-367)
    q, k = _operands(query, key)
    lib = _lib.load()
    dev = query.device
    index = dev.index if dev.index is not None else torch.cuda.current_device()
    lse = torch.empty(_lse_floats(index, b, h, m, n, q.shape[3]), device=dev, dtype=torch.float32)
    sums = torch.empty((b, h, n), device=dev, dtype=res_dtype)
    maxs = torch.empty((b, h, n), device=dev, dtype=res_dtype)
    with torch.cuda.device(index):
        _lib.check(lib.fcr_colreduce_sum_max_to(
            q.data_ptr(), k.data_ptr(), sums.data_ptr(), maxs.data_ptr(), _DTYPES[res_dtype], lse.data_ptr(),
            _DTYPES[q.dtype], b, h, m, n, q.shape[3], _lib.strides4(q.stride()), _lib.strides4(k.stride()), float(scale),
            _REDUCTIONS[sum_reduction], 1 if is_causal else 0, _raw_stream(dev)))
    return sums, maxs


def _launch(query, key, kinds, is_causal, scale):
    """Runs the row kernel once and the column kernel for the entries of `kinds` ('sum' / 'max').

    Returns ([fp32 (B*H, N) per kind], fp32 lse (B*H*M,)).  All device memory comes from torch.
    """
    b, h, m, d = query.shape
    n = key.shape[2]
    if scale is None:
        scale = 1 / math.sqrt(d)  # the unpadded D (flash.py:366-367)
    q, k = _operands(query, key)
    lib = _lib.load()
    dev = query.device
    # the row statistics, followed by whatever scratch the row kernel wants for this shape
    index = dev.index if dev.index is not None else torch.cuda.current_device()
    lse = torch.empty(_lse_floats(index, b, h, m, n, q.shape[3]), device=dev, dtype=torch.float32)
    outs = [torch.empty((b * h, n), device=dev, dtype=torch.float32) for _ in kinds]
    if b * h * m * n == 0:
        lse.fill_(float("-inf"))
        for o in outs:
            o.zero_()
    else:
        with torch.cuda.device(dev):
            stream = torch.cuda.current_stream(dev).cuda_stream
            common = (_DTYPES[q.dtype], b, h, m, n, q.shape[3], _lib.strides4(q.stride()), _lib.strides4(k.stride()),
                      float(scale))
            causal = int(bool(is_causal))
            if len(kinds) == 1:
                red = _lib.REDUCE_MAX if kinds[0] == "max" else _lib.REDUCE_SUM
                _lib.check(lib.fcr_colreduce(q.data_ptr(), k.data_ptr(), outs[0].data_ptr(), lse.data_ptr(),
                                             *common, red, causal, stream))
            elif sorted(kinds) == ["max", "sum"]:
                # both kinds from one column sweep (few queries against many keys: from the single sweep)
                by_kind = dict(zip(kinds, outs))
                _lib.check(lib.fcr_colreduce_sum_max(q.data_ptr(), k.data_ptr(), by_kind["sum"].data_ptr(),
                                                     by_kind["max"].data_ptr(), lse.data_ptr(), *common, causal, stream))
            else:
                _lib.check(lib.fcr_row_lse(q.data_ptr(), k.data_ptr(), lse.data_ptr(), *common, causal, stream))
                for kind, o in zip(kinds, outs):
                    red = _lib.REDUCE_MAX if kind == "max" else _lib.REDUCE_SUM
                    _lib.check(lib.fcr_col_reduce(q.data_ptr(), k.data_ptr(), lse.data_ptr(), o.data_ptr(),
                                                  *common, red, causal, stream))
    return outs, lse[: b * h * m]


def _countdown(count: int, device: torch.device) -> torch.Tensor:
    """count, count-1, .., 1: the causal mean divisor from the offset on (flash.py:381-382).

    Built on the device by every call, on the caller's stream.  A tensor kept between calls would be
    wrong under HIP graph capture (its fill would only be recorded, and its memory would belong to the
    graph's pool) and would be shared between streams without an event."""
    return torch.arange(count, 0, -1, device=device)


def _finish(acc, reduction, query, m, n, is_causal, res_dtype, shared=False):
    """Cast of the fp32 accumulation and the mean epilogue, as flash.py:308 and 377-385.

    `shared`: the accumulation also feeds other results, so it must not be divided in place."""
    b, h = query.shape[0], query.shape[1]
    scores = acc.view(b, h, n).to(res_dtype, copy=shared)
    if reduction == "mean":
        # M for keys left of the offset, N-j from the offset on
        if is_causal:
            c = max(n - m, 0)
            scores[..., :c] /= m
            scores[..., c:] /= _countdown(n - c, query.device)
        else:
            scores /= m
    return scores


def flash_colreduce(
    query: torch.Tensor,
    key: torch.Tensor,
    reduction: str,
    is_causal: bool = False,
    scale: Optional[float] = None,
    *,
    out_dtype: Optional[torch.dtype] = None,
) -> torch.Tensor:
    """Per-key sum / mean / max over queries of softmax(Q K^T * scale), shape (B, H, N).

    Args follow the reference (flash.py:311-352): query (B,H,M,D), key (B,H,N,D), fp16, bf16 or
    fp32 on the GPU, rows of at most 1 KiB: D <= 512, D <= 256 for fp32 (fp32 operands are multiplied in fp32); `is_causal` applies the right-aligned mask (key j visible to query i iff
    j <= i + max(N-M, 0)); `scale` defaults to 1/sqrt(D).

    `out_dtype` (keyword only, not in the reference) selects the result dtype.  None reproduces
    the reference: the fp32 accumulation is cast to query.dtype and, for 'mean', divided in that
    dtype (flash.py:308, 377-385).  torch.float32 returns the kernel's fp32 result, with the
    mean division done in fp32.
    """
    _validate(query, key, reduction)
    b, h, m, _ = query.shape
    n = key.shape[2]
    res_dtype = query.dtype if out_dtype is None else out_dtype
    if m == 0 and n > 0 and b * h > 0 and reduction == "max":
        raise ValueError("reduction='max' needs at least one query row.")
    if m > 0 and b * h * n > 0 and res_dtype in _DTYPES:
        return _launch_to(query, key, reduction, is_causal, scale, res_dtype)
    if m == 0:
        acc = torch.zeros((b * h, n), device=query.device, dtype=torch.float32)
    else:
        (acc,), _ = _launch(query, key, ["max" if reduction == "max" else "sum"], is_causal, scale)
    return _finish(acc, reduction, query, m, n, is_causal, res_dtype)


def flash_colreduce_multi(
    query: torch.Tensor,
    key: torch.Tensor,
    reductions,
    is_causal: bool = False,
    scale: Optional[float] = None,
    *,
    out_dtype: Optional[torch.dtype] = None,
):
    """Several reductions of the same attention matrix; returns one (B, H, N) tensor per entry.

    Not in the reference, whose callers ask for one reduction per call and recompute everything
    (flash.py:311-385).  Here the row statistics are computed once and one column sweep produces the
    sums ('sum', 'mean') and the maxima together: 'mean' + 'max' costs two kernels instead of four.
    Results agree with flash_colreduce for each reduction (sums up to the order of fp32 additions).
    """
    reductions = list(reductions)
    if not reductions:
        raise ValueError("reductions must name at least one of 'sum', 'mean', 'max'.")
    _validate(query, key, reductions[0])
    for r in reductions[1:]:
        if r not in ("sum", "mean", "max"):
            raise ValueError(f"Invalid reduction: {r}. Must be 'sum', 'mean', or 'max'.")
    b, h, m, _ = query.shape
    n = key.shape[2]
    res_dtype = query.dtype if out_dtype is None else out_dtype
    if m == 0 and n > 0 and b * h > 0 and "max" in reductions:
        raise ValueError("reduction='max' needs at least one query row.")
    wanted = set(reductions)
    if m > 0 and b * h * n > 0 and res_dtype in _DTYPES and wanted in ({"sum", "max"}, {"mean", "max"}):
        # the usual pair: both results leave the kernel in their final form (fcr_colreduce_sum_max_to)
        sums, maxs = _launch_pair_to(query, key, "mean" if "mean" in wanted else "sum", is_causal, scale, res_dtype)
        out, seen = [], set()
        for r in reductions:   # an entry named twice gets a tensor of its own
            t = maxs if r == "max" else sums
            out.append(t.clone() if r in seen else t)
            seen.add(r)
        return tuple(out)
    kinds = []
    for r in reductions:
        kind = "max" if r == "max" else "sum"
        if kind not in kinds:
            kinds.append(kind)
    if m == 0:
        accs = [torch.zeros((b * h, n), device=query.device, dtype=torch.float32) for _ in kinds]
    else:
        accs, _ = _launch(query, key, kinds, is_causal, scale)
    by_kind = dict(zip(kinds, accs))
    return tuple(_finish(by_kind["max" if r == "max" else "sum"], r, query, m, n, is_causal, res_dtype,
                         shared=True) for r in reductions)


def row_lse2(query: torch.Tensor, key: torch.Tensor, is_causal: bool = False,
             scale: Optional[float] = None) -> torch.Tensor:
    """Base-2 log-sum-exp of every query row over its visible keys, fp32 (B, H, M).

    The hand-over between the two kernels, exposed for tests and for callers that want the
    softmax normaliser; the reference keeps it in registers (flash.py:242).
    """
    _validate(query, key, None)
    b, h, m, _ = query.shape
    _, lse = _launch(query, key, [], is_causal, scale)
    return lse.view(b, h, m)


def topk_keep_mask(scores: torch.Tensor, k: int, return_threshold: bool = False):
    """Boolean mask of the k largest entries along the last dimension (ties: lower index wins; a NaN
    ranks above +inf, as in torch.topk).

    The step a pruning caller takes on the (B, H, N) result of flash_colreduce; not part of the
    reference's package.  `scores` is a float32, float16 or bfloat16 GPU tensor; the result has its shape.
    With return_threshold also returns the k-th largest value per row, shape scores.shape[:-1].
    """
    if not scores.is_cuda:
        raise ValueError("scores must be on CUDA device.")
    if scores.dtype not in _DTYPES or scores.dim() < 1:
        raise ValueError(f"scores must be a float32, float16 or bfloat16 tensor with at least one dimension. "
                         f"Got {scores.dtype}.")
    s = scores.contiguous()   # 16-bit scores (what flash_colreduce returns for 16-bit operands) are read as they are
    n = s.shape[-1]
    rows = s.numel() // n if n else 0
    if rows > 0 and n > 0:
        mask = torch.empty(s.shape, device=s.device, dtype=torch.bool)   # the kernel writes every entry
    else:
        mask = torch.zeros(s.shape, device=s.device, dtype=torch.bool)
    thr = torch.empty(s.shape[:-1], device=s.device, dtype=torch.float32) if return_threshold else None   # always fp32
    if rows > 0 and n > 0:
        lib = _lib.load()
        nbytes = lib.fcr_topk_bytes(rows, n)   # > 0 for long rows: scratch that lets workgroups share a row
        ws = torch.empty(nbytes, device=s.device, dtype=torch.uint8) if nbytes else None
        with torch.cuda.device(s.device):
            _lib.check(lib.fcr_topk_mask_typed(s.data_ptr(), _DTYPES[s.dtype], mask.data_ptr(),
                                               thr.data_ptr() if thr is not None else None, rows, n, int(k),
                                               ws.data_ptr() if ws is not None else None, nbytes,
                                               torch.cuda.current_stream(s.device).cuda_stream))
    return (mask, thr) if return_threshold else mask
