"""Latency / peak-memory sweep over the reference's 20 benchmark shapes.

    python -m flash_colreduce_amd.benchmark [--budget SECONDS] [--no-naive] [--rows 0,13] [--dtype fp16|bf16|fp32] [--out FILE]
    python -m flash_colreduce_amd.benchmark --shape 1,32,8192,8192,128,1 [--constant]     (one shape B,H,M,N,D,causal)
    python -m flash_colreduce_amd.benchmark --topk

Same shapes and method as the reference's harness (benchmarks/run.py:11-92): fp16, H = 32, D = 128,
reduction = "sum"; per implementation one call, a 10-call calibration, then `iters` warm-up calls and
`iters` timed calls between device synchronisations; peak memory is torch's max_memory_allocated
around one call.  `iters = max(int(budget / t_call), 10)`; the reference uses a 10 s budget, the
default here is 2 s.  Prints a plain-text table (the reference renders the same columns with rich).
"""
from __future__ import annotations

import argparse
import sys
import time

import torch

from . import flash_colreduce, naive_colreduce
from .flash import topk_keep_mask

CONFIGS = (
    [dict(b=b, h=32, m=1024, n=1024, d=128, is_causal=False) for b in (1, 4, 16, 64, 256)]
    + [dict(b=1, h=32, m=n, n=n, d=128, is_causal=False) for n in (1024, 2048, 4096, 8192, 16384)]
    + [dict(b=b, h=32, m=64, n=16384, d=128, is_causal=True) for b in (1, 4, 16, 64, 256)]
    + [dict(b=1, h=32, m=512, n=n, d=128, is_causal=True) for n in (16384, 32768, 65536, 131072, 262144)]
)


def _now() -> float:
    torch.cuda.synchronize()
    return time.perf_counter()


def measure_latency(fn, budget: float) -> float:
    fn()
    t0 = _now()
    for _ in range(10):
        fn()
    per_call = (_now() - t0) / 10
    iters = max(int(budget / max(per_call, 1e-9)), 10)
    for _ in range(iters):
        fn()
    t0 = _now()
    for _ in range(iters):
        fn()
    return (_now() - t0) / iters * 1e3


def measure_memory(fn) -> float:
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    torch.cuda.reset_peak_memory_stats()
    fn()
    torch.cuda.synchronize()
    return torch.cuda.max_memory_allocated() / 2**20


DTYPES = {"fp16": torch.float16, "bf16": torch.bfloat16, "fp32": torch.float32}


def run(budget: float = 2.0, with_naive: bool = True, out=sys.stdout, only=None, dtype: str = "fp16", shapes=CONFIGS,
        constant: bool = False):
    name = torch.cuda.get_device_name(0)
    print(f"Benchmark results on {name} ({dtype}, reduction=sum)", file=out)
    head = (f"{'configuration':<48} {'flash ms':>10} {'naive ms':>10} {'speedup':>8} {'flash MB':>10} "
            f"{'naive MB':>10} {'mem saving':>10} {'TFLOP/s':>9}")
    print(head, file=out)
    print("-" * len(head), file=out)
    rows = []
    with torch.inference_mode():
        for index, cfg in enumerate(shapes):
            if only is not None and index not in only:
                continue
            b, h, m, n, d, causal = (cfg[k] for k in ("b", "h", "m", "n", "d", "is_causal"))
            g = torch.Generator(device="cuda").manual_seed(0)
            q = torch.randn(b, h, m, d, device="cuda", dtype=DTYPES[dtype], generator=g)
            k = torch.randn(b, h, n, d, device="cuda", dtype=DTYPES[dtype], generator=g)
            if constant:   # every element 0.5: the same instructions on operands that toggle no bits
                q.fill_(0.5)
                k.fill_(0.5)
            flash = lambda: flash_colreduce(q, k, reduction="sum", is_causal=causal)  # noqa: E731
            naive = lambda: naive_colreduce(q, k, reduction="sum", is_causal=causal)  # noqa: E731
            f_ms, f_mb = measure_latency(flash, budget), measure_memory(flash)
            n_ms = n_mb = float("nan")
            if with_naive:
                try:
                    n_ms, n_mb = measure_latency(naive, budget), measure_memory(naive)
                except torch.OutOfMemoryError:
                    torch.cuda.empty_cache()
            # visible scores: right-aligned mask hides a triangle of side m-1 when causal
            visible = m * n - (m * (m - 1) // 2 if causal else 0)
            tflops = 4.0 * b * h * visible * d / (f_ms * 1e-3) / 1e12
            label = ",".join(f"{key}={val}" for key, val in cfg.items())
            print(f"{label:<48} {f_ms:>10.3f} {n_ms:>10.3f} {n_ms / f_ms:>8.2f} {f_mb:>10.1f} {n_mb:>10.1f} "
                  f"{n_mb / f_mb:>10.2f} {tflops:>9.1f}", file=out, flush=True)
            rows.append(dict(cfg, flash_ms=f_ms, naive_ms=n_ms, flash_mb=f_mb, naive_mb=n_mb, tflops=tflops))
            del q, k
            torch.cuda.empty_cache()
    return rows


TOPK_SHAPES = ((32, 8192, 2048), (32, 8192, 64), (32, 32768, 8192), (32, 32768, 512), (256, 8192, 2048),
               (32, 262144, 65536), (8, 1048576, 100000))


def run_topk(out=sys.stdout):
    """The step a pruning caller takes on the reduced columns: keep-mask of the k largest of every row,
    against torch.topk (+ the scatter that turns its indices into a mask) on the same GPU.  Times are
    events around 50 calls after 10 warm-up calls, host overhead of the call included."""
    def timed(fn):
        for _ in range(10):
            fn()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(50):
            fn()
        b.record()
        b.synchronize()
        return a.elapsed_time(b) / 50 * 1e3

    print(f"{'rows x columns, k':<34} {'topk_keep_mask us':>18} {'torch.topk us':>14} {'topk+scatter us':>16}", file=out)
    g = torch.Generator(device="cuda").manual_seed(0)
    cases = [(r, n, k, torch.float32) for r, n, k in TOPK_SHAPES]
    # 16-bit rows, what flash_colreduce returns for 16-bit operands (many ties: the masks may differ in which
    # of the equal values they keep, so only the number kept and the threshold are compared)
    cases += [(32, 8192, 2048, torch.float16), (32, 32768, 8192, torch.bfloat16), (32, 262144, 65536, torch.float16)]
    for rows, n, k, dt in cases:
        s = torch.rand(rows, n, device="cuda", generator=g).to(dt)

        def via_torch():
            idx = torch.topk(s, k, dim=-1).indices
            return torch.zeros_like(s, dtype=torch.bool).scatter_(1, idx, True)

        t_ours = timed(lambda: topk_keep_mask(s, k))
        t_topk = timed(lambda: torch.topk(s, k, dim=-1))
        t_mask = timed(via_torch)
        if dt == torch.float32:
            assert torch.equal(topk_keep_mask(s, k), via_torch())   # distinct values: both masks are the same set
        else:
            mask, thr = topk_keep_mask(s, k, return_threshold=True)
            assert bool((mask.sum(-1) == k).all()) and torch.equal(thr, torch.topk(s, k, dim=-1).values[:, -1].float())
        label = f"[{rows}, {n}], k={k} {str(dt)[6:]}"
        print(f"{label:<34} {t_ours:>18.1f} {t_topk:>14.1f} {t_mask:>16.1f}", file=out, flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--budget", type=float, default=2.0, help="seconds of timed calls per implementation")
    ap.add_argument("--no-naive", action="store_true", help="skip the materialising implementation")
    ap.add_argument("--rows", default=None, help="comma separated indices (0..19) of the shapes to run; default all")
    ap.add_argument("--out", default=None, help="also write the table to this file")
    ap.add_argument("--dtype", default="fp16", choices=sorted(DTYPES), help="element type of q and k (the reference's table is fp16)")
    ap.add_argument("--topk", action="store_true", help="time the top-k keep-mask against torch.topk instead")
    ap.add_argument("--shape", default=None, help="B,H,M,N,D,causal (0 or 1): this one shape instead of the table")
    ap.add_argument("--constant", action="store_true",
                    help="operands filled with 0.5 instead of N(0,1) draws (the clock the GPU keeps depends on the data)")
    args = ap.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("benchmark needs a GPU")
    if args.topk:
        run_topk()
        return
    only = None if args.rows is None else {int(r) for r in args.rows.split(",")}
    shapes = CONFIGS
    if args.shape:
        b, h, m, n, d, causal = (int(x) for x in args.shape.split(","))
        shapes, only = [dict(b=b, h=h, m=m, n=n, d=d, is_causal=bool(causal))], None
    kw = dict(only=only, dtype=args.dtype, shapes=shapes, constant=args.constant)
    if args.out:
        with open(args.out, "w") as f:
            run(args.budget, not args.no_naive, out=f, **kw)
        print(open(args.out).read())
    else:
        run(args.budget, not args.no_naive, **kw)


if __name__ == "__main__":
    main()
