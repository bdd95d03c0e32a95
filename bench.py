#!/usr/bin/env python3
"""Benchmark of the column-reduction hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--cpu-heads H]

One step = one fcr_colreduce call (row-statistics kernel + column-reduce kernel) on the headline
workload: causal, B=1, H=32, M=N=8192, D=128, fp16, reduction=sum, inputs
resident in HBM, buffers preallocated.  Prints ONE JSON line.

value        effective TFLOP/s = (4*B*H*M*N*D / 2) / time per call (flop convention of the metric).
roofline     the slower of the two kernels, timed alone with events on the launch stream, against
             the dense fp16 MFMA peak; `kernels` lists both.
cpu_baseline the CPU oracle (fp32 matmul, mask, softmax, column sum; chunked over query rows)
             timed on this host's cores on a sample of heads of the same workload; the same
             sample is used to check the GPU result against the tolerance of the metric.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP16_DENSE_TFLOPS = 2516.6  # 256 CU x 2.4 GHz x 4096 flop/CU/clk, MI355X published dense fp16
# HBM bytes per launch on the headline workload, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs
# scaled by the same counters on a 256 MiB device copy (FETCH unit 2 KiB, WRITE unit 1 KiB);
# the summary of those runs is profiles/headline_causal_8192_fp16.md.
HBM_TRAFFIC_BYTES = {"row_lse_kernel": 198.1e6 + 1.05e6, "col_reduce_kernel": 186.0e6 + 1.05e6}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--cpu-heads", type=int, default=32,
                    help="heads of the workload the CPU oracle is timed on (0 = skip)")
    ap.add_argument("--copy-calib", action="store_true",
                    help="also run one plain 256 MiB device copy, as the known-size reference for "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE counters")
    ap.add_argument("--traffic-bytes", type=float, default=None,
                    help="override roofline.traffic (HBM bytes per launch of the dominant kernel)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (every (b,h) pair is independent and would shard "
              "across GPUs without any exchange, but no multi-GPU path is built); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from flash_colreduce_amd import _lib
    from tests import _inputs

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    lib = _lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    B, H, M, N, D = 1, 32, 8192, 8192, 128
    q_cpu, k_cpu = _inputs.headline()
    q, k = q_cpu.to(dev), k_cpu.to(dev)
    out = torch.empty(B * H, N, device=dev, dtype=torch.float32)
    lse = torch.empty(lib.fcr_lse_bytes(B, H, M, N, D) // 4, device=dev, dtype=torch.float32)
    scale = 1.0 / (D ** 0.5)
    stream = torch.cuda.current_stream(dev).cuda_stream
    common = (_lib.DTYPE_F16, B, H, M, N, D, _lib.strides4(q.stride()), _lib.strides4(k.stride()), scale)

    def both():
        _lib.check(lib.fcr_colreduce(q.data_ptr(), k.data_ptr(), out.data_ptr(), lse.data_ptr(), *common,
                                     _lib.REDUCE_SUM, 1, stream))

    def pass1():
        _lib.check(lib.fcr_row_lse(q.data_ptr(), k.data_ptr(), lse.data_ptr(), *common, 1, stream))

    def pass2():
        _lib.check(lib.fcr_col_reduce(q.data_ptr(), k.data_ptr(), lse.data_ptr(), out.data_ptr(), *common,
                                      _lib.REDUCE_SUM, 1, stream))

    for _ in range(args.warmup):
        both()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        both()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    def event_ms(fn, reps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        fn()
        a.record()
        for _ in range(reps):
            fn()
        b.record()
        b.synchronize()
        return a.elapsed_time(b) / reps

    reps = max(args.steps, 10)
    k1_ms, k2_ms = event_ms(pass1, reps), event_ms(pass2, reps)
    if args.copy_calib:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()

    flop_call = 4.0 * B * H * M * N * D / 2.0       # two masked GEMMs, causal halves the work
    flop_kernel = flop_call / 2.0
    value = flop_call / (ms_per_step * 1e-3) / 1e12
    kernels = {
        "row_lse_kernel": {"ms": k1_ms, "tflops": flop_kernel / (k1_ms * 1e-3) / 1e12},
        "col_reduce_kernel": {"ms": k2_ms, "tflops": flop_kernel / (k2_ms * 1e-3) / 1e12},
    }
    dom = max(kernels, key=lambda n: kernels[n]["ms"])
    roofline = {"bound": "mfma", "kernel": dom, "achieved": kernels[dom]["tflops"],
                "peak": PEAK_FP16_DENSE_TFLOPS, "unit": "TFLOP/s",
                "frac": kernels[dom]["tflops"] / PEAK_FP16_DENSE_TFLOPS, "traffic": args.traffic_bytes if args.traffic_bytes is not None else HBM_TRAFFIC_BYTES[dom],
                "kernels": kernels, "whole_call_frac": value / PEAK_FP16_DENSE_TFLOPS}

    cpu_baseline = None
    parity = None
    if args.cpu_heads > 0:
        from oracle.colreduce_oracle import colreduce_ref
        hs = min(args.cpu_heads, H)
        cores = os.cpu_count() or 1
        cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
        torch.set_num_threads(cores)
        qs, ks = q_cpu[:, :hs].float(), k_cpu[:, :hs].float()
        colreduce_ref(qs[:, :1], ks[:, :1], "sum", True)  # warm the thread pool
        t0 = time.perf_counter()
        want = colreduce_ref(qs, ks, "sum", True)
        cpu_s = time.perf_counter() - t0
        cpu_baseline = {"value": (flop_call * hs / H) / cpu_s / 1e12, "unit": "TFLOP/s", "cores": cores,
                        "kind": "port",
                        "sample": f"{hs} of {H} heads of the same workload, fp32 torch-CPU oracle "
                                  f"(matmul, mask, softmax, column sum; 4096-row chunks), {cpu_s:.2f} s",
                        "ms_per_call_extrapolated": cpu_s * 1e3 * H / hs}
        got = out.view(B, H, N)[:, :hs].cpu()
        err = (got - want).abs()
        ok = bool((err <= 1e-5 + 2e-3 * want.abs()).all())
        parity = {"heads_checked": hs, "rtol": 2e-3, "atol": 1e-5, "pass": ok,
                  "max_abs_err": float(err.max()), "max_rel_err": float((err / want.abs().clamp_min(1e-30)).max())}

    line = {
        "metric": "effective TFLOP/s (4*B*H*M*N*D, halved for causal) of flash_colreduce sum, "
                  "causal B1 H32 M=N=8192 d128 fp16",
        "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp16", "accumulate": "fp32", "data": "synthetic",
        "config": {"workload": "causal B=1 H=32 M=N=8192 D=128 fp16, reduction=sum, seed 0 N(0,1)",
                   "flop_per_call": flop_call, "frac_of_fp16_dense_peak": value / PEAK_FP16_DENSE_TFLOPS},
        "roofline": roofline, "cpu_baseline": cpu_baseline, "parity": parity,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
