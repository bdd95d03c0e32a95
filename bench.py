#!/usr/bin/env python3
"""Benchmark of the column-reduction hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--cpu-heads H] [--no-configs]

One step = one fcr_colreduce call (row-statistics kernel + column-reduce kernel) on the headline
workload: causal, B=1, H=32, M=N=8192, D=128, fp16, reduction=sum, inputs resident in HBM, buffers
preallocated.  Prints ONE JSON line.

value        effective TFLOP/s = (4*B*H*M*N*D / 2) / wall time per step over exactly K steps between
             device synchronisations, after W warm-up steps.  Before the warm-up an untimed conditioning
             phase (`config.conditioning`) runs the same call for a fixed time so that the GPU has left
             its idle clocks; it is outside both `warmup` and `steps`.  `ms_per_step_events` times the
             same K steps with events on the launch stream.
roofline     the slower of the two kernels, timed alone with events on the launch stream, against
             the dense fp16 MFMA peak; `kernels` lists both.
cpu_baseline the CPU oracle (fp32 matmul, mask, softmax, column sum; chunked over query rows)
             timed on this host's cores on a sample of heads of the same workload; the same
             sample is used to check the GPU result against the tolerance of the metric.
configs      the five named workloads of the benchmark set: ms per call (events, after 0.25 s of untimed
             calls of the same workload), TFLOP/s by the
             metric's convention, fraction of the MFMA (and, for the decode-shaped one, HBM) roofline,
             the CPU oracle timed on a sample of heads, and the tolerance verdict per reduction.
             `kernel_us` is the same problem through the C ABI with preallocated buffers, many calls back to
             back between two events: the time of the call's kernels on the GPU as long as the host issues a
             call faster than that (`host_issue_us`); `ms` is the Python operator, torch allocations included.
             `--configs 2,3` restricts the set (and `--no-headline` skips the headline) for profiler runs.
decode       the HBM-bound shape of the reference's own benchmark table (causal B=64 H=32 M=64 N=16384 D=128
             fp16, sum; benchmarks/run.py:34-55): ms per call, and a `roofline` object of its own, the
             algorithmic bytes over the time of the call's kernels against the 8 TB/s HBM peak.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP16_DENSE_TFLOPS = 2516.6  # 256 CU x 2.4 GHz x 4096 flop/CU/clk, MI355X published dense fp16 (= bf16)
PEAK_HBM_TBPS = 8.0
# HBM bytes per launch on the headline workload, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs
# scaled by the same counters on a 256 MiB device copy (FETCH unit 2 KiB, WRITE unit 1 KiB);
# the summary of those runs is profiles/headline_causal_8192_fp16.md.  Against the 135.3 MB a launch has
# to move (q, k, the fp32 result) that is 1.70 times the bytes for the row sweep and 1.48 for the column
# sweep: streamed tiles that several workgroups ask for and that do not all meet in a cache.
HBM_TRAFFIC_BYTES = {"row_lse_kernel": 229.5e6 + 1.05e6, "col_reduce_kernel": 199.7e6 + 1.05e6}
# the same for the single sweep on the decode workload (profiles/decode_b64_m64_n16384_fp16.md): 9.00 GB read
# (1.045 times the keys and queries), 84.4 MB written
DECODE_TRAFFIC_BYTES = 9.00e9 + 84.4e6
CONDITIONING_SECONDS = 0.4
CONFIG_CONDITIONING_SECONDS = 0.25   # per workload and reduction of the configs array, untimed


def _events_ms(torch, fn, reps):
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        fn()
    b.record()
    b.synchronize()
    return a.elapsed_time(b) / reps


def _close(torch, got, want, reduction):
    """Tolerance of the metric: rtol 2e-3 / atol 1e-5 for sum and mean, 2e-3 relative for max."""
    err = (got - want).abs()
    if reduction == "max":
        rel = float((err / want.abs().clamp_min(1e-30)).max())
        return rel <= 2e-3, rel
    ok = bool((err <= 1e-5 + 2e-3 * want.abs()).all())
    return ok, float((err / (1e-5 + 2e-3 * want.abs())).max())   # worst error in units of the tolerance


def _c_abi_us(torch, qd, kd, red, causal, reps):
    """The call through the C ABI with preallocated buffers (fcr_colreduce_to, fp32 result), `reps` times back to
    back.  Returns (microseconds per call between two events on the stream, microseconds the host needs to
    issue one call).  While the host is the faster of the two the first number is the time of the call's
    kernels on the GPU."""
    from flash_colreduce_amd import _lib
    lib = _lib.load()
    b, h, m, d = qd.shape
    n = kd.shape[2]
    out = torch.empty(b, h, n, device=qd.device, dtype=torch.float32)
    lse = torch.empty(lib.fcr_lse_bytes(b, h, m, n, d) // 4, device=qd.device, dtype=torch.float32)
    dt = {torch.float16: _lib.DTYPE_F16, torch.bfloat16: _lib.DTYPE_BF16, torch.float32: _lib.DTYPE_F32}[qd.dtype]
    code = {"sum": _lib.REDUCE_SUM, "max": _lib.REDUCE_MAX, "mean": _lib.REDUCE_MEAN}[red]
    qs, ks = _lib.strides4(qd.stride()), _lib.strides4(kd.stride())
    stream = torch.cuda.current_stream(qd.device).cuda_stream
    args = (qd.data_ptr(), kd.data_ptr(), out.data_ptr(), _lib.DTYPE_F32, lse.data_ptr(), dt, b, h, m, n, d, qs, ks,
            1.0 / d ** 0.5, code, int(causal), stream)
    call = lambda: lib.fcr_colreduce_to(*args)
    for _ in range(3):
        _lib.check(call())
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    t0 = time.perf_counter()
    for _ in range(reps):
        call()
    host = (time.perf_counter() - t0) / reps * 1e6
    e1.record()
    e1.synchronize()
    return e0.elapsed_time(e1) / reps * 1e3, host


def run_decode(torch, fca, colreduce_ref):
    """The HBM-bound shape of the reference's benchmark table (benchmarks/run.py:34-55): causal B=64 H=32 M=64
    N=16384 D=128 fp16, sum.  The single sweep reads the 8.6 GB of keys once; its roofline is the HBM peak.
    Timed with events through the Python operator and through the C ABI; parity on two (b,h) pairs."""
    dev = torch.device("cuda:0")
    b, h, m, n, d = 64, 32, 64, 16384, 128
    g = torch.Generator(device="cuda").manual_seed(13)
    qd = torch.randn(b, h, m, d, device=dev, dtype=torch.float16, generator=g)
    kd = torch.randn(b, h, n, d, device=dev, dtype=torch.float16, generator=g)
    fn = lambda: fca.flash_colreduce(qd, kd, "sum", is_causal=True, out_dtype=torch.float32)
    got = fn()
    for _ in range(5):
        fn()
    torch.cuda.synchronize()
    ms = _events_ms(torch, fn, 20)
    kernel_us, host_us = _c_abi_us(torch, qd, kd, "sum", True, 20)
    pick = [(0, 0), (63, 31)]
    qs = torch.stack([qd[i, j] for i, j in pick]).unsqueeze(0).float().cpu()
    ks = torch.stack([kd[i, j] for i, j in pick]).unsqueeze(0).float().cpu()
    want = colreduce_ref(qs, ks, "sum", True)
    ok, worst = _close(torch, torch.stack([got[i, j] for i, j in pick]).unsqueeze(0).cpu(), want, "sum")
    bytes_alg = b * h * (m + n) * d * 2 + b * h * n * 4
    return {"name": "decode_b64_m64_n16384", "shape": {"B": b, "H": h, "M": m, "N": n, "D": d}, "dtype": "float16",
            "causal": True, "reduction": "sum", "algorithmic_bytes": bytes_alg, "ms": ms, "kernel_us": kernel_us,
            "host_issue_us": host_us, "launches_per_call": 2,
            "roofline": {"bound": "hbm", "kernel": "col_fused_kernel", "achieved": bytes_alg / (kernel_us * 1e-6) / 1e9,
                         "peak": PEAK_HBM_TBPS * 1e3, "unit": "GB/s",
                         "frac": bytes_alg / (kernel_us * 1e-6) / 1e12 / PEAK_HBM_TBPS,
                         "traffic": DECODE_TRAFFIC_BYTES},
            "pass": ok, "worst_err_over_tol": worst}


def run_configs(torch, fca, colreduce_ref, inputs, cores, only=None):
    """The five named workloads.  GPU: flash_colreduce (fp32 result) timed with events; CPU: the oracle
    on a head sample, timed once (configs 4, 5) or best of three (1-3); parity on that sample."""
    dev = torch.device("cuda:0")
    specs = [
        ("config1", inputs.config1, False, ("sum", "mean", "max"), None),
        ("config2", inputs.config2, False, ("sum", "mean", "max"), None),
        ("config3", inputs.config3, True, ("sum", "mean", "max"), None),
        ("config4", inputs.config4, True, ("sum",), [0, 10, 21, 31]),
        ("config5", inputs.config5, True, ("mean", "max"), [0, 9, 17, 31]),
    ]
    out = []
    for name, make, causal, reductions, heads in specs:
        if only is not None and int(name[-1]) not in only:
            continue
        q, k = make()
        b, h, m, d = q.shape
        n = k.shape[2]
        qd, kd = q.to(dev), k.to(dev)
        flop = 4.0 * b * h * m * n * d * (0.5 if causal else 1.0)
        bytes_alg = b * h * (m + n) * d * q.element_size() + b * h * n * 4
        hs = list(range(h)) if heads is None else heads
        qs, ks = q[:, hs].float(), k[:, hs].float()
        entry = {"name": name, "shape": {"B": b, "H": h, "M": m, "N": n, "D": d}, "dtype": str(q.dtype).split(".")[-1],
                 "causal": causal, "flop_per_call": flop, "algorithmic_bytes": bytes_alg,
                 "cpu_heads": len(hs), "cpu_cores": cores, "reductions": {}}
        for red in reductions:
            fn = lambda: fca.flash_colreduce(qd, kd, red, is_causal=causal, out_dtype=torch.float32)
            got = fn()
            torch.cuda.synchronize()
            reps = 5 if flop > 2e12 else (20 if flop > 1e11 else 100)
            # the CPU oracle ran in between: the same conditioning as for the headline before timing
            t0 = time.perf_counter()
            while time.perf_counter() - t0 < CONFIG_CONDITIONING_SECONDS:
                for _ in range(max(2, reps // 4)):
                    fn()
                torch.cuda.synchronize()
            ms = _events_ms(torch, fn, reps)
            kernel_us, host_us = _c_abi_us(torch, qd, kd, red, causal, max(reps, 50))
            cpu_s = None
            for _ in range(1 if flop > 1e11 else 3):
                t0 = time.perf_counter()
                want = colreduce_ref(qs, ks, red, causal)
                dt = time.perf_counter() - t0
                cpu_s = dt if cpu_s is None else min(cpu_s, dt)
            ok, worst = _close(torch, got[:, hs].cpu(), want, red)
            r = {"ms": ms, "kernel_us": kernel_us, "host_issue_us": host_us, "tflops": flop / (ms * 1e-3) / 1e12,
                 "frac_mfma_peak": flop / (ms * 1e-3) / 1e12 / PEAK_FP16_DENSE_TFLOPS,
                 "cpu_ms_per_call_extrapolated": cpu_s * 1e3 * h / len(hs),
                 "cpu_tflops": flop * len(hs) / h / cpu_s / 1e12, "pass": ok,
                 ("max_rel_err" if red == "max" else "worst_err_over_tol"): worst}
            if name == "config3":
                # decode shaped: bound by reading K; also the flop count of the scores actually visible
                visible = sum(min(n, i + max(n - m, 0) + 1) for i in range(m)) / float(m * n)
                r["tflops_visible_scores"] = 4.0 * b * h * m * n * d * visible / (ms * 1e-3) / 1e12
                r["frac_hbm_peak"] = bytes_alg / (ms * 1e-3) / 1e12 / PEAK_HBM_TBPS
                r["frac_hbm_peak_kernels"] = bytes_alg / (kernel_us * 1e-6) / 1e12 / PEAK_HBM_TBPS
            entry["reductions"][red] = r
        entry["pass"] = all(r["pass"] for r in entry["reductions"].values())
        out.append(entry)
        del qd, kd, q, k, qs, ks
        torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--cpu-heads", type=int, default=32,
                    help="heads of the workload the CPU oracle is timed on (0 = skip)")
    ap.add_argument("--no-configs", action="store_true", help="skip the five named workloads")
    ap.add_argument("--configs", type=str, default=None, help="comma separated subset of the named workloads, e.g. 2,3")
    ap.add_argument("--no-headline", action="store_true",
                    help="skip the headline workload (value, roofline and cpu_baseline are then null); for profiler runs")
    ap.add_argument("--conditioning", type=float, default=CONDITIONING_SECONDS,
                    help="seconds of untimed calls before the warm-up (0 = none)")
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
    import flash_colreduce_amd as fca
    from flash_colreduce_amd import _lib
    from flash_colreduce_amd import workloads as _inputs

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    lib = _lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    only = None if args.configs is None else {int(x) for x in args.configs.split(",") if x}
    METRIC = ("effective TFLOP/s (4*B*H*M*N*D, halved for causal) of flash_colreduce sum, causal B1 H32 M=N=8192 "
              "d128 fp16; one step = one fcr_colreduce call of the C ABI (both kernels, preallocated buffers, fp32 "
              "result); the Python operator on the same tensors is ms_per_step_python_api")
    if args.no_headline:
        from oracle.colreduce_oracle import colreduce_ref
        cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
        torch.set_num_threads(cores)
        configs = run_configs(torch, fca, colreduce_ref, _inputs, cores, only)
        print(json.dumps({"metric": METRIC, "value": None, "unit": "TFLOP/s", "n_gpus": 1, "steps": 0, "warmup": 0,
                          "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "fp16",
                          "data": "synthetic", "config": {"workload": "named workloads only (--no-headline)"},
                          "roofline": None, "cpu_baseline": None, "configs": configs}), flush=True)
        return

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

    # conditioning: the same call, untimed, until the clocks have left idle
    cond_calls = 0
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < args.conditioning:
        for _ in range(20):
            both()
        torch.cuda.synchronize()
        cond_calls += 20

    for _ in range(args.warmup):
        both()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        both()
    e1.record()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    ms_per_step_events = e0.elapsed_time(e1) / args.steps

    # the reference's own call on the same tensors: torch allocations, both kernels, fp16 result
    api = lambda: fca.flash_colreduce(q, k, "sum", is_causal=True)
    for _ in range(args.warmup):
        api()
    torch.cuda.synchronize()
    ms_per_step_python_api = _events_ms(torch, api, args.steps)

    reps = max(args.steps, 10)
    pass1()
    k1_ms = _events_ms(torch, pass1, reps)
    pass2()
    k2_ms = _events_ms(torch, pass2, reps)
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
                "frac": kernels[dom]["tflops"] / PEAK_FP16_DENSE_TFLOPS,
                "traffic": args.traffic_bytes if args.traffic_bytes is not None else HBM_TRAFFIC_BYTES[dom],
                "kernels": kernels, "whole_call_frac": value / PEAK_FP16_DENSE_TFLOPS}

    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    cpu_baseline = None
    parity = None
    from oracle.colreduce_oracle import colreduce_ref
    if args.cpu_heads > 0:
        hs = min(args.cpu_heads, H)
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
    del q, k, out, lse
    torch.cuda.empty_cache()

    configs = None if args.no_configs else run_configs(torch, fca, colreduce_ref, _inputs, cores, only)
    decode = None if args.no_configs else run_decode(torch, fca, colreduce_ref)

    line = {
        "metric": METRIC,
        "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "ms_per_step_events": ms_per_step_events,
        "ms_per_step_python_api": ms_per_step_python_api,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp16", "accumulate": "fp32", "data": "synthetic",
        "config": {"workload": "causal B=1 H=32 M=N=8192 D=128 fp16, reduction=sum, seed 0 N(0,1)",
                   "flop_per_call": flop_call, "frac_of_fp16_dense_peak": value / PEAK_FP16_DENSE_TFLOPS,
                   "conditioning": f"{cond_calls} untimed calls of the same workload over {args.conditioning} s "
                                   "before the warm-up (GPU clocks leave idle); not part of warmup or steps"},
        "roofline": roofline, "cpu_baseline": cpu_baseline, "parity": parity, "configs": configs,
        "decode": decode,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
