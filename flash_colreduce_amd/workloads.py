"""Seeded synthetic inputs shared by the benchmark, the smoke test and the GPU parity tests.

Everything is drawn from the CPU generator in fp32 and then cast, so the CPU oracle and the
GPU kernel see identical bits.  config1..config5 and headline are the benchmark set's named workloads.
"""
from __future__ import annotations

import torch


def randn_pair(b, h, m, n, d, seed, dtype=torch.float16):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(b, h, m, d, generator=g, dtype=torch.float32)
    k = torch.randn(b, h, n, d, generator=g, dtype=torch.float32)
    return q.to(dtype), k.to(dtype)


def config1():
    """fp32 CPU case: [1,2,256,64] x [1,2,256,64], non-causal."""
    return randn_pair(1, 2, 256, 256, 64, seed=1, dtype=torch.float32)


def config2():
    """Non-causal fp16 [8,16,512,64]."""
    return randn_pair(8, 16, 512, 512, 64, seed=2, dtype=torch.float16)


def config3():
    """Causal decode-style fp16: q [1,32,128,128], k [1,32,4096,128]."""
    return randn_pair(1, 32, 128, 4096, 128, seed=3, dtype=torch.float16)


def config4(heads=32, n=8192):
    """Visual-token pruning prefill, causal bf16, heavy-hitter key columns."""
    g = torch.Generator().manual_seed(4)
    q = torch.randn(1, heads, n, 128, generator=g, dtype=torch.float32)
    k = torch.randn(1, heads, n, 128, generator=g, dtype=torch.float32)
    idx = torch.randperm(n, generator=g)[: max(1, n // 100)]
    k0 = k[:, :, 0, :].clone()
    k[:, :, idx, :] *= 4
    k[:, :, 0, :] = 8 * k0
    return q.to(torch.bfloat16), k.to(torch.bfloat16)


def config5(heads=32, n=32768):
    """Long-context KV pruning, causal bf16, per-head key mean offset ~ N(0, 0.5)."""
    g = torch.Generator().manual_seed(5)
    q = torch.randn(1, heads, n, 128, generator=g, dtype=torch.float32)
    k = torch.randn(1, heads, n, 128, generator=g, dtype=torch.float32)
    k += 0.5 * torch.randn(1, heads, 1, 128, generator=g, dtype=torch.float32)
    return q.to(torch.bfloat16), k.to(torch.bfloat16)


def headline():
    """The benchmark configuration: causal fp16 [1,32,8192,128] x 2."""
    return randn_pair(1, 32, 8192, 8192, 128, seed=0, dtype=torch.float16)
