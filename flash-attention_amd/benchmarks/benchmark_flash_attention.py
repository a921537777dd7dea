#!/usr/bin/env python3
"""Forward, backward and forward + backward throughput over the reference's own sweep
(benchmarks/benchmark_flash_attention.py:70-78 there): fp16, hidden size 2048, head dim 64 / 128,
(batch, seqlen) in {(32, 512), (16, 1k), (8, 2k), (4, 4k), (2, 8k), (1, 16k)}, causal or not,
dropout 0.  FLOPs as the reference counts them (:27-30): forward 4 b s^2 h d (halved if causal),
backward 2.5 x forward.  Timed with HIP events on the current stream after a warm-up.

    python flash-attention_amd/benchmarks/benchmark_flash_attention.py [--dtype bf16] [--repeats 30]
"""
import argparse
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from flash_attn import flash_attn_qkvpacked_func  # noqa: E402


def flops(batch, seqlen, headdim, nheads, causal, mode="fwd"):
    f = 4 * batch * seqlen ** 2 * nheads * headdim // (2 if causal else 1)
    return f if mode == "fwd" else (2.5 * f if mode == "bwd" else 3.5 * f)


def timed(fn, repeats, warmup=5):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(repeats):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / repeats * 1e-3


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--dtype", choices=["fp16", "bf16"], default="fp16")
    ap.add_argument("--repeats", type=int, default=30)
    a = ap.parse_args()
    dtype = torch.float16 if a.dtype == "fp16" else torch.bfloat16
    dim = 2048
    print("%-7s %-7s %-6s %-7s | %9s %9s %9s   (TFLOP/s)" % ("causal", "headdim", "batch", "seqlen", "fwd", "bwd", "fwd+bwd"))
    for causal in (False, True):
        for headdim in (64, 128):
            for batch, seqlen in ((32, 512), (16, 1024), (8, 2048), (4, 4096), (2, 8192), (1, 16384)):
                nheads = dim // headdim
                qkv = torch.randn(batch, seqlen, 3, nheads, headdim, device="cuda", dtype=dtype, requires_grad=True)
                out = flash_attn_qkvpacked_func(qkv, causal=causal)
                g = torch.randn_like(out)
                t_f = timed(lambda: flash_attn_qkvpacked_func(qkv, causal=causal), a.repeats)
                t_b = timed(lambda: out.backward(g, retain_graph=True), a.repeats)
                qkv.grad = None
                print("%-7s %-7d %-6d %-7d | %9.1f %9.1f %9.1f" % (
                    causal, headdim, batch, seqlen,
                    flops(batch, seqlen, headdim, nheads, causal, "fwd") / t_f / 1e12,
                    flops(batch, seqlen, headdim, nheads, causal, "bwd") / t_b / 1e12,
                    flops(batch, seqlen, headdim, nheads, causal, "fwd_bwd") / (t_f + t_b) / 1e12), flush=True)


if __name__ == "__main__":
    main()
