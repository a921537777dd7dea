#!/usr/bin/env python3
"""Benchmark of the MI355X FlashAttention forward path (one GPU).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-decode] [--no-backward] [--no-cpu]

One "step" is one forward pass over one synthetic batch already resident in HBM:
  * prefill  -- flash_attn_func, bf16, batch 4, seqlen 8192, 32 heads, head dim 128, causal
                (the configuration the headline metric is quoted on); value = TFLOP/s with the
                reference's FLOP convention 4*b*s^2*h*d/2 (benchmarks/benchmark_flash_attention.py:27-30);
  * decode   -- flash_attn_with_kvcache, bf16, batch 64, 1 new token appended with rotary, caches
                (64, 32768, 8, 128), 64 query heads, cache_seqlens uniform in [1024, 32767] at the start of
                every timed block and one longer after every step (a decoding loop: each step appends where
                the last one stopped); reported as achieved HBM GB/s over the algorithmic bytes.
  * rotary   -- apply_rotary_emb in place on (8, 8192, 32, 128) bf16 (the standalone rotary kernel), GB/s
                over 2 x the tensor's bytes;
  * backward -- gradients of the prefill workload (rowsum(dO o O), dQ pass, dK/dV pass); reported under
                "backward" at the conventional 2.5 x forward FLOP count.
  * fwd_bwd  -- the one kernel metric the reference publishes (forward + backward together, fp16, causal,
                head dim 128, seqlen 8k, batch 2, 16 heads: 182 TFLOP/s on A100, 308 on H100), FLOPs
                counted as 3.5 x forward like the reference's benchmark script;
  * varlen   -- flash_attn_varlen_func, bf16, 64 packed sequences with lengths uniform in [128, 4096]
                (seed 0), 16 heads, head dim 128 and 256, causal; FLOPs over the visible (row, key) pairs;
  * gqa_window -- flash_attn_func, bf16, batch 2, seqlen 16384, 32 query / 8 kv heads, head dim 128, causal
                with window (4096, 0); FLOPs over the visible pairs (sum_i min(i + 1, 4097) per head);
  * config1  -- flash_attn_func, fp16, batch 2, seqlen 512, 8 heads, head dim 64, non-causal (the reference's own
                CPU-runnable case): 1 GFLOP per call, so what is measured is the latency of one launch;
Prints ONE JSON line.  The CPU baseline is the oracle (a restatement of the reference's
attention_ref) timed on the host cores on a bounded sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "flash-attention_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E


def _traffic(key):
    """Measured HBM bytes per launch from the committed rocprofv3 --pmc summaries, if recorded."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    try:
        with open(path) as f:
            return json.load(f).get(key)
    except (OSError, ValueError):
        return None


BLOCKS = 3   # timed blocks of `steps` launches each; the median block is reported, the fastest beside it


class Timing(tuple):
    """(ms, wall_ms) of the median block, with .ms_min = the fastest block's ms per step."""
    def __new__(cls, ms, wall_ms, ms_min):
        t = super().__new__(cls, (ms, wall_ms))
        t.ms_min = ms_min
        return t


def time_steps(fn, steps, warmup, before_block=None):
    """`warmup` untimed calls, then BLOCKS blocks of exactly `steps` calls, each bracketed by HIP events
    on the stream the kernels are launched on (torch's current stream) and by a device synchronisation.
    `before_block` runs (untimed) ahead of the warm-up and of every block: a workload whose steps move its
    state puts the state back there."""
    import torch
    if before_block is not None:
        before_block()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    blocks = []
    for _ in range(BLOCKS):
        if before_block is not None:
            before_block()
            torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3
        blocks.append((e0.elapsed_time(e1) / steps, wall_ms / steps))
    blocks.sort()
    med = blocks[len(blocks) // 2]
    return Timing(med[0], med[1], blocks[0][0])


def bench_prefill(steps, warmup):
    import torch
    import flash_attn
    b, s, h, d = 4, 8192, 32, 128
    torch.manual_seed(0)
    q, k, v = (torch.randn(b, s, h, d, device="cuda", dtype=torch.bfloat16) for _ in range(3))
    fn = lambda: flash_attn.flash_attn_func(q, k, v, causal=True)
    tm = time_steps(fn, steps, warmup)
    ms, wall_ms = tm
    flops = 4.0 * b * s * s * h * d / 2
    tflops = flops / (ms * 1e-3) / 1e12
    return {
        "ms": ms, "ms_min": tm.ms_min, "wall_ms": wall_ms, "tflops": tflops, "tokens_per_s": b * s / (ms * 1e-3),
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": tflops / PEAK_BF16_TFLOPS, "traffic": _traffic("prefill_bf16_d128_causal_8k"), "traffic_source": "profiles/traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, not measured in this run)",
                     "kernel": "fa::prefill_pp16_kernel<bf16,128,64,128,2>", "flops_per_launch": flops},
    }


def bench_head_dims(steps, warmup):
    """Head dims between the buckets (bf16 causal, 4 x 8192, 32 heads): 96 runs on the 128-wide tiles and 192
    on the 256-wide ones with the k-steps and output column blocks past the head dim left out; FLOPs are
    counted at the real head dim."""
    import torch
    import flash_attn
    b, s, h = 4, 8192, 32
    res = {}
    for d, kern in ((96, "fa::prefill_pp16_kernel<bf16,128,64,96,2>"), (192, "fa::prefill_pp16_kernel<bf16,256,32,192,2>")):
        torch.manual_seed(0)
        q, k, v = (torch.randn(b, s, h, d, device="cuda", dtype=torch.bfloat16, requires_grad=True) for _ in range(3))
        with torch.no_grad():
            tm = time_steps(lambda: flash_attn.flash_attn_func(q, k, v, causal=True), steps, warmup)
        o = flash_attn.flash_attn_func(q, k, v, causal=True)
        do = torch.randn_like(o)
        tb = time_steps(lambda: torch.autograd.grad(o, (q, k, v), do, retain_graph=True), max(1, steps // 3), max(1, warmup // 3))
        flops = 4.0 * b * s * s * h * d / 2
        tf, tfb = flops / (tm[0] * 1e-3) / 1e12, 2.5 * flops / (tb[0] * 1e-3) / 1e12
        res["d%d" % d] = {
            "ms": tm[0], "ms_min": tm.ms_min, "tflops": tf,
            "roofline": {"bound": "mfma", "achieved": tf, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": tf / PEAK_BF16_TFLOPS,
                         "traffic": _traffic("head_dim_%d_bf16_causal_8k" % d),
                         "traffic_source": "profiles/traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, not measured in this run)",
                         "kernel": kern, "flops_per_launch": flops},
            "backward": {"ms": tb[0], "ms_min": tb.ms_min, "tflops": tfb, "frac": tfb / PEAK_BF16_TFLOPS},
        }
        del q, k, v, o, do
    return res


def bench_mfma_peak(steps, warmup):
    """What the matrix pipes sustain on MFMAs alone (fa_mfma_peak in the library): the clock of the fully
    loaded part follows the switching activity of the operands, so the figure is taken on random bf16
    operands (comparable to Gaussian q, k, v) and on zeros."""
    import ctypes
    import torch
    from flash_attn import _native as nat
    lib = nat.lib
    lib.fa_mfma_peak_shape.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.POINTER(ctypes.c_int64), ctypes.c_void_p]
    lib.fa_mfma_peak_shape.restype = ctypes.c_int
    sink = torch.zeros(1, dtype=torch.float32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    res = {"kernel": "fa::mfma_peak_kernel (independent v_mfma_f32_32x32x16_bf16 -- and, under \"shape_16x16x32\", v_mfma_f32_16x16x32_bf16 --, 4 waves per SIMD, operands in registers)"}

    def leg(rnd, shape):
        flops = ctypes.c_int64(0)

        def fn():
            rc = lib.fa_mfma_peak_shape(sink.data_ptr(), 1500, rnd, shape, ctypes.byref(flops), stream)
            if rc != 0:
                raise RuntimeError("fa_mfma_peak_shape failed: %d" % rc)
        tm = time_steps(fn, max(3, steps // 3), max(2, warmup // 3))
        return {"ms": tm[0], "ms_min": tm.ms_min, "tflops": flops.value / (tm[0] * 1e-3) / 1e12,
                "frac_of_published_peak": flops.value / (tm[0] * 1e-3) / 1e12 / PEAK_BF16_TFLOPS}
    for name, rnd in (("random_bf16", 1), ("zeros", 0)):
        res[name] = leg(rnd, 0)
    res["shape_16x16x32"] = {"random_bf16": leg(1, 1), "zeros": leg(0, 1)}
    return res


def bench_hbm_peak(steps, warmup):
    """What a kernel that only reads sustains from HBM (fa_hbm_read_peak in the library) over as many bytes as
    the decode step moves, with ordinary and with non-temporal loads."""
    import ctypes
    import torch
    from flash_attn import _native as nat
    lib = nat.lib
    lib.fa_hbm_read_peak.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p]
    lib.fa_hbm_read_peak.restype = ctypes.c_int
    nbytes = 4544733184 // 16 * 16
    src = torch.empty(nbytes // 2, dtype=torch.bfloat16, device="cuda").normal_()
    sink = torch.zeros(1, dtype=torch.int32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    res = {"kernel": "fa::hbm_read_peak_kernel (16-byte loads, 8 in flight per lane, a contiguous share per workgroup, nothing written)", "bytes_per_launch": nbytes}
    for name, nt in (("nontemporal", 1), ("ordinary", 0)):
        def fn():
            rc = lib.fa_hbm_read_peak(src.data_ptr(), nbytes, nt, sink.data_ptr(), stream)
            if rc != 0:
                raise RuntimeError("fa_hbm_read_peak failed: %d" % rc)
        tm = time_steps(fn, max(3, steps // 3), max(2, warmup // 3))
        gbs = nbytes / (tm[0] * 1e-3) / 1e9
        res[name] = {"ms": tm[0], "ms_min": tm.ms_min, "gb_per_s": gbs, "frac_of_published_peak": gbs / PEAK_HBM_GBS}
    return res


def bench_lds_peak(steps, warmup):
    """What the LDS of a CU delivers to 16-byte-per-lane reads (fa_lds_read_peak in the library), with one and
    with two waves per SIMD, in bytes per shader clock; at the full matrix rate the operand fragments of the
    attention kernels need 128."""
    import ctypes
    import torch
    from flash_attn import _native as nat
    lib = nat.lib
    lib.fa_lds_read_peak.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.POINTER(ctypes.c_int64),
                                     ctypes.c_void_p, ctypes.c_void_p]
    lib.fa_lds_read_peak.restype = ctypes.c_int
    wgs = 256
    cycles = torch.zeros(wgs, dtype=torch.int64, device="cuda")
    sink = torch.zeros(1, dtype=torch.int32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    res = {"kernel": "fa::lds_read_peak_kernel (ds_read_b128, 1 KB per wave instruction, no bank conflicts, one workgroup per CU)"}
    for waves in (4, 8):
        nbytes = ctypes.c_int64(0)
        for _ in range(3):
            rc = lib.fa_lds_read_peak(cycles.data_ptr(), wgs, waves, 5000, ctypes.byref(nbytes), sink.data_ptr(), stream)
            if rc != 0:
                raise RuntimeError("fa_lds_read_peak failed: %d" % rc)
        torch.cuda.synchronize()
        res["waves_per_simd_%d" % (waves // 4)] = {"bytes_per_clock_per_cu": nbytes.value / cycles.double().mean().item()}
    return res


def bench_rotary(steps, warmup):
    import torch
    from flash_attn.layers.rotary import apply_rotary
    b, s, h, d = 8, 8192, 32, 128
    torch.manual_seed(0)
    x = torch.randn(b, s, h, d, device="cuda", dtype=torch.bfloat16)
    ang = torch.rand(s, d // 2, device="cuda") * 6.28
    cos, sin = torch.cos(ang).to(torch.bfloat16), torch.sin(ang).to(torch.bfloat16)
    fn = lambda: apply_rotary(x, cos, sin, inplace=True)
    tm = time_steps(fn, steps, warmup)
    ms, wall_ms = tm
    algo_bytes = 2 * x.numel() * x.element_size()
    gbs = algo_bytes / (ms * 1e-3) / 1e9
    return {
        "ms": ms, "ms_min": tm.ms_min, "wall_ms": wall_ms, "gb_per_s": gbs,
        "workload": "apply_rotary_emb bf16 (8, 8192, 32, 128) rotary_dim 128 in place",
        "roofline": {"bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS,
                     "traffic": _traffic("rotary_bf16_8x8192x32x128_inplace"),
                     "traffic_source": "profiles/traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, not measured in this run)",
                     "kernel": "fa::rotary_kernel<bf16,bf16,u32,stream>", "bytes_per_launch": algo_bytes},
    }


def bench_backward(steps, warmup):
    import torch
    from flash_attn import _native as nat
    b, s, h, d = 4, 8192, 32, 128
    torch.manual_seed(0)
    q, k, v, dout = (torch.randn(b, s, h, d, device="cuda", dtype=torch.bfloat16) for _ in range(4))
    scale = d ** -0.5
    out, _, _, _, _, lse, _, _ = nat.fwd(q, k, v, None, 0.0, scale, True, -1, -1, False, None)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    fn = lambda: nat.bwd(dout, q, k, v, out, lse, dq, dk, dv, 0.0, scale, True, -1, -1, None, None)
    tm = time_steps(fn, steps, warmup)
    ms, wall_ms = tm
    flops = 2.5 * 4.0 * b * s * s * h * d / 2      # 5 products of 2 b h s^2 d / 2 (causal)
    tflops = flops / (ms * 1e-3) / 1e12
    return {
        "ms": ms, "ms_min": tm.ms_min, "wall_ms": wall_ms, "tflops": tflops,
        "workload": "flash_attn_func bwd bf16 batch=4 seqlen=8192 nheads=32 headdim=128 causal (dot + dQ + dK/dV kernels)",
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": tflops / PEAK_BF16_TFLOPS, "traffic": _traffic("backward_bf16_d128_causal_8k"),
                     "traffic_source": "profiles/traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, not measured in this run)",
                     "kernel": "fa::bwd_dkv3_kernel<bf16,128,64> + fa::bwd_dq_kernel<bf16,128,32> (7 tile products executed for 5 counted)",
                     "flops_per_launch": flops},
    }


def bench_varlen(steps, warmup):
    import torch
    import flash_attn
    torch.manual_seed(0)
    lens = torch.randint(128, 4097, (64,))
    cu = torch.cat([torch.zeros(1, dtype=torch.long), lens.cumsum(0)]).to(torch.int32)
    total, mx, h = int(cu[-1]), int(lens.max()), 16
    cu_d = cu.cuda()
    res = {"workload": "flash_attn_varlen_func fwd bf16 64 sequences U[128,4096] (%d tokens) nheads=16 causal" % total}
    for d in (128, 256):
        q, k, v = (torch.randn(total, h, d, device="cuda", dtype=torch.bfloat16) for _ in range(3))
        fn = lambda: flash_attn.flash_attn_varlen_func(q, k, v, cu_d, cu_d, mx, mx, causal=True)
        tm = time_steps(fn, steps, warmup)
        ms, wall_ms = tm
        flops = sum(4.0 * h * d * (int(l) * (int(l) + 1) / 2) for l in lens)
        tflops = flops / (ms * 1e-3) / 1e12
        res["d%d" % d] = {"ms": ms, "ms_min": tm.ms_min, "wall_ms": wall_ms, "tflops": tflops, "tokens_per_s": total / (ms * 1e-3),
                          "roofline": {"bound": "mfma", "achieved": tflops, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                                       "frac": tflops / PEAK_BF16_TFLOPS, "traffic": _traffic("varlen_bf16_d%d_64seq_h16" % d),
                                       "traffic_source": "profiles/traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, not measured in this run)",
                                       "kernel": "fa::prefill_pp16_kernel<bf16,128,64,128,2>" if d == 128 else "fa::prefill_pp16_kernel<bf16,256,32,256,1>",
                                       "flops_per_launch": flops}}
        del q, k, v
    return res


def bench_gqa_window(steps, warmup):
    import torch
    import flash_attn
    b, s, h, hk, d, wl = 2, 16384, 32, 8, 128, 4096
    torch.manual_seed(0)
    q = torch.randn(b, s, h, d, device="cuda", dtype=torch.bfloat16)
    k, v = (torch.randn(b, s, hk, d, device="cuda", dtype=torch.bfloat16) for _ in range(2))
    fn = lambda: flash_attn.flash_attn_func(q, k, v, causal=True, window_size=(wl, 0))
    tm = time_steps(fn, steps, warmup)
    ms, wall_ms = tm
    pairs = (wl + 1) * (wl + 2) // 2 + (s - wl - 1) * (wl + 1)       # sum_i min(i + 1, wl + 1)
    flops = 4.0 * d * pairs * b * h
    tflops = flops / (ms * 1e-3) / 1e12
    return {
        "ms": ms, "ms_min": tm.ms_min, "wall_ms": wall_ms, "tflops": tflops, "tokens_per_s": b * s / (ms * 1e-3),
        "workload": "flash_attn_func fwd bf16 batch=2 seqlen=16384 nheads=32 nheads_kv=8 headdim=128 causal window=(4096,0)",
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": tflops / PEAK_BF16_TFLOPS, "traffic": _traffic("gqa_window_bf16_d128_2x16k_w4096"),
                     "traffic_source": "profiles/traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, not measured in this run)",
                     "kernel": "fa::prefill_pp16_kernel<bf16,128,64,128,2>", "flops_per_launch": flops},
    }


def bench_config1(steps, warmup):
    """The reference's CPU-runnable case: fp16, batch 2 x 512 x 8 heads x 64, non-causal.  1.07 GFLOP and 3 MB per
    call: neither roofline is in sight, what a call costs is the launch (host side + one kernel of 64 workgroups on
    256 CUs).  Reported as microseconds per call on the stream and calls per second of host wall time."""
    import torch
    import flash_attn
    b, s, h, d = 2, 512, 8, 64
    torch.manual_seed(0)
    q, k, v = (torch.randn(b, s, h, d, device="cuda", dtype=torch.float16) for _ in range(3))
    fn = lambda: flash_attn.flash_attn_func(q, k, v)
    tm = time_steps(fn, max(steps, 200), max(warmup, 20))
    ms, wall_ms = tm
    flops = 4.0 * b * s * s * h * d
    tflops = flops / (ms * 1e-3) / 1e12
    return {
        "us_per_call": ms * 1e3, "us_per_call_min": tm.ms_min * 1e3, "host_us_per_call": wall_ms * 1e3, "calls_per_s": 1e3 / wall_ms, "tflops": tflops,
        "workload": "flash_attn_func fwd fp16 batch=2 seqlen=512 nheads=8 headdim=64 non-causal",
        "bound": "launch latency (64 workgroups of one 128-row block each; 1.07 GFLOP)",
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": tflops / PEAK_BF16_TFLOPS,
                     "traffic": _traffic("config1_fp16_d64_2x512x8"), "traffic_source": "profiles/traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, not measured in this run)",
                     "kernel": "fa::prefill_il_kernel<fp16,ILCfg<fp16,64,64>>", "flops_per_launch": flops},
    }


def bench_fwd_bwd(steps, warmup):
    import torch
    from flash_attn import _native as nat
    b, s, h, d = 2, 8192, 16, 128
    torch.manual_seed(0)
    q, k, v, dout = (torch.randn(b, s, h, d, device="cuda", dtype=torch.float16) for _ in range(4))
    scale = d ** -0.5
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)

    def fn():
        out, _, _, _, _, lse, _, _ = nat.fwd(q, k, v, None, 0.0, scale, True, -1, -1, False, None)
        nat.bwd(dout, q, k, v, out, lse, dq, dk, dv, 0.0, scale, True, -1, -1, None, None)

    tm = time_steps(fn, steps, warmup)
    ms, wall_ms = tm
    flops = 3.5 * 4.0 * b * s * s * h * d / 2
    tflops = flops / (ms * 1e-3) / 1e12
    return {
        "ms": ms, "ms_min": tm.ms_min, "wall_ms": wall_ms, "tflops": tflops,
        "workload": "flash_attn_func fwd+bwd fp16 batch=2 seqlen=8192 nheads=16 headdim=128 causal",
        "published": {"a100_tflops": 182.0, "h100_tflops": 308.0, "vs_a100": tflops / 182.0, "vs_h100": tflops / 308.0,
                      "source": "reference assets/flash2_a100_fwd_bwd_benchmark.png, flash2_h100_fwd_bwd_benchmark.png, panel (d)"},
    }


def bench_decode(steps, warmup):
    import torch
    import flash_attn
    b, cap, hk, h, d = 64, 32768, 8, 64, 128
    torch.manual_seed(0)
    k_cache = torch.randn(b, cap, hk, d, device="cuda", dtype=torch.bfloat16)
    v_cache = torch.randn(b, cap, hk, d, device="cuda", dtype=torch.bfloat16)
    q = torch.randn(b, 1, h, d, device="cuda", dtype=torch.bfloat16)
    kn = torch.randn(b, 1, hk, d, device="cuda", dtype=torch.bfloat16)
    vn = torch.randn(b, 1, hk, d, device="cuda", dtype=torch.bfloat16)
    start = torch.randint(1024, cap, (b,), dtype=torch.int32).cuda()          # [1024, 32767]
    # A decoding loop: every step appends one token where the last step stopped.  The lengths go back to `start`
    # ahead of every timed block; a sequence drawn within `steps` tokens of the end of the cache starts that many
    # tokens earlier, so that no block runs past the cache.
    start = torch.clamp(start, max=cap - 1 - max(steps, warmup))
    cache_seqlens = start.clone()
    # cos / sin of position x inverse frequency, base 10000, as flash_attn/layers/rotary.py builds its cache
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
    ang = torch.outer(torch.arange(cap, dtype=torch.float32), inv_freq)
    cos, sin = torch.cos(ang).to(torch.bfloat16).cuda(), torch.sin(ang).to(torch.bfloat16).cuda()

    def fn():
        flash_attn.flash_attn_with_kvcache(q, k_cache, v_cache, kn, vn, cos, sin, cache_seqlens, causal=True, rotary_interleaved=True)
        cache_seqlens.add_(1)          # (part of the step: a decoding loop does this too)

    tm = time_steps(fn, steps, warmup, before_block=lambda: cache_seqlens.copy_(start))
    ms, wall_ms = tm
    # keys read by the average step of a block: step t of a block sees start + t + 1 keys
    t = torch.arange(steps, device="cuda", dtype=torch.int64)[:, None]
    keys = float((start.long()[None, :] + t + 1).sum().item()) / steps
    algo_bytes = keys * hk * d * 2 * 2 + 2 * b * h * d * 2 + 2 * b * hk * d * 2 * 2
    gbs = algo_bytes / (ms * 1e-3) / 1e9
    return {
        "ms": ms, "ms_min": tm.ms_min, "wall_ms": wall_ms, "gb_per_s": gbs, "tokens_per_s": b / (ms * 1e-3),
        "workload": "flash_attn_with_kvcache bf16 b64 cache(64,32768,8,128) hq64 append1+rotary128 causal, lengths advancing by one per step",
        "roofline": {"bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": gbs / PEAK_HBM_GBS, "traffic": _traffic("decode_bf16_d128_b64_32k"), "traffic_source": "profiles/traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, not measured in this run)",
                     "kernel": "fa::decode_persistent_kernel<bf16,128,append,stream> (step = that kernel, which also appends the new rows, + fa::combine_kernel + the length update)", "bytes_per_launch": algo_bytes},
    }


def bench_decode_variants(steps, warmup):
    """Decoding shapes beside config 5 that take other paths of the library: four query positions at once on the
    config 5 caches (a draft of four tokens: 32 (position, head) rows per kv head, laid out as the rows of one
    tiled problem per kv head) and one position on a multi-query cache (32 q heads on 1 kv head: the grouped
    heads become the rows).  Both run the tiled kernel under the ticket schedule (chunks that hold keys, drawn
    from a counter).  Bytes: the cached K/V rows the masks let the queries see, once."""
    import torch
    import flash_attn
    res = {}
    for name, (b, cap, hk, h, d, sq, lo, kern) in (
            ("four_positions_gqa8", (64, 32768, 8, 64, 128, 4, 1024, "fa::prefill_persistent_kernel<bf16,128,stream>")),
            ("one_position_mqa32", (16, 65536, 1, 32, 128, 1, 30000, "fa::prefill_persistent_kernel<bf16,128,stream>"))):
        torch.manual_seed(0)
        k_cache = torch.randn(b, cap, hk, d, device="cuda", dtype=torch.bfloat16)
        v_cache = torch.randn(b, cap, hk, d, device="cuda", dtype=torch.bfloat16)
        q = torch.randn(b, sq, h, d, device="cuda", dtype=torch.bfloat16)
        cache_seqlens = torch.randint(lo, cap - sq, (b,), dtype=torch.int32).cuda()
        fn = lambda: flash_attn.flash_attn_with_kvcache(q, k_cache, v_cache, cache_seqlens=cache_seqlens, causal=True)
        tm = time_steps(fn, steps, warmup)
        ms = tm[0]
        algo_bytes = int(cache_seqlens.long().sum().item()) * hk * d * 2 * 2 + 2 * b * sq * h * d * 2
        gbs = algo_bytes / (ms * 1e-3) / 1e9
        res[name] = {"ms": ms, "ms_min": tm.ms_min, "gb_per_s": gbs,
                     "workload": "flash_attn_with_kvcache bf16 b%d cache(%d,%d,%d,%d) hq%d seqlen_q %d causal" % (b, b, cap, hk, d, h, sq),
                     "roofline": {"bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS,
                                  "traffic": _traffic("decode_variant_" + name),
                                  "traffic_source": "profiles/traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, not measured in this run)",
                                  "kernel": kern + " + fa::combine_kernel", "bytes_per_launch": algo_bytes}}
        del k_cache, v_cache
    return res


def cpu_baseline():
    """Oracle on the host cores: 1 batch entry x 4 heads of the prefill workload (1/32 of the
    (batch, head) pairs, which are independent), repeated for about 12 s."""
    import torch
    from oracle import attention_oracle as orc
    b, s, h, d = 4, 8192, 32, 128
    hs = 4
    torch.manual_seed(0)
    q, k, v = (torch.randn(1, s, hs, d).to(torch.bfloat16) for _ in range(3))
    t0 = time.perf_counter()
    reps = 0
    while True:
        orc.attention_forward(q, k, v, causal=True, head_block=1)
        reps += 1
        if time.perf_counter() - t0 > 12.0 or reps >= 64:
            break
    dt = (time.perf_counter() - t0) / reps
    flops_sample = 4.0 * 1 * s * s * hs * d / 2
    return {"value": flops_sample / dt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(),
            "host_cpus": os.cpu_count(), "kind": "port",
            "sample": "attention oracle (fp32 upcast) on 1 batch x %d heads of the prefill workload "
                      "(%d repeats, %.2f s each); whole batch would take %.0f s" % (hs, reps, dt, dt * b * h / hs)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-decode", action="store_true")
    ap.add_argument("--no-backward", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--only", default=None,
                    choices=["prefill", "config1", "mfma_peak", "hbm_peak", "lds_peak", "decode", "decode_variants", "rotary", "backward", "fwd_bwd", "varlen", "gqa_window", "head_dims"],
                    help="run one leg alone and print its record (for profiler runs: the trace then holds that leg's kernels only)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy, so that hardware-counter readings of "
                         "FETCH_SIZE / WRITE_SIZE can be scaled against a kernel of known traffic")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this build measures one GPU only (the hot path uses no collectives); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    import flash_attn  # noqa: F401  fails loudly if the HIP library is missing

    if a.calibrate_copy:
        src = torch.empty(1 << 29, dtype=torch.bfloat16, device="cuda").normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if a.only:
        leg = {"prefill": bench_prefill, "config1": bench_config1, "mfma_peak": bench_mfma_peak, "hbm_peak": bench_hbm_peak, "lds_peak": bench_lds_peak, "decode": bench_decode, "decode_variants": bench_decode_variants, "rotary": bench_rotary,
               "backward": bench_backward, "fwd_bwd": bench_fwd_bwd, "varlen": bench_varlen, "gqa_window": bench_gqa_window,
               "head_dims": bench_head_dims}[a.only]
        print(json.dumps({"only": a.only, "steps": a.steps, "warmup": a.warmup, a.only: leg(a.steps, a.warmup)}))
        return
    pre = bench_prefill(a.steps, a.warmup)
    peak = bench_mfma_peak(a.steps, a.warmup)
    # the kernel's own instruction shape (16x16x32) on random operands: the most this part sustains on such data
    pre["roofline"]["measured_peak"] = peak["shape_16x16x32"]["random_bf16"]["tflops"]
    pre["roofline"]["frac_of_measured_peak"] = pre["tflops"] / peak["shape_16x16x32"]["random_bf16"]["tflops"]
    lds = bench_lds_peak(a.steps, a.warmup)
    out = {
        "metric": "fwd TFLOP/s (bf16, hdim128, causal, 8k)",
        "value": pre["tflops"], "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": pre["ms"], "ms_min": pre["ms_min"], "timed_blocks": BLOCKS, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "flash_attn_func fwd bf16 batch=4 seqlen=8192 nheads=32 headdim=128 causal",
                   "global_batch": 4, "seq_len": 8192},
        "tokens_per_s": pre["tokens_per_s"],
        "roofline": pre["roofline"],
        "mfma_peak": peak,
        "lds_peak": lds,
    }
    if not a.no_decode:
        dec = bench_decode(a.steps, a.warmup)
        hbm = bench_hbm_peak(a.steps, a.warmup)
        dec["roofline"]["measured_peak"] = hbm["nontemporal"]["gb_per_s"]
        dec["roofline"]["frac_of_measured_peak"] = dec["gb_per_s"] / hbm["nontemporal"]["gb_per_s"]
        out["decode"] = dec
        out["hbm_peak"] = hbm
        out["decode_variants"] = bench_decode_variants(a.steps, a.warmup)
    if not a.no_backward:
        out["rotary"] = bench_rotary(a.steps, a.warmup)
        out["backward"] = bench_backward(max(1, a.steps // 2), max(1, a.warmup // 2))
        out["fwd_bwd"] = bench_fwd_bwd(a.steps, a.warmup)
        out["varlen"] = bench_varlen(a.steps, a.warmup)
        out["gqa_window"] = bench_gqa_window(a.steps, a.warmup)
        out["head_dims"] = bench_head_dims(a.steps, a.warmup)
        out["config1"] = bench_config1(a.steps, a.warmup)
    if not a.no_cpu:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
