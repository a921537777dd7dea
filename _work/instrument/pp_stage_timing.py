"""Where the time of fa::prefill_pp_kernel<bf16,128,64> goes, from the kernel's own clocks.

Needs a measurement build of the library, in which every workgroup records when it passes the stages of
the kernel (shader-clock counter), when it starts and ends (constant 100 MHz counter), which CU runs it and
how many key tiles it visits:

    python flash-attention_amd/build.py -D FA_PP_TIMING --out /tmp/libfa_timing.so --obj-dir /tmp/fa_timing_obj
    FLASH_ATTN_MI355X_LIB=/tmp/libfa_timing.so python flash-attention_amd/benchmarks/pp_stage_timing.py dense
    FLASH_ATTN_MI355X_LIB=/tmp/libfa_timing.so python flash-attention_amd/benchmarks/pp_stage_timing.py varlen 0

Prints the average shader clock, the cycles per stage, the cost of a key tile, the share of the time outside
the key loop, for every XCD when its CUs were busy and when it finished, and how long a CU waits between
two workgroups.  (The stamps cost about 10 % of the kernel's speed; the ordinary build has none.)
"""
import ctypes
import os
import sys

import numpy as np
import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
import flash_attn  # noqa: E402

SLOTS = 16            # int64 slots per (workgroup, wave group); see FA_PP_STAMP in csrc/fa_prefill_pp.h
BLOCKS = 32768        # FA_PP_DBG_BLOCKS


def records():
    lib = ctypes.CDLL(os.environ["FLASH_ATTN_MI355X_LIB"])
    buf = np.zeros(BLOCKS * 2 * SLOTS, dtype=np.int64)
    rc = lib.fa_pp_debug_read(buf.ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(buf.nbytes))
    if rc != 0:
        raise RuntimeError("fa_pp_debug_read failed: %d" % rc)
    x = buf.reshape(-1, 2, SLOTS)[:, 0, :]
    bid = np.arange(len(x))
    ok = (x[:, 5] > x[:, 0]) & (x[:, 7] > x[:, 6])
    ok &= x[:, 6] > x[ok][:, 6].max() - 1000000        # the last launch only (starts within 10 ms of the newest)
    return x[ok], bid[ok]


def report(name, ms):
    x, bid = records()
    cyc = (x[:, 5] - x[:, 0]).astype(np.float64)
    real = (x[:, 7] - x[:, 6]).astype(np.float64)
    loop = (x[:, 4] - x[:, 3]).astype(np.float64)
    nt = x[:, 11].astype(np.float64)
    print("%s: kernel %.3f ms, %d workgroups with work, shader clock %.2f GHz" % (name, ms, len(x), cyc.sum() / real.sum() * 0.1))
    stages = (("work item known", 8, 0), ("sequence bounds", 9, 8), ("first K/V tiles requested", 1, 9), ("Q loads issued", 10, 1),
              ("registers set up, tiles landed, barrier", 2, 10), ("first S tile", 3, 2), ("key loop", 4, 3), ("epilogue", 5, 4))
    print("   mean cycles per workgroup: " + " | ".join("%s %.0f" % (n, (x[:, a] - x[:, b]).mean()) for n, a, b in stages))
    slope, icpt = np.linalg.lstsq(np.vstack([nt, np.ones_like(nt)]).T, loop, rcond=None)[0]
    print("   key tiles per workgroup %.1f; key loop = %.0f cycles per tile + %.0f; outside the loop %.0f cycles = %.1f %% of the busy time"
          % (nt.mean(), slope, icpt, (cyc - loop).mean(), 100 * (cyc - loop).sum() / cyc.sum()))
    t0 = x[:, 6].min()
    hw = x[:, 12]
    cu = ((hw >> 8) & 0xf) | (((hw >> 12) & 1) << 4) | (((hw >> 13) & 7) << 5)       # CU, shader array, shader engine
    print("   per XCD (block id mod 8): workgroups, busy time / 32 CUs, all CUs busy until, last workgroup ends [ms]; wait of a CU between two workgroups [us]")
    for xc in range(8):
        m = (bid & 7) == xc
        ends = np.sort(x[m, 7])
        gaps = []
        for c in np.unique(cu[m]):
            mm = m & (cu == c)
            o = np.argsort(x[mm, 6])
            gaps.append(x[mm, 6][o][1:] - x[mm, 7][o][:-1])
        g = np.concatenate(gaps) / 100.0
        print("      xcd %d: %5d  %.3f  %.3f  %.3f   wait mean %.2f median %.2f p90 %.2f" %
              (xc, m.sum(), (x[m, 7] - x[m, 6]).sum() / 1e5 / 32, (ends[-32] - t0) / 1e5 if len(ends) >= 32 else 0.0,
               (ends[-1] - t0) / 1e5, g.mean(), np.median(g), np.percentile(g, 90)))


def timed(fn):
    for _ in range(5):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1)


def dense(b=4, s=8192, h=32, d=128):
    torch.manual_seed(0)
    q, k, v = (torch.randn(b, s, h, d, device="cuda", dtype=torch.bfloat16) for _ in range(3))
    report("flash_attn_func bf16 (%d, %d, %d, %d) causal" % (b, s, h, d), timed(lambda: flash_attn.flash_attn_func(q, k, v, causal=True)))


def varlen(seed, h=16, d=128):
    torch.manual_seed(seed)
    lens = torch.randint(128, 4097, (64,))
    cu = torch.cat([torch.zeros(1, dtype=torch.long), lens.cumsum(0)]).int()
    total, mx = int(cu[-1]), int(lens.max())
    q, k, v = (torch.randn(total, h, d, device="cuda", dtype=torch.bfloat16) for _ in range(3))
    cu_d = cu.cuda()
    report("flash_attn_varlen_func bf16 64 sequences U[128,4096] (seed %d, %d tokens) %d heads causal" % (seed, total, h),
           timed(lambda: flash_attn.flash_attn_varlen_func(q, k, v, cu_d, cu_d, mx, mx, causal=True)))


if __name__ == "__main__":
    if "FLASH_ATTN_MI355X_LIB" not in os.environ:
        sys.exit("set FLASH_ATTN_MI355X_LIB to a library built with -D FA_PP_TIMING (see the top of this file)")
    if len(sys.argv) > 1 and sys.argv[1] == "varlen":
        varlen(int(sys.argv[2]) if len(sys.argv) > 2 else 0)
    else:
        dense()
