"""GPU parity on rows built to defeat the kernels' running-maximum shortcuts.

The long-sequence kernels do not take a row maximum per key tile.  They exponentiate a tile against the reference
maximum the row already has and look at the tile's row sum; only a sum above 2^14 (or a non-finite one: no reference
yet) makes them form the exact maximum, move the reference when it lags by more than 2^8, and redo the tile
(csrc/fa_prefill_pp.h, csrc/fa_prefill_il.h; the reference's rule is softmax_rescale_o,
csrc/flash_attn/src/flash_fwd_kernel.h:24-53, with scale_apply_exp2, softmax.h:65-84).  On i.i.d. Gaussian inputs at
the default scale that branch fires on a row's first tiles only.  The rows here make it fire again and again, and late:

  * rising / falling: every query has a common component u and the keys carry a ramp along u, so the scores of a row
    climb (or fall) by 60 standard deviations over the key range, in the order the kernel walks it or against it;
  * spike_first / spike_middle / spike_last: one key 30 standard deviations above the rest in the first, a middle or
    the last key tile;
  * scale1: softmax_scale = 1 at the real head dim (scores with a standard deviation of sqrt(d));
  * x8: q, k and v multiplied by 8 (scores x 64, outputs x 8);
  * dead_tiles: seqlen_q != seqlen_k under a two-sided window, with the ramp: for many rows the first key tiles the
    workgroup visits are masked out entirely, then finite scores begin, then tiles are masked out again.

Each runs on the general tiled kernel, the software-pipelined kernel (head dims 64 and 128), the 8-wave ping-pong
kernel and the head-dim-256 kernel, in bf16 and fp16, dense, causal and windowed, and the kernel is asserted.
Acceptance is the usual rule (max|out - ref| <= 2 max|lowprec - ref| + 1e-5, log-sum-exp within 1e-3 relative)."""
import math
import sys

import pytest
import torch

from oracle import attention_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def _fa():
    import flash_attn
    return flash_attn


# kernel -> (d, b, h, hk, sq, sk by mask mode); sized by the dispatch rules (csrc/fa_prefill_inst.hip, plan() in
# csrc/fa_api.hip): ping-pong needs 2048+ keys and more than 256 row blocks of 256 rows under a mask (128 and 769+
# keys without), the pipelined kernels 96+ rows in a launch that is not split
_SHAPES = {
    "tiled": (128, 2, 4, 2, 80, 1000),
    "pipelined": (128, 4, 8, 2, 512, 1024),
    "pipelined64": (64, 4, 8, 2, 512, 1024),
    "pingpong": (128, 1, 32, 4, 4352, 4352),
    "pingpong96": (96, 1, 32, 4, 4352, 4352),
    "wide": (256, 4, 8, 2, 512, 1024),
    "wide32": (192, 1, 32, 4, 2816, 2816),            # 11 x 32 blocks of 256 rows (9 x 32 with fewer queries than keys): the 32-rows-per-wave form
}
_KERNEL_OF = {"tiled": "tiled", "pipelined": "pipelined", "pipelined64": "pipelined", "pingpong": "pingpong",
              "pingpong96": "pingpong", "wide": "pingpong_wide", "wide32": "pingpong_wide32"}
_PATTERNS = ["rising", "falling", "spike_first", "spike_middle", "spike_last", "scale1", "x8"]


def _inputs(pattern, dtype, d, b, h, hk, sq, sk, seed=0):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(b, sq, h, d, generator=g)
    k = torch.randn(b, sk, hk, d, generator=g)
    v = torch.randn(b, sk, hk, d, generator=g)
    scale = 1.0 / math.sqrt(d)
    u = torch.randn(d, generator=g)
    u = u / u.norm()
    amp = 30.0 / (4.0 * scale)            # q.u = 4, k.u = amp: 30 standard deviations of a scaled score
    if pattern in ("rising", "falling", "dead_tiles"):
        ramp = torch.linspace(-amp, amp, sk)
        if pattern == "falling":
            ramp = ramp.flip(0)
        q = q + 4.0 * u
        k = k + ramp[None, :, None, None] * u
    elif pattern.startswith("spike"):
        j = {"spike_first": 5, "spike_middle": sk // 2 + 3, "spike_last": sk - 7}[pattern]
        q = q + 4.0 * u
        k[:, j] += amp * u
    elif pattern == "scale1":
        scale = 1.0
    elif pattern == "x8":
        q, k, v = q * 8, k * 8, v * 8
    return q.to(dtype), k.to(dtype), v.to(dtype), scale


def _run_and_check(kernel, pattern, dtype, mode, rect=False):
    d, b, h, hk, sq, sk = _SHAPES[kernel]
    if rect:
        sq = sq - sq // 4 - 37               # seqlen_q < seqlen_k, not a multiple of anything
    q, k, v, scale = _inputs(pattern, dtype, d, b, h, hk, sq, sk)
    causal = mode == "causal"
    window = (-1, -1)
    if mode == "local":
        window = (sk // 3 + 11, sk // 9 + 5)         # (1461, 488) at 4352 keys: wider than the narrow-window cut
    out, lse, _ = _fa().flash_attn_func(q.to(DEV), k.to(DEV), v.to(DEV), softmax_scale=scale, causal=causal,
                                        window_size=window, return_attn_probs=True)
    from flash_attn import _native as nat
    got = nat.last_kernel()
    _say("   kernel", got)
    assert got[0] == _KERNEL_OF[kernel], got
    assert not torch.isnan(out).any()
    # the (batch, head) pairs are independent problems: a sample is checked (two pairs of the big launches in fp16,
    # whose low-precision CPU run is slow)
    pairs = [(0, 0), (b - 1, h - 1), (b // 2, h // 2 + 1)]
    if sq * sk > 1 << 21 and dtype == torch.float16:
        pairs = pairs[:2]
    group = h // hk
    worst = 0.0
    for (bb, hh) in pairs:
        sl = lambda t, x: t[bb:bb + 1, :, x:x + 1]
        o_ref, l_ref, o_pt = orc.attention_reference_pair(sl(q, hh), sl(k, hh // group), sl(v, hh // group), causal=causal,
                                                          window_size=window, softmax_scale=scale)
        ok, err, bound = orc.tolerance_ok(sl(out, hh).cpu(), o_ref, o_pt, 2.0, 1e-5)
        assert ok, ("output", kernel, pattern, mode, bb, hh, err, bound)
        okl, rel = orc.lse_ok(lse[bb:bb + 1, hh:hh + 1].cpu(), l_ref)
        assert okl, ("lse", kernel, pattern, mode, bb, hh, rel)
        worst = max(worst, rel)
    _say("   %d pairs, worst lse rel %.2e" % (len(pairs), worst))


@pytest.mark.parametrize("pattern", _PATTERNS)
@pytest.mark.parametrize("kernel", ["tiled", "pipelined", "pipelined64", "pingpong", "pingpong96", "wide", "wide32"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
def test_adversarial_rows_causal(kernel, pattern, dtype):
    _say("softmax stress causal", kernel, pattern, dtype)
    _run_and_check(kernel, pattern, dtype, "causal")


@pytest.mark.parametrize("pattern", ["rising", "falling", "spike_middle", "scale1"])
@pytest.mark.parametrize("kernel", ["pipelined", "pingpong", "wide", "wide32"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
def test_adversarial_rows_dense(kernel, pattern, dtype):
    _say("softmax stress dense", kernel, pattern, dtype)
    _run_and_check(kernel, pattern, dtype, "full")


@pytest.mark.parametrize("pattern", ["rising", "falling", "spike_first", "spike_last", "x8", "dead_tiles"])
@pytest.mark.parametrize("kernel", ["tiled", "pipelined", "pipelined64", "pingpong", "wide", "wide32"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
def test_adversarial_rows_under_a_window(kernel, pattern, dtype):
    """dead_tiles: seqlen_q < seqlen_k, so the window of the first rows starts far into the keys"""
    _say("softmax stress window", kernel, pattern, dtype)
    _run_and_check(kernel, pattern, dtype, "local", rect=(pattern == "dead_tiles"))
