"""GPU parity tests sized for the long-sequence kernels (not the general 4-wave one and not the split path), each
asserting through fa_last_kernel() that the launch reached the kernel the case was written for.  Dispatch as the
library has it (csrc/fa_prefill_inst.hip), for an unsplit launch of 96+ query rows (32+ above head dim 128):

  * ping-pong kernel (fa_prefill_pp.h): head dim 65..128, keys from 2048 on under a mask / beyond 768 without,
    more than 256 (masked) / 128 (unmasked) row blocks of 256 rows in the launch, and no window whose two bounds
    span 768 keys or fewer;
  * software-pipelined kernel (fa_prefill_il.h): everything else up to head dim 128;
  * head dim 129..256: the 8-wave kernel with 16 query rows per wave ("pingpong_wide"), or, up to head dim 192 in a
    launch of more than 128 blocks of 256 rows (256 under a mask when sequences span several blocks) with more
    than 128 queries per sequence, with 32 rows per wave ("pingpong_wide32"); pairs of waves with dropout.

Launches are made large enough for those thresholds with many query heads on few kv heads; the CPU oracle then checks
a sample of (batch, head) pairs, which are independent problems.  Cases follow the reference's own test dimensions
(tests/test_flash_attn.py:530-657, 1295-1402): ragged lengths, seqlen_q != seqlen_k both ways, causal / local masks,
MQA/GQA, padded head dims, fp16 and bf16, strided packed inputs, packed variable-length batches.  Acceptance: the
reference's rule (max|out - ref| <= 2 max|lowprec - ref| + 1e-5) and log-sum-exp within 1e-3 relative."""
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


def _gen(shape, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=torch.float32).to(dtype)


def _ran(name, head_dims=None, dropout=False):
    """the last forward launch of this thread took kernel `name` (flash_attn._native.last_kernel)"""
    from flash_attn import _native as nat
    got = nat.last_kernel()
    _say("   kernel", got)
    assert got[0] == name and got[1] == dropout and not got[2], got
    if head_dims is not None:
        assert got[3] == head_dims, got


def _check_pairs(out, lse, q, k, v, pairs, **kw):
    """oracle check of sampled (batch, q head) pairs; k / v heads follow the GQA mapping"""
    group = q.shape[2] // k.shape[2]
    for (b, h) in pairs:
        sl = lambda t, hh: t[b:b + 1, :, hh:hh + 1]
        _say("   (b=%d, h=%d)" % (b, h))
        _check(sl(out, h), lse[b:b + 1, h:h + 1], sl(q, h), sl(k, h // group), sl(v, h // group), **kw)


def _check(out, lse, q, k, v, **kw):
    out_ref, lse_ref, out_pt = orc.attention_reference_pair(q, k, v, **kw)
    ok, err, bound = orc.tolerance_ok(out.cpu(), out_ref, out_pt, 2.0, 1e-5)
    _say("   out err %.3e bound %.3e" % (err, bound))
    assert not torch.isnan(out).any()
    assert ok, "output error %g exceeds bound %g" % (err, bound)
    okl, rel = orc.lse_ok(lse.cpu(), lse_ref)
    _say("   lse rel %.3e" % rel)
    assert okl, "lse relative error %g" % rel


def _window(mode, sk, seed):
    if mode != "local":
        return (-1, -1)
    g = torch.Generator().manual_seed(seed)
    return tuple(torch.randint(0, sk, (2,), generator=g).tolist())


@pytest.mark.parametrize("d", [24, 32, 40, 64, 96, 128])
@pytest.mark.parametrize("s", [512, 777, 1024])
@pytest.mark.parametrize("mode", ["full", "causal", "local"])
def test_pipelined_kernel_square(d, s, mode):
    _say("pipelined square", d, s, mode)
    dtype = torch.bfloat16
    b, h, hk = 4, 16, 4          # 4 row blocks x 64 at s = 512: exactly the 256 blocks that avoid the split path
    q = _gen((b, s, h, d), dtype, 1); k = _gen((b, s, hk, d), dtype, 2); v = _gen((b, s, hk, d), dtype, 3)
    window = _window(mode, s, d * 1000 + s)
    out, lse, _ = _fa().flash_attn_func(q.to(DEV), k.to(DEV), v.to(DEV), causal=(mode == "causal"),
                                        window_size=window, return_attn_probs=True)
    # (without a mask, keys beyond 768 at head dim 65..128 are the ping-pong kernel's)
    _ran("pingpong" if (mode == "full" and d > 64 and s >= 769) else "pipelined", 32 if d <= 32 else 64 if d <= 64 else 96 if d <= 96 else 128)
    _check(out, lse, q, k, v, causal=(mode == "causal"), window_size=window)


@pytest.mark.parametrize("sq,sk,dtype", [(600, 1500, torch.float16), (600, 1500, torch.bfloat16), (1500, 600, torch.float16),
                                         (1500, 600, torch.bfloat16), (513, 4000, torch.bfloat16), (1100, 1101, torch.bfloat16)])
@pytest.mark.parametrize("mode", ["causal", "local"])
def test_pipelined_kernel_rectangular(sq, sk, dtype, mode):
    """seqlen_q != seqlen_k: bottom-right alignment, rows without any visible key (sq > sk).  (fp16 only on
    the smaller shapes: the low-precision CPU oracle is slow in fp16.)"""
    _say("pipelined rect", sq, sk, mode, dtype)
    d, b, h = 128, 2, 32
    q = _gen((b, sq, h, d), dtype, 1); k = _gen((b, sk, 1, d), dtype, 2); v = _gen((b, sk, 1, d), dtype, 3)   # MQA
    window = _window(mode, sk, sq * 7 + sk)
    out, lse, _ = _fa().flash_attn_func(q.to(DEV), k.to(DEV), v.to(DEV), causal=(mode == "causal"),
                                        window_size=window, return_attn_probs=True)
    _ran("pipelined", 128)
    _check(out, lse, q, k, v, causal=(mode == "causal"), window_size=window)


# name: (dtype, d, b, h, hk, sq, sk, causal, window); every case has more than 256 row blocks of 256 rows (128 without
# a mask), 2048+ keys under a mask, and no window narrower than 769 keys
_PP_CASES = {
    "full_2304": (torch.bfloat16, 128, 2, 8, 2, 2304, 2304, False, (-1, -1)),
    "causal_4200": (torch.bfloat16, 128, 1, 16, 2, 4200, 4200, True, (-1, -1)),
    "local_4500": (torch.bfloat16, 128, 1, 16, 2, 4500, 4500, False, (1000, 300)),
    "left_only_4500": (torch.bfloat16, 128, 1, 16, 1, 4500, 4500, False, (900, -1)),
    "rect_causal": (torch.bfloat16, 128, 3, 16, 2, 2000, 4500, True, (-1, -1)),        # sq < sk
    "rect_causal_tall": (torch.bfloat16, 128, 2, 8, 1, 4300, 2100, True, (-1, -1)),    # sq > sk: leading rows see nothing
    "rect_local": (torch.bfloat16, 128, 2, 8, 2, 4300, 2100, False, (900, 200)),       # sq > sk, two-sided window
    "rect_local_wide": (torch.bfloat16, 128, 3, 16, 4, 2000, 4500, False, (1500, 400)),  # sq < sk, two-sided window
    "ragged_causal": (torch.bfloat16, 128, 3, 16, 2, 1531, 3977, True, (-1, -1)),      # no length a multiple of a tile
    "fp16_causal": (torch.float16, 128, 1, 16, 2, 4200, 4200, True, (-1, -1)),
    "fp16_rect_local": (torch.float16, 128, 3, 16, 2, 2000, 4500, False, (1200, 100)),
    "fp16_full": (torch.float16, 128, 2, 8, 2, 2304, 2304, False, (-1, -1)),
    "d96_full": (torch.bfloat16, 96, 2, 8, 2, 2100, 2100, False, (-1, -1)),            # head dims 65..96: the 96-column variant
    "d96_causal": (torch.bfloat16, 96, 1, 16, 2, 4200, 4200, True, (-1, -1)),
    "d80_local": (torch.bfloat16, 80, 1, 16, 2, 4500, 4500, False, (1000, 300)),
    "d72_rect_causal": (torch.bfloat16, 72, 3, 16, 2, 2000, 4500, True, (-1, -1)),
    "d88_fp16_rect_tall_local": (torch.float16, 88, 2, 8, 1, 4300, 2100, False, (1100, 64)),
    "d104_causal": (torch.bfloat16, 104, 1, 16, 2, 4200, 4200, True, (-1, -1)),        # 97..128: all 128 columns, 104 real
    "d120_rect_local": (torch.bfloat16, 120, 3, 16, 2, 2000, 4500, False, (1500, 400)),
}


@pytest.mark.parametrize("case", sorted(_PP_CASES))
def test_pingpong_kernel(case):
    _say("ping-pong", case)
    dtype, d, b, h, hk, sq, sk, causal, window = _PP_CASES[case]
    q = _gen((b, sq, h, d), dtype, 1); k = _gen((b, sk, hk, d), dtype, 2); v = _gen((b, sk, hk, d), dtype, 3)
    out, lse, _ = _fa().flash_attn_func(q.to(DEV), k.to(DEV), v.to(DEV), causal=causal, window_size=window,
                                        return_attn_probs=True)
    _ran("pingpong", 96 if d <= 96 else 128)
    assert not torch.isnan(out).any()
    # first and last head of the launch, and one in the middle of a kv group (two pairs in fp16, whose
    # low-precision CPU run is slow)
    pairs = [(0, 0), (b - 1, h - 1), (b // 2, h // 2 + 1)]
    _check_pairs(out, lse, q, k, v, pairs[:2] if dtype == torch.float16 else pairs, causal=causal, window_size=window)


@pytest.mark.parametrize("d", [136, 160, 192, 224, 256])
@pytest.mark.parametrize("sq,sk,mode", [(777, 777, "causal"), (512, 512, "full"), (600, 1500, "causal"),
                                         (1500, 600, "local"), (1024, 1024, "local")])
def test_wide_kernel_head_dims_above_128(d, sq, sk, mode):
    _say("head dims above 128", d, sq, sk, mode)
    dtype = torch.float16 if d == 160 and sq <= 777 else torch.bfloat16
    b, h, hk = 4, 16, 2
    q = _gen((b, sq, h, d), dtype, 1); k = _gen((b, sk, hk, d), dtype, 2); v = _gen((b, sk, hk, d), dtype, 3)
    window = _window(mode, sk, d * 31 + sq)
    out, lse, _ = _fa().flash_attn_func(q.to(DEV), k.to(DEV), v.to(DEV), causal=(mode == "causal"),
                                        window_size=window, return_attn_probs=True)
    blocks256 = (sq + 255) // 256 * h * b
    rows32 = d <= 192 and blocks256 > (256 if mode != "full" else 128)       # (1500, 600, local) below head dim 193
    _ran("pingpong_wide32" if rows32 else "pingpong_wide",
         160 if d <= 160 else 192 if d <= 192 else 224 if d <= 224 else 256)      # the reference's buckets above 128
    _check(out, lse, q, k, v, causal=(mode == "causal"), window_size=window)


# The 32-rows-per-wave form of the wide kernel (head dims 129-192): launches of more than 256 blocks of 256 rows under
# a mask, more than 128 without.  (dtype, d, b, h, hk, sq, sk, causal, window)
_WIDE32_CASES = {
    "d192_causal": (torch.bfloat16, 192, 1, 32, 4, 2300, 2300, True, (-1, -1)),
    "d192_causal_fp16": (torch.float16, 192, 2, 32, 8, 1300, 1300, True, (-1, -1)),
    "d160_full_ragged": (torch.bfloat16, 160, 3, 16, 2, 777, 1111, False, (-1, -1)),
    "d136_more_keys_causal": (torch.bfloat16, 136, 2, 32, 4, 1100, 2900, True, (-1, -1)),
    "d176_fewer_keys_causal": (torch.bfloat16, 176, 2, 32, 4, 1500, 700, True, (-1, -1)),
    "d192_two_sided_window": (torch.bfloat16, 192, 1, 48, 6, 1600, 1600, False, (1000, 300)),
    "d160_rect_local_fp16": (torch.float16, 160, 2, 32, 2, 1200, 2600, False, (900, 0)),
    "d192_narrow_window": (torch.bfloat16, 192, 2, 32, 4, 1400, 1400, False, (100, 60)),
    "d144_one_block_per_sequence": (torch.bfloat16, 144, 24, 8, 2, 200, 1800, True, (-1, -1)),
}


@pytest.mark.parametrize("case", sorted(_WIDE32_CASES))
def test_wide_kernel_with_32_rows_per_wave(case):
    _say("wide, 32 rows per wave", case)
    dtype, d, b, h, hk, sq, sk, causal, window = _WIDE32_CASES[case]
    q = _gen((b, sq, h, d), dtype, 1); k = _gen((b, sk, hk, d), dtype, 2); v = _gen((b, sk, hk, d), dtype, 3)
    out, lse, _ = _fa().flash_attn_func(q.to(DEV), k.to(DEV), v.to(DEV), causal=causal, window_size=window,
                                        return_attn_probs=True)
    _ran("pingpong_wide32", 160 if d <= 160 else 192)
    assert not torch.isnan(out).any()
    pairs = [(0, 0), (b - 1, h - 1), (b // 2, h // 2 + 1)]
    _check_pairs(out, lse, q, k, v, pairs[:2] if dtype == torch.float16 else pairs, causal=causal, window_size=window)


def test_wide_kernel_with_32_rows_per_wave_packed_sequences():
    """Variable-length batch at head dim 192 with empty, one-row and ragged sequences: row blocks are aligned to the
    end of each sequence, so the first block of most sequences starts before its first row."""
    _say("wide, 32 rows per wave, varlen")
    dtype, h, hk, d = torch.bfloat16, 16, 4, 192
    lens = [0, 1, 255, 256, 257, 700, 0, 1300, 2100, 129, 513, 1999, 31, 1024]
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    total, mx = int(cu[-1]), max(lens)
    q = _gen((total, h, d), dtype, 1); k = _gen((total, hk, d), dtype, 2); v = _gen((total, hk, d), dtype, 3)
    out, lse, _ = _fa().flash_attn_varlen_func(q.to(DEV), k.to(DEV), v.to(DEV), cu.to(DEV), cu.to(DEV), mx, mx,
                                               causal=True, return_attn_probs=True)
    _ran("pingpong_wide32", 192)                # 9 blocks of 256 rows x 16 heads x 14 sequences
    assert not torch.isnan(out).any()
    for i, n in enumerate(lens):
        if n == 0:
            continue
        a, e = int(cu[i]), int(cu[i + 1])
        _check_pairs(out[a:e][None], lse[i:i + 1, :, :n], q[a:e][None], k[a:e][None], v[a:e][None], [(0, 0), (0, h - 1)],
                     causal=True)


def test_wide_kernel_with_32_rows_per_wave_chunked_prefill_on_a_cache():
    """A 512-token chunk appended to K/V caches that hold different lengths (flash_attn_with_kvcache with new keys,
    head dim 160, GQA): per-batch key lengths that are not prefix sums, more keys than queries, causal mask aligned
    to the end of each cache entry."""
    _say("wide, 32 rows per wave, kv cache")
    from flash_attn import _native as nat
    dtype, b, h, hk, d, sq, cap = torch.bfloat16, 8, 32, 4, 160, 512, 3000
    q = _gen((b, sq, h, d), dtype, 1)
    kc = _gen((b, cap, hk, d), dtype, 2); vc = _gen((b, cap, hk, d), dtype, 3)
    kn = _gen((b, sq, hk, d), dtype, 4); vn = _gen((b, sq, hk, d), dtype, 5)
    lens = torch.tensor([0, 1, 300, 1111, 2047, 2488, 64, 777], dtype=torch.int32)
    kd, vd = kc.to(DEV), vc.to(DEV)
    out, lse = nat.fwd_kvcache(q.to(DEV), kd, vd, kn.to(DEV), vn.to(DEV), lens.to(DEV), None, None, None, None, d ** -0.5,
                               True, -1, -1, True, 0)
    _ran("pingpong_wide32", 160)                # 2 blocks of 256 rows x 32 heads x 8 entries
    assert not torch.isnan(out).any()
    out, lse = out.cpu(), lse.cpu()
    for i in (0, 1, 3, 5):
        sl = slice(i, i + 1)
        for hh in (0, h - 1):
            g = hh // (h // hk)
            o_ref, l_ref, k_after, v_after = orc.kvcache_forward(q[sl, :, hh:hh + 1], kc[sl, :, g:g + 1], vc[sl, :, g:g + 1],
                                                                 kn[sl, :, g:g + 1], vn[sl, :, g:g + 1], None, None, lens[sl], causal=True)
            o_pt, _, _, _ = orc.kvcache_forward(q[sl, :, hh:hh + 1], kc[sl, :, g:g + 1], vc[sl, :, g:g + 1], kn[sl, :, g:g + 1],
                                                vn[sl, :, g:g + 1], None, None, lens[sl], causal=True, upcast=False, reorder_ops=True)
            ok, err, bound = orc.tolerance_ok(out[sl, :, hh:hh + 1], o_ref, o_pt, 2.0, 1e-5)
            _say("   entry %d head %d: err %.3e bound %.3e" % (i, hh, err, bound))
            assert ok
            assert orc.lse_ok(lse[sl, hh:hh + 1], l_ref)[0]
            assert torch.equal(kd[sl, :, g:g + 1].cpu(), k_after.to(dtype)) and torch.equal(vd[sl, :, g:g + 1].cpu(), v_after.to(dtype))


@pytest.mark.parametrize("s,d", [(1024, 64), (2304, 128), (1024, 256)])
def test_long_kernels_take_strided_packed_input(s, d):
    """q, k, v as strided views of one (b, s, 3, h, d) tensor: row stride 3*h*d."""
    _say("packed long", s, d)
    dtype = torch.bfloat16
    b, h = 2, 16
    qkv = _gen((b, s, 3, h, d), dtype, 5)
    out, lse, _ = _fa().flash_attn_qkvpacked_func(qkv.to(DEV), causal=True, return_attn_probs=True)
    _ran({64: "pipelined", 128: "pingpong", 256: "pingpong_wide"}[d])        # (d 128: 9 row blocks x 16 heads x 2 = 288)
    _check(out, lse, qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2], causal=True)


@pytest.mark.parametrize("d", [64, 128, 256])
def test_varlen_long_with_empty_and_tiny_sequences(d):
    _say("varlen long", d)
    dtype, h = torch.bfloat16, 16
    lens = [0, 1, 63, 64, 65, 700, 0, 1300, 2100, 129, 512, 1999]
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    total, mx = int(cu[-1]), max(lens)
    q = _gen((total, h, d), dtype, 1); k = _gen((total, h, d), dtype, 2); v = _gen((total, h, d), dtype, 3)
    out, lse, _ = _fa().flash_attn_varlen_func(q.to(DEV), k.to(DEV), v.to(DEV), cu.to(DEV), cu.to(DEV), mx, mx,
                                               causal=True, return_attn_probs=True)
    _ran({64: "pipelined", 128: "pingpong", 256: "pingpong_wide"}[d])        # (d 128: 9 row blocks x 16 heads x 12 sequences)
    assert out.shape == q.shape and lse.shape == (len(lens), h, mx)
    assert not torch.isnan(out).any()
    for i, L in enumerate(lens):
        if L == 0:
            continue
        a, e = int(cu[i]), int(cu[i + 1])
        o_ref, l_ref, o_pt = orc.attention_reference_pair(q[a:e][None], k[a:e][None], v[a:e][None], causal=True)
        ok, err, bound = orc.tolerance_ok(out[a:e][None].cpu(), o_ref, o_pt, 2.0, 1e-5)
        _say("   seq %d (len %d): err %.3e bound %.3e" % (i, L, err, bound))
        assert ok
        assert orc.lse_ok(lse[i, :, :L][None].cpu(), l_ref)[0]
