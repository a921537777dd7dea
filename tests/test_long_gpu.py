"""GPU parity tests sized so that the two long-sequence kernels run (not the general 4-wave one and not
the split path): at least 512 query rows and at least 256 row blocks in the launch.

  * software-pipelined kernel (fa_prefill_il.h): head dim <= 64 at any length, head dim <= 128 up to
    4096 keys (causal / windowed) or 2048 keys (full attention);
  * ping-pong kernel (fa_prefill_pp.h): head dim 65..128 beyond those key counts;
  * the pair form of the software-pipelined kernel (two waves split the head dimension): head dim
    129..256.

Cases follow the reference's own test dimensions (tests/test_flash_attn.py:530-657, 1295-1402): ragged
lengths, seqlen_q != seqlen_k both ways, causal / local masks, MQA/GQA, padded head dims, fp16 and
bf16, strided packed inputs, packed variable-length batches.  Acceptance: the reference's rule
(max|out - ref| <= 2 max|lowprec - ref| + 1e-5) and log-sum-exp within 1e-3 relative."""
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


@pytest.mark.parametrize("d", [40, 64, 96, 128])
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
    _check(out, lse, q, k, v, causal=(mode == "causal"), window_size=window)


@pytest.mark.parametrize("case", ["full_2304", "causal_4200", "local_4500", "rect_causal", "rect_local", "d96_full",
                                  "d96_causal", "d80_local", "d72_rect_causal"])
def test_pingpong_kernel(case):
    _say("ping-pong", case)
    dtype = torch.bfloat16
    d, hk = 128, 2
    if case == "full_2304":
        b, h, sq, sk, causal, window = 2, 8, 2304, 2304, False, (-1, -1)
    elif case == "causal_4200":
        b, h, sq, sk, causal, window = 1, 8, 4200, 4200, True, (-1, -1)
    elif case == "local_4500":
        b, h, sq, sk, causal, window = 1, 8, 4500, 4500, False, (1000, 300)
    elif case == "rect_causal":
        b, h, sq, sk, causal, window = 3, 8, 2000, 4500, True, (-1, -1)     # 192 row blocks of 256: more than half the CUs
    elif case == "rect_local":
        b, h, sq, sk, causal, window = 2, 8, 4300, 2100, False, (700, 50)      # sq > sk: leading rows see nothing
    elif case == "d96_causal":       # head dims 65..96 take the kernel's 96-column variant
        b, h, sq, sk, causal, window, d = 1, 8, 4200, 4200, True, (-1, -1), 96
    elif case == "d80_local":
        b, h, sq, sk, causal, window, d = 1, 8, 4500, 4500, False, (1000, 300), 80
    elif case == "d72_rect_causal":
        b, h, sq, sk, causal, window, d = 3, 8, 2000, 4500, True, (-1, -1), 72
    else:
        b, h, sq, sk, causal, window, d = 2, 8, 2100, 2100, False, (-1, -1), 96
    q = _gen((b, sq, h, d), dtype, 1); k = _gen((b, sk, hk, d), dtype, 2); v = _gen((b, sk, hk, d), dtype, 3)
    out, lse, _ = _fa().flash_attn_func(q.to(DEV), k.to(DEV), v.to(DEV), causal=causal, window_size=window,
                                        return_attn_probs=True)
    _check(out, lse, q, k, v, causal=causal, window_size=window)


@pytest.mark.parametrize("d", [136, 160, 192, 224, 256])
@pytest.mark.parametrize("sq,sk,mode", [(777, 777, "causal"), (512, 512, "full"), (600, 1500, "causal"),
                                         (1500, 600, "local"), (1024, 1024, "local")])
def test_pair_kernel_head_dims_above_128(d, sq, sk, mode):
    _say("pair kernel", d, sq, sk, mode)
    dtype = torch.float16 if d == 160 and sq <= 777 else torch.bfloat16
    b, h, hk = 4, 16, 2
    q = _gen((b, sq, h, d), dtype, 1); k = _gen((b, sk, hk, d), dtype, 2); v = _gen((b, sk, hk, d), dtype, 3)
    window = _window(mode, sk, d * 31 + sq)
    out, lse, _ = _fa().flash_attn_func(q.to(DEV), k.to(DEV), v.to(DEV), causal=(mode == "causal"),
                                        window_size=window, return_attn_probs=True)
    _check(out, lse, q, k, v, causal=(mode == "causal"), window_size=window)


@pytest.mark.parametrize("s,d", [(1024, 64), (2304, 128), (1024, 256)])
def test_long_kernels_take_strided_packed_input(s, d):
    """q, k, v as strided views of one (b, s, 3, h, d) tensor: row stride 3*h*d."""
    _say("packed long", s, d)
    dtype = torch.bfloat16
    b, h = 2, 16
    qkv = _gen((b, s, 3, h, d), dtype, 5)
    out, lse, _ = _fa().flash_attn_qkvpacked_func(qkv.to(DEV), causal=True, return_attn_probs=True)
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
