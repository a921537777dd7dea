"""GPU tests of dropout on the attention probabilities, forward and backward.

The reference's method (tests/test_flash_attn.py:583-657, 905-1010): run with dropout_p = 0.17 and
return_attn_probs=True, read the mask that the kernel used out of S_dmask (negative = dropped), feed
that mask to the oracle, and require output and gradients to agree under the usual rule; the fraction
of dropped entries must be within 0.01 of dropout_p (:652-655).  Here S_dmask is in plain (row, key)
order, so no fragment-layout decoding is needed.  Gradient parity is what shows that the backward
regenerates the very mask of the forward from rng_state: both of its kernels walk the score matrix
in a different register geometry than the forward."""
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


def _ran(name, head_dims=None):
    """the forward launch before this call took the dropout instantiation of kernel `name`"""
    from flash_attn import _native as nat
    got = nat.last_kernel()
    _say("   kernel", got)
    assert got[0] == name and got[1] and not got[2], got
    if head_dims is not None:
        assert got[3] == head_dims, got


def _check_all(out, lse, S, grads, q, k, v, dout, p, causal, window, entries=None):
    """entries: batch entries to check (independent problems), default all"""
    if entries is not None:
        for e in entries:
            _say("   batch entry", e)
            sl = lambda t: t[e:e + 1]
            _check_all(sl(out), sl(lse), sl(S), [sl(g) for g in grads], sl(q), sl(k), sl(v), sl(dout), p, causal, window)
        return
    b, sq, h, d = q.shape
    sk = k.shape[1]
    S = S[:, :, :sq, :sk].float().cpu()
    mask = ~torch.signbit(S)
    vis = orc.visible_mask(sq, sk, window, causal)
    n = int(vis.sum()) * b * h
    frac = 1.0 - mask[:, :, vis].float().mean().item()
    _say("   dropped fraction %.4f over %d entries" % (frac, n))
    # the reference's 0.01, widened by four standard deviations where few entries are visible
    assert abs(frac - p) < 0.01 + 4.0 * (p * (1 - p) / max(n, 1)) ** 0.5
    kw = dict(causal=causal, window_size=window, dropout_p=p, dropout_mask=mask)
    o_ref, lse_ref = orc.attention_forward(q.float(), k.float(), v.float(), **kw)
    o_pt, _ = orc.attention_forward(q, k, v, upcast=False, reorder_ops=True, **kw)
    ok, err, bound = orc.tolerance_ok(out.cpu(), o_ref, o_pt, 2.0, 1e-5)
    _say("   out err %.3e bound %.3e" % (err, bound))
    assert ok
    assert orc.lse_ok(lse.cpu(), lse_ref)[0]          # dropout does not touch the log-sum-exp
    # |S_dmask| is the softmax probability itself
    hk = k.shape[2]
    s = torch.einsum("bthd,bshd->bhts", q.float(), k.float().repeat_interleave(h // hk, 2)) * d ** -0.5
    probs = torch.nan_to_num(torch.softmax(s.masked_fill(~vis, float("-inf")), -1), 0.0)
    assert (S.abs() - probs).abs().max().item() < 4e-3
    ref = orc.attention_backward(q, k, v, dout, **kw)
    pt = orc.attention_backward_autograd(q, k, v, dout, upcast=False, reorder_ops=True, **kw)
    for name, a, r, p_ in zip(("dq", "dk", "dv"), grads, ref, pt):
        e = (a.float().cpu() - r).abs().max().item()
        bnd = 2 * (p_.float() - r).abs().max().item() + 1e-5
        _say("   %s err %.3e bound %.3e" % (name, e, bnd))
        assert e <= bnd, name


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("mode", ["full", "causal", "local"])
@pytest.mark.parametrize("d", [32, 59, 64, 96, 128, 192, 256])
@pytest.mark.parametrize("sq,sk", [(113, 203), (128, 217), (256, 512), (384, 256), (1, 239)])
def test_dropout_forward_backward(sq, sk, d, mode, dtype):
    _say("dropout", sq, sk, d, mode, dtype)
    b, h, p = 2, 6, 0.17
    hk = {0: 6, 1: 2, 2: 1}[(d // 32 + sq) % 3]
    q = _gen((b, sq, h, d), dtype, 1); k = _gen((b, sk, hk, d), dtype, 2); v = _gen((b, sk, hk, d), dtype, 3)
    dout = _gen((b, sq, h, d), dtype, 4)
    window = (-1, -1)
    if mode == "local":
        g = torch.Generator().manual_seed(d + sq)
        window = tuple(torch.randint(0, sk, (2,), generator=g).tolist())
    qd, kd, vd = [t.to(DEV).requires_grad_() for t in (q, k, v)]
    out, lse, S = _fa().flash_attn_func(qd, kd, vd, dropout_p=p, causal=(mode == "causal"), window_size=window,
                                        return_attn_probs=True)
    assert S.shape == (b, h, (sq + 127) // 128 * 128, (sk + 127) // 128 * 128) and S.dtype == dtype
    grads = torch.autograd.grad(out, (qd, kd, vd), dout.to(DEV))
    _check_all(out, lse, S, grads, q, k, v, dout, p, mode == "causal", window)


@pytest.mark.parametrize("d", [64, 128, 256])
@pytest.mark.parametrize("p", [0.1, 0.5])
def test_dropout_on_the_long_sequence_kernels(d, p):
    """From 96 query rows on the forward runs on the software-pipelined kernels (pairs of waves at
    head dim 256), which walk the score matrix in steps of their own."""
    _say("dropout long", d, p)
    dtype, b, h, s = torch.bfloat16, 1, 4, 1100
    q = _gen((b, s, h, d), dtype, 1); k = _gen((b, s, h, d), dtype, 2); v = _gen((b, s, h, d), dtype, 3)
    dout = _gen((b, s, h, d), dtype, 4)
    qd, kd, vd = [t.to(DEV).requires_grad_() for t in (q, k, v)]
    out, lse, S = _fa().flash_attn_func(qd, kd, vd, dropout_p=p, causal=True, return_attn_probs=True)
    _ran("wide_pair" if d == 256 else "pipelined")
    grads = torch.autograd.grad(out, (qd, kd, vd), dout.to(DEV))
    _check_all(out, lse, S, grads, q, k, v, dout, p, True, (-1, -1))


# The dropout instantiation of the 8-wave ping-pong kernel, which applies the mask in its own register geometry (one
# query row per lane).  Dispatch sends a launch there at head dim 65..128 with keys beyond 768 (no mask) / from 2048
# on (masked), more than 128 / 256 row blocks of 256 rows and no window spanning 768 keys or fewer: the batch makes
# the launch that large, and three batch entries (independent problems) are checked.
@pytest.mark.parametrize("sq,sk,d,mode,dtype,b,h,hk", [
    (640, 2300, 128, "full", torch.bfloat16, 24, 2, 1),          # 3 x 2 x 24 = 144 row blocks, no mask
    (600, 4200, 96, "causal", torch.float16, 44, 2, 2),          # 3 x 2 x 44 = 264; sq < sk; 96 of the 128 columns
    (1030, 4300, 128, "local", torch.bfloat16, 26, 2, 1),        # 5 x 2 x 26 = 260; two-sided window of 1800 keys
    (1300, 2100, 128, "causal", torch.float16, 22, 2, 2),        # 6 x 2 x 22 = 264; fp16 at all 128 columns
    (2200, 2100, 80, "causal", torch.bfloat16, 15, 2, 1),        # 9 x 2 x 15 = 270; sq > sk: leading rows see nothing
])
def test_dropout_on_the_pingpong_kernel(sq, sk, d, mode, dtype, b, h, hk):
    _say("dropout ping-pong", sq, sk, d, mode, dtype)
    p = 0.17
    q = _gen((b, sq, h, d), dtype, 1); k = _gen((b, sk, hk, d), dtype, 2); v = _gen((b, sk, hk, d), dtype, 3)
    dout = _gen((b, sq, h, d), dtype, 4)
    window = (1500, 300) if mode == "local" else (-1, -1)
    qd, kd, vd = [t.to(DEV).requires_grad_() for t in (q, k, v)]
    out, lse, S = _fa().flash_attn_func(qd, kd, vd, dropout_p=p, causal=(mode == "causal"), window_size=window,
                                        return_attn_probs=True)
    _ran("pingpong", 128)       # (the dropout instantiation always runs all 128 columns)
    grads = torch.autograd.grad(out, (qd, kd, vd), dout.to(DEV))
    _check_all(out, lse, S, grads, q, k, v, dout, p, mode == "causal", window, entries=[0, b - 1, b // 2])


def test_dropout_qkvpacked_and_varlen():
    _say("dropout packed / varlen")
    dtype, h, d, p = torch.float16, 4, 64, 0.17
    lens = [130, 1, 257, 64]
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    total = int(cu[-1])
    qkv = _gen((total, 3, h, d), dtype, 7); dout = _gen((total, h, d), dtype, 8)
    x = qkv.to(DEV).requires_grad_()
    out, lse, S = _fa().flash_attn_varlen_qkvpacked_func(x, cu.to(DEV), max(lens), dropout_p=p, causal=True,
                                                         return_attn_probs=True)
    (dqkv,) = torch.autograd.grad(out, x, dout.to(DEV))
    assert S.shape == (len(lens), h, 384, 384)
    for i, L in enumerate(lens):
        a, e = int(cu[i]), int(cu[i + 1])
        Si = S[i:i + 1, :, :L, :L].float().cpu()
        mask = ~torch.signbit(Si)
        kw = dict(causal=True, dropout_p=p, dropout_mask=mask)
        qi, ki, vi, gi = qkv[a:e, 0][None], qkv[a:e, 1][None], qkv[a:e, 2][None], dout[a:e][None]
        o_ref, _ = orc.attention_forward(qi.float(), ki.float(), vi.float(), **kw)
        o_pt, _ = orc.attention_forward(qi, ki, vi, upcast=False, reorder_ops=True, **kw)
        assert orc.tolerance_ok(out[a:e][None].cpu(), o_ref, o_pt, 2.0, 1e-5)[0]
        ref = orc.attention_backward(qi, ki, vi, gi, **kw)
        pt = orc.attention_backward_autograd(qi, ki, vi, gi, upcast=False, reorder_ops=True, **kw)
        # The one-token sequence has P = 1, so dS = P (dP - D) vanishes only as far as D = rowsum(dO o O)
        # equals dP = dO . (r v): with dropout O = r v is rounded to 16 bits before D is formed (in the
        # reference's algorithm too), which leaves |dP| 2^-11 where torch's softmax gradient is exactly 0.
        atol = 1e-3 if L == 1 else 1e-5
        for j in range(3):
            err = (dqkv[a:e, j][None].float().cpu() - ref[j]).abs().max().item()
            assert err <= 2 * (pt[j].float() - ref[j]).abs().max().item() + atol
    # dense packed form
    qkv4 = _gen((2, 200, 3, h, d), dtype, 9)
    x4 = qkv4.to(DEV).requires_grad_()
    out4, lse4, S4 = _fa().flash_attn_qkvpacked_func(x4, dropout_p=p, return_attn_probs=True)
    g4 = _gen((2, 200, h, d), dtype, 10)
    (dqkv4,) = torch.autograd.grad(out4, x4, g4.to(DEV))
    _check_all(out4, lse4, S4, (dqkv4[:, :, 0], dqkv4[:, :, 1], dqkv4[:, :, 2]), qkv4[:, :, 0], qkv4[:, :, 1],
               qkv4[:, :, 2], g4, p, False, (-1, -1))


def test_dropout_mask_follows_the_generator():
    """Same generator state => same mask and output; the state advances with every call; masks of
    different calls, heads and batch entries are unrelated (agreement about p_keep^2 + p_drop^2)."""
    _say("dropout generator")
    dtype, b, s, h, d, p = torch.float16, 2, 256, 4, 64, 0.25
    q = _gen((b, s, h, d), dtype, 1).to(DEV); k = _gen((b, s, h, d), dtype, 2).to(DEV); v = _gen((b, s, h, d), dtype, 3).to(DEV)
    torch.cuda.manual_seed(1234)
    o1, _, S1 = _fa().flash_attn_func(q, k, v, dropout_p=p, return_attn_probs=True)
    o2, _, S2 = _fa().flash_attn_func(q, k, v, dropout_p=p, return_attn_probs=True)
    torch.cuda.manual_seed(1234)
    o3, _, S3 = _fa().flash_attn_func(q, k, v, dropout_p=p, return_attn_probs=True)
    assert torch.equal(o1, o3) and torch.equal(S1, S3)
    m1, m2 = ~torch.signbit(S1.float()), ~torch.signbit(S2.float())
    expect = (1 - p) ** 2 + p ** 2
    assert abs((m1 == m2).float().mean().item() - expect) < 0.01
    assert abs((m1[0] == m1[1]).float().mean().item() - expect) < 0.01          # batch entries
    assert abs((m1[:, 0] == m1[:, 1]).float().mean().item() - expect) < 0.01    # heads
    assert abs((m1[:, :, :-1] == m1[:, :, 1:]).float().mean().item() - expect) < 0.01   # neighbouring rows
    assert abs((m1[..., :-1] == m1[..., 1:]).float().mean().item() - expect) < 0.01     # neighbouring keys
    # every row and every column keeps about 1 - p of its entries
    assert (m1.float().mean(-1) - (1 - p)).abs().max().item() < 0.15
    assert (m1.float().mean(-2) - (1 - p)).abs().max().item() < 0.15


def test_return_attn_probs_needs_dropout_and_kvcache_has_none():
    from flash_attn import _native as nat
    q = torch.zeros(1, 8, 2, 64, dtype=torch.float16, device=DEV)
    out, lse, S = _fa().flash_attn_func(q, q, q, return_attn_probs=True)        # dropout 0: S is None, as the reference
    assert S is None
    with pytest.raises(RuntimeError, match="return_softmax is only supported when p_dropout > 0.0"):
        nat.fwd(q, q, q, None, 0.0, 0.125, False, -1, -1, True, None)
