"""GPU parity of the backward pass (fa_bwd / fa_varlen_bwd behind the six autograd functions) against
the CPU oracle.  Cases follow the reference's tests/test_flash_attn.py (:530-657 packed qkv, :660-1010
q / kv / separate, :1013-1292 variable length, :1295-1402 causal with seqlen_q != seqlen_k): fp16 and
bf16, head dims 32..256 including ones that are padded, MHA / GQA / MQA, full / causal / local masks,
ragged lengths.  Acceptance is the reference's rule (:1006-1008):
max|dx - dx_ref| <= 2 max|dx_pt - dx_ref| (+1e-5 absolute), dx_ref the fp32 oracle and dx_pt torch
autograd through an ordinary implementation in the input precision."""
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


def _window(mode, sk, seed):
    if mode != "local":
        return (-1, -1)
    g = torch.Generator().manual_seed(seed)
    return tuple(torch.randint(0, sk, (2,), generator=g).tolist())


def _check_grads(got, q, k, v, dout, **kw):
    ref = orc.attention_backward(q, k, v, dout, **kw)
    pt = orc.attention_backward_autograd(q, k, v, dout, upcast=False, reorder_ops=True, **kw)
    for name, a, r, p_ in zip(("dq", "dk", "dv"), got, ref, pt):
        assert a.shape == r.shape, name
        assert not torch.isnan(a).any(), name
        err = (a.float().cpu() - r).abs().max().item()
        bound = 2 * (p_.float() - r).abs().max().item() + 1e-5
        _say("   %s err %.3e bound %.3e" % (name, err, bound))
        assert err <= bound, "%s error %g exceeds bound %g" % (name, err, bound)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("mode", ["full", "causal", "local"])
@pytest.mark.parametrize("d", [32, 59, 64, 80, 96, 128, 160, 192, 224, 256])
@pytest.mark.parametrize("sq,sk", [(113, 203), (128, 217), (108, 256), (256, 512), (1, 147), (257, 1), (384, 256)])
def test_backward_separate_qkv(sq, sk, d, mode, dtype):
    _say("bwd", sq, sk, d, mode, dtype)
    b, h = 3, 6
    hk = {0: 6, 1: 2, 2: 1}[(d // 32 + sq) % 3]               # MHA / GQA / MQA in turn
    q = _gen((b, sq, h, d), dtype, 1); k = _gen((b, sk, hk, d), dtype, 2); v = _gen((b, sk, hk, d), dtype, 3)
    dout = _gen((b, sq, h, d), dtype, 4)
    window = _window(mode, sk, d + sq)
    qd, kd, vd = [t.to(DEV).requires_grad_() for t in (q, k, v)]
    out = _fa().flash_attn_func(qd, kd, vd, causal=(mode == "causal"), window_size=window)
    got = torch.autograd.grad(out, (qd, kd, vd), dout.to(DEV))
    _check_grads(got, q, k, v, dout, causal=(mode == "causal"), window_size=window)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("mode", ["full", "causal", "local"])
@pytest.mark.parametrize("d", [40, 64, 128, 256])
@pytest.mark.parametrize("s", [97, 128, 200, 384, 768])
def test_backward_qkvpacked(s, d, mode, dtype):
    """Gradient of the packed (b, s, 3, h, d) input: dq, dk, dv are written as strided views of one tensor."""
    _say("bwd qkvpacked", s, d, mode, dtype)
    b, h = 2, 4
    qkv = _gen((b, s, 3, h, d), dtype, 5)
    dout = _gen((b, s, h, d), dtype, 6)
    window = _window(mode, s, d + s)
    x = qkv.to(DEV).requires_grad_()
    out = _fa().flash_attn_qkvpacked_func(x, causal=(mode == "causal"), window_size=window)
    (dqkv,) = torch.autograd.grad(out, x, dout.to(DEV))
    assert dqkv.shape == qkv.shape
    _check_grads((dqkv[:, :, 0], dqkv[:, :, 1], dqkv[:, :, 2]), qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2], dout,
                 causal=(mode == "causal"), window_size=window)


@pytest.mark.parametrize("mode", ["full", "causal", "local"])
@pytest.mark.parametrize("d", [64, 96, 128])
def test_backward_kvpacked_gqa(d, mode):
    _say("bwd kvpacked", d, mode)
    dtype, b, sq, sk, h, hk = torch.bfloat16, 2, 300, 421, 8, 2
    q = _gen((b, sq, h, d), dtype, 1); kv = _gen((b, sk, 2, hk, d), dtype, 2); dout = _gen((b, sq, h, d), dtype, 3)
    window = _window(mode, sk, d)
    qd, kvd = q.to(DEV).requires_grad_(), kv.to(DEV).requires_grad_()
    out = _fa().flash_attn_kvpacked_func(qd, kvd, causal=(mode == "causal"), window_size=window)
    dq, dkv = torch.autograd.grad(out, (qd, kvd), dout.to(DEV))
    _check_grads((dq, dkv[:, :, 0], dkv[:, :, 1]), q, kv[:, :, 0], kv[:, :, 1], dout, causal=(mode == "causal"),
                 window_size=window)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("mode", ["full", "causal", "local"])
@pytest.mark.parametrize("d", [32, 64, 96, 111, 128, 160, 256])
def test_backward_varlen(d, mode, dtype):
    """Packed sequences with different q and k lengths per sequence, an empty and a one-token one.
    Each sequence's gradients equal those of that sequence attended alone."""
    _say("bwd varlen", d, mode, dtype)
    h, hk = 4, 2
    lens_q = [0, 1, 63, 129, 200, 77, 256]
    lens_k = [5, 1, 200, 64, 333, 0, 256]
    cu_q = torch.tensor([0] + list(torch.tensor(lens_q).cumsum(0)), dtype=torch.int32)
    cu_k = torch.tensor([0] + list(torch.tensor(lens_k).cumsum(0)), dtype=torch.int32)
    tq, tk = int(cu_q[-1]), int(cu_k[-1])
    q = _gen((tq, h, d), dtype, 1); k = _gen((tk, hk, d), dtype, 2); v = _gen((tk, hk, d), dtype, 3)
    dout = _gen((tq, h, d), dtype, 4)
    window = _window(mode, 64, d)
    qd, kd, vd = [t.to(DEV).requires_grad_() for t in (q, k, v)]
    out = _fa().flash_attn_varlen_func(qd, kd, vd, cu_q.to(DEV), cu_k.to(DEV), max(lens_q), max(lens_k),
                                       causal=(mode == "causal"), window_size=window)
    dq, dk, dv = torch.autograd.grad(out, (qd, kd, vd), dout.to(DEV))
    assert not (torch.isnan(dq).any() or torch.isnan(dk).any() or torch.isnan(dv).any())
    for i in range(len(lens_q)):
        a, e, c, f = int(cu_q[i]), int(cu_q[i + 1]), int(cu_k[i]), int(cu_k[i + 1])
        if e == a or f == c:
            # nothing attends, or nothing is attended to: the gradients of this sequence are zero
            assert not dq[a:e].any() and not dk[c:f].any() and not dv[c:f].any()
            continue
        _say("  seq", i, lens_q[i], lens_k[i])
        _check_grads((dq[a:e][None], dk[c:f][None], dv[c:f][None]), q[a:e][None], k[c:f][None], v[c:f][None],
                     dout[a:e][None], causal=(mode == "causal"), window_size=window)


@pytest.mark.parametrize("d", [64, 128])
def test_backward_varlen_packed_forms(d):
    _say("bwd varlen packed", d)
    dtype, h = torch.float16, 4
    lens = [130, 1, 257, 64]
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    total = int(cu[-1])
    qkv = _gen((total, 3, h, d), dtype, 7); dout = _gen((total, h, d), dtype, 8)
    x = qkv.to(DEV).requires_grad_()
    out = _fa().flash_attn_varlen_qkvpacked_func(x, cu.to(DEV), max(lens), causal=True)
    (dqkv,) = torch.autograd.grad(out, x, dout.to(DEV))
    qd, kvd = qkv[:, 0].to(DEV).requires_grad_(), qkv[:, 1:].contiguous().to(DEV).requires_grad_()
    out2 = _fa().flash_attn_varlen_kvpacked_func(qd, kvd, cu.to(DEV), cu.to(DEV), max(lens), max(lens), causal=True)
    dq2, dkv2 = torch.autograd.grad(out2, (qd, kvd), dout.to(DEV))
    # same kernels, same inputs: the two packings agree bit for bit
    assert torch.equal(dqkv[:, 0], dq2) and torch.equal(dqkv[:, 1:], dkv2)
    for i in range(len(lens)):
        a, e = int(cu[i]), int(cu[i + 1])
        _check_grads((dqkv[a:e, 0][None], dqkv[a:e, 1][None], dqkv[a:e, 2][None]), qkv[a:e, 0][None], qkv[a:e, 1][None],
                     qkv[a:e, 2][None], dout[a:e][None], causal=True)


@pytest.mark.parametrize("d", [64, 80, 96, 128, 160, 192, 256])
@pytest.mark.parametrize("mode", ["causal", "local"])
def test_backward_long_sequences(d, mode):
    """Lengths at which the forward runs its long-sequence kernels and the backward streams many tiles."""
    _say("bwd long", d, mode)
    dtype, b, h, hk, sq, sk = torch.bfloat16, 1, 4, 2, 1100, 1500
    q = _gen((b, sq, h, d), dtype, 1); k = _gen((b, sk, hk, d), dtype, 2); v = _gen((b, sk, hk, d), dtype, 3)
    dout = _gen((b, sq, h, d), dtype, 4)
    window = (300, 200) if mode == "local" else (-1, -1)
    qd, kd, vd = [t.to(DEV).requires_grad_() for t in (q, k, v)]
    out = _fa().flash_attn_func(qd, kd, vd, causal=(mode == "causal"), window_size=window)
    got = torch.autograd.grad(out, (qd, kd, vd), dout.to(DEV))
    _check_grads(got, q, k, v, dout, causal=(mode == "causal"), window_size=window)


def test_backward_is_deterministic_and_returns_softmax_d():
    """No atomics anywhere: two runs agree bit for bit; softmax_d is rowsum(dout * out) as the
    reference returns it (flash_api.cpp:741, 810)."""
    _say("bwd deterministic")
    from flash_attn import _native as nat
    dtype, b, sq, sk, h, hk, d = torch.bfloat16, 2, 300, 700, 8, 2, 128
    q = _gen((b, sq, h, d), dtype, 1).to(DEV); k = _gen((b, sk, hk, d), dtype, 2).to(DEV)
    v = _gen((b, sk, hk, d), dtype, 3).to(DEV); dout = _gen((b, sq, h, d), dtype, 4).to(DEV)
    out, _, _, _, _, lse, _, _ = nat.fwd(q, k, v, None, 0.0, d ** -0.5, True, -1, -1, False, None)
    r1 = nat.bwd(dout, q, k, v, out, lse, None, None, None, 0.0, d ** -0.5, True, -1, -1, None, None)
    r2 = nat.bwd(dout, q, k, v, out, lse, None, None, None, 0.0, d ** -0.5, True, -1, -1, None, None)
    for a, c in zip(r1, r2):
        assert torch.equal(a, c)
    softmax_d = r1[3]
    assert softmax_d.shape == (b, h, 384) and softmax_d.dtype == torch.float32
    want = (dout.float() * out.float()).sum(-1).permute(0, 2, 1)
    assert torch.allclose(softmax_d[:, :, :sq], want, rtol=1e-4, atol=1e-4)


def test_backward_rejects_missing_rng_state_and_bad_shapes():
    _say("bwd errors")
    from flash_attn import _native as nat
    q = torch.zeros(1, 8, 2, 64, dtype=torch.float16, device=DEV)
    lse = torch.zeros(1, 2, 8, dtype=torch.float32, device=DEV)
    with pytest.raises(RuntimeError, match="rng_state"):        # dropout needs the forward's seed and offset
        nat.bwd(q, q, q, q, q, lse, None, None, None, 0.1, 0.125, False, -1, -1, None, None)
    with pytest.raises(RuntimeError, match="dq has the wrong shape"):
        nat.bwd(q, q, q, q, q, lse, q[:, :4], None, None, 0.0, 0.125, False, -1, -1, None, None)
    with pytest.raises(RuntimeError, match="same dtype"):
        nat.bwd(q, q, q.to(torch.bfloat16), q, q, lse, None, None, None, 0.0, 0.125, False, -1, -1, None, None)


def test_forward_and_backward_replay_from_a_hip_graph():
    """A training step's attention (forward + backward, no dropout) captured once and replayed with new
    inputs copied into the static tensors: every replay must equal the eager result.  Nothing in the
    two entry points synchronises, allocates outside torch's graph pool or depends on device values
    on the host."""
    _say("bwd graph")
    dtype, b, s, h, hk, d = torch.bfloat16, 2, 384, 4, 2, 128
    fa = _fa()
    q = torch.zeros(b, s, h, d, device=DEV, dtype=dtype, requires_grad=True)
    k = torch.zeros(b, s, hk, d, device=DEV, dtype=dtype, requires_grad=True)
    v = torch.zeros(b, s, hk, d, device=DEV, dtype=dtype, requires_grad=True)
    dout = torch.zeros(b, s, h, d, device=DEV, dtype=dtype)

    def step():
        out = fa.flash_attn_func(q, k, v, causal=True)
        return (out,) + torch.autograd.grad(out, (q, k, v), dout)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
        side.synchronize()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static = step()
    for seed in (1, 2, 3):
        with torch.no_grad():
            q.copy_(_gen((b, s, h, d), dtype, seed)); k.copy_(_gen((b, s, hk, d), dtype, seed + 10))
            v.copy_(_gen((b, s, hk, d), dtype, seed + 20)); dout.copy_(_gen((b, s, h, d), dtype, seed + 30))
        graph.replay()
        torch.cuda.synchronize()
        eager = step()
        torch.cuda.synchronize()
        for a, c in zip(static, eager):
            assert torch.equal(a, c)
