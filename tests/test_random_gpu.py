"""Seeded random sweeps of the three entry points against the oracle, beyond the fixed grids of the
other GPU tests: shapes, masks, head groupings, dtypes, dropout, packed lengths (empty sequences
included), cache lengths, appended tokens, rotary, cache_batch_idx and split counts are drawn at
random; the rules are the usual ones (tests/test_flash_attn.py:583-657 for the tolerances).

Rows that see fewer than a handful of keys are kept out of the dropout cases, and problems with
fewer than 8 rows or keys get 3x instead of 2x on the gradients: there dS = P o (dP - D) is a small
difference of large terms and D = rowsum(dO o O) comes, as in the reference
(csrc/flash_attn/src/flash_bwd_kernel.h:74-180), from the 16-bit O, so the deviation from the exact
gradient is that of the algorithm, not of its implementation (exact arithmetic on that definition
reproduces it)."""
import math
import random
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


def _grad_check(tag, got, ref, pt, extra=0.0, mult=2.0):
    for name, a, r, p_ in zip(("dq", "dk", "dv"), got, ref, pt):
        e = (a.float().cpu() - r).abs().max().item()
        bnd = mult * (p_.float() - r).abs().max().item() + 1e-5 + extra
        assert not torch.isnan(a).any(), (tag, name)
        assert e <= bnd, "%s %s error %g exceeds bound %g" % (tag, name, e, bnd)


@pytest.mark.parametrize("block", range(6))
def test_random_dense_forward_backward(block):
    rnd = random.Random(100 + block)
    for it in range(10):
        d = rnd.choice([8, 16, 24, 32, 40, 56, 64, 72, 96, 104, 128, 136, 160, 192, 200, 256])
        hk = rnd.choice([1, 2, 3]); h = hk * rnd.choice([1, 2, 4])
        b = rnd.choice([1, 2, 3])
        sq = rnd.choice([1, 2, 7, 31, 32, 33, 63, 64, 65, 100, 127, 128, 129, 200, 255, 256, 257, 300, 511, 513, 600, 1024, 1100])
        sk = rnd.choice([1, 2, 7, 31, 32, 33, 63, 64, 65, 100, 127, 128, 129, 200, 255, 256, 257, 300, 511, 513, 700, 1100, 2300])
        mode = rnd.choice(["full", "causal", "local", "local_l", "local_r"])
        dtype = rnd.choice([torch.float16, torch.bfloat16])
        p = rnd.choice([0.0, 0.0, 0.2])
        if sk < 16 or (mode != "full" and sk < sq + 16):
            p = 0.0
        window = (-1, -1)
        if mode == "local": window = (rnd.randint(0, sk), rnd.randint(0, sk))
        if mode == "local_l": window = (rnd.randint(0, sk), -1)
        if mode == "local_r": window = (-1, rnd.randint(0, sk))
        if p > 0 and mode.startswith("local"):
            window = tuple(w if w < 0 else max(w, 16) for w in window)
        causal = mode == "causal"
        g = torch.Generator().manual_seed(block * 100 + it)
        q = torch.randn(b, sq, h, d, generator=g).to(dtype); k = torch.randn(b, sk, hk, d, generator=g).to(dtype)
        v = torch.randn(b, sk, hk, d, generator=g).to(dtype); do = torch.randn(b, sq, h, d, generator=g).to(dtype)
        tag = "dense %d.%d b%d sq%d sk%d h%d/%d d%d %s %s %s p%.1f" % (block, it, b, sq, sk, h, hk, d, mode, window, str(dtype)[6:], p)
        _say(tag)
        qd, kd, vd = [t.to(DEV).requires_grad_() for t in (q, k, v)]
        out, lse, S = _fa().flash_attn_func(qd, kd, vd, dropout_p=p, causal=causal, window_size=window, return_attn_probs=True)
        grads = torch.autograd.grad(out, (qd, kd, vd), do.to(DEV))
        kw = dict(causal=causal, window_size=window)
        if p > 0:
            kw.update(dropout_p=p, dropout_mask=~torch.signbit(S[:, :, :sq, :sk].float().cpu()))
        o_ref, lse_ref = orc.attention_forward(q.float(), k.float(), v.float(), **kw)
        o_pt, _ = orc.attention_forward(q, k, v, upcast=False, reorder_ops=True, **kw)
        ok, err, bound = orc.tolerance_ok(out.detach().cpu(), o_ref, o_pt, 2.0, 1e-5)
        assert ok, "%s out error %g exceeds bound %g" % (tag, err, bound)
        assert orc.lse_ok(lse.cpu(), lse_ref)[0], tag
        ref = orc.attention_backward(q, k, v, do, **kw)
        pt = orc.attention_backward_autograd(q, k, v, do, upcast=False, reorder_ops=True, **kw)
        # problems of a few rows or keys are entirely in the regime the module docstring describes: 3x there
        _grad_check(tag, grads, ref, pt, 1e-3 if p > 0 else 0.0, 3.0 if min(sq, sk) < 8 else 2.0)


@pytest.mark.parametrize("block", range(4))
def test_random_packed_forward_backward(block):
    rnd = random.Random(200 + block)
    for it in range(8):
        d = rnd.choice([32, 40, 64, 96, 128, 160, 256])
        hk = rnd.choice([1, 2]); h = hk * rnd.choice([1, 2, 4])
        b = rnd.choice([1, 2, 3, 5])
        lens = [8, 64, 65, 127, 128, 129, 200, 300, 511, 512, 513, 700, 1030]
        if it % 3 == 0:
            lens = lens + [0, 0, 1]
        lq = [rnd.choice(lens) for _ in range(b)]
        lk = lq if rnd.random() < 0.5 else [max(rnd.choice(lens), x) for x in lq]   # keys at least as long as queries
        mode = rnd.choice(["full", "causal", "local"])
        dtype = rnd.choice([torch.float16, torch.bfloat16])
        window = (rnd.randint(8, 300), rnd.randint(8, 300)) if mode == "local" else (-1, -1)
        causal = mode == "causal"
        cq = torch.tensor([0] + lq).cumsum(0).int(); ck = torch.tensor([0] + lk).cumsum(0).int()
        tq, tk = int(cq[-1]), int(ck[-1])
        if tq == 0 or tk == 0:
            continue
        g = torch.Generator().manual_seed(2000 + block * 100 + it)
        q = torch.randn(tq, h, d, generator=g).to(dtype); k = torch.randn(tk, hk, d, generator=g).to(dtype)
        v = torch.randn(tk, hk, d, generator=g).to(dtype); do = torch.randn(tq, h, d, generator=g).to(dtype)
        tag = "packed %d.%d lq %s lk %s h%d/%d d%d %s %s %s" % (block, it, lq, lk, h, hk, d, mode, window, str(dtype)[6:])
        _say(tag)
        qd, kd, vd = [t.to(DEV).requires_grad_() for t in (q, k, v)]
        out, lse, _ = _fa().flash_attn_varlen_func(qd, kd, vd, cq.to(DEV), ck.to(DEV), max(lq), max(lk), causal=causal,
                                                   window_size=window, return_attn_probs=True)
        dq, dk, dv = torch.autograd.grad(out, (qd, kd, vd), do.to(DEV))
        o_ref, _ = orc.attention_varlen_forward(q.float(), k.float(), v.float(), cq, ck, max(lq), causal=causal, window_size=window)
        o_pt, _ = orc.attention_varlen_forward(q, k, v, cq, ck, max(lq), causal=causal, window_size=window, upcast=False,
                                               reorder_ops=True)
        ok, err, bound = orc.tolerance_ok(out.detach().cpu(), o_ref, o_pt, 2.0, 1e-5)
        assert ok, "%s out error %g exceeds bound %g" % (tag, err, bound)
        for i in range(b):
            q0, q1, k0, k1 = int(cq[i]), int(cq[i + 1]), int(ck[i]), int(ck[i + 1])
            if q1 == q0 or k1 == k0:       # nothing flows through an empty side
                assert k1 == k0 or (dk[k0:k1].abs().max() == 0 and dv[k0:k1].abs().max() == 0), tag
                assert q1 == q0 or dq[q0:q1].abs().max() == 0, tag
                continue
            kw = dict(causal=causal, window_size=window)
            args = (q[q0:q1][None], k[k0:k1][None], v[k0:k1][None], do[q0:q1][None])
            ref = orc.attention_backward(*args, **kw)
            pt = orc.attention_backward_autograd(*args, upcast=False, reorder_ops=True, **kw)
            _grad_check("%s seq %d" % (tag, i), (dq[q0:q1][None], dk[k0:k1][None], dv[k0:k1][None]), ref, pt,
                        mult=3.0 if min(q1 - q0, k1 - k0) < 8 else 2.0)


@pytest.mark.parametrize("block", range(6))
def test_random_kvcache(block):
    rnd = random.Random(300 + block)
    for it in range(10):
        g = torch.Generator().manual_seed(3000 + block * 100 + it)
        gen = lambda shape, dtype: torch.randn(*shape, generator=g, dtype=torch.float32).to(dtype)
        d = rnd.choice([32, 64, 80, 96, 128, 160, 256])
        seqlen_q = rnd.choice([1, 1, 1, 2, 3, 5, 16, 17, 64, 100, 130, 260])
        seqlen_k = max(rnd.choice([1, 17, 128, 129, 255, 256, 339, 1000, 1024, 3000, 5000, 8200, 12000]), seqlen_q + 3)
        b = rnd.choice([1, 2, 3, 7])
        hk = rnd.choice([1, 2, 3]); h = hk * rnd.choice([1, 2, 4, 8, 8, 17, 32])
        has_idx = rnd.random() < 0.3
        bc = b * 2 if has_idx else b
        new_kv = rnd.random() < 0.5
        mode = rnd.choice(["full", "causal", "local"])
        dtype = rnd.choice([torch.float16, torch.bfloat16])
        rotary_dim = math.floor(int((rnd.choice([0.0, 0.0, 0.5, 1.0]) if new_kv else 0.0) * d) / 16) * 16
        inter = rnd.random() < 0.5
        num_splits = rnd.choice([0, 0, 1, 3])
        window = (-1, -1) if mode != "local" else (rnd.randint(0, seqlen_k), rnd.randint(0, seqlen_k))
        causal = mode == "causal"
        seqlen_new = rnd.randint(1, seqlen_q) if new_kv else 0
        q = gen((b, seqlen_q, h, d), dtype)
        k = v = None
        if new_kv:
            k = gen((b, seqlen_new, hk, d), dtype); v = gen((b, seqlen_new, hk, d), dtype)
        kc = gen((bc, seqlen_k, hk, d), dtype); vc = gen((bc, seqlen_k, hk, d), dtype)
        hi = (seqlen_k - (seqlen_q if mode != "full" and rotary_dim > 1 else seqlen_new) + 1) if new_kv else seqlen_k + 1
        cache_seqlens = torch.randint(0, max(hi, 1), (b,), generator=g, dtype=torch.int32)
        idx = torch.randperm(bc, generator=g, dtype=torch.int32)[:b] if has_idx else None
        cos = sin = None
        if rotary_dim > 0:
            angle = torch.rand(seqlen_k, rotary_dim // 2, generator=g) * 2 * math.pi
            cos, sin = torch.cos(angle).to(dtype), torch.sin(angle).to(dtype)
        tag = "kvcache %d.%d b%d sq%d sk%d new%d h%d/%d d%d %s %s rot%d/%d idx%d splits%d %s" % (
            block, it, b, seqlen_q, seqlen_k, seqlen_new, h, hk, d, mode, window, rotary_dim, inter, has_idx, num_splits, str(dtype)[6:])
        _say(tag)
        kc_d, vc_d = kc.to(DEV), vc.to(DEV)
        to = lambda t: None if t is None else t.to(DEV)
        out = _fa().flash_attn_with_kvcache(to(q), kc_d, vc_d, to(k), to(v), to(cos), to(sin), to(cache_seqlens), to(idx),
                                            causal=causal, window_size=window, rotary_interleaved=inter, num_splits=num_splits)
        kw = dict(causal=causal, window_size=window, rotary_interleaved=inter)
        o_ref, _, k_ref, v_ref = orc.kvcache_forward(q, kc, vc, k, v, cos, sin, cache_seqlens, idx, **kw)
        o_pt, _, _, _ = orc.kvcache_forward(q, kc, vc, k, v, cos, sin, cache_seqlens, idx, upcast=False, reorder_ops=True, **kw)
        assert not torch.isnan(out).any(), tag
        ok, err, bound = orc.tolerance_ok(out.cpu(), o_ref, o_pt, 3.0, 1e-5)
        assert ok, "%s out error %g exceeds bound %g" % (tag, err, bound)
        if new_kv:
            assert torch.equal(vc_d.cpu(), v_ref), tag
            assert torch.allclose(kc_d.cpu().float(), k_ref.float(), rtol=1e-3, atol=1e-3), tag
        else:
            assert torch.equal(vc_d.cpu(), vc) and torch.equal(kc_d.cpu(), kc), tag
