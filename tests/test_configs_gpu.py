"""The five benchmark configurations at their full sizes on the GPU.

The whole problem runs through the public API; the CPU oracle then checks a SAMPLE of (batch, head)
pairs / sequences / cache rows (the units are independent, and the full score tensors would be tens
of GB): fixed corner units plus units drawn anew on every run (the draw's seed is printed, and
FA_SAMPLE_SEED replays it), under the reference's tolerance rule (tests/test_flash_attn.py:648-650) with
log-sum-exp within 1e-3 relative.  Size-independent properties (bit-repeatability, split-count
invariance, appended cache rows) are checked on the whole output."""
import math
import os
import random
import sys
import time

import pytest
import torch

from oracle import attention_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def _drawn(n, *ranges):
    """n index tuples drawn anew on every run, one index below each of `ranges`"""
    seed = int(os.environ.get("FA_SAMPLE_SEED", time.time_ns() % (1 << 31)))
    rng = random.Random(seed)
    picks = [tuple(rng.randrange(r) for r in ranges) for _ in range(n)]
    _say("   sample drawn with FA_SAMPLE_SEED=%d: %s" % (seed, picks))
    return picks


def _fa():
    import flash_attn
    return flash_attn


def _check_heads(out, lse, q, k, v, pairs, group, mult=2.0, **kw):
    """Compare (batch, q-head) pairs against the oracle; k/v heads follow the GQA mapping."""
    for (b, h) in pairs:
        qs = q[b:b + 1, :, h:h + 1].cpu()
        ks = k[b:b + 1, :, h // group:h // group + 1].cpu()
        vs = v[b:b + 1, :, h // group:h // group + 1].cpu()
        o_ref, l_ref, o_pt = orc.attention_reference_pair(qs, ks, vs, **kw)
        ok, err, bound = orc.tolerance_ok(out[b:b + 1, :, h:h + 1].cpu(), o_ref, o_pt, mult, 1e-5)
        _say("   (b=%d,h=%d) out err %.3e bound %.3e" % (b, h, err, bound))
        assert ok, (b, h, err, bound)
        if lse is not None:
            okl, rel = orc.lse_ok(lse[b:b + 1, h:h + 1].cpu(), l_ref)
            assert okl, (b, h, rel)


def test_config2_bf16_causal_8k():
    """bf16, batch 4, seqlen 8192, 32 heads, head dim 128, causal, scale 1/sqrt(128); out + lse."""
    _say("config2")
    torch.manual_seed(0)
    b, s, h, d = 4, 8192, 32, 128
    q, k, v = (torch.randn(b, s, h, d, device=DEV, dtype=torch.bfloat16) for _ in range(3))
    fa = _fa()
    out, lse, _ = fa.flash_attn_func(q, k, v, softmax_scale=1 / math.sqrt(128), causal=True, return_attn_probs=True)
    assert not torch.isnan(out).any() and torch.isfinite(lse).all()
    _check_heads(out, lse, q, k, v, [(0, 0), (3, 31), (1, 17)] + _drawn(2, b, h), 1, causal=True, softmax_scale=1 / math.sqrt(128))
    out2, lse2, _ = fa.flash_attn_func(q, k, v, softmax_scale=1 / math.sqrt(128), causal=True, return_attn_probs=True)
    assert torch.equal(out, out2) and torch.equal(lse, lse2)
    # first row of every (batch, head) sees exactly one key: out = v[0], lse = scale * q0.k0
    assert torch.equal(out[:, 0], v[:, 0])
    s00 = (q[:, 0].float() * k[:, 0].float()).sum(-1) / math.sqrt(128)
    assert torch.allclose(lse[:, :, 0], s00, rtol=1e-3, atol=1e-3)


def test_config2_dense_matches_qkvpacked():
    _say("config2 dense / qkvpacked")
    torch.manual_seed(1)
    b, s, h, d = 2, 4096, 16, 128
    qkv = torch.randn(b, s, 3, h, d, device=DEV, dtype=torch.bfloat16)
    fa = _fa()
    o1 = fa.flash_attn_qkvpacked_func(qkv)
    o2 = fa.flash_attn_func(qkv[:, :, 0].contiguous(), qkv[:, :, 1].contiguous(), qkv[:, :, 2].contiguous())
    assert torch.equal(o1, o2)
    _check_heads(o1, None, qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2], [(1, 5)], 1)


def test_config3_gqa_sliding_window_16k():
    """bf16, batch 2, seqlen 16384, 32 q heads / 8 kv heads, head dim 128, causal, window (4096, 0)."""
    _say("config3")
    torch.manual_seed(0)
    b, s, h, hk, d = 2, 16384, 32, 8, 128
    q = torch.randn(b, s, h, d, device=DEV, dtype=torch.bfloat16)
    k = torch.randn(b, s, hk, d, device=DEV, dtype=torch.bfloat16)
    v = torch.randn(b, s, hk, d, device=DEV, dtype=torch.bfloat16)
    out, lse, _ = _fa().flash_attn_func(q, k, v, causal=True, window_size=(4096, 0), return_attn_probs=True)
    assert not torch.isnan(out).any()
    _check_heads(out, lse, q, k, v, [(0, 3), (1, 30)] + _drawn(1, b, h), h // hk, causal=True, window_size=(4096, 0))


@pytest.mark.parametrize("d", [128, 256])
def test_config4_varlen_64_sequences(d):
    """bf16, 64 packed sequences with lengths uniform in [128, 4096], 16 heads, causal."""
    _say("config4", d)
    torch.manual_seed(0)
    h = 16
    lens = torch.randint(128, 4097, (64,))
    cu = torch.cat([torch.zeros(1, dtype=torch.long), lens.cumsum(0)]).int()
    total, mx = int(cu[-1]), int(lens.max())
    q, k, v = (torch.randn(total, h, d, device=DEV, dtype=torch.bfloat16) for _ in range(3))
    cu_d = cu.to(DEV)
    out, lse, _ = _fa().flash_attn_varlen_func(q, k, v, cu_d, cu_d, mx, mx, causal=True, return_attn_probs=True)
    assert out.shape == q.shape and lse.shape == (64, h, mx)
    assert not torch.isnan(out).any()
    order = torch.argsort(lens)
    units = [(int(order[j]), hh) for j in (0, 31, -1) for hh in (0, 11)] + [(7, 0), (7, 11)]   # shortest, median, longest, one more
    for i, hh in units + _drawn(3, 64, h):
        a, e = int(cu[i]), int(cu[i + 1])
        qs, ks, vs = (t[a:e, hh:hh + 1][None].cpu() for t in (q, k, v))
        o_ref, l_ref, o_pt = orc.attention_reference_pair(qs, ks, vs, causal=True)
        ok, err, bound = orc.tolerance_ok(out[a:e, hh:hh + 1][None].cpu(), o_ref, o_pt, 2.0, 1e-5)
        _say("   seq %d (len %d) head %d: err %.3e bound %.3e" % (i, e - a, hh, err, bound))
        assert ok
        assert orc.lse_ok(lse[i, hh:hh + 1, : e - a][None].cpu(), l_ref)[0]


def test_config5_decode_kvcache_rotary():
    """bf16 decode: batch 64, caches (64, 32768, 8, 128), 64 q heads (GQA 8:1), one new token
    appended with rotary (dim 128, base 10000, interleaved), cache_seqlens uniform in [1024, 32767]."""
    _say("config5")
    torch.manual_seed(0)
    b, cap, hk, h, d = 64, 32768, 8, 64, 128
    kc = torch.randn(b, cap, hk, d, device=DEV, dtype=torch.bfloat16)
    vc = torch.randn(b, cap, hk, d, device=DEV, dtype=torch.bfloat16)
    q = torch.randn(b, 1, h, d, device=DEV, dtype=torch.bfloat16)
    kn = torch.randn(b, 1, hk, d, device=DEV, dtype=torch.bfloat16)
    vn = torch.randn(b, 1, hk, d, device=DEV, dtype=torch.bfloat16)
    lens = torch.randint(1024, cap, (b,), dtype=torch.int32)
    lens[0], lens[1] = 1024, cap - 1
    cos, sin = orc.rotary_table(cap, d, dtype=torch.bfloat16)
    sample = sorted(set([0, 1, 17, 63] + [i for (i,) in _drawn(2, b)]))
    before_k = {i: kc[i, : int(lens[i]) + 2].cpu() for i in sample}
    before_v = {i: vc[i, : int(lens[i]) + 2].cpu() for i in sample}
    lens_d = lens.to(DEV)
    fa = _fa()
    # the native entry point behind flash_attn_with_kvcache, which also returns the log-sum-exp
    # (mha_fwd_kvcache, csrc/flash_attn/flash_api.cpp:1278)
    import flash_attn._native as nat
    out, lse = nat.fwd_kvcache(q, kc, vc, kn, vn, lens_d, cos.to(DEV), sin.to(DEV), None, None, d ** -0.5, True, -1, -1,
                               True, 0)
    assert not torch.isnan(out).any() and lse.shape == (b, h, 1)
    for i in sample:
        L = int(lens[i])
        o_ref, l_ref, k_ref, v_ref = orc.kvcache_forward(q[i:i + 1].cpu(), before_k[i][None], before_v[i][None],
                                                         kn[i:i + 1].cpu(), vn[i:i + 1].cpu(), cos, sin,
                                                         torch.tensor([L], dtype=torch.int32), causal=True)
        o_pt, _, _, _ = orc.kvcache_forward(q[i:i + 1].cpu(), before_k[i][None], before_v[i][None],
                                            kn[i:i + 1].cpu(), vn[i:i + 1].cpu(), cos, sin,
                                            torch.tensor([L], dtype=torch.int32), causal=True, upcast=False,
                                            reorder_ops=True)
        ok, err, bound = orc.tolerance_ok(out[i:i + 1].cpu(), o_ref, o_pt, 3.0, 1e-5)
        _say("   batch %d (len %d): err %.3e bound %.3e" % (i, L, err, bound))
        assert ok
        assert orc.lse_ok(lse[i:i + 1].cpu(), l_ref, 1e-3)[0]                    # persistent kernel + merge
        assert torch.equal(vc[i, : L + 2].cpu(), v_ref[0])                       # V rows bit-exact
        assert torch.allclose(kc[i, : L + 2].cpu().float(), k_ref[0].float(), rtol=1e-3, atol=1e-3)
    # the appended V row of EVERY batch entry is the new value, bit for bit
    rows = vc[torch.arange(b, device=DEV), lens_d.long()]
    assert torch.equal(rows, vn[:, 0])
    # split-count invariance on the whole output (cache already holds the appended token: no k/v now)
    lens1 = lens_d + 1
    outs = [fa.flash_attn_with_kvcache(q, kc, vc, cache_seqlens=lens1, num_splits=n).float() for n in (0, 1, 5)]
    assert (outs[0] - outs[1]).abs().max().item() < 2e-2 and (outs[0] - outs[2]).abs().max().item() < 2e-2


def test_decode_ticket_schedule_matches_one_workgroup_per_chunk(monkeypatch):
    """The decode call takes the persistent, ticket-scheduled kernel when the caller passes a scratch
    word and the one-workgroup-per-chunk kernel when it does not (work_counter == NULL at the C
    boundary); both must give the same attention output (up to fp32 re-association of the combine)
    and agree with the oracle."""
    _say("decode: ticket schedule vs plain")
    from flash_attn import _native as nat
    torch.manual_seed(3)
    b, cap, hk, h, d = 16, 32768, 8, 64, 128
    kc = torch.randn(b, cap, hk, d, device=DEV, dtype=torch.bfloat16)
    vc = torch.randn(b, cap, hk, d, device=DEV, dtype=torch.bfloat16)
    q = torch.randn(b, 1, h, d, device=DEV, dtype=torch.bfloat16)
    lens = torch.randint(1, cap + 1, (b,), dtype=torch.int32)
    lens[0], lens[1], lens[2] = 1, cap, 4097
    lens_d = lens.to(DEV)
    fa = _fa()
    out_ticket = fa.flash_attn_with_kvcache(q, kc, vc, cache_seqlens=lens_d, causal=True)

    seen = []

    # the plan must be made with the same (absent) scratch word as the launch: patch before planning
    def plan_without(params, api, batch, heads, seqlen_q, dd, device):
        import ctypes
        n = ctypes.c_int32(0)
        params.work_counter = None
        rc = nat.lib.fa_plan_splits(ctypes.byref(params), api, ctypes.byref(n))
        assert rc == 0
        seen.append(n.value)
        keep = ()
        if n.value > 1:
            lse_accum = torch.empty((n.value, batch, heads, seqlen_q), dtype=torch.float32, device=device)
            o_accum = torch.empty((n.value, batch, heads, seqlen_q, (dd + 31) // 32 * 32), dtype=torch.float32, device=device)
            params.lse_accum = lse_accum.data_ptr()
            params.o_accum = o_accum.data_ptr()
            keep = (lse_accum, o_accum)
        return keep
    monkeypatch.setattr(nat, "_plan_and_alloc", plan_without)
    out_plain = fa.flash_attn_with_kvcache(q, kc, vc, cache_seqlens=lens_d, causal=True)
    monkeypatch.undo()
    assert seen and seen[0] > 1                      # the plain path did split
    assert not torch.isnan(out_ticket).any() and not torch.isnan(out_plain).any()
    diff = (out_ticket.float() - out_plain.float()).abs().max().item()
    _say("   max |ticket - plain| = %.3e" % diff)
    assert diff < 2e-2
    for i in (0, 1, 2, 9):
        L = int(lens[i])
        o_ref, _, o_pt = orc.attention_reference_pair(q[i:i + 1].cpu(), kc[i:i + 1, :L].cpu(), vc[i:i + 1, :L].cpu(), causal=True)
        for name, o in (("ticket", out_ticket), ("plain", out_plain)):
            ok, err, bound = orc.tolerance_ok(o[i:i + 1].cpu(), o_ref, o_pt, 3.0, 1e-5)
            _say("   batch %d (len %d) %s: err %.3e bound %.3e" % (i, L, name, err, bound))
            assert ok
