"""GPU parity tests of the HIP forward path against the CPU oracle, through the public API (and so
through the C ABI).  Cases and the acceptance rule follow the reference's own test-suite
(tests/test_flash_attn.py): max|out - ref_fp32| <= 2 * max|ref_lowprec - ref_fp32| (+1e-5), with
log-sum-exp within 1e-3 relative on top (the reference never pins its values)."""
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


def _gen(shape, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=torch.float32).to(dtype)


def _check(out, lse, q, k, v, mult=2.0, extra=1e-5, **kw):
    out_ref, lse_ref, out_pt = orc.attention_reference_pair(q, k, v, **kw)
    ok, err, bound = orc.tolerance_ok(out.cpu(), out_ref, out_pt, mult, extra)
    _say("   out err %.3e bound %.3e" % (err, bound))
    assert not torch.isnan(out).any()
    assert ok, "output error %g exceeds bound %g" % (err, bound)
    if lse is not None:
        okl, rel = orc.lse_ok(lse.cpu(), lse_ref)
        _say("   lse rel %.3e" % rel)
        assert okl, "lse relative error %g" % rel


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("d", [64, 128, 256])
@pytest.mark.parametrize("causal", [False, True])
def test_dense_basic(dtype, d, causal):
    _say("dense_basic", dtype, d, causal)
    b, s, h = 2, 256, 4
    q, k, v = (_gen((b, s, h, d), dtype, i) for i in (1, 2, 3))
    out, lse, _ = _fa().flash_attn_func(q.to(DEV), k.to(DEV), v.to(DEV), causal=causal, return_attn_probs=True)
    assert out.shape == q.shape and lse.shape == (b, h, s)
    _check(out, lse, q, k, v, causal=causal)


def test_config1_fp16_dense():
    """The smallest benchmark configuration: fp16, batch 2, seqlen 512, 8 heads, headdim 64, non-causal."""
    _say("config1")
    torch.manual_seed(0)
    q, k, v = (_gen((2, 512, 8, 64), torch.float16, i) for i in (1, 2, 3))
    out, lse, _ = _fa().flash_attn_func(q.to(DEV), k.to(DEV), v.to(DEV), return_attn_probs=True)
    _check(out, lse, q, k, v)


@pytest.mark.parametrize("d", [32, 40, 59, 64, 80, 96, 111, 128, 160, 192, 224, 256])
@pytest.mark.parametrize("causal,local", [(False, False), (True, False), (False, True)])
def test_head_dims_and_masks(d, causal, local):
    """Head-dim sweep of tests/test_flash_attn.py:530-657 with ragged sequence lengths."""
    _say("head_dims", d, causal, local)
    dtype = torch.bfloat16
    b, sq, sk, h = 2, 217, 339, 3
    window = (-1, -1)
    if local:
        g = torch.Generator().manual_seed(d)
        window = tuple(torch.randint(0, sk, (2,), generator=g).tolist())
    q = _gen((b, sq, h, d), dtype, 1); k = _gen((b, sk, h, d), dtype, 2); v = _gen((b, sk, h, d), dtype, 3)
    out, lse, _ = _fa().flash_attn_func(q.to(DEV), k.to(DEV), v.to(DEV), causal=causal, window_size=window,
                                        return_attn_probs=True)
    _check(out, lse, q, k, v, causal=causal, window_size=window)


@pytest.mark.parametrize("sq,sk", [(1, 239), (3, 799), (127, 512), (127, 513), (113, 203), (128, 217),
                                   (113, 211), (108, 256), (256, 512), (1023, 1024), (239, 1), (799, 3),
                                   (513, 127), (1024, 1023)])
@pytest.mark.parametrize("mode", ["causal", "local"])
def test_bottom_right_alignment(sq, sk, mode):
    """seqlen_q != seqlen_k both ways: pins bottom-right mask alignment and zero rows
    (tests/test_flash_attn.py:1295-1402)."""
    _say("alignment", sq, sk, mode)
    dtype, d, b, h = torch.float16, 64, 2, 4
    window = (-1, -1)
    if mode == "local":
        g = torch.Generator().manual_seed(sq * 7 + sk)
        window = tuple(torch.randint(0, max(sk, 2), (2,), generator=g).tolist())
    q = _gen((b, sq, h, d), dtype, 1); k = _gen((b, sk, h, d), dtype, 2); v = _gen((b, sk, h, d), dtype, 3)
    out, lse, _ = _fa().flash_attn_func(q.to(DEV), k.to(DEV), v.to(DEV), causal=(mode == "causal"),
                                        window_size=window, return_attn_probs=True)
    _check(out, lse, q, k, v, causal=(mode == "causal"), window_size=window)


@pytest.mark.parametrize("mha_type", ["mqa", "gqa"])
@pytest.mark.parametrize("packed", ["none", "kv"])
def test_gqa_and_packed(mha_type, packed):
    _say("gqa", mha_type, packed)
    dtype, d, b, sq, sk, h = torch.bfloat16, 128, 2, 300, 421, 6
    hk = 1 if mha_type == "mqa" else 3
    q = _gen((b, sq, h, d), dtype, 1); k = _gen((b, sk, hk, d), dtype, 2); v = _gen((b, sk, hk, d), dtype, 3)
    fa = _fa()
    if packed == "kv":
        kv = torch.stack([k, v], dim=2).to(DEV)
        out, lse, _ = fa.flash_attn_kvpacked_func(q.to(DEV), kv, causal=True, return_attn_probs=True)
    else:
        out, lse, _ = fa.flash_attn_func(q.to(DEV), k.to(DEV), v.to(DEV), causal=True, return_attn_probs=True)
    _check(out, lse, q, k, v, causal=True)


def test_qkvpacked_strided_views():
    _say("qkvpacked")
    dtype, d, b, s, h = torch.float16, 96, 3, 200, 5
    qkv = _gen((b, s, 3, h, d), dtype, 5)
    out = _fa().flash_attn_qkvpacked_func(qkv.to(DEV), causal=True, softmax_scale=0.2)
    _check(out, None, qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2], causal=True, softmax_scale=0.2)


@pytest.mark.parametrize("d", [64, 128, 256])
@pytest.mark.parametrize("causal", [False, True])
def test_varlen(d, causal):
    """Packed sequences (tests/test_flash_attn.py:1011-1292): each attends alone; lse rows beyond a
    sequence's length are not compared."""
    _say("varlen", d, causal)
    dtype, h, hk = torch.bfloat16, 4, 2
    g = torch.Generator().manual_seed(d)
    lens_q = torch.randint(1, 400, (7,), generator=g)
    lens_k = lens_q.clone() if causal else torch.randint(1, 500, (7,), generator=g)
    lens_q[3] = 0 if not causal else lens_q[3]
    cu_q = torch.cat([torch.zeros(1, dtype=torch.long), lens_q.cumsum(0)]).int()
    cu_k = torch.cat([torch.zeros(1, dtype=torch.long), lens_k.cumsum(0)]).int()
    tq, tk = int(cu_q[-1]), int(cu_k[-1])
    mq, mk = int(lens_q.max()), int(lens_k.max())
    q = _gen((tq, h, d), dtype, 1); k = _gen((tk, hk, d), dtype, 2); v = _gen((tk, hk, d), dtype, 3)
    out, lse, _ = _fa().flash_attn_varlen_func(q.to(DEV), k.to(DEV), v.to(DEV), cu_q.to(DEV), cu_k.to(DEV),
                                              mq, mk, causal=causal, return_attn_probs=True)
    assert lse.shape == (7, h, mq)
    o_ref, l_ref = orc.attention_varlen_forward(q, k, v, cu_q, cu_k, mq, causal=causal)
    o_pt, _ = orc.attention_varlen_forward(q, k, v, cu_q, cu_k, mq, causal=causal, upcast=False, reorder_ops=True)
    ok, err, bound = orc.tolerance_ok(out.cpu(), o_ref, o_pt, 2.0, 1e-5)
    _say("   out err %.3e bound %.3e" % (err, bound))
    assert ok
    lse = lse.cpu()
    for i in range(7):
        n = int(lens_q[i])
        if n:
            assert orc.lse_ok(lse[i, :, :n], l_ref[i, :, :n])[0]


def test_varlen_qkvpacked():
    _say("varlen_qkvpacked")
    dtype, h, d = torch.float16, 3, 64
    lens = torch.tensor([5, 130, 64, 257])
    cu = torch.cat([torch.zeros(1, dtype=torch.long), lens.cumsum(0)]).int()
    qkv = _gen((int(cu[-1]), 3, h, d), dtype, 9)
    out = _fa().flash_attn_varlen_qkvpacked_func(qkv.to(DEV), cu.to(DEV), int(lens.max()), causal=True)
    o_ref, _ = orc.attention_varlen_forward(qkv[:, 0], qkv[:, 1], qkv[:, 2], cu, cu, int(lens.max()), causal=True)
    o_pt, _ = orc.attention_varlen_forward(qkv[:, 0], qkv[:, 1], qkv[:, 2], cu, cu, int(lens.max()), causal=True,
                                           upcast=False, reorder_ops=True)
    assert orc.tolerance_ok(out.cpu(), o_ref, o_pt, 2.0, 1e-5)[0]


@pytest.mark.parametrize("sq,sk", [(3, 1024), (1, 339), (64, 800), (3, 799), (64, 2048), (16, 20000), (128, 128)])
@pytest.mark.parametrize("causal,local", [(False, False), (True, False), (False, True)])
def test_splitkv_small_grids(sq, sk, causal, local):
    """Small grids make the planner split the key range (tests/test_flash_attn.py:1555-1659)."""
    _say("splitkv", sq, sk, causal, local)
    dtype, d, b, h = torch.float16, 128, 1, 12
    window = (-1, -1)
    if local:
        g = torch.Generator().manual_seed(sq + sk)
        window = tuple(torch.randint(0, sk, (2,), generator=g).tolist())
    q = _gen((b, sq, h, d), dtype, 1); k = _gen((b, sk, h, d), dtype, 2); v = _gen((b, sk, h, d), dtype, 3)
    out, lse, _ = _fa().flash_attn_func(q.to(DEV), k.to(DEV), v.to(DEV), causal=causal, window_size=window,
                                        return_attn_probs=True)
    _check(out, lse, q, k, v, causal=causal, window_size=window)


def _kvcache_case(seqlen_q, seqlen_k, d, has_batch_idx, rotary_fraction, rotary_interleaved, seqlen_new_eq,
                  causal, local, new_kv, mha_type, num_splits, dtype, seed=0):
    """Input construction of tests/test_flash_attn.py:1704-1860 on the CPU, run on the GPU, compared
    with the oracle: output (3x rule), V cache bit-exact, K cache within 1e-3."""
    g = torch.Generator().manual_seed(seed)
    batch_size = 2
    bc = batch_size if not has_batch_idx else batch_size * 2
    nheads = 6
    rotary_dim = math.floor(int(rotary_fraction * d) / 16) * 16
    hk = nheads if mha_type == "mha" else (1 if mha_type == "mqa" else 3)
    window = (-1, -1) if not local else tuple(torch.randint(0, seqlen_k, (2,), generator=g).tolist())
    q = _gen((batch_size, seqlen_q, nheads, d), dtype, seed + 1)
    seqlen_new = seqlen_q if seqlen_new_eq else int(torch.randint(1, seqlen_q + 1, (1,), generator=g))
    k = v = None
    if new_kv:
        k = _gen((batch_size, seqlen_new, hk, d), dtype, seed + 2)
        v = _gen((batch_size, seqlen_new, hk, d), dtype, seed + 3)
    kc = _gen((bc, seqlen_k, hk, d), dtype, seed + 4)
    vc = _gen((bc, seqlen_k, hk, d), dtype, seed + 5)
    hi = (seqlen_k - (seqlen_q if (causal or local) and rotary_dim > 1 else seqlen_new) + 1) if new_kv else (seqlen_k + 1)
    cache_seqlens = torch.randint(0, hi, (batch_size,), generator=g, dtype=torch.int32)
    idx = torch.randperm(bc, generator=g, dtype=torch.int32)[:batch_size] if has_batch_idx else None
    cos = sin = None
    if rotary_dim > 0:
        angle = torch.rand(seqlen_k, rotary_dim // 2, generator=g) * 2 * math.pi
        cos, sin = torch.cos(angle).to(dtype), torch.sin(angle).to(dtype)
    kc_d, vc_d = kc.to(DEV), vc.to(DEV)
    to = lambda t: None if t is None else t.to(DEV)
    out = _fa().flash_attn_with_kvcache(to(q), kc_d, vc_d, to(k), to(v), to(cos), to(sin), to(cache_seqlens),
                                        to(idx), causal=causal, window_size=window,
                                        rotary_interleaved=rotary_interleaved, num_splits=num_splits)
    kw = dict(causal=causal, window_size=window, rotary_interleaved=rotary_interleaved)
    o_ref, _, k_ref, v_ref = orc.kvcache_forward(q, kc, vc, k, v, cos, sin, cache_seqlens, idx, **kw)
    o_pt, _, _, _ = orc.kvcache_forward(q, kc, vc, k, v, cos, sin, cache_seqlens, idx, upcast=False,
                                        reorder_ops=True, **kw)
    assert not torch.isnan(out).any()
    ok, err, bound = orc.tolerance_ok(out.cpu(), o_ref, o_pt, 3.0, 1e-5)
    _say("   out err %.3e bound %.3e" % (err, bound))
    assert ok
    if new_kv:
        assert torch.equal(vc_d.cpu(), v_ref)
        assert torch.allclose(kc_d.cpu().float(), k_ref.float(), rtol=1e-3, atol=1e-3)
    else:
        assert torch.equal(vc_d.cpu(), vc) and torch.equal(kc_d.cpu(), kc)


@pytest.mark.parametrize("num_splits", [1, 0])
@pytest.mark.parametrize("mha_type", ["mha", "mqa", "gqa"])
@pytest.mark.parametrize("new_kv", [False, True])
@pytest.mark.parametrize("causal,local", [(False, False), (True, False), (False, True)])
@pytest.mark.parametrize("seqlen_q,seqlen_k", [(1, 128), (1, 339), (3, 1024), (64, 800), (16, 20000), (128, 128)])
def test_kvcache_matrix(seqlen_q, seqlen_k, new_kv, causal, local, mha_type, num_splits):
    _say("kvcache", seqlen_q, seqlen_k, new_kv, causal, local, mha_type, num_splits)
    _kvcache_case(seqlen_q, seqlen_k, 128, False, 0.0, True, True, causal, local, new_kv, mha_type, num_splits,
                  torch.float16)


@pytest.mark.parametrize("rotary_interleaved", [False, True])
@pytest.mark.parametrize("rotary_fraction", [0.5, 1.0])
@pytest.mark.parametrize("has_batch_idx", [False, True])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("seqlen_q,seqlen_k,d", [(1, 339, 128), (3, 1024, 64), (64, 800, 128), (2, 500, 256), (1, 256, 80)])
def test_kvcache_rotary_batch_idx(seqlen_q, seqlen_k, d, causal, has_batch_idx, rotary_fraction, rotary_interleaved):
    _say("kvcache_rotary", seqlen_q, seqlen_k, d, causal, has_batch_idx, rotary_fraction, rotary_interleaved)
    _kvcache_case(seqlen_q, seqlen_k, d, has_batch_idx, rotary_fraction, rotary_interleaved, False, causal, False,
                  True, "gqa", 0, torch.bfloat16, seed=3)


def test_kvcache_int_seqlens_and_no_seqlens():
    _say("kvcache_int")
    dtype, d = torch.float16, 64
    q = _gen((2, 1, 4, d), dtype, 1); kc = _gen((2, 300, 2, d), dtype, 2); vc = _gen((2, 300, 2, d), dtype, 3)
    fa = _fa()
    out = fa.flash_attn_with_kvcache(q.to(DEV), kc.to(DEV), vc.to(DEV), cache_seqlens=123)
    o_ref, _, _, _ = orc.kvcache_forward(q, kc, vc, cache_seqlens=123)
    o_pt, _, _, _ = orc.kvcache_forward(q, kc, vc, cache_seqlens=123, upcast=False, reorder_ops=True)
    assert orc.tolerance_ok(out.cpu(), o_ref, o_pt, 3.0, 1e-5)[0]
    out = fa.flash_attn_with_kvcache(q.to(DEV), kc.to(DEV), vc.to(DEV))
    o_ref, _, _, _ = orc.kvcache_forward(q, kc, vc)
    o_pt, _, _, _ = orc.kvcache_forward(q, kc, vc, upcast=False, reorder_ops=True)
    assert orc.tolerance_ok(out.cpu(), o_ref, o_pt, 3.0, 1e-5)[0]


@pytest.mark.parametrize("seqlen_q", [1, 40])
def test_kvcache_lengths_outside_the_cache_are_clamped(seqlen_q):
    """cache_seqlens beyond the capacity or negative are a caller error the reference does not check
    (flash_attn_interface.py:944-946).  Here they are clamped to [0, capacity]: no key, table row or
    appended row outside the cache is touched, and the result is that of the clamped lengths."""
    _say("kvcache_clamped", seqlen_q)
    dtype, d, cap = torch.float16, 64, 300
    q = _gen((2, seqlen_q, 4, d), dtype, 1); kc = _gen((2, cap, 2, d), dtype, 2); vc = _gen((2, cap, 2, d), dtype, 3)
    fa = _fa()
    bad = torch.tensor([cap + 100, -5], dtype=torch.int32)
    good = torch.tensor([cap, 0], dtype=torch.int32)
    out_bad = fa.flash_attn_with_kvcache(q.to(DEV), kc.to(DEV), vc.to(DEV), cache_seqlens=bad.to(DEV))
    out_good = fa.flash_attn_with_kvcache(q.to(DEV), kc.to(DEV), vc.to(DEV), cache_seqlens=good.to(DEV))
    assert torch.equal(out_bad, out_good)
    assert torch.equal(out_bad[1], torch.zeros_like(out_bad[1]))          # no visible key
    # with one new token: nothing is appended past the capacity, row 0 of the empty sequence is
    kn = _gen((2, 1, 2, d), dtype, 4); vn = _gen((2, 1, 2, d), dtype, 5)
    kc_d, vc_d = kc.to(DEV), vc.to(DEV)
    out = fa.flash_attn_with_kvcache(q[:, :1].to(DEV), kc_d, vc_d, k=kn.to(DEV), v=vn.to(DEV), cache_seqlens=bad.to(DEV))
    assert torch.equal(kc_d[0].cpu(), kc[0]) and torch.equal(vc_d[0].cpu(), vc[0])
    assert torch.equal(vc_d[1, 0].cpu(), vn[1, 0]) and torch.equal(vc_d[1, 1:].cpu(), vc[1, 1:])
    assert torch.allclose(out[1, 0].float().cpu(), vn[1, 0].float().repeat_interleave(2, dim=0), atol=1e-3)


@pytest.mark.parametrize("seqlen_q", [1, 40])
def test_kvcache_rotary_positions_stay_inside_the_table(seqlen_q):
    """A full (or nearly full) cache puts cache length + query row past the capacity; the rotary tables
    are only required to cover the capacity (flash_api.cpp:1214), so q positions stop at the last
    table row.  The tables here are the first `cap` rows of a buffer whose following rows are NaN: a
    read past the table would poison the output.  The result must equal the one obtained with
    tables that continue with copies of their last row."""
    _say("kvcache_rotary_clamp", seqlen_q)
    dtype, d, cap = torch.bfloat16, 64, 300
    q = _gen((2, seqlen_q, 4, d), dtype, 1); kc = _gen((2, cap, 2, d), dtype, 2); vc = _gen((2, cap, 2, d), dtype, 3)
    kn = _gen((2, seqlen_q, 2, d), dtype, 4); vn = _gen((2, seqlen_q, 2, d), dtype, 5)
    cos, sin = orc.rotary_table(cap, d, dtype=dtype)
    lens = torch.tensor([cap, cap - 3], dtype=torch.int32).to(DEV)
    fa = _fa()
    outs = []
    for tail in (float("nan"), None):
        big_c = torch.full((cap + 64, d // 2), float("nan"), dtype=dtype)
        big_s = torch.full((cap + 64, d // 2), float("nan"), dtype=dtype)
        big_c[:cap], big_s[:cap] = cos, sin
        if tail is None:
            big_c[cap:], big_s[cap:] = cos[-1], sin[-1]
        big_c, big_s = big_c.to(DEV), big_s.to(DEV)
        tc, ts = (big_c[:cap], big_s[:cap]) if tail is not None else (big_c, big_s)
        kc_d, vc_d = kc.to(DEV), vc.to(DEV)
        outs.append(fa.flash_attn_with_kvcache(q.to(DEV), kc_d, vc_d, kn.to(DEV), vn.to(DEV), tc, ts, lens, causal=True,
                                               rotary_interleaved=False))
        assert not torch.isnan(kc_d).any()
    assert not torch.isnan(outs[0]).any()
    assert torch.equal(outs[0], outs[1])


def test_kvcache_strided_cache_views():
    """K and V caches as strided views of one (b, s, 2, h_k, d) tensor, as the reference's MHA module
    passes them (flash_attn/modules/mha.py:459-477)."""
    _say("kvcache_strided")
    dtype, d = torch.bfloat16, 128
    kv = _gen((2, 700, 2, 2, d), dtype, 4)
    q = _gen((2, 1, 8, d), dtype, 5)
    lens = torch.tensor([650, 13], dtype=torch.int32)
    kv_d = kv.to(DEV)
    out = _fa().flash_attn_with_kvcache(q.to(DEV), kv_d[:, :, 0], kv_d[:, :, 1], cache_seqlens=lens.to(DEV))
    o_ref, _, _, _ = orc.kvcache_forward(q, kv[:, :, 0], kv[:, :, 1], cache_seqlens=lens)
    o_pt, _, _, _ = orc.kvcache_forward(q, kv[:, :, 0], kv[:, :, 1], cache_seqlens=lens, upcast=False, reorder_ops=True)
    assert orc.tolerance_ok(out.cpu(), o_ref, o_pt, 3.0, 1e-5)[0]


def test_num_splits_invariance():
    """Result independent of the split count up to fp32 re-association."""
    _say("num_splits_invariance")
    dtype, d = torch.bfloat16, 128
    q = _gen((2, 1, 16, d), dtype, 1); kc = _gen((2, 5000, 2, d), dtype, 2); vc = _gen((2, 5000, 2, d), dtype, 3)
    lens = torch.tensor([4999, 1234], dtype=torch.int32).to(DEV)
    fa = _fa()
    outs = [fa.flash_attn_with_kvcache(q.to(DEV), kc.to(DEV), vc.to(DEV), cache_seqlens=lens, num_splits=n).float()
            for n in (1, 2, 7, 0, 128)]
    for o in outs[1:]:
        assert (o - outs[0]).abs().max().item() < 1e-2
    o_ref, _, _, _ = orc.kvcache_forward(q, kc, vc, cache_seqlens=lens.cpu())
    o_pt, _, _, _ = orc.kvcache_forward(q, kc, vc, cache_seqlens=lens.cpu(), upcast=False, reorder_ops=True)
    for o in outs:
        assert orc.tolerance_ok(o.cpu(), o_ref, o_pt, 3.0, 1e-5)[0]


def test_repeatability():
    """Bit-identical out and lse over repeats (tests/test_flash_attn.py:1863-1930)."""
    _say("repeatability")
    dtype, d = torch.float16, 128
    q, k, v = (_gen((4, 333, 6, d), dtype, i).to(DEV) for i in (1, 2, 3))
    fa = _fa()
    o0, l0, _ = fa.flash_attn_func(q, k, v, causal=True, return_attn_probs=True)
    for _ in range(50):
        o, l, _ = fa.flash_attn_func(q, k, v, causal=True, return_attn_probs=True)
        assert torch.equal(o, o0) and torch.equal(l, l0)


def test_errors_surface_as_exceptions():
    _say("errors")
    fa = _fa()
    q = torch.randn(1, 8, 2, 64, device=DEV, dtype=torch.float16)
    with pytest.raises(RuntimeError):
        fa.flash_attn_func(q.float(), q.float(), q.float())
    with pytest.raises(RuntimeError):
        fa.flash_attn_func(q, q[:, :, :1].expand(1, 8, 3, 64), q)
    with pytest.raises(RuntimeError):
        fa.flash_attn_func(q, q, q, dropout_p=1.0)
    big = torch.randn(1, 8, 2, 264, device=DEV, dtype=torch.float16)
    with pytest.raises(RuntimeError):
        fa.flash_attn_func(big, big, big)
    with pytest.raises(RuntimeError):       # the KV-cache entry point has no dropout: the C ABI rejects it
        import ctypes
        from flash_attn import _native as nat
        p = nat.FaFwdParams()
        p.q = p.k = p.v = p.o = p.softmax_lse = q.data_ptr()
        p.b, p.h, p.h_k, p.d, p.seqlen_q, p.seqlen_k, p.dtype, p.p_dropout = 1, 2, 2, 64, 8, 8, 0, 0.1
        p.rng_state = q.data_ptr()
        nat._call(nat.lib.fa_fwd_kvcache, p, 0)
