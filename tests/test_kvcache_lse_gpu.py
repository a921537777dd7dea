"""Log-sum-exp of the KV-cache path against the oracle (1e-3 relative, infinities exact).

flash_attn_with_kvcache returns only `out`; the native entry point behind it returns
[out, softmax_lse] like mha_fwd_kvcache (csrc/flash_attn/flash_api.cpp:1278).  Each case below names
the kernel it is sized to reach: the persistent ticket-scheduled decode kernel with its merge of
the partial results, the one-workgroup-per-chunk decode kernel (split and unsplit), and the tiled
kernel in its split form (more than 16 packed query rows)."""
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


def _fa_func():
    import flash_attn
    return flash_attn.flash_attn_func


def _nat():
    import flash_attn._native as nat
    return nat


def _gen(shape, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g).to(dtype)


def _run(q, kc, vc, lens, kn=None, vn=None, cos=None, sin=None, causal=False, window=(-1, -1), num_splits=0,
         interleaved=True):
    nat = _nat()
    d = q.shape[-1]
    dev = lambda t: None if t is None else t.to(DEV)
    kc_d, vc_d = kc.to(DEV), vc.to(DEV)
    out, lse = nat.fwd_kvcache(dev(q), kc_d, vc_d, dev(kn), dev(vn), dev(lens), dev(cos), dev(sin), None, None,
                               d ** -0.5, causal, window[0], window[1], interleaved, num_splits)
    o_ref, l_ref, _, _ = orc.kvcache_forward(q, kc, vc, kn, vn, cos, sin, lens, causal=causal, window_size=window,
                                             rotary_interleaved=interleaved)
    o_pt, _, _, _ = orc.kvcache_forward(q, kc, vc, kn, vn, cos, sin, lens, causal=causal, window_size=window,
                                        rotary_interleaved=interleaved, upcast=False, reorder_ops=True)
    ok, err, bound = orc.tolerance_ok(out.cpu(), o_ref, o_pt, 3.0, 1e-5)
    assert ok, (err, bound)
    assert lse.shape == (q.shape[0], q.shape[2], q.shape[1])
    ok, rel = orc.lse_ok(lse.cpu(), l_ref, 1e-3)
    assert ok, rel
    return lse.cpu(), l_ref


@pytest.mark.parametrize("with_new", [False, True])
def test_lse_persistent_decode_and_merge(with_new):
    """One decode step over caches large enough for the ticket-scheduled kernel (it takes over from
    about 4 million cached key rows per launch: 8 x 32768 x 16 here, chunks of 2048 keys): sequences
    with many complete chunks plus a ragged remainder, one chunk plus a few keys, less than one chunk,
    and an empty cache.  Every batch entry is checked against the oracle on its own slice."""
    _say("kvcache_lse persistent", with_new)
    nat = _nat()
    dtype, d, cap, b, h = torch.bfloat16, 64, 32768, 8, 16
    torch.manual_seed(5)
    kc = torch.randn(b, cap, h, d, device=DEV, dtype=dtype)
    vc = torch.randn(b, cap, h, d, device=DEV, dtype=dtype)
    q = torch.randn(b, 1, h, d, device=DEV, dtype=dtype)
    lens = torch.tensor([cap - 1, 1100, 3000, 5, 0, 20000, 2048, 2051], dtype=torch.int32)
    kn = vn = cos = sin = None
    if with_new:
        kn = torch.randn(b, 1, h, d, device=DEV, dtype=dtype)
        vn = torch.randn(b, 1, h, d, device=DEV, dtype=dtype)
        cos, sin = orc.rotary_table(cap, d, dtype=dtype)
    before = {i: (kc[i, : int(lens[i]) + 2].cpu(), vc[i, : int(lens[i]) + 2].cpu()) for i in range(b)}
    # the plan the library makes for this call must be the persistent one, or the test proves nothing
    p = nat.FaFwdParams()
    p.b, p.h, p.h_k, p.seqlen_q, p.seqlen_k, p.d, p.dtype = b, h, h, 1, cap, d, 1
    p.is_seqlens_k_cumulative = 0
    p.softmax_scale = d ** -0.5
    p.window_left = p.window_right = -1
    for name in ("q", "k", "v", "o", "softmax_lse", "work_counter", "cu_seqlens_k"):
        setattr(p, name, 256)          # non-null placeholders: planning reads no memory
    p.work_counter_len = nat.WORK_COUNTER_WORDS
    import ctypes
    n = ctypes.c_int32(0)
    assert nat.lib.fa_plan_splits(ctypes.byref(p), 2, ctypes.byref(n)) == 0
    assert n.value == cap // 2048 + 4, n.value      # 16 complete-chunk slots + 4 remainder slots of 512 keys
    dev = lambda t: None if t is None else t.to(DEV)
    out, lse = nat.fwd_kvcache(q, kc, vc, kn, vn, lens.to(DEV), dev(cos), dev(sin), None, None, d ** -0.5, True, -1, -1,
                               True, 0)
    for i in range(b):
        L = torch.tensor([int(lens[i])], dtype=torch.int32)
        sl = lambda t: None if t is None else t[i:i + 1].cpu()
        args = (q[i:i + 1].cpu(), before[i][0][None], before[i][1][None], sl(kn), sl(vn), cos, sin, L)
        o_ref, l_ref, _, _ = orc.kvcache_forward(*args, causal=True)
        o_pt, _, _, _ = orc.kvcache_forward(*args, causal=True, upcast=False, reorder_ops=True)
        ok, err, bound = orc.tolerance_ok(out[i:i + 1].cpu(), o_ref, o_pt, 3.0, 1e-5)
        assert ok, (i, err, bound)
        ok, rel = orc.lse_ok(lse[i:i + 1].cpu(), l_ref, 1e-3)
        _say("   batch %d (len %d): err %.3e bound %.3e lse rel %.3e" % (i, int(lens[i]), err, bound, rel))
        assert ok, (i, rel)
    if not with_new:
        assert torch.isposinf(lse[4]).all() and (out[4] == 0).all()      # empty cache, nothing appended


@pytest.mark.parametrize("num_splits", [1, 4])
def test_lse_decode_kernel_one_workgroup_per_chunk(num_splits):
    """Explicit split counts take the one-workgroup-per-chunk decode kernel (unsplit, and split with
    the stand-alone merge); the empty sequence sees no key: lse = +inf, out = 0."""
    _say("kvcache_lse decode", num_splits)
    dtype, d, cap, b, h, hk = torch.float16, 64, 1500, 3, 8, 2
    q = _gen((b, 2, h, d), dtype, 1); kc = _gen((b, cap, hk, d), dtype, 2); vc = _gen((b, cap, hk, d), dtype, 3)
    lens = torch.tensor([1500, 0, 333], dtype=torch.int32)
    lse, l_ref = _run(q, kc, vc, lens, num_splits=num_splits)
    assert torch.isposinf(lse[1]).all() and torch.isposinf(l_ref[1]).all()


def test_lse_tiled_split_kernel():
    """40 query rows x 4 grouped heads do not fit the decode kernel's 16 packed rows: the tiled kernel
    runs in its split form.  With a causal mask and 10 cached keys the first rows of the second
    sequence see nothing."""
    _say("kvcache_lse tiled split")
    dtype, d, cap, b, h, hk = torch.bfloat16, 128, 3000, 2, 8, 2
    q = _gen((b, 40, h, d), dtype, 1); kc = _gen((b, cap, hk, d), dtype, 2); vc = _gen((b, cap, hk, d), dtype, 3)
    lens = torch.tensor([2900, 10], dtype=torch.int32)
    lse, l_ref = _run(q, kc, vc, lens, causal=True, num_splits=3)
    assert torch.isposinf(l_ref[1, :, :30]).all() and torch.isposinf(lse[1, :, :30]).all()
    _run(q, kc, vc, lens, causal=True, window=(100, 0), num_splits=0)


@pytest.mark.parametrize("mode", ["plain", "causal", "append_rotary", "window_right", "window_left"])
@pytest.mark.parametrize("h,hk,d", [(32, 1, 128), (64, 2, 64), (40, 2, 128), (24, 1, 256), (17, 1, 96)])
def test_single_query_with_more_than_16_grouped_heads(h, hk, d, mode):
    """One query position and more grouped q heads per kv head than the decode kernel packs (16): the library
    reads q and out with the grouped heads as rows (the reference's seqlen_q <-> ngroups swap,
    csrc/flash_attn/flash_api.cpp:1096-1104), so K/V are fetched once per kv head.  Output, log-sum-exp and the
    appended rows must be those of the plain problem; a left window bound keeps the plain form."""
    _say("single query, many grouped heads", h, hk, d, mode)
    nat = _nat()
    dtype, cap, b = torch.bfloat16, 5000, 3
    torch.manual_seed(h + d)
    kc = torch.randn(b, cap, hk, d, dtype=dtype)
    vc = torch.randn(b, cap, hk, d, dtype=dtype)
    q = torch.randn(b, 1, h, d, dtype=dtype)
    lens = torch.tensor([4096, 37, 2500], dtype=torch.int32)
    kn = vn = cos = sin = None
    causal, wl, wr = mode == "causal", -1, -1
    if mode == "append_rotary":
        kn = torch.randn(b, 1, hk, d, dtype=dtype)
        vn = torch.randn(b, 1, hk, d, dtype=dtype)
        cos, sin = orc.rotary_table(cap, d, dtype=dtype)
        causal = True
    if mode == "window_right":
        wr = 7
    if mode == "window_left":
        wl = 300
    dev = lambda t: None if t is None else t.to(DEV)
    kc_d, vc_d = kc.to(DEV), vc.to(DEV)
    out, lse = nat.fwd_kvcache(q.to(DEV), kc_d, vc_d, dev(kn), dev(vn), lens.to(DEV), dev(cos), dev(sin), None, None, d ** -0.5,
                               causal, wl, wr, True, 0)
    kw = dict(causal=causal, window_size=(wl, wr))
    o_ref, l_ref, k_ref, v_ref = orc.kvcache_forward(q, kc, vc, kn, vn, cos, sin, lens, **kw)
    o_pt, _, _, _ = orc.kvcache_forward(q, kc, vc, kn, vn, cos, sin, lens, upcast=False, reorder_ops=True, **kw)
    ok, err, bound = orc.tolerance_ok(out.cpu(), o_ref, o_pt, 3.0, 1e-5)
    _say("   out err %.3e bound %.3e" % (err, bound))
    assert ok
    assert lse.shape == (b, h, 1) and orc.lse_ok(lse.cpu(), l_ref, 1e-3)[0]
    assert torch.equal(vc_d.cpu(), v_ref)
    assert torch.allclose(kc_d.cpu().float(), k_ref.float(), rtol=1e-3, atol=1e-3)
    # the same through the public call without a cache argument (mha_fwd path), one batch entry at its length
    if mode in ("plain", "causal"):
        L = int(lens[2])
        o2 = _fa_func()(q[2:3].to(DEV), kc[2:3, :L].to(DEV), vc[2:3, :L].to(DEV), causal=causal)
        assert orc.tolerance_ok(o2.cpu(), o_ref[2:3], o_pt[2:3], 3.0, 1e-5)[0]


def _planned_splits(nat, b, h, hk, sq, cap, d):
    """partial slots the library plans for a kv-cache call with per-batch cache lengths and automatic splits"""
    import ctypes
    p = nat.FaFwdParams()
    p.b, p.h, p.h_k, p.seqlen_q, p.seqlen_k, p.d, p.dtype = b, h, hk, sq, cap, d, 1
    p.is_seqlens_k_cumulative = 0
    p.softmax_scale = d ** -0.5
    p.window_left = p.window_right = -1
    for name in ("q", "k", "v", "o", "softmax_lse", "work_counter", "cu_seqlens_k"):
        setattr(p, name, 256)          # non-null placeholders: planning reads no memory
    p.q_head_stride = p.o_head_stride = d
    p.work_counter_len = nat.WORK_COUNTER_WORDS
    n = ctypes.c_int32(0)
    assert nat.lib.fa_plan_splits(ctypes.byref(p), 2, ctypes.byref(n)) == 0
    return n.value


@pytest.mark.parametrize("num_splits,cap", [(0, 3000), (1, 3000), (0, 9000)])
@pytest.mark.parametrize("mode", ["plain", "causal", "append_rotary", "window_right", "window_left", "local"])
@pytest.mark.parametrize("sq,h,hk,d", [(4, 64, 8, 128), (2, 32, 2, 64), (5, 12, 3, 128), (16, 8, 4, 96), (33, 6, 2, 128),
                                        (100, 4, 2, 64), (3, 48, 1, 256), (127, 2, 1, 128)])
def test_few_query_positions_with_grouped_heads(sq, h, hk, d, mode, num_splits, cap):
    """2..127 query positions with grouped q heads and more than 16 (position, head) rows per kv head (a draft of
    several tokens checked at once, a short chunk of a prompt): the library lays those rows out as the rows of
    one problem per kv head, so K/V are fetched once and not once per q head.  Masks and rotary positions follow
    the position of a row, softmax_lse keeps its (batch, head, position) layout.  Caches of 9000 rows take the
    ticket-scheduled form of the tiled kernel (a launch this small: chunks of 512 keys, remainders in pieces of 256; lengths with
    complete chunks and a remainder, less than a chunk, a whole number of chunks)."""
    _say("few positions, grouped heads", sq, h, hk, d, mode, num_splits, cap)
    nat = _nat()
    dtype, b = torch.bfloat16, 3
    if cap == 9000 and sq * (h // hk) <= 128:      # (more rows than one row block holds: the plain split form)
        assert _planned_splits(nat, b, h, hk, sq, cap, d) == 18 + 2     # 18 chunk slots + 2 remainder slots
    torch.manual_seed(sq * 7 + h)
    kc = torch.randn(b, cap, hk, d, dtype=dtype)
    vc = torch.randn(b, cap, hk, d, dtype=dtype)
    q = torch.randn(b, sq, h, d, dtype=dtype)
    lens = torch.tensor([2500, max(sq, 37), 1203] if cap == 3000 else [8700, max(sq, 37), 4096 + sq], dtype=torch.int32)
    kn = vn = cos = sin = None
    causal, wl, wr = mode in ("causal", "append_rotary"), -1, -1
    if mode == "append_rotary":
        kn = torch.randn(b, sq, hk, d, dtype=dtype)
        vn = torch.randn(b, sq, hk, d, dtype=dtype)
        cos, sin = orc.rotary_table(cap, d - d % 16, dtype=dtype)
        lens = lens - sq                   # the cache holds the older tokens, the call appends these
    if mode == "window_right":
        wr = 2
    if mode == "window_left":
        wl = 300
    if mode == "local":
        wl, wr = 150, 1
    dev = lambda t: None if t is None else t.to(DEV)
    kc_d, vc_d = kc.to(DEV), vc.to(DEV)
    out, lse = nat.fwd_kvcache(q.to(DEV), kc_d, vc_d, dev(kn), dev(vn), lens.to(DEV), dev(cos), dev(sin), None, None, d ** -0.5,
                               causal, wl, wr, True, num_splits)
    kw = dict(causal=causal, window_size=(wl, wr))
    o_ref, l_ref, k_ref, v_ref = orc.kvcache_forward(q, kc, vc, kn, vn, cos, sin, lens, **kw)
    o_pt, _, _, _ = orc.kvcache_forward(q, kc, vc, kn, vn, cos, sin, lens, upcast=False, reorder_ops=True, **kw)
    ok, err, bound = orc.tolerance_ok(out.cpu(), o_ref, o_pt, 3.0, 1e-5)
    _say("   out err %.3e bound %.3e" % (err, bound))
    assert ok
    assert lse.shape == (b, h, sq) and orc.lse_ok(lse.cpu(), l_ref, 1e-3)[0]
    assert torch.equal(vc_d.cpu(), v_ref)
    assert torch.allclose(kc_d.cpu().float(), k_ref.float(), rtol=1e-3, atol=1e-3)
    if mode in ("plain", "causal", "local") and num_splits == 0:
        # the same problem through flash_attn_func on one batch entry (q as a strided view of a wider tensor)
        L = int(lens[0])
        wide = torch.zeros(1, sq, h + 2, d, dtype=dtype)
        wide[:, :, 1:h + 1] = q[0:1]
        o2 = _fa_func()(wide.to(DEV)[:, :, 1:h + 1], kc[0:1, :L].to(DEV), vc[0:1, :L].to(DEV), causal=causal, window_size=(wl, wr))
        assert orc.tolerance_ok(o2.cpu(), o_ref[0:1], o_pt[0:1], 3.0, 1e-5)[0]


@pytest.mark.parametrize("num_splits", [0, 1])
@pytest.mark.parametrize("sq,h,hk,b,cap", [(4, 64, 8, 16, 16384), (1, 24, 1, 64, 32768), (40, 2, 2, 16, 65536), (1, 32, 1, 16, 49152)])
def test_caches_of_a_gibibyte_take_the_streaming_tile_loop(sq, h, hk, b, cap, num_splits):
    """K/V caches of 384 MiB and more (three of 1 GiB, one of 384 MiB) whose rows one workgroup reads (one row block per kv head) are fetched with
    non-temporal loads, requested two tiles ahead: the key loop of that variant has its own prologue and runs
    two tiles per trip.  Lengths of 1, 2, 3 and 4 tiles, an odd and an even long one, and an empty entry; a few
    batch entries are checked against the oracle, out and softmax_lse, with and without split keys."""
    _say("gibibyte caches", sq, h, hk, b, cap, num_splits)
    nat = _nat()
    dtype, d = torch.bfloat16, 128
    assert 4 * b * cap * hk * d >= 3 << 27
    torch.manual_seed(sq + 11 * num_splits)
    kc = torch.randn(b, cap, hk, d, dtype=dtype)
    vc = torch.randn(b, cap, hk, d, dtype=dtype)
    q = torch.randn(b, sq, h, d, dtype=dtype)
    lens = torch.randint(cap // 4, cap - sq, (b,), dtype=torch.int32)
    picks = [0, 1, 2, 3, 4, 5, 6, b - 1]
    lens[:7] = torch.tensor([max(sq, 40), 100, 130, 250, cap - 1, cap - 64 - 7, 0 if sq == 1 else sq], dtype=torch.int32)
    out, lse = nat.fwd_kvcache(q.to(DEV), kc.to(DEV), vc.to(DEV), None, None, lens.to(DEV), None, None, None, None, d ** -0.5,
                               True, -1, -1, True, num_splits)
    out, lse = out.cpu(), lse.cpu()
    assert torch.isfinite(out.float()).all()
    for i in picks:
        sl = slice(i, i + 1)
        o_ref, l_ref, _, _ = orc.kvcache_forward(q[sl], kc[sl], vc[sl], None, None, None, None, lens[sl], causal=True)
        o_pt, _, _, _ = orc.kvcache_forward(q[sl], kc[sl], vc[sl], None, None, None, None, lens[sl], causal=True,
                                            upcast=False, reorder_ops=True)
        ok, err, bound = orc.tolerance_ok(out[sl], o_ref, o_pt, 3.0, 1e-5)
        _say("   entry %d length %d: out err %.3e bound %.3e" % (i, int(lens[i]), err, bound))
        assert ok
        assert orc.lse_ok(lse[sl], l_ref, 1e-3)[0]


@pytest.mark.parametrize("mode", ["causal", "full", "local"])
@pytest.mark.parametrize("inter", [False, True])
@pytest.mark.parametrize("sq,h,hk,d,rot", [(128, 64, 8, 128, 128), (300, 32, 32, 64, 32), (97, 72, 8, 96, 64), (200, 32, 4, 256, 256)])
def test_appended_chunk_with_rotary_on_the_long_sequence_kernels(sq, h, hk, d, rot, inter, mode):
    """A chunk of 97..300 tokens appended with rotary to caches, in a launch that is not split (256+ row blocks):
    the q rows are rotated into the output tensor by a pass of their own and the long-sequence kernels read them
    from there.  Out, softmax_lse and the cache contents against the oracle; q must come back untouched."""
    _say("appended chunk with rotary", sq, h, hk, d, rot, inter, mode)
    nat = _nat()
    dtype, cap, b = torch.bfloat16, 1500, 4
    assert (sq + 127) // 128 * h * b >= 256
    torch.manual_seed(sq + d)
    kc = torch.randn(b, cap, hk, d, dtype=dtype)
    vc = torch.randn(b, cap, hk, d, dtype=dtype)
    q = torch.randn(b, sq, h, d, dtype=dtype)
    kn = torch.randn(b, sq, hk, d, dtype=dtype)
    vn = torch.randn(b, sq, hk, d, dtype=dtype)
    lens = torch.tensor([cap - sq, 0, 700, 1], dtype=torch.int32)
    cos, sin = orc.rotary_table(cap, rot, dtype=dtype)
    causal, wl, wr = mode == "causal", -1, -1
    if mode == "local":
        wl, wr = 200, 30
    q_d, kc_d, vc_d = q.to(DEV), kc.to(DEV), vc.to(DEV)
    out, lse = nat.fwd_kvcache(q_d, kc_d, vc_d, kn.to(DEV), vn.to(DEV), lens.to(DEV), cos.to(DEV), sin.to(DEV), None, None, d ** -0.5,
                               causal, wl, wr, inter, 0)
    assert torch.equal(q_d.cpu(), q)
    kw = dict(causal=causal, window_size=(wl, wr), rotary_interleaved=inter)
    o_ref, l_ref, k_ref, v_ref = orc.kvcache_forward(q, kc, vc, kn, vn, cos, sin, lens, **kw)
    o_pt, _, _, _ = orc.kvcache_forward(q, kc, vc, kn, vn, cos, sin, lens, upcast=False, reorder_ops=True, **kw)
    ok, err, bound = orc.tolerance_ok(out.cpu(), o_ref, o_pt, 3.0, 1e-5)
    _say("   out err %.3e bound %.3e" % (err, bound))
    assert ok
    assert orc.lse_ok(lse.cpu(), l_ref, 1e-3)[0]
    assert torch.equal(vc_d.cpu(), v_ref)
    assert torch.allclose(kc_d.cpu().float(), k_ref.float(), rtol=1e-3, atol=1e-3)


def _kernel():
    return _nat().last_kernel()


@pytest.mark.parametrize("out_layout", ["own", "q_itself", "interleaved_with_q"])
def test_rotary_chunk_when_out_shares_memory_with_q(out_layout):
    """The long-sequence path of a chunk appended with rotary parks the rotated q rows in `out` first.  It may do
    so only when out and q share no memory: with out == q, or out and q as views of one tensor, the kernel that
    rotates while it loads must run instead (fa_last_kernel says which did) and the results must be the same."""
    _say("rotary chunk, out layout", out_layout)
    nat = _nat()
    dtype, cap, b, sq, h, hk, d = torch.bfloat16, 1500, 4, 128, 64, 8, 128
    torch.manual_seed(7)
    kc = torch.randn(b, cap, hk, d, dtype=dtype)
    vc = torch.randn(b, cap, hk, d, dtype=dtype)
    q = torch.randn(b, sq, h, d, dtype=dtype)
    kn = torch.randn(b, sq, hk, d, dtype=dtype)
    vn = torch.randn(b, sq, hk, d, dtype=dtype)
    lens = torch.tensor([cap - sq, 0, 700, 1], dtype=torch.int32)
    cos, sin = orc.rotary_table(cap, d, dtype=dtype)
    if out_layout == "interleaved_with_q":
        both = torch.zeros(b, sq, 2, h, d, dtype=dtype, device=DEV)     # q and out as the two slices of one tensor
        both[:, :, 0] = q.to(DEV)
        q_d, out_d = both[:, :, 0], both[:, :, 1]
    else:
        q_d = q.to(DEV)
        out_d = q_d if out_layout == "q_itself" else None
    out, lse = nat.fwd_kvcache(q_d, kc.to(DEV), vc.to(DEV), kn.to(DEV), vn.to(DEV), lens.to(DEV), cos.to(DEV), sin.to(DEV), None,
                               out_d, d ** -0.5, True, -1, -1, False, 0)
    name = _kernel()[0]
    _say("   kernel", name)
    assert name == ("pipelined" if out_layout == "own" else "tiled")
    if out_layout == "interleaved_with_q":
        assert torch.equal(q_d.cpu(), q)
    kw = dict(causal=True, rotary_interleaved=False)
    o_ref, l_ref, _, _ = orc.kvcache_forward(q, kc, vc, kn, vn, cos, sin, lens, **kw)
    o_pt, _, _, _ = orc.kvcache_forward(q, kc, vc, kn, vn, cos, sin, lens, upcast=False, reorder_ops=True, **kw)
    ok, err, bound = orc.tolerance_ok(out.cpu(), o_ref, o_pt, 3.0, 1e-5)
    _say("   out err %.3e bound %.3e" % (err, bound))
    assert ok
    assert orc.lse_ok(lse.cpu(), l_ref, 1e-3)[0]


@pytest.mark.parametrize("sq,h,hk,d,cap,b", [(14, 64, 8, 128, 8192, 32), (1, 16, 16, 64, 32768, 8), (4, 32, 4, 128, 8192, 32)])
def test_ticket_counters_left_in_use_are_treated_as_fresh(sq, h, hk, d, cap, b):
    """The ticket-scheduled kernels (decode and tiled) find their counter words as a launch that never finished
    would leave them -- or as a caller that did not clear them would pass them: non-zero counts under a foreign
    tag.  The launch must schedule every item all the same (each call tags the counters with a number of its own
    and takes anything else for zero), match the oracle, and leave the words zero; a second call right after
    must too.  All kernels run to their normal end: nothing is torn down to set this up, the words are written
    from the host."""
    _say("poisoned ticket words", sq, h, hk, d, cap, b)
    nat = _nat()
    dtype = torch.bfloat16
    torch.manual_seed(3 + sq)
    kc = torch.randn(b, cap, hk, d, dtype=dtype)
    vc = torch.randn(b, cap, hk, d, dtype=dtype)
    q = torch.randn(b, sq, h, d, dtype=dtype)
    lens = torch.randint(sq, cap + 1, (b,), dtype=torch.int32)
    lens[0], lens[1], lens[2] = cap, sq, 4096 + 5
    q_d, kc_d, vc_d, lens_d = q.to(DEV), kc.to(DEV), vc.to(DEV), lens.to(DEV)
    nat.fwd_kvcache(q_d, kc_d, vc_d, None, None, lens_d, None, None, None, None, d ** -0.5, True, -1, -1, True, 0)   # makes the words
    name, _, split, _ = _kernel()
    assert name == ("decode_tickets" if sq * (h // hk) <= 16 else "tiled_tickets") and split, (name, split)
    torch.cuda.synchronize()
    key = (torch.cuda.current_device(), nat._stream(q_d.device))
    words = nat._COUNTERS[key]
    assert not words[:nat.WORK_COUNTER_WORDS].any()
    outs = []
    for poison in ([1000, 0x7eadbeef, 3, 0x7eadbeef], [5, 0, 77, 0], [-1, -1, -1, -1], [0, 0, 0, 0]):
        words[:4] = torch.tensor(poison, dtype=torch.int32, device=DEV)
        out, lse = nat.fwd_kvcache(q_d, kc_d, vc_d, None, None, lens_d, None, None, None, None, d ** -0.5, True, -1, -1, True, 0)
        torch.cuda.synchronize()
        assert not words[:nat.WORK_COUNTER_WORDS].any(), (poison, words[:4].tolist())
        outs.append((out.cpu(), lse.cpu()))
    for o, l in outs[:-1]:           # same items whatever the words held
        assert (o.float() - outs[-1][0].float()).abs().max().item() < 2e-2
    for i in (0, 1, 2, b - 1):
        sl = slice(i, i + 1)
        o_ref, l_ref, _, _ = orc.kvcache_forward(q[sl], kc[sl], vc[sl], None, None, None, None, lens[sl], causal=True)
        o_pt, _, _, _ = orc.kvcache_forward(q[sl], kc[sl], vc[sl], None, None, None, None, lens[sl], causal=True,
                                            upcast=False, reorder_ops=True)
        for o, l in outs:
            ok, err, bound = orc.tolerance_ok(o[sl], o_ref, o_pt, 3.0, 1e-5)
            assert ok, (i, err, bound)
            assert orc.lse_ok(l[sl], l_ref, 1e-3)[0]


@pytest.mark.parametrize("sq,h,hk,b,cap,expect", [
    (14, 64, 8, 32, 8192, "tiled_tickets"),        # 112 (position, head) rows per kv head, 256 row blocks, long caches
    (16, 64, 8, 64, 16384, "tiled_tickets"),       # 128 rows, 512 row blocks
    (112, 8, 8, 32, 8192, "pipelined"),            # the same count of rows as plain query positions: left whole
    (4, 64, 8, 32, 8192, "tiled_tickets"),
])
def test_split_plan_is_the_plan_that_runs(sq, h, hk, b, cap, expect):
    """fa_plan_splits and the call itself must make the same plan: the caller sizes the partial buffers by the
    former.  (position, grouped head) rows numbering 96-128 per kv head are the case where the two once differed:
    the call saw its own already packed problem as plain query rows and left it whole on the general kernel.)"""
    _say("plan == run", sq, h, hk, b, cap)
    nat = _nat()
    dtype, d = torch.bfloat16, 128
    planned = _planned_splits(nat, b, h, hk, sq, cap, d)
    torch.manual_seed(1)
    kc = torch.randn(b, cap, hk, d, dtype=dtype)
    vc = torch.randn(b, cap, hk, d, dtype=dtype)
    q = torch.randn(b, sq, h, d, dtype=dtype)
    lens = torch.randint(cap // 2, cap + 1, (b,), dtype=torch.int32)
    out, lse = nat.fwd_kvcache(q.to(DEV), kc.to(DEV), vc.to(DEV), None, None, lens.to(DEV), None, None, None, None, d ** -0.5,
                               True, -1, -1, True, 0)
    name, _, split, _ = _kernel()
    _say("   planned %d partial slots; ran %s, split %s" % (planned, name, split))
    assert name == expect and split == (planned > 1)
    out, lse = out.cpu(), lse.cpu()
    for i in (0, b - 1):
        sl = slice(i, i + 1)
        o_ref, l_ref, _, _ = orc.kvcache_forward(q[sl], kc[sl], vc[sl], None, None, None, None, lens[sl], causal=True)
        o_pt, _, _, _ = orc.kvcache_forward(q[sl], kc[sl], vc[sl], None, None, None, None, lens[sl], causal=True,
                                            upcast=False, reorder_ops=True)
        ok, err, bound = orc.tolerance_ok(out[sl], o_ref, o_pt, 3.0, 1e-5)
        assert ok, (i, err, bound)
        assert orc.lse_ok(lse[sl], l_ref, 1e-3)[0]
