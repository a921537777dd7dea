"""Pins the CPU oracle against things the reference or the mathematics fix, so that a dropped
term, a wrong sign/index or a transposed operand fails at least one check.  CPU only."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import attention_oracle as orc


def _randn(*shape, dtype=torch.float32, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=torch.float32).to(dtype)


def brute_force(q, k, v, causal, window, scale, sk_len=None):
    """Scalar-loop attention in float64 for one (batch) of tiny shapes."""
    b, sq, h, d = q.shape
    sk, hk = k.shape[1], k.shape[2]
    g = h // hk
    left, right = window
    if causal:
        right = 0
    out = torch.zeros(b, sq, h, d, dtype=torch.float64)
    lse = torch.zeros(b, h, sq, dtype=torch.float64)
    for ib in range(b):
        L = sk if sk_len is None else int(sk_len[ib])
        for ih in range(h):
            for i in range(sq):
                scores, js = [], []
                for j in range(L):
                    if right >= 0 and j > i + L - sq + right:
                        continue
                    if left >= 0 and j < i + L - sq - left:
                        continue
                    scores.append(sum(float(q[ib, i, ih, e]) * float(k[ib, j, ih // g, e]) for e in range(d)) * scale)
                    js.append(j)
                if not js:
                    lse[ib, ih, i] = float("inf")
                    continue
                m = max(scores)
                z = sum(math.exp(s - m) for s in scores)
                lse[ib, ih, i] = m + math.log(z)
                for s, j in zip(scores, js):
                    out[ib, i, ih] += math.exp(s - m) / z * v[ib, j, ih // g].double()
    return out, lse


def test_docstring_masks():
    # flash_attn/flash_attn_interface.py:611-621
    m = orc.visible_mask(2, 5, causal=True)
    assert m.int().tolist() == [[1, 1, 1, 1, 0], [1, 1, 1, 1, 1]]
    m = orc.visible_mask(5, 2, causal=True)
    assert m.int().tolist() == [[0, 0], [0, 0], [0, 0], [1, 0], [1, 1]]


def test_window_inequality():
    # flash_attn/flash_attn_interface.py:623-625: keys in [i+sk-sq-l, i+sk-sq+r] inclusive
    sq, sk, l, r = 7, 11, 2, 1
    m = orc.visible_mask(sq, sk, (l, r))
    for i in range(sq):
        for j in range(sk):
            assert bool(m[i, j]) == (i + sk - sq - l <= j <= i + sk - sq + r)
    # one-sided windows: negative bound = unbounded
    m = orc.visible_mask(sq, sk, (-1, 0))
    assert torch.equal(m, orc.visible_mask(sq, sk, causal=True))
    m = orc.visible_mask(sq, sk, (3, -1))
    for i in range(sq):
        for j in range(sk):
            assert bool(m[i, j]) == (j >= i + sk - sq - 3)


@pytest.mark.parametrize("causal", [False, True])
def test_against_sdpa(causal):
    q, k, v = _randn(2, 33, 4, 16, seed=1), _randn(2, 33, 4, 16, seed=2), _randn(2, 33, 4, 16, seed=3)
    out, lse = orc.attention_forward(q, k, v, causal=causal)
    ref = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2),
                                         is_causal=causal).transpose(1, 2)
    assert torch.allclose(out, ref, atol=2e-6, rtol=1e-5)
    s = torch.einsum("bthd,bshd->bhts", q, k) / math.sqrt(16)
    if causal:
        s = s.masked_fill(torch.triu(torch.ones(33, 33, dtype=torch.bool), 1), float("-inf"))
    assert torch.allclose(lse, torch.logsumexp(s, -1), atol=1e-5)


@pytest.mark.parametrize("sq,sk", [(3, 7), (7, 3), (5, 5), (1, 6)])
@pytest.mark.parametrize("mode", ["dense", "causal", "local", "local_left"])
def test_against_brute_force(sq, sk, mode):
    h, hk, d = 4, 2, 8
    q, k, v = _randn(2, sq, h, d, seed=4), _randn(2, sk, hk, d, seed=5), _randn(2, sk, hk, d, seed=6)
    causal = mode == "causal"
    window = {"dense": (-1, -1), "causal": (-1, -1), "local": (2, 1), "local_left": (1, -1)}[mode]
    scale = 0.37
    out, lse = orc.attention_forward(q, k, v, causal=causal, window_size=window, softmax_scale=scale)
    bo, bl = brute_force(q, k, v, causal, window, scale)
    assert torch.allclose(out.double(), bo, atol=1e-5)
    assert torch.equal(torch.isinf(lse), torch.isinf(bl))
    fin = ~torch.isinf(bl)
    assert torch.allclose(lse.double()[fin], bl[fin], atol=1e-5)
    assert (lse[~fin] > 0).all()  # +inf, not -inf


def test_fully_masked_rows_zero_and_lse_inf():
    q, k, v = _randn(1, 5, 2, 8), _randn(1, 2, 2, 8, seed=1), _randn(1, 2, 2, 8, seed=2)
    out, lse = orc.attention_forward(q, k, v, causal=True)
    assert (out[:, :3] == 0).all() and (lse[:, :, :3] == float("inf")).all()
    assert torch.isfinite(lse[:, :, 3:]).all()


def test_uniform_closed_form():
    # zero queries -> uniform weights over visible keys: out = mean of visible V, lse = log(count)
    sq, sk, d = 4, 9, 8
    q = torch.zeros(1, sq, 1, d)
    k, v = _randn(1, sk, 1, d, seed=1), _randn(1, sk, 1, d, seed=2)
    out, lse = orc.attention_forward(q, k, v, causal=True)
    for i in range(sq):
        n = i + sk - sq + 1
        assert torch.allclose(out[0, i, 0], v[0, :n, 0].mean(0), atol=1e-6)
        assert abs(lse[0, 0, i].item() - math.log(n)) < 1e-6


def test_gqa_equals_repeated_heads():
    q, k, v = _randn(2, 9, 6, 8, seed=1), _randn(2, 12, 2, 8, seed=2), _randn(2, 12, 2, 8, seed=3)
    out, lse = orc.attention_forward(q, k, v, causal=True)
    out2, lse2 = orc.attention_forward(q, k.repeat_interleave(3, 2), v.repeat_interleave(3, 2), causal=True)
    assert torch.equal(out, out2) and torch.equal(lse, lse2)


def test_key_lengths_equal_truncation():
    q, k, v = _randn(2, 4, 2, 8, seed=1), _randn(2, 10, 2, 8, seed=2), _randn(2, 10, 2, 8, seed=3)
    lens = torch.tensor([6, 10])
    out, lse = orc.attention_forward(q, k, v, causal=True, seqlens_k=lens)
    for b in range(2):
        o, l = orc.attention_forward(q[b:b + 1], k[b:b + 1, : lens[b]], v[b:b + 1, : lens[b]], causal=True)
        assert torch.allclose(out[b], o[0], atol=1e-6) and torch.allclose(lse[b], l[0], atol=1e-6)


def test_varlen_equals_per_sequence():
    lens_q, lens_k = [3, 0, 5], [4, 2, 5]
    cu_q = torch.tensor([0, 3, 3, 8]); cu_k = torch.tensor([0, 4, 6, 11])
    q, k, v = _randn(8, 2, 8, seed=1), _randn(11, 2, 8, seed=2), _randn(11, 2, 8, seed=3)
    out, lse = orc.attention_varlen_forward(q, k, v, cu_q, cu_k, 5, causal=True)
    o0, l0 = orc.attention_forward(q[None, 0:3], k[None, 0:4], v[None, 0:4], causal=True)
    o2, l2 = orc.attention_forward(q[None, 3:8], k[None, 6:11], v[None, 6:11], causal=True)
    assert torch.equal(out[0:3], o0[0]) and torch.equal(out[3:8], o2[0])
    assert torch.equal(lse[0, :, :3], l0[0]) and torch.equal(lse[2, :, :5], l2[0])


@pytest.mark.parametrize("interleaved", [False, True])
def test_rotary_closed_forms(interleaved):
    b, s, h, d, rd = 2, 5, 3, 16, 8
    x = _randn(b, s, h, d, seed=1)
    ang = torch.rand(32, rd // 2, generator=torch.Generator().manual_seed(2)) * 6.28
    cos, sin = torch.cos(ang), torch.sin(ang)
    pos = torch.tensor([[3, 4, 5, 6, 7], [10, 11, 12, 13, 14]])
    y = orc.rotary_apply(x, cos, sin, pos, interleaved)
    # pass-through dims and norm preservation of each rotated pair
    assert torch.equal(y[..., rd:], x[..., rd:])
    if interleaved:
        pairs_x = x[..., :rd].reshape(b, s, h, rd // 2, 2)
        pairs_y = y[..., :rd].reshape(b, s, h, rd // 2, 2)
    else:
        pairs_x = torch.stack((x[..., : rd // 2], x[..., rd // 2: rd]), -1)
        pairs_y = torch.stack((y[..., : rd // 2], y[..., rd // 2: rd]), -1)
    assert torch.allclose(pairs_x.norm(dim=-1), pairs_y.norm(dim=-1), atol=1e-5)
    # complex-number form: (x0 + i x1) * exp(i*angle)
    zc = torch.complex(pairs_x[..., 0], pairs_x[..., 1]) * torch.polar(torch.ones_like(ang), ang)[pos].unsqueeze(2)
    assert torch.allclose(pairs_y[..., 0], zc.real, atol=1e-5)
    assert torch.allclose(pairs_y[..., 1], zc.imag, atol=1e-5)
    # the textbook formula x*cos + rotate_half(x)*sin (flash_attn/layers/rotary.py:11-32)
    if not interleaved:
        xr = x[..., :rd]
        rot_half = torch.cat((-xr[..., rd // 2:], xr[..., : rd // 2]), -1)
        c2 = torch.cat((cos, cos), -1)[pos].unsqueeze(2); s2 = torch.cat((sin, sin), -1)[pos].unsqueeze(2)
        assert torch.allclose(y[..., :rd], xr * c2 + rot_half * s2, atol=1e-6)


def test_rotary_table_known_values():
    cos, sin = orc.rotary_table(8, 4, base=10000.0)
    assert cos.shape == (8, 2)
    assert torch.allclose(cos[:, 0], torch.cos(torch.arange(8.0)))          # inv_freq[0] = 1
    assert torch.allclose(sin[:, 1], torch.sin(torch.arange(8.0) * 0.01))   # inv_freq[1] = 10000^-0.5


def test_kvcache_semantics():
    b, sk, hk, h, d, new = 2, 12, 2, 4, 16, 2
    q = _randn(b, 2, h, d, seed=1)
    kc, vc = _randn(4, sk, hk, d, seed=2), _randn(4, sk, hk, d, seed=3)
    k, v = _randn(b, new, hk, d, seed=4), _randn(b, new, hk, d, seed=5)
    lens = torch.tensor([3, 7], dtype=torch.int32)
    idx = torch.tensor([2, 0], dtype=torch.int32)
    cos, sin = orc.rotary_table(sk, 8)
    out, lse, ka, va = orc.kvcache_forward(q, kc, vc, k, v, cos, sin, lens, idx, causal=True,
                                           rotary_interleaved=False)
    # untouched rows/batches are bit-identical, V rows are the new values bit-exact
    assert torch.equal(ka[1], kc[1]) and torch.equal(ka[3], kc[3])
    assert torch.equal(va[2, 3:5], v[0]) and torch.equal(va[0, 7:9], v[1])
    assert torch.equal(ka[2, :3], kc[2, :3]) and torch.equal(ka[2, 5:], kc[2, 5:])
    # equivalent dense problem built by hand for batch 1
    kpos = torch.tensor([[7, 8]]); qpos = torch.tensor([[7, 8]])
    k_ro = orc.rotary_apply(k[1:2], cos, sin, kpos, False)
    q_ro = orc.rotary_apply(q[1:2], cos, sin, qpos, False)
    kk = torch.cat((kc[0:1, :7], k_ro), 1); vv = torch.cat((vc[0:1, :7], v[1:2]), 1)
    o, l = orc.attention_forward(q_ro, kk, vv, causal=True)
    assert torch.allclose(out[1], o[0], atol=1e-6) and torch.allclose(lse[1], l[0], atol=1e-6)
    # non-causal: every q row rotated at the same position
    out2, _, _, _ = orc.kvcache_forward(q, kc, vc, k, v, cos, sin, lens, idx, causal=False,
                                        rotary_interleaved=False)
    q_ro2 = orc.rotary_apply(q[1:2], cos, sin, torch.tensor([[7, 7]]), False)
    o2, _ = orc.attention_forward(q_ro2, kk, vv)
    assert torch.allclose(out2[1], o2[0], atol=1e-6)


def test_combine_splits_matches_unsplit():
    q, k, v = _randn(1, 4, 2, 8, seed=1), _randn(1, 24, 2, 8, seed=2), _randn(1, 24, 2, 8, seed=3)
    full, lse_full = orc.attention_forward(q, k, v)
    parts, lses = [], []
    for s in range(3):
        o, l = orc.attention_forward(q, k[:, 8 * s: 8 * s + 8], v[:, 8 * s: 8 * s + 8],
                                     softmax_scale=1 / math.sqrt(8))
        parts.append(o.transpose(1, 2)); lses.append(l)
    # an empty split contributes lse = -inf, out = 0
    parts.append(torch.zeros_like(parts[0])); lses.append(torch.full_like(lses[0], float("-inf")))
    o, l = orc.combine_splits(torch.stack(parts), torch.stack(lses))
    assert torch.allclose(o.transpose(1, 2), full, atol=1e-6) and torch.allclose(l, lse_full, atol=1e-6)
    o, l = orc.combine_splits(torch.zeros(2, 3, 4), torch.full((2, 3), float("-inf")))
    assert (o == 0).all() and (l == float("inf")).all()


def test_num_splits_heuristic_known_answer():
    # worked example in csrc/flash_attn/flash_api.cpp:206-211: 48 blocks on 108 SMs -> 2 splits
    assert orc.num_splits_heuristic_reference(48, 108, 64, 128) == 2
    assert orc.num_splits_heuristic_reference(100, 108, 64, 128) == 1      # >= 0.8 * SMs
    assert orc.num_splits_heuristic_reference(1, 108, 1, 128) == 1          # a single key block
    # never exceeds any of its caps
    for blocks in (1, 3, 17):
        for nb in (1, 2, 5, 300):
            s = orc.num_splits_heuristic_reference(blocks, 108, nb, 128)
            assert 1 <= s <= min(128, 108, nb)


def test_flops_convention():
    # benchmarks/benchmark_flash_attention.py:27-30
    assert orc.attention_flops(2, 512, 512, 8, 64) == 4 * 2 * 512 ** 2 * 8 * 64
    f = orc.attention_flops(4, 8192, 8192, 32, 128, causal=True)
    assert abs(f / (4 * 4 * 8192 ** 2 * 32 * 128 / 2) - 1) < 2e-4
    # windowed config: sum_i min(i+1, 4097) pairs per (b, h)
    f = orc.attention_flops(2, 16384, 16384, 32, 128, causal=True, window_size=(4096, 0))
    assert f == 4 * 128 * 58734592 * 2 * 32


def test_tolerance_rule_detects_errors():
    q, k, v = (_randn(1, 64, 2, 32, dtype=torch.bfloat16, seed=s) for s in (1, 2, 3))
    ref, lse, pt = orc.attention_reference_pair(q, k, v, causal=True)
    ok, err, bound = orc.tolerance_ok(pt, ref, pt)
    assert ok and bound > 0
    ok, _, _ = orc.tolerance_ok(ref + 0.05, ref, pt)
    assert not ok
    assert orc.lse_ok(lse * (1 + 5e-4), lse)[0] and not orc.lse_ok(lse * 1.01, lse)[0]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("sq,sk,d,kw", [(64, 64, 32, dict(causal=True)), (128, 512, 64, dict()),
                                        (96, 777, 128, dict(window_size=(100, 20))), (256, 2048, 128, dict(causal=True))])
def test_tolerance_rule_is_bounded_above(dtype, sq, sk, d, kw):
    """The allowance the rule hands to a kernel is `mult` x the error of the low-precision CPU run, so that
    run must not be loose.  Every output is a convex combination of rows of v: rounding it to the 16-bit
    type costs at most eps/2 * max|v|, and on these inputs the products and the softmax in 16-bit
    arithmetic add less than as much again.  So the run stays within one eps * max|v| of the fp32 run
    (measured: 0.03-0.5), and a kernel held to twice that is held to two units in the last place of the
    largest output."""
    eps = torch.finfo(dtype).eps
    for seed in range(3):
        q, k, v = (_randn(1, s, 2, d, dtype=dtype, seed=10 * seed + i) for i, s in enumerate((sq, sk, sk)))
        ref, _, pt = orc.attention_reference_pair(q, k, v, **kw)
        err = (pt.float() - ref.float()).abs().max().item()
        assert 0 < err <= eps * v.float().abs().max().item(), (seed, err)


# ---------------------------------------------------------------------------------------------
# backward restatement
# ---------------------------------------------------------------------------------------------
def _loss(q, k, v, w, **kw):
    """sum(out * w) with out from a scalar-loop softmax attention in fp64: the function whose gradient
    the backward restatement claims to be."""
    b, sq, h, d = q.shape
    sk, hk = k.shape[1], k.shape[2]
    g = h // hk
    scale = kw.get("softmax_scale") or d ** -0.5
    vis = orc.visible_mask(sq, sk, kw.get("window_size", (-1, -1)), kw.get("causal", False))
    total = 0.0
    for ib in range(b):
        for ih in range(h):
            s = (q[ib, :, ih] @ k[ib, :, ih // g].T) * scale
            for i in range(sq):
                cols = [j for j in range(sk) if vis[i, j]]
                if not cols:
                    continue
                e = torch.exp(s[i, cols] - s[i, cols].max())
                p = e / e.sum()
                total = total + ((p[:, None] * v[ib, cols, ih // g]).sum(0) * w[ib, i, ih]).sum()
    return total


@pytest.mark.parametrize("kw", [dict(), dict(causal=True), dict(window_size=(2, 1)), dict(window_size=(-1, 0), softmax_scale=0.3)])
def test_backward_against_central_differences(kw):
    """Every entry of dq, dk, dv against (L(x + e) - L(x - e)) / 2e of a scalar-loop forward in fp64;
    seqlen_q > seqlen_k under causal gives rows that see nothing (gradient exactly zero)."""
    g = torch.Generator().manual_seed(3)
    b, sq, sk, h, hk, d = 1, 5, 4, 2, 1, 3
    q = torch.randn(b, sq, h, d, generator=g, dtype=torch.float64)
    k = torch.randn(b, sk, hk, d, generator=g, dtype=torch.float64)
    v = torch.randn(b, sk, hk, d, generator=g, dtype=torch.float64)
    w = torch.randn(b, sq, h, d, generator=g, dtype=torch.float64)
    grads = orc.attention_backward(q, k, v, w, dtype=torch.float64, **kw)
    eps = 1e-6
    for x, gx in zip((q, k, v), grads):
        flat = x.view(-1)
        for idx in range(flat.numel()):
            old = flat[idx].item()
            flat[idx] = old + eps
            up = _loss(q, k, v, w, **kw)
            flat[idx] = old - eps
            dn = _loss(q, k, v, w, **kw)
            flat[idx] = old
            assert abs((up - dn).item() / (2 * eps) - gx.view(-1)[idx].item()) < 1e-7


@pytest.mark.parametrize("kw", [dict(causal=True), dict(window_size=(5, 3)), dict(),
                                dict(causal=True, seqlens_q=torch.tensor([7, 13]), seqlens_k=torch.tensor([17, 6]))])
def test_backward_against_autograd(kw):
    """Library check: torch autograd through the forward restatement (fp64, GQA, padded lengths)."""
    g = torch.Generator().manual_seed(4)
    q = torch.randn(2, 13, 6, 16, generator=g, dtype=torch.float64)
    k = torch.randn(2, 17, 2, 16, generator=g, dtype=torch.float64)
    v = torch.randn(2, 17, 2, 16, generator=g, dtype=torch.float64)
    do = torch.randn(2, 13, 6, 16, generator=g, dtype=torch.float64)
    a = orc.attention_backward(q, k, v, do, dtype=torch.float64, **kw)
    c = orc.attention_backward_autograd(q, k, v, do, upcast=False, **kw)
    for x, y in zip(a, c):
        assert (x - y).abs().max() < 1e-12


def test_backward_closed_forms():
    """One key: P = 1, so dV = sum of dO over rows and heads of the group, dQ = dK = 0.
    Zero queries: uniform attention, dV[j] = mean-weighted sum of dO and dK = 0 exactly when dO V^T is
    constant along keys (V rows equal)."""
    g = torch.Generator().manual_seed(5)
    q = torch.randn(2, 6, 4, 8, generator=g); do = torch.randn(2, 6, 4, 8, generator=g)
    k = torch.randn(2, 1, 2, 8, generator=g); v = torch.randn(2, 1, 2, 8, generator=g)
    dq, dk, dv = orc.attention_backward(q, k, v, do)
    assert dq.abs().max() < 1e-6 and dk.abs().max() < 1e-6
    want = do.view(2, 6, 2, 2, 8).sum(dim=(1, 3))
    assert torch.allclose(dv[:, 0], want, atol=1e-5)
    sk = 5
    k = torch.randn(2, sk, 2, 8, generator=g)
    v = torch.randn(2, 1, 2, 8, generator=g).expand(2, sk, 2, 8).contiguous()
    dq, dk, dv = orc.attention_backward(torch.zeros_like(q), k, v, do)
    assert dk.abs().max() < 1e-6
    assert torch.allclose(dv, (want / sk)[:, None].expand_as(dv), atol=1e-5)


def test_dropout_restatement():
    """Dropout in the oracle: the forward zeroes masked probabilities after the softmax and scales
    by 1 / (1 - p) (so an all-kept mask with p = 0.5 doubles the output and leaves lse alone), and
    the backward formulas with the mask equal autograd through that forward."""
    g = torch.Generator().manual_seed(6)
    q = torch.randn(2, 9, 4, 8, generator=g, dtype=torch.float64)
    k = torch.randn(2, 11, 2, 8, generator=g, dtype=torch.float64)
    v = torch.randn(2, 11, 2, 8, generator=g, dtype=torch.float64)
    do = torch.randn(2, 9, 4, 8, generator=g, dtype=torch.float64)
    o0, l0 = orc.attention_forward(q, k, v, causal=True, upcast=False)
    o1, l1 = orc.attention_forward(q, k, v, causal=True, upcast=False, dropout_p=0.5,
                                   dropout_mask=torch.ones(2, 4, 9, 11, dtype=torch.bool))
    assert torch.allclose(o1, 2 * o0) and torch.equal(l0, l1)
    m = torch.rand(2, 4, 9, 11, generator=g) > 0.3
    # one dropped key: the output loses exactly that key's share
    a = orc.attention_backward(q, k, v, do, dtype=torch.float64, causal=True, dropout_p=0.3, dropout_mask=m)
    c = orc.attention_backward_autograd(q, k, v, do, upcast=False, causal=True, dropout_p=0.3, dropout_mask=m)
    for x, y in zip(a, c):
        assert (x - y).abs().max() < 1e-12
