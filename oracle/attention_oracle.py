"""CPU oracle for the FlashAttention-2 forward and backward path.  TEST INFRASTRUCTURE ONLY.

This module is the checker, never the product: only the test-suite, the smoke entry and the
benchmark's CPU-baseline leg may import it.  Nothing in the shipped package routes through it.

It restates, in plain PyTorch on the CPU, the semantics that the reference pins for this path:

* masked softmax attention as written in the reference's test oracle
  (`tests/test_flash_attn.py:153-180` mask, `:183-259` attention) -- fp32 "upcast" form and the
  low-precision "re-ordered" form (scale applied to K, no upcast) that supplies the right-hand
  side of the tolerance rule (`tests/test_flash_attn.py:648-650`);
* log-sum-exp as the kernels define it (`csrc/flash_attn/src/flash_fwd_kernel.h:509-516`):
  natural log of the sum of exp(scale * s), +inf for a row with no visible key;
* rotary embedding (`flash_attn/layers/rotary.py:11-32`) at per-batch position offsets, and the
  KV-cache append + attention semantics of `flash_attn_with_kvcache`
  (`flash_attn/flash_attn_interface.py:922-1042`, `tests/test_flash_attn.py:1759-1834`);
* packed variable-length attention as "each sequence attends alone"
  (`tests/test_flash_attn.py:229-258`);
* the reference's split-count heuristic (`csrc/flash_attn/flash_api.cpp:212-246`);
* the gradients of q, k, v by the formulas the backward kernel evaluates
  (`csrc/flash_attn/src/flash_bwd_kernel.h:79-780`: dV = P^T dO, dP = dO V^T, dS = P o (dP - D) with
  D = rowsum(dO o O), dQ = scale dS K, dK = scale dS^T Q), pinned against torch autograd through
  the forward restatement and against central finite differences in fp64.

How each function is pinned (none is "parity unpinned"): see tests/test_oracle.py -- library
routine `scaled_dot_product_attention`, brute-force scalar loops on tiny shapes, the docstring
mask matrices (`flash_attn/flash_attn_interface.py:611-621`), closed forms (uniform attention
for zero scores, rotation norm preservation / composition), the heuristic's own worked
example (`flash_api.cpp:206-211`), and for the gradients and dropout: central differences of a
scalar-loop forward in fp64, torch autograd through the forward restatement, one-key and equal-value
closed forms, an all-kept mask (output scales by 1 / (1 - p), log-sum-exp unchanged).

The score tensor of the reference form is (b, h, sq, sk) fp32, tens of GB at benchmark sizes, so
every routine here walks (batch, head-block) chunks, which are independent.
"""
import math
from typing import Optional, Tuple

import torch


# --------------------------------------------------------------------------------------------
# masks
# --------------------------------------------------------------------------------------------
def visible_mask(seqlen_q: int, seqlen_k: int, window_size=(-1, -1), causal: bool = False,
                 sq_actual=None, sk_actual=None) -> torch.Tensor:
    """Boolean (…, seqlen_q, seqlen_k) tensor, True where query row i may see key column j.

    Bottom-right aligned window: i + sk - sq - left <= j <= i + sk - sq + right, j < sk, with a
    negative bound meaning "unbounded" and causal forcing right = 0
    (`flash_attn/flash_attn_interface.py:611-625`, `tests/test_flash_attn.py:153-180`).
    sq_actual / sk_actual are optional (b,) integer tensors of per-batch true lengths inside a
    padded (seqlen_q, seqlen_k) frame; the result then has a leading batch dimension.
    """
    left, right = int(window_size[0]), int(window_size[1])
    if causal:
        right = 0
    rows = torch.arange(seqlen_q, dtype=torch.long).view(-1, 1)
    cols = torch.arange(seqlen_k, dtype=torch.long).view(1, -1)
    if sq_actual is None and sk_actual is None:
        sq, sk = seqlen_q, seqlen_k
    else:
        sq = (torch.as_tensor(sq_actual, dtype=torch.long).view(-1, 1, 1)
              if sq_actual is not None else seqlen_q)
        sk = (torch.as_tensor(sk_actual, dtype=torch.long).view(-1, 1, 1)
              if sk_actual is not None else seqlen_k)
    shift = sk - sq
    vis = (cols < sk) & torch.ones(seqlen_q, seqlen_k, dtype=torch.bool)
    if right >= 0:
        vis = vis & (cols <= rows + shift + right)
    if left >= 0:
        vis = vis & (cols >= rows + shift - left)
    return vis


# --------------------------------------------------------------------------------------------
# dense attention
# --------------------------------------------------------------------------------------------
def attention_forward(q, k, v, causal=False, window_size=(-1, -1), softmax_scale=None,
                      seqlens_q=None, seqlens_k=None, upcast=True, reorder_ops=False,
                      head_block: int = 4, dropout_p: float = 0.0,
                      dropout_mask=None) -> Tuple[torch.Tensor, torch.Tensor]:
    """out (b, sq, h, d) in q's dtype and lse (b, h, sq) fp32.

    Follows the reference oracle (`tests/test_flash_attn.py:183-259`): with `upcast` the inputs are
    promoted to fp32, Q is scaled, scores = Q K^T, masked entries are -inf, softmax, rows with no
    visible key give zeros, out = P V, one final rounding.  With `upcast=False, reorder_ops=True`
    everything stays in the input dtype and K is scaled instead (`:225-228`): that run measures the
    rounding noise of an ordinary low-precision implementation.  GQA/MQA: query head h reads
    key/value head h // (H / H_k) (`:222-223`).  seqlens_q / seqlens_k give per-batch valid lengths
    (the reference's padding masks, `:229-258`): padded keys are invisible, padded query rows give 0.
    dropout_mask (b, h, sq, sk) bool, True = keep: probabilities are zeroed where False and the rest
    scaled by 1 / (1 - dropout_p) AFTER the softmax, so the log-sum-exp is that of the undropped
    scores (`:247-251`).
    """
    b, sq, h, d = q.shape
    _, sk, hk, _ = k.shape
    assert h % hk == 0
    g = h // hk
    scale = (1.0 / math.sqrt(d)) if softmax_scale is None else float(softmax_scale)
    dtype_og = q.dtype
    if upcast:
        q, k, v = q.float(), k.float(), v.float()
    out = torch.empty(b, sq, h, v.shape[-1], dtype=dtype_og)
    lse = torch.empty(b, h, sq, dtype=torch.float32)
    need_mask = causal or window_size[0] >= 0 or window_size[1] >= 0 \
        or seqlens_k is not None or seqlens_q is not None
    vis_all = None
    if need_mask:
        vis_all = visible_mask(sq, sk, window_size, causal, seqlens_q, seqlens_k)
    for ib in range(b):
        vis = None
        if need_mask:
            vis = vis_all[ib] if vis_all.dim() == 3 else vis_all
        for h0 in range(0, h, head_block):
            h1 = min(h, h0 + head_block)
            qh = q[ib, :, h0:h1]                                    # (sq, hb, d)
            kv_idx = torch.arange(h0, h1) // g
            kh = k[ib][:, kv_idx]                                   # (sk, hb, d)
            vh = v[ib][:, kv_idx]
            scaled = (lambda x: x / math.sqrt(d)) if softmax_scale is None else (lambda x: x * scale)
            if not reorder_ops:
                s = torch.einsum("thd,shd->hts", scaled(qh), kh)
            else:
                s = torch.einsum("thd,shd->hts", qh, scaled(kh))
            if vis is not None:
                s = s.masked_fill(~vis, float("-inf"))
            lse_blk = torch.logsumexp(s.float(), dim=-1)              # -inf where nothing visible
            p = torch.softmax(s, dim=-1)
            if vis is not None:
                dead = ~vis.any(dim=-1, keepdim=True)
                p = p.masked_fill(dead, 0.0)
                lse_blk = torch.where(dead.squeeze(-1).expand_as(lse_blk),
                                      torch.full_like(lse_blk, float("inf")), lse_blk)
            if dropout_mask is not None:
                p = p.masked_fill(~dropout_mask[ib, h0:h1], 0.0) * (1.0 / (1.0 - dropout_p))
            o = torch.einsum("hts,shd->thd", p, vh)
            if seqlens_q is not None:
                pad_rows = torch.arange(sq) >= int(seqlens_q[ib])
                o = o.masked_fill(pad_rows.view(-1, 1, 1), 0.0)
            out[ib, :, h0:h1] = o.to(dtype_og)
            lse[ib, h0:h1] = lse_blk
    return out, lse


def attention_backward(q, k, v, dout, causal=False, window_size=(-1, -1), softmax_scale=None,
                       seqlens_q=None, seqlens_k=None, dtype=torch.float32, dropout_p: float = 0.0,
                       dropout_mask=None):
    """(dq, dk, dv) in `dtype` (fp32, or fp64 for the finite-difference check), unrounded.

    The backward kernel's own formulas (`csrc/flash_attn/src/flash_bwd_kernel.h:79-780`), evaluated per
    (batch, head) on the full score matrix: P = softmax(scale Q K^T) over the visible keys (0 for a row
    that sees none), dV = P^T dO, dP = dO V^T, D_i = sum_d dO[i,d] O[i,d], dS = P o (dP - D),
    dQ = scale dS K, dK = scale dS^T Q; with GQA / MQA the dK, dV of a key head are summed over the
    query heads that read it (`csrc/flash_attn/flash_api.cpp:799-803`).  Padded query rows
    (seqlens_q) contribute nothing and get dQ = 0; padded keys get dK = dV = 0.
    With dropout (mask M, r = 1 / (1 - p)): O = (P o M r) V, so dV = (P o M r)^T dO and
    dP = (dO V^T) o M r, with D still rowsum(dO o O) (`flash_bwd_kernel.h:411-460`)."""
    b, sq, h, d = q.shape
    _, sk, hk, _ = k.shape
    g = h // hk
    scale = (1.0 / math.sqrt(d)) if softmax_scale is None else float(softmax_scale)
    qf, kf, vf, gf = q.to(dtype), k.to(dtype), v.to(dtype), dout.to(dtype)
    dq, dk, dv = torch.zeros_like(qf), torch.zeros_like(kf), torch.zeros_like(vf)
    vis_all = visible_mask(sq, sk, window_size, causal, seqlens_q, seqlens_k)
    for ib in range(b):
        vis = vis_all[ib] if vis_all.dim() == 3 else vis_all
        if seqlens_q is not None:
            vis = vis & (torch.arange(sq) < int(seqlens_q[ib])).view(-1, 1)
        dead = ~vis.any(dim=-1, keepdim=True)
        for ih in range(h):
            jk = ih // g
            s = (qf[ib, :, ih] @ kf[ib, :, jk].T) * scale
            s = s.masked_fill(~vis, float("-inf"))
            p = torch.softmax(s, dim=-1).masked_fill(dead, 0.0)
            pd = p
            if dropout_mask is not None:
                keep = dropout_mask[ib, ih].to(dtype) * (1.0 / (1.0 - dropout_p))
                pd = p * keep
            o = pd @ vf[ib, :, jk]
            do = gf[ib, :, ih]
            dv[ib, :, jk] += pd.T @ do
            dp = do @ vf[ib, :, jk].T
            if dropout_mask is not None:
                dp = dp * keep
            dsum = (do * o).sum(dim=-1, keepdim=True)
            ds = p * (dp - dsum)
            dq[ib, :, ih] = scale * (ds @ kf[ib, :, jk])
            dk[ib, :, jk] += scale * (ds.T @ qf[ib, :, ih])
    return dq, dk, dv


def attention_backward_autograd(q, k, v, dout, upcast=True, reorder_ops=False, **kw):
    """(dq, dk, dv) by torch autograd through `attention_forward`.  With upcast=False,
    reorder_ops=True this is the ordinary low-precision implementation whose error supplies the
    right-hand side of the gradient tolerance rule (`tests/test_flash_attn.py:1006-1008`)."""
    q, k, v = [t.detach().clone().requires_grad_() for t in (q, k, v)]
    out, _ = attention_forward(q, k, v, upcast=upcast, reorder_ops=reorder_ops, **kw)
    return torch.autograd.grad(out, (q, k, v), dout.to(out.dtype))


def attention_reference_pair(q, k, v, **kw):
    """(out_fp32path, lse, out_lowprecision): the two runs the tolerance rule needs."""
    out_ref, lse = attention_forward(q, k, v, upcast=True, reorder_ops=False, **kw)
    out_pt, _ = attention_forward(q, k, v, upcast=False, reorder_ops=True, **kw)
    return out_ref, lse, out_pt


def tolerance_ok(out, out_ref, out_pt, mult: float = 2.0, extra: float = 0.0):
    """The reference's acceptance rule (`tests/test_flash_attn.py:648-650`; `+1e-5` at `:1397`;
    `3x + 1e-5` for the KV-cache API at `:1860`).  Returns (ok, err, bound)."""
    err = (out.float() - out_ref.float()).abs().max().item()
    bound = mult * (out_pt.float() - out_ref.float()).abs().max().item() + extra
    return err <= bound, err, bound


def lse_ok(lse, lse_ref, rtol: float = 1e-3):
    """log-sum-exp within `rtol` relative (absolute floor of rtol for values near 0); infinities
    must coincide exactly."""
    lse, lse_ref = lse.float(), lse_ref.float()
    inf_ref = torch.isinf(lse_ref)
    if not torch.equal(torch.isinf(lse), inf_ref):
        return False, float("inf")
    if not torch.equal(lse[inf_ref], lse_ref[inf_ref]):
        return False, float("inf")
    fin = ~inf_ref
    if fin.sum() == 0:
        return True, 0.0
    diff = (lse[fin] - lse_ref[fin]).abs()
    rel = (diff / lse_ref[fin].abs().clamp_min(1.0)).max().item()
    return rel <= rtol, rel


# --------------------------------------------------------------------------------------------
# packed variable-length attention
# --------------------------------------------------------------------------------------------
def attention_varlen_forward(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, causal=False,
                             window_size=(-1, -1), softmax_scale=None, upcast=True,
                             reorder_ops=False):
    """q (total_q, h, d), k/v (total_k, h_k, d), cu_seqlens int (b+1,).  Sequence i occupies rows
    cu[i]:cu[i+1] and attends only to its own keys.  Returns out (total_q, h, d) and lse
    (b, h, max_seqlen_q) with rows beyond a sequence's length set to 0 (the kernels leave them
    unwritten, `csrc/flash_attn/flash_api.cpp:527`)."""
    bsz = len(cu_seqlens_q) - 1
    h = q.shape[1]
    out = torch.zeros(q.shape[0], h, v.shape[-1], dtype=q.dtype)
    lse = torch.zeros(bsz, h, max_seqlen_q, dtype=torch.float32)
    for i in range(bsz):
        q0, q1 = int(cu_seqlens_q[i]), int(cu_seqlens_q[i + 1])
        k0, k1 = int(cu_seqlens_k[i]), int(cu_seqlens_k[i + 1])
        if q1 == q0:
            continue
        if k1 == k0:
            lse[i, :, : q1 - q0] = float("inf")
            continue
        o, l = attention_forward(q[q0:q1][None], k[k0:k1][None], v[k0:k1][None], causal=causal,
                                 window_size=window_size, softmax_scale=softmax_scale,
                                 upcast=upcast, reorder_ops=reorder_ops)
        out[q0:q1] = o[0]
        lse[i, :, : q1 - q0] = l[0]
    return out, lse


# --------------------------------------------------------------------------------------------
# rotary embedding
# --------------------------------------------------------------------------------------------
def rotary_apply(x, cos, sin, positions, interleaved: bool):
    """x (b, s, h, d); cos/sin (seqlen_ro, rotary_dim/2); positions (b, s) long: table row per token.

    out[..., :rd] = x * cos + rotate_half(x) * sin, remaining dims pass through
    (`flash_attn/layers/rotary.py:11-32`).  Math in fp32 on the (possibly low-precision) table
    values, one rounding to x.dtype at the end, as the kernels do
    (`csrc/flash_attn/src/utils.h:427-431, 499-501`).
    interleaved pairs dims (2i, 2i+1); otherwise dims (i, i + rd/2).
    """
    rd = cos.shape[-1] * 2
    assert rd <= x.shape[-1]
    c = cos.float()[positions]            # (b, s, rd/2)
    s_ = sin.float()[positions]
    xf = x.float()
    xr = xf[..., :rd]
    if interleaved:
        x0, x1 = xr[..., 0::2], xr[..., 1::2]
        c, s_ = c.unsqueeze(2), s_.unsqueeze(2)
        o0 = x0 * c - x1 * s_
        o1 = x0 * s_ + x1 * c
        rot = torch.stack((o0, o1), dim=-1).flatten(-2)
    else:
        x0, x1 = xr[..., : rd // 2], xr[..., rd // 2:]
        c, s_ = c.unsqueeze(2), s_.unsqueeze(2)
        rot = torch.cat((x0 * c - x1 * s_, x1 * c + x0 * s_), dim=-1)
    return torch.cat((rot, xf[..., rd:]), dim=-1).to(x.dtype)


def rotary_table(seqlen: int, rotary_dim: int, base: float = 10000.0, dtype=torch.float32):
    """cos/sin (seqlen, rotary_dim/2): cos(outer(t, base^(-2i/rd))) computed in fp32, then cast
    (`flash_attn/layers/rotary.py:362-401`)."""
    inv_freq = 1.0 / (base ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))
    t = torch.arange(seqlen, dtype=torch.float32)
    freqs = torch.outer(t, inv_freq)
    return torch.cos(freqs).to(dtype), torch.sin(freqs).to(dtype)


# --------------------------------------------------------------------------------------------
# KV-cache API
# --------------------------------------------------------------------------------------------
def kvcache_forward(q, k_cache, v_cache, k=None, v=None, rotary_cos=None, rotary_sin=None,
                    cache_seqlens=None, cache_batch_idx=None, softmax_scale=None, causal=False,
                    window_size=(-1, -1), rotary_interleaved=True, upcast=True, reorder_ops=False):
    """Semantics of `flash_attn_with_kvcache` (`flash_attn/flash_attn_interface.py:922-1042`) as the
    reference's test builds them (`tests/test_flash_attn.py:1759-1834`).

    Returns (out, lse, k_cache_after, v_cache_after) where the caches are full updated copies
    (indexed like the inputs, i.e. rows `cache_batch_idx` are the ones touched).
    * new keys are rotated at positions cache_seqlens + t and written at those rows; new values
      are written unrotated (bit-exact);
    * q is rotated at cache_seqlens + i when causal or local, else at cache_seqlens for every row;
    * attention covers keys [0, cache_seqlens + seqlen_new) of the selected cache row.
    """
    b, sq, h, d = q.shape
    sk_cap = k_cache.shape[1]
    if cache_seqlens is None:
        lens = torch.full((b,), sk_cap, dtype=torch.long)
    elif isinstance(cache_seqlens, int):
        lens = torch.full((b,), cache_seqlens, dtype=torch.long)
    else:
        lens = cache_seqlens.long()
    idx = torch.arange(b) if cache_batch_idx is None else cache_batch_idx.long()
    k_after, v_after = k_cache.clone(), v_cache.clone()
    seqlen_new = 0 if k is None else k.shape[1]
    local = window_size[0] >= 0 or window_size[1] >= 0
    q_use = q
    if rotary_cos is not None:
        assert k is not None
        if causal or local:
            qpos = lens.view(-1, 1) + torch.arange(sq).view(1, -1)
        else:
            qpos = lens.view(-1, 1).expand(b, sq)
        q_use = rotary_apply(q, rotary_cos, rotary_sin, qpos, rotary_interleaved)
    if k is not None:
        kpos = lens.view(-1, 1) + torch.arange(seqlen_new).view(1, -1)
        k_use = k if rotary_cos is None else rotary_apply(k, rotary_cos, rotary_sin, kpos,
                                                          rotary_interleaved)
        for ib in range(b):
            L = int(lens[ib])
            k_after[idx[ib], L:L + seqlen_new] = k_use[ib]
            v_after[idx[ib], L:L + seqlen_new] = v[ib]
    eff = lens + seqlen_new
    out, lse = attention_forward(q_use, k_after[idx], v_after[idx], causal=causal,
                                 window_size=window_size, softmax_scale=softmax_scale,
                                 seqlens_k=eff, upcast=upcast, reorder_ops=reorder_ops)
    return out, lse, k_after, v_after


# --------------------------------------------------------------------------------------------
# split-KV merge and the reference's split-count heuristic
# --------------------------------------------------------------------------------------------
def combine_splits(o_parts, lse_parts):
    """Merge per-split normalised partial outputs (S, …, d) with their lse (S, …): the closed form
    behind `combine_attn_seqk_parallel` (`csrc/flash_attn/src/flash_fwd_kernel.h:1227-1298`):
    lse = logsumexp_s lse_s, out = sum_s exp(lse_s - lse) o_s; all -inf gives lse = +inf, out = 0."""
    lse = torch.logsumexp(lse_parts, dim=0)
    w = torch.exp(lse_parts - lse.unsqueeze(0))
    w = torch.nan_to_num(w, nan=0.0)
    out = (w.unsqueeze(-1) * o_parts).sum(0)
    lse = torch.where(torch.isneginf(lse), torch.full_like(lse, float("inf")), lse)
    return out, lse


def num_splits_heuristic_reference(batch_nheads_mblocks: int, num_sms: int, num_n_blocks: int,
                                   max_splits: int) -> int:
    """The reference's rule (`csrc/flash_attn/flash_api.cpp:212-246`): one split if the grid
    already fills 80 % of the SMs; otherwise the smallest eligible split count whose wave
    efficiency reaches 85 % of the best one."""
    if batch_nheads_mblocks >= 0.8 * num_sms:
        return 1
    max_splits = min(max_splits, num_sms, num_n_blocks)
    cdiv = lambda a, b_: (a + b_ - 1) // b_

    def eligible(s):
        return s == 1 or cdiv(num_n_blocks, s) != cdiv(num_n_blocks, s - 1)

    effs = []
    best = 0.0
    for s in range(1, max_splits + 1):
        if not eligible(s):
            effs.append(0.0)
            continue
        waves = float(batch_nheads_mblocks * s) / num_sms
        eff = waves / math.ceil(waves)
        best = max(best, eff)
        effs.append(eff)
    for s in range(1, max_splits + 1):
        if eligible(s) and effs[s - 1] >= 0.85 * best:
            return s
    return 1


def attention_flops(batch, seqlen_q, seqlen_k, nheads, headdim, causal=False, window_size=(-1, -1)):
    """Forward FLOPs: 4 * d * (visible (i, j) pairs) * b * h.  For dense / square-causal inputs this
    equals the reference's convention 4*b*s^2*h*d (/2 if causal)
    (`benchmarks/benchmark_flash_attention.py:27-30`) up to the diagonal term."""
    left, right = window_size
    if causal:
        right = 0
    rows = torch.arange(seqlen_q, dtype=torch.long)
    shift = seqlen_k - seqlen_q
    hi = torch.full_like(rows, seqlen_k - 1) if right < 0 else torch.clamp(rows + shift + right, max=seqlen_k - 1)
    lo = torch.zeros_like(rows) if left < 0 else torch.clamp(rows + shift - left, min=0)
    pairs = torch.clamp(hi - lo + 1, min=0).sum().item()
    return 4.0 * headdim * pairs * batch * nheads
