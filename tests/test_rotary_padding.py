"""CPU checks of the host-side pieces around the variable-length and rotary paths: padding helpers,
the plain-torch rotary restatement against the oracle, the rotary layer's cos / sin cache, and the
argument checks of `fa_rotary` (no kernel is launched)."""
import ctypes

import pytest
import torch

from oracle import attention_oracle as orc


def test_unpad_pad_round_trip_and_cu_seqlens():
    from flash_attn.bert_padding import index_first_axis, index_put_first_axis, pad_input, unpad_input
    g = torch.Generator().manual_seed(0)
    b, s = 6, 37
    lens = torch.tensor([0, 1, 37, 5, 36, 20])
    mask = torch.arange(s)[None, :] < lens[:, None]
    x = torch.randn(b, s, 3, 8, generator=g)
    packed, indices, cu, mx = unpad_input(x, mask)
    assert packed.shape == (int(lens.sum()), 3, 8)
    assert cu.dtype == torch.int32 and cu.tolist() == [0] + lens.cumsum(0).tolist()
    assert mx == 37
    # brute force: token t of sequence i sits at packed row cu[i] + t
    for i in range(b):
        for t in range(int(lens[i])):
            assert torch.equal(packed[cu[i] + t], x[i, t])
            assert int(indices[cu[i] + t]) == i * s + t
    back = pad_input(packed, indices, b, s)
    assert torch.equal(back, x * mask[:, :, None, None])
    assert torch.equal(index_first_axis(x.reshape(b * s, 3, 8), indices), packed)
    assert torch.equal(index_put_first_axis(packed, indices, b * s).reshape(b, s, 3, 8), back)


def test_unpad_with_holes_in_mask_and_int_mask():
    """The mask need not be a prefix: any non-zero entry keeps its token, in row-major order."""
    from flash_attn.bert_padding import pad_input, unpad_input
    mask = torch.tensor([[0, 1, 1, 0], [1, 0, 0, 1], [0, 0, 0, 0]], dtype=torch.int64)
    x = torch.arange(12, dtype=torch.float32).reshape(3, 4, 1)
    packed, indices, cu, mx = unpad_input(x, mask)
    assert packed.flatten().tolist() == [1, 2, 4, 7]
    assert indices.tolist() == [1, 2, 4, 7] and cu.tolist() == [0, 2, 4, 4] and mx == 2
    assert torch.equal(pad_input(packed, indices, 3, 4), x * mask[:, :, None])


def test_padding_helpers_are_differentiable():
    from flash_attn.bert_padding import pad_input, unpad_input
    mask = torch.tensor([[1, 1, 0], [1, 0, 0]], dtype=torch.bool)
    x = torch.randn(2, 3, 4, requires_grad=True)
    packed, indices, _, _ = unpad_input(x, mask)
    w = torch.randn(2, 3, 4)
    (pad_input(packed * 2.0, indices, 2, 3) * w).sum().backward()
    assert torch.equal(x.grad, 2.0 * w * mask[:, :, None])


@pytest.mark.parametrize("interleaved", [False, True])
@pytest.mark.parametrize("rotary_dim", [32, 64])
def test_torch_restatement_matches_oracle(interleaved, rotary_dim):
    from flash_attn.layers.rotary import apply_rotary_emb_torch
    g = torch.Generator().manual_seed(1)
    b, s, h, d = 2, 19, 3, 64
    x = torch.randn(b, s, h, d, generator=g)
    cos, sin = orc.rotary_table(s, rotary_dim)
    pos = torch.arange(s)[None, :].expand(b, s)
    got = apply_rotary_emb_torch(x, cos, sin, interleaved=interleaved)
    assert torch.allclose(got, orc.rotary_apply(x, cos, sin, pos, interleaved), atol=1e-6, rtol=0)
    # a rotation: norms of rotated pairs are preserved, and position 0 is the identity
    assert torch.allclose(got.norm(dim=-1), x.norm(dim=-1), rtol=1e-5)
    assert torch.equal(got[:, 0], x[:, 0])


def test_rotary_embedding_cache_matches_table_and_xpos_cancels():
    from flash_attn.layers.rotary import RotaryEmbedding
    rot = RotaryEmbedding(64, base=10000.0)
    rot._update_cos_sin_cache(50, device=torch.device("cpu"), dtype=torch.float32)
    cos, sin = orc.rotary_table(50, 64)
    assert torch.equal(rot._cos_cached, cos) and torch.equal(rot._sin_cached, sin)
    rot._update_cos_sin_cache(20, device=torch.device("cpu"), dtype=torch.float32)    # never shrinks
    assert rot._cos_cached.shape[0] == 50
    xp = RotaryEmbedding(64, scale_base=512)
    xp._update_cos_sin_cache(33, device=torch.device("cpu"), dtype=torch.float32)
    cos, sin = orc.rotary_table(33, 64)
    # q's table times k's table gives back the unscaled one; the middle position is unscaled
    assert torch.allclose(xp._cos_cached * xp._cos_k_cached, cos * cos, atol=1e-6)
    assert torch.allclose(xp._sin_cached * xp._sin_k_cached, sin * sin, atol=1e-6)
    assert torch.allclose(xp._cos_cached[33 // 2], cos[33 // 2], atol=1e-7)


def test_rotary_entry_point_rejects_bad_arguments():
    import flash_attn._native as nat
    assert nat.lib.fa_sizeof_rotary_params() == ctypes.sizeof(nat.FaRotaryParams)
    p = nat.FaRotaryParams()
    assert nat.lib.fa_rotary(ctypes.byref(p), None) != 0           # null pointers
    assert nat.lib.fa_last_error()
    p.x = p.out = p.cos = p.sin = 16                               # never dereferenced: checks fail first
    p.b, p.seqlen, p.h, p.d, p.rotary_dim, p.seqlen_ro = 1, 4, 1, 64, 72, 4
    p.dtype, p.cs_dtype = nat.FA_DTYPE_BF16, nat.FA_DTYPE_FP32
    assert nat.lib.fa_rotary(ctypes.byref(p), None) != 0           # rotary_dim > d
    p.rotary_dim = 24
    assert nat.lib.fa_rotary(ctypes.byref(p), None) != 0           # not a multiple of 16
    p.rotary_dim, p.dtype = 32, 7
    assert nat.lib.fa_rotary(ctypes.byref(p), None) != 0           # unknown dtype


def test_unpad_for_concatenated_sequences_docstring_example():
    """The reference documents this function by one example (flash_attn/bert_padding.py:131-170): batch 3, seqlen 6,
    lengths [[2, 3, 0, 0, 0, 0], [3, 2, 0, 0, 0, 0], [6, 0, 0, 0, 0, 0]] stand for the block-diagonal causal masks
    drawn there.  Known answer: five sequences of 2, 3, 3, 2, 6 tokens; the first row's last token is padding.
    The masks themselves: packed causal attention over the returned cu_seqlens must equal dense attention under
    the documented 3D mask."""
    from flash_attn.bert_padding import pad_input, unpad_input_for_concatenated_sequences
    lengths = torch.tensor([[2, 3, 0, 0, 0, 0], [3, 2, 0, 0, 0, 0], [6, 0, 0, 0, 0, 0]], dtype=torch.int32)
    x = torch.arange(3 * 6 * 2, dtype=torch.float32).reshape(3, 6, 2)
    packed, indices, cu, mx = unpad_input_for_concatenated_sequences(x, lengths)
    assert cu.dtype == torch.int32 and cu.tolist() == [0, 2, 5, 8, 10, 16] and mx == 6
    assert indices.tolist() == [0, 1, 2, 3, 4, 6, 7, 8, 9, 10, 12, 13, 14, 15, 16, 17]
    assert torch.equal(packed, x.reshape(18, 2)[indices])
    back = pad_input(packed, indices, 3, 6)
    assert torch.equal(back[0, :5], x[0, :5]) and not back[0, 5].any() and torch.equal(back[1:, :5], x[1:, :5])
    # the documented 3D masks, row by row
    doc = torch.tensor([
        [[1, 0, 0, 0, 0, 0], [1, 1, 0, 0, 0, 0], [0, 0, 1, 0, 0, 0], [0, 0, 1, 1, 0, 0], [0, 0, 1, 1, 1, 0], [0, 0, 0, 0, 0, 1]],
        [[1, 0, 0, 0, 0, 0], [1, 1, 0, 0, 0, 0], [1, 1, 1, 0, 0, 0], [0, 0, 0, 1, 0, 0], [0, 0, 0, 1, 1, 0], [0, 0, 0, 0, 0, 1]],
        [[1, 0, 0, 0, 0, 0], [1, 1, 0, 0, 0, 0], [1, 1, 1, 0, 0, 0], [1, 1, 1, 1, 0, 0], [1, 1, 1, 1, 1, 0], [1, 1, 1, 1, 1, 1]],
    ], dtype=torch.bool)
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(3, 6, 1, 8, generator=g) for _ in range(3))
    qp, kp, vp = (unpad_input_for_concatenated_sequences(t, lengths)[0] for t in (q, k, v))
    out_packed, _ = orc.attention_varlen_forward(qp, kp, vp, cu, cu, mx, causal=True)
    dense = torch.zeros(3, 6, 1, 8)
    for b in range(3):
        s = torch.einsum("thd,shd->hts", q[b], k[b]) * 8 ** -0.5
        p = torch.softmax(s.masked_fill(~doc[b], float("-inf")), -1)
        dense[b] = torch.einsum("hts,shd->thd", p, v[b])
    got = pad_input(out_packed, indices, 3, 6)
    real = pad_input(torch.ones(16, 1), indices, 3, 6).bool().squeeze(-1)
    assert torch.allclose(got[real], dense[real], atol=1e-5)


def test_index_first_axis_residual_gradient():
    from flash_attn.bert_padding import index_first_axis_residual
    x = torch.randn(7, 3, requires_grad=True)
    idx = torch.tensor([5, 0, 5, 2])
    rows, whole = index_first_axis_residual(x, idx)
    assert torch.equal(rows, x[idx]) and whole is x
    (rows.sum() * 2 + (whole * 3).sum()).backward()
    want = torch.full((7, 3), 3.0)
    want[5] += 4.0
    want[0] += 2.0
    want[2] += 2.0
    assert torch.equal(x.grad, want)


def test_speculative_sampling_keeps_the_verifying_distribution():
    """The point of speculative sampling: whatever the drafting distribution, the first token that comes out is
    distributed as the VERIFYING model's first position, and when the first draft stands, the second as its second
    (Leviathan et al., theorem 1).  Checked empirically on a vocabulary of 6 with 400k independent rows, plus the
    two greedy known answers: equal argmax -> the draft stands, different -> the verifier's argmax replaces it."""
    from flash_attn.utils.generation import sample_speculative
    torch.manual_seed(0)
    vocab, rows = 6, 400000
    lp = torch.randn(1, 2, vocab) * 1.5
    lq = torch.randn(1, 1, vocab) * 1.5
    p, q = lp.softmax(-1)[0], lq.softmax(-1)[0]
    drafts = torch.multinomial(q[0], rows, replacement=True).unsqueeze(1)
    tokens, counted = sample_speculative(lp.expand(rows, 2, vocab), lq.expand(rows, 1, vocab), drafts, top_k=0)
    first = torch.bincount(tokens[:, 0], minlength=vocab).float() / rows
    assert (first - p[0]).abs().max().item() < 4e-3, (first, p[0])
    stood = counted == 2
    assert abs(stood.float().mean().item() - torch.minimum(p[0], q[0]).sum().item()) < 4e-3     # acceptance rate = sum min(p, q)
    second = torch.bincount(tokens[stood, 1], minlength=vocab).float() / int(stood.sum())
    assert (second - p[1]).abs().max().item() < 6e-3
    # greedy
    lg = torch.tensor([[[0.0, 3.0, 1.0], [2.0, 0.0, 1.0], [0.0, 1.0, 5.0]]])
    t, n = sample_speculative(lg, lg[:, :2] + 0.1, torch.tensor([[1, 0]]), top_k=1)
    assert t.tolist() == [[1, 0, 2]] and n.tolist() == [3]
    t, n = sample_speculative(lg, torch.tensor([[[0.0, 1.0, 3.0], [2.0, 0.0, 1.0]]]), torch.tensor([[2, 0]]), top_k=1)
    assert t[0, 0].item() == 1 and n.tolist() == [1]
