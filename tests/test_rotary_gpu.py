"""GPU parity of the standalone rotary op (`fa_rotary` behind flash_attn.layers.rotary) against the
CPU oracle.  Cases and acceptance follow the reference's tests/test_rotary.py:46-250: fp16 / bf16,
seqlen_offsets as 0 / int / per-sequence tensor, rotary_dim = headdim or headdim / 2, interleaved or
not, in place or not, packed q/k/v and k/v tensors, packed variable-length input; forward and the
gradient (the inverse rotation).  Tolerance: rtol 1e-3 plus twice the rounding step of the expected
values (`|(y + 0.3 - 0.3) - y|` max), as the reference has it."""
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


def _table(rows, rotary_dim, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    angle = torch.rand(rows, rotary_dim // 2, generator=g) * 2 * math.pi
    return torch.cos(angle).to(dtype), torch.sin(angle).to(dtype)


def _offsets(kind, batch, seqlen, seed):
    g = torch.Generator().manual_seed(seed)
    if kind == "zero":
        return 0
    if kind == "int":
        return int(torch.randint(0, seqlen + 1, (1,), generator=g))
    return torch.randint(0, seqlen + 1, (batch,), generator=g, dtype=torch.int32)


def _positions(offsets, batch, seqlen):
    off = offsets.long() if isinstance(offsets, torch.Tensor) else torch.full((batch,), offsets, dtype=torch.long)
    return off[:, None] + torch.arange(seqlen)[None, :]


def _close(got, want, what):
    got = got.float().cpu()
    step = ((want + 0.3 - 0.3) - want).float().abs().max().item()      # in want's own 16-bit type
    diff = (got - want.float()).abs().max().item()
    _say("   %s max diff %.3e (rounding step %.3e)" % (what, diff, step))
    assert torch.allclose(got, want.float(), rtol=1e-3, atol=2 * step), what


def _dev(offsets):
    return offsets.to(DEV) if isinstance(offsets, torch.Tensor) else offsets


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("offsets_kind", ["zero", "int", "tensor"])
@pytest.mark.parametrize("fraction", [1.0, 0.5])
@pytest.mark.parametrize("interleaved", [False, True])
@pytest.mark.parametrize("inplace", [False, True])
def test_rotary_emb_func(inplace, interleaved, fraction, offsets_kind, dtype):
    from flash_attn.layers.rotary import apply_rotary_emb
    _say("rotary func", inplace, interleaved, fraction, offsets_kind, dtype)
    b, s, h, d = 32, 217, 4, 128
    rd = int(fraction * d)
    g = torch.Generator().manual_seed(42)
    x_cpu = torch.randn(b, s, h, d, generator=g).to(dtype)
    cos, sin = _table(2 * s, rd, dtype, 7)
    offsets = _offsets(offsets_kind, b, s, 11)
    pos = _positions(offsets, b, s)
    x = x_cpu.to(DEV).requires_grad_()
    out = apply_rotary_emb(x, cos.to(DEV), sin.to(DEV), seqlen_offsets=_dev(offsets), interleaved=interleaved,
                           inplace=inplace)
    if inplace:
        assert out.data_ptr() == x.data_ptr()
    else:
        assert torch.equal(x.detach().cpu(), x_cpu)
    _close(out.detach(), orc.rotary_apply(x_cpu, cos, sin, pos, interleaved), "out")
    gout = torch.randn(b, s, h, d, generator=g).to(dtype)
    out.backward(gout.to(DEV))
    _close(x.grad, orc.rotary_apply(gout, cos, -sin, pos, interleaved), "grad")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("offsets_kind", ["zero", "int", "tensor"])
@pytest.mark.parametrize("fraction", [1.0, 0.5])
@pytest.mark.parametrize("interleaved", [False, True])
@pytest.mark.parametrize("contiguous", [True, False])
def test_rotary_emb_qkv(contiguous, interleaved, fraction, offsets_kind, dtype):
    """Packed (b, s, 3, h, d): q and k rotated in place, v untouched.  Dense input takes the single
    launch over 2h heads, a strided view takes one launch each for q and k."""
    from flash_attn.layers.rotary import apply_rotary_emb_qkv_
    _say("rotary qkv", contiguous, interleaved, fraction, offsets_kind, dtype)
    b, s, h, d = 8, 512, 4, 128
    rd = int(fraction * d)
    g = torch.Generator().manual_seed(42)
    qkv_cpu = torch.randn(b, s, 3, h, d, generator=g).to(dtype)
    cos, sin = _table(2 * s, rd, dtype, 7)
    offsets = _offsets(offsets_kind, b, s, 13)
    pos = _positions(offsets, b, s)
    leaf = qkv_cpu.to(DEV).requires_grad_()
    if contiguous:
        inp = leaf
    else:
        wide = torch.zeros(b, s, 3, h, d + 8, dtype=dtype, device=DEV)
        inp = wide[..., :d]
        inp.copy_(leaf)            # differentiable copy into a view with row pitch d + 8
        assert not inp.is_contiguous()
    out = apply_rotary_emb_qkv_(inp, cos.to(DEV), sin.to(DEV), interleaved=interleaved, seqlen_offsets=_dev(offsets))
    want = torch.stack([orc.rotary_apply(qkv_cpu[:, :, 0], cos, sin, pos, interleaved),
                        orc.rotary_apply(qkv_cpu[:, :, 1], cos, sin, pos, interleaved), qkv_cpu[:, :, 2]], dim=2)
    _close(out.detach(), want, "out")
    assert torch.equal(out.detach()[:, :, 2].cpu(), qkv_cpu[:, :, 2])
    gout = torch.randn(b, s, 3, h, d, generator=g).to(dtype)
    out.backward(gout.to(DEV))
    gwant = torch.stack([orc.rotary_apply(gout[:, :, 0], cos, -sin, pos, interleaved),
                         orc.rotary_apply(gout[:, :, 1], cos, -sin, pos, interleaved), gout[:, :, 2]], dim=2)
    _close(leaf.grad, gwant, "grad")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("offsets_kind", ["zero", "int", "tensor"])
@pytest.mark.parametrize("fraction", [1.0, 0.5])
@pytest.mark.parametrize("interleaved", [False, True])
def test_rotary_emb_kv(interleaved, fraction, offsets_kind, dtype):
    from flash_attn.layers.rotary import apply_rotary_emb_kv_
    _say("rotary kv", interleaved, fraction, offsets_kind, dtype)
    b, s, h, d = 8, 781, 4, 64
    rd = int(fraction * d)
    g = torch.Generator().manual_seed(42)
    kv_cpu = torch.randn(b, s, 2, h, d, generator=g).to(dtype)
    cos, sin = _table(2 * s, rd, dtype, 7)
    offsets = _offsets(offsets_kind, b, s, 17)
    pos = _positions(offsets, b, s)
    leaf = kv_cpu.to(DEV).requires_grad_()
    out = apply_rotary_emb_kv_(leaf, cos.to(DEV), sin.to(DEV), interleaved=interleaved,
                               seqlen_offsets=_dev(offsets))
    want = torch.stack([orc.rotary_apply(kv_cpu[:, :, 0], cos, sin, pos, interleaved), kv_cpu[:, :, 1]], dim=2)
    _close(out.detach(), want, "out")
    gout = torch.randn(b, s, 2, h, d, generator=g).to(dtype)
    out.backward(gout.to(DEV))
    gwant = torch.stack([orc.rotary_apply(gout[:, :, 0], cos, -sin, pos, interleaved), gout[:, :, 1]], dim=2)
    _close(leaf.grad, gwant, "grad")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("offsets_kind", ["zero", "int", "tensor"])
@pytest.mark.parametrize("fraction", [1.0, 0.5])
@pytest.mark.parametrize("interleaved", [False, True])
@pytest.mark.parametrize("inplace", [False, True])
def test_rotary_emb_varlen_func(inplace, interleaved, fraction, offsets_kind, dtype):
    """Packed (total, h, d) with cu_seqlens; one sequence is empty and one has a single token."""
    from flash_attn.bert_padding import pad_input, unpad_input
    from flash_attn.layers.rotary import apply_rotary_emb
    _say("rotary varlen", inplace, interleaved, fraction, offsets_kind, dtype)
    b, s, h, d = 32, 217, 4, 128
    rd = int(fraction * d)
    g = torch.Generator().manual_seed(42)
    x_cpu = torch.randn(b, s, h, d, generator=g).to(dtype)
    lengths = torch.randint(max(1, s - 20), s + 1, (b,), generator=g)
    lengths[3], lengths[9] = 0, 1
    mask = torch.arange(s)[None, :] < lengths[:, None]
    cos, sin = _table(2 * s, rd, dtype, 7)
    offsets = _offsets(offsets_kind, b, s, 19)
    pos = _positions(offsets, b, s)
    x_unpad, indices, cu, mx = unpad_input(x_cpu.to(DEV), mask.to(DEV))
    assert mx == int(lengths.max())
    keep = x_unpad.clone()
    leaf = x_unpad.requires_grad_()
    out_unpad = apply_rotary_emb(leaf, cos.to(DEV), sin.to(DEV), seqlen_offsets=_dev(offsets), interleaved=interleaved,
                                 inplace=inplace, cu_seqlens=cu, max_seqlen=mx)
    if not inplace:
        assert torch.equal(leaf.detach(), keep)
    out = pad_input(out_unpad, indices, b, s)
    want = orc.rotary_apply(x_cpu, cos, sin, pos, interleaved) * mask[:, :, None, None]
    _close(out.detach(), want, "out")
    gout = torch.randn(b, s, h, d, generator=g).to(dtype)
    out.backward(gout.to(DEV))
    gwant = orc.rotary_apply(gout, cos, -sin, pos, interleaved) * mask[:, :, None, None]
    _close(pad_input(leaf.grad, indices, b, s), gwant, "grad")


@pytest.mark.parametrize("varlen", [False, True])
@pytest.mark.parametrize("inplace", [False, True])
@pytest.mark.parametrize("interleaved", [False, True])
@pytest.mark.parametrize("h,d,rd", [(16, 128, 128), (32, 128, 64), (40, 64, 64), (24, 256, 96), (128, 32, 32)])
def test_rotary_many_heads(h, d, rd, interleaved, inplace, varlen):
    """With 128 or more 16-byte work items per token the kernel hands whole tokens to workgroups (one index
    division per item instead of four); same results required, dense and packed, with per-sequence offsets
    and positions that run past the table."""
    from flash_attn.layers.rotary import apply_rotary_emb
    _say("rotary many heads", h, d, rd, interleaved, inplace, varlen)
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(h + d)
    lens = [5, 1, 77, 130] if varlen else [61, 61, 61]
    b, mx = len(lens), max(lens)
    cos, sin = _table(mx + 20, rd, dtype, 3)
    offsets = torch.tensor([0, 19, 3, 40][:b], dtype=torch.int32)       # the last packed sequence runs past the table
    if varlen:
        cu = torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32)
        x_cpu = torch.randn(int(cu[-1]), h, d, generator=g).to(dtype)
        x = x_cpu.to(DEV)
        out = apply_rotary_emb(x, cos.to(DEV), sin.to(DEV), seqlen_offsets=offsets.to(DEV), cu_seqlens=cu.to(DEV),
                               max_seqlen=mx, interleaved=interleaved, inplace=inplace)
        pieces = [(x_cpu[int(cu[i]):int(cu[i + 1])][None], int(offsets[i]), lens[i]) for i in range(b)]
    else:
        x_cpu = torch.randn(b, mx, h, d, generator=g).to(dtype)
        x = x_cpu.to(DEV)
        out = apply_rotary_emb(x, cos.to(DEV), sin.to(DEV), seqlen_offsets=offsets.to(DEV), interleaved=interleaved,
                               inplace=inplace)
        pieces = [(x_cpu[i:i + 1], int(offsets[i]), mx) for i in range(b)]
    if not inplace:
        assert torch.equal(x.cpu(), x_cpu)
    got = out.cpu()
    row = 0
    for i, (xi, off, n) in enumerate(pieces):
        pos = (off + torch.arange(n))[None]
        inside = pos[0] < cos.shape[0]
        want = xi.clone()
        if inside.any():
            want[:, inside] = orc.rotary_apply(xi[:, inside], cos, sin, pos[:, inside], interleaved)
        gi = got[row:row + n][None] if varlen else got[i:i + 1]
        _close(gi, want, "sequence %d" % i)
        row += n


@pytest.mark.parametrize("interleaved,inplace", [(False, True), (True, False)])
def test_rotary_half_gigabyte_tensor(interleaved, inplace):
    """From 384 MiB on the kernel moves x and out with non-temporal accesses (another instantiation): the
    benchmark shape (8, 8192, 32, 128), checked on sampled (batch, head) slices, and everything else of an
    out-of-place result must be finite."""
    from flash_attn.layers.rotary import apply_rotary_emb
    _say("rotary 0.5 GB", interleaved, inplace)
    b, s, h, d = 8, 8192, 32, 128
    torch.manual_seed(5)
    x = torch.randn(b, s, h, d, device=DEV, dtype=torch.bfloat16)
    cos, sin = _table(s + 7, d, torch.bfloat16, 9)
    sample = [(0, 0), (7, 31), (3, 17)]
    before = {bh: x[bh[0], :, bh[1]].cpu() for bh in sample}
    out = apply_rotary_emb(x, cos.to(DEV), sin.to(DEV), seqlen_offsets=7, interleaved=interleaved, inplace=inplace)
    assert (out.data_ptr() == x.data_ptr()) == inplace
    assert torch.isfinite(out).all()
    pos = _positions(7, 1, s)
    for (bi, hi) in sample:
        want = orc.rotary_apply(before[(bi, hi)][None, :, None], cos, sin, pos, interleaved)
        _close(out[bi, :, hi][None, :, None], want, "batch %d head %d" % (bi, hi))
        if not inplace:
            assert torch.equal(x[bi, :, hi].cpu(), before[(bi, hi)])


@pytest.mark.parametrize("d,rd", [(64, 16), (96, 48), (256, 256), (40, 32)])
@pytest.mark.parametrize("interleaved", [False, True])
def test_rotary_fp32_tables_and_other_head_dims(d, rd, interleaved):
    """fp32 cos / sin (as the KV-cache path of a model in mixed precision holds them) and head dims
    other than 64 / 128; 16-byte granules straddle nothing since rotary_dim is a multiple of 16."""
    from flash_attn.layers.rotary import apply_rotary_emb
    _say("rotary fp32 tables", d, rd, interleaved)
    b, s, h = 3, 333, 5
    g = torch.Generator().manual_seed(3)
    x = torch.randn(b, s, h, d, generator=g).to(torch.bfloat16)
    cos, sin = _table(s + 50, rd, torch.float32, 5)
    out = apply_rotary_emb(x.to(DEV), cos.to(DEV), sin.to(DEV), seqlen_offsets=50, interleaved=interleaved)
    _close(out, orc.rotary_apply(x, cos, sin, _positions(50, b, s), interleaved), "out")


def test_rotary_embedding_module_matches_oracle_on_q_and_kv():
    """The layer: table built on the device, q rotated through the (q, kv) form with GQA-shaped kv,
    and XPos tables (k's table is the inverse scale of q's)."""
    from flash_attn.layers.rotary import RotaryEmbedding
    _say("rotary module")
    b, s, h, hk, d = 2, 300, 8, 2, 64
    g = torch.Generator().manual_seed(9)
    q = torch.randn(b, s, h, d, generator=g).to(torch.float16)
    kv = torch.randn(b, s, 2, hk, d, generator=g).to(torch.float16)
    pos = _positions(5, b, s)
    for scale_base in (None, 512):
        rot = RotaryEmbedding(d, interleaved=False, scale_base=scale_base, device=DEV)
        q_out, kv_out = rot(q.to(DEV).clone(), kv.to(DEV).clone(), seqlen_offset=5)
        cq, sq_ = rot._cos_cached.cpu(), rot._sin_cached.cpu()
        ck = cq if scale_base is None else rot._cos_k_cached.cpu()
        sk_ = sq_ if scale_base is None else rot._sin_k_cached.cpu()
        if scale_base is None:
            c_ref, s_ref = orc.rotary_table(s + 5, d, dtype=torch.float16)
            # device cos / sin may differ from the host's in the last fp32 bit before rounding to fp16
            assert (cq.float() - c_ref.float()).abs().max() <= 2 ** -10
            assert (sq_.float() - s_ref.float()).abs().max() <= 2 ** -10
        _close(q_out, orc.rotary_apply(q, cq, sq_, pos, False), "q")
        _close(kv_out[:, :, 0], orc.rotary_apply(kv[:, :, 0], ck, sk_, pos, False), "k")
        assert torch.equal(kv_out[:, :, 1].cpu(), kv[:, :, 1])


def test_rotary_positions_past_the_table_pass_through():
    """Per-sequence offsets may push a padded batch's trailing positions past the table (the reference
    kernel masks those loads to cos = 1, sin = 0: flash_attn/ops/triton/rotary.py:80-85)."""
    from flash_attn.layers.rotary import apply_rotary_emb
    _say("rotary past table")
    b, s, h, d = 2, 64, 2, 64
    g = torch.Generator().manual_seed(4)
    x = torch.randn(b, s, h, d, generator=g).to(torch.float16)
    cos, sin = _table(s, d, torch.float16, 6)
    offsets = torch.tensor([0, 40], dtype=torch.int32)
    out = apply_rotary_emb(x.to(DEV), cos.to(DEV), sin.to(DEV), seqlen_offsets=offsets.to(DEV)).cpu()
    pos = _positions(offsets, b, s)
    want = orc.rotary_apply(x, cos, sin, pos.clamp(max=s - 1), False)
    want[1, s - 40:] = x[1, s - 40:]
    _close(out, want, "out")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("d,rd", [(64, 24), (128, 42), (80, 80), (36, 36), (100, 50), (64, 2), (256, 200), (30, 30)])
@pytest.mark.parametrize("interleaved", [False, True])
@pytest.mark.parametrize("inplace", [False, True])
def test_rotary_any_even_dim_and_any_head_dim(d, rd, interleaved, inplace, dtype):
    """Rotary dimensions that are even but not multiples of 16, head dims that are not multiples of 8 (so rows
    start at odd 4-byte offsets), as the reference's op takes them (flash_attn/ops/triton/rotary.py:176-208; its
    test grid has rotary fractions 1.0 and 0.5 of head dims 128: tests/test_rotary.py:46-50).  These take the
    element-wise kernel; forward with per-sequence offsets, and the gradient (the inverse rotation)."""
    from flash_attn.layers.rotary import apply_rotary_emb
    _say("rotary general", d, rd, interleaved, inplace, dtype)
    b, s, h = 3, 77, 5
    g = torch.Generator().manual_seed(d + rd)
    x = torch.randn(b, s, h, d, generator=g).to(dtype)
    cos, sin = _table(s + 40, rd, dtype, 8)
    offsets = torch.tensor([0, 13, 40], dtype=torch.int32)
    xd = x.to(DEV).clone().requires_grad_(not inplace)
    out = apply_rotary_emb(xd, cos.to(DEV), sin.to(DEV), seqlen_offsets=offsets.to(DEV), interleaved=interleaved, inplace=inplace)
    pos = _positions(offsets, b, s)
    want = orc.rotary_apply(x, cos, sin, pos, interleaved)
    _close(out.detach(), want, "out")
    if inplace:
        assert out.data_ptr() == xd.data_ptr()
    else:
        assert torch.equal(xd.detach().cpu(), x)
        go = torch.randn(b, s, h, d, generator=g).to(dtype)
        (gx,) = torch.autograd.grad(out, xd, go.to(DEV))
        # the gradient of a rotation is the rotation by the opposite angle
        _close(gx, orc.rotary_apply(go, cos, -sin, pos, interleaved), "grad")


def test_rotary_general_kernel_on_packed_and_strided_input():
    """the element-wise kernel with packed variable-length rows and with x as a view whose strides are not
    multiples of 8 elements (a slice of a wider tensor)"""
    from flash_attn.layers.rotary import apply_rotary_emb
    _say("rotary general packed / strided")
    h, d, rd = 3, 44, 20
    lens = [5, 0, 31, 1, 18]
    cu = torch.tensor([0] + lens).cumsum(0).to(torch.int32)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(int(cu[-1]), h, d, generator=g).to(torch.float16)
    cos, sin = _table(max(lens), rd, torch.float16, 3)
    out = apply_rotary_emb(x.to(DEV), cos.to(DEV), sin.to(DEV), interleaved=True, cu_seqlens=cu.to(DEV), max_seqlen=max(lens))
    for i, L in enumerate(lens):
        if L:
            a = int(cu[i])
            want = orc.rotary_apply(x[a:a + L][None], cos, sin, torch.arange(L)[None], True)
            _close(out[a:a + L][None], want, "sequence %d" % i)
    wide = torch.randn(2, 50, 4, 67, generator=g).to(torch.bfloat16)      # row stride 4 * 67, head stride 67
    xs = wide[..., 3:3 + 64]
    cos, sin = _table(50, 32, torch.bfloat16, 4)
    out = apply_rotary_emb(xs.to(DEV)[...], cos.to(DEV), sin.to(DEV))
    wide_d = wide.to(DEV)
    out2 = apply_rotary_emb(wide_d[..., 3:3 + 64], cos.to(DEV), sin.to(DEV))
    want = orc.rotary_apply(xs, cos, sin, _positions(0, 2, 50), False)
    _close(out, want, "contiguous copy")
    _close(out2, want, "strided view")
