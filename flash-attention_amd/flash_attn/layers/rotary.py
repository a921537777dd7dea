"""Rotary position embedding on the MI355X HIP kernel.

Mirrors the reference's flash_attn/layers/rotary.py: `apply_rotary_emb` (:94-124, autograd function
:34-91), `apply_rotary_emb_qkv_` (:131-233), `apply_rotary_emb_kv_` (:236-296), the `RotaryEmbedding`
module with its cos/sin cache and XPos scaling (:299-480), `apply_rotary_emb_torch` (:19-31, a plain
torch restatement) and `rotate_half` (:11-16).  The reference runs a Triton kernel (flash_attn/ops/triton/rotary.py);
here the work is done by `fa_rotary` of libfa_mi355x.so.  The backward pass is the same kernel with
the rotation inverted (`conjugate`), as in the reference (:70-85).
"""
import ctypes
from typing import Optional, Union

import torch

from flash_attn import _native as nat


def rotate_half(x, interleaved=False):
    if not interleaved:
        x1, x2 = x.chunk(2, dim=-1)
        return torch.cat((-x2, x1), dim=-1)
    x1, x2 = x[..., 0::2], x[..., 1::2]
    return torch.stack((-x2, x1), dim=-1).flatten(-2)


def apply_rotary_emb_torch(x, cos, sin, interleaved=False):
    """x (batch, seqlen, nheads, headdim); cos, sin (seqlen, rotary_dim / 2) or
    (batch, seqlen, rotary_dim / 2).  Plain torch, any device."""
    ro_dim = cos.shape[-1] * 2
    assert ro_dim <= x.shape[-1]
    if interleaved:
        cos_f = cos.repeat_interleave(2, dim=-1).unsqueeze(-2)
        sin_f = sin.repeat_interleave(2, dim=-1).unsqueeze(-2)
    else:
        cos_f = torch.cat((cos, cos), dim=-1).unsqueeze(-2)
        sin_f = torch.cat((sin, sin), dim=-1).unsqueeze(-2)
    rot = x[..., :ro_dim] * cos_f + rotate_half(x[..., :ro_dim], interleaved) * sin_f
    return torch.cat((rot, x[..., ro_dim:]), dim=-1)


def apply_rotary(x, cos, sin, seqlen_offsets: Union[int, torch.Tensor] = 0, cu_seqlens: Optional[torch.Tensor] = None,
                 max_seqlen: Optional[int] = None, interleaved=False, inplace=False, conjugate=False):
    """Same contract as the reference's Triton entry (flash_attn/ops/triton/rotary.py:144-240)."""
    is_varlen = cu_seqlens is not None
    if not is_varlen:
        batch, seqlen, nheads, headdim = x.shape
    else:
        assert max_seqlen is not None, "If cu_seqlens is passed in, then max_seqlen must be passed"
        total_seqlen, nheads, headdim = x.shape
        batch = cu_seqlens.shape[0] - 1
        seqlen = max_seqlen
    seqlen_ro, rotary_dim = cos.shape
    assert sin.shape == cos.shape
    rotary_dim *= 2
    assert rotary_dim <= headdim, "rotary_dim must be <= headdim"
    assert headdim <= 256, "Only support headdim <= 256"
    assert seqlen_ro >= seqlen, "seqlen_ro must be >= seqlen"
    assert cos.dtype == sin.dtype, "cos and sin must have the same dtype"
    assert x.dtype in (torch.float16, torch.bfloat16), "rotary supports fp16 and bf16 input"
    assert x.is_cuda and cos.is_cuda and sin.is_cuda, "tensors must be on the GPU"
    assert x.stride(-1) == 1
    cos, sin = cos.contiguous(), sin.contiguous()
    if isinstance(seqlen_offsets, torch.Tensor):
        assert seqlen_offsets.shape == (batch,)
        assert seqlen_offsets.dtype in (torch.int32, torch.int64)
        seqlen_offsets = seqlen_offsets.to(torch.int32).contiguous()
    else:
        assert seqlen_offsets + seqlen <= seqlen_ro
    out = x if inplace else torch.empty_like(x)

    p = nat.FaRotaryParams()
    p.x, p.out, p.cos, p.sin = x.data_ptr(), out.data_ptr(), cos.data_ptr(), sin.data_ptr()
    p.cu_seqlens = None
    if is_varlen:
        cu32 = cu_seqlens.to(torch.int32).contiguous()
        p.cu_seqlens = cu32.data_ptr()
        p.x_batch_stride, p.x_row_stride, p.x_head_stride = 0, x.stride(0), x.stride(1)
        p.o_batch_stride, p.o_row_stride, p.o_head_stride = 0, out.stride(0), out.stride(1)
    else:
        p.x_batch_stride, p.x_row_stride, p.x_head_stride = x.stride(0), x.stride(1), x.stride(2)
        p.o_batch_stride, p.o_row_stride, p.o_head_stride = out.stride(0), out.stride(1), out.stride(2)
    if isinstance(seqlen_offsets, torch.Tensor):
        p.seqlen_offsets, p.seqlen_offset = seqlen_offsets.data_ptr(), 0
    else:
        p.seqlen_offsets, p.seqlen_offset = None, int(seqlen_offsets)
    p.cs_row_stride = cos.stride(0)
    p.b, p.seqlen, p.h, p.d = batch, seqlen, nheads, headdim
    p.rotary_dim, p.seqlen_ro = rotary_dim, seqlen_ro
    p.interleaved, p.conjugate = int(bool(interleaved)), int(bool(conjugate))
    p.dtype = nat._dtype_code(x.dtype)
    p.cs_dtype = {torch.float16: nat.FA_DTYPE_FP16, torch.bfloat16: nat.FA_DTYPE_BF16, torch.float32: nat.FA_DTYPE_FP32}[cos.dtype]
    with nat._on_device(x.device):
        rc = nat.lib.fa_rotary(ctypes.byref(p), ctypes.c_void_p(nat._stream(x.device)))
    if rc != 0:
        raise RuntimeError(nat.lib.fa_last_error().decode() or "libfa_mi355x: error %d" % rc)
    return out


class ApplyRotaryEmb(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, cos, sin, interleaved=False, inplace=False, seqlen_offsets: Union[int, torch.Tensor] = 0,
                cu_seqlens: Optional[torch.Tensor] = None, max_seqlen: Optional[int] = None):
        out = apply_rotary(x, cos, sin, seqlen_offsets=seqlen_offsets, cu_seqlens=cu_seqlens, max_seqlen=max_seqlen,
                           interleaved=interleaved, inplace=inplace)
        if isinstance(seqlen_offsets, int):
            ctx.save_for_backward(cos, sin, cu_seqlens)
            ctx.seqlen_offsets = seqlen_offsets
        else:
            ctx.save_for_backward(cos, sin, cu_seqlens, seqlen_offsets)
            ctx.seqlen_offsets = None
        ctx.interleaved, ctx.inplace, ctx.max_seqlen = interleaved, inplace, max_seqlen
        # as in the reference, the rotated input is returned without marking it dirty, so a leaf that
        # requires grad may be rotated in place
        return out

    @staticmethod
    def backward(ctx, do):
        seqlen_offsets = ctx.seqlen_offsets
        if seqlen_offsets is None:
            cos, sin, cu_seqlens, seqlen_offsets = ctx.saved_tensors
        else:
            cos, sin, cu_seqlens = ctx.saved_tensors
        if do.stride(-1) != 1:
            do = do.contiguous()
        dx = apply_rotary(do, cos, sin, seqlen_offsets=seqlen_offsets, cu_seqlens=cu_seqlens, max_seqlen=ctx.max_seqlen,
                          interleaved=ctx.interleaved, inplace=ctx.inplace, conjugate=True)
        return dx, None, None, None, None, None, None, None


def apply_rotary_emb(x, cos, sin, interleaved=False, inplace=False, seqlen_offsets: Union[int, torch.Tensor] = 0,
                     cu_seqlens: Optional[torch.Tensor] = None, max_seqlen: Optional[int] = None):
    """x (batch_size, seqlen, nheads, headdim), or (total_seqlen, nheads, headdim) with cu_seqlens;
    cos, sin (seqlen_rotary, rotary_dim / 2); rotates the first rotary_dim columns of x.
    interleaved: pairs (2i, 2i+1) (GPT-J style) instead of (i, i + rotary_dim/2) (GPT-NeoX style).
    seqlen_offsets: int or (batch_size,) tensor, position of the first token of each sequence."""
    return ApplyRotaryEmb.apply(x, cos, sin, interleaved, inplace, seqlen_offsets, cu_seqlens, max_seqlen)


apply_rotary_emb_func = apply_rotary_emb


def _save_offsets(ctx, tensors, seqlen_offsets):
    if isinstance(seqlen_offsets, torch.Tensor):
        ctx.save_for_backward(*tensors, seqlen_offsets)
        ctx.int_offset = None
    else:
        ctx.save_for_backward(*tensors)
        ctx.int_offset = seqlen_offsets


def _saved_offsets(ctx):
    saved = ctx.saved_tensors
    if ctx.int_offset is None:
        return saved[:-1], saved[-1]
    return saved, ctx.int_offset


def _rotate_q_and_k_(qkv, cos, sin, cos_k, sin_k, interleaved, seqlen_offsets, conjugate):
    """Rotate q = qkv[:, :, 0] and k = qkv[:, :, 1] in place.  With one table for both and a dense
    tensor, q and k heads are one run of 2 * nheads heads per token: one launch."""
    batch, seqlen, three, nheads, headdim = qkv.shape
    if cos_k is None and sin_k is None and qkv.is_contiguous():
        qk = qkv.view(batch, seqlen, 3 * nheads, headdim)[:, :, : 2 * nheads]
        apply_rotary(qk, cos, sin, seqlen_offsets=seqlen_offsets, interleaved=interleaved, inplace=True,
                     conjugate=conjugate)
        return
    apply_rotary(qkv[:, :, 0], cos, sin, seqlen_offsets=seqlen_offsets, interleaved=interleaved, inplace=True,
                 conjugate=conjugate)
    apply_rotary(qkv[:, :, 1], cos if cos_k is None else cos_k, sin if sin_k is None else sin_k,
                 seqlen_offsets=seqlen_offsets, interleaved=interleaved, inplace=True, conjugate=conjugate)


class ApplyRotaryEmbQKV_(torch.autograd.Function):
    @staticmethod
    def forward(ctx, qkv, cos, sin, cos_k=None, sin_k=None, interleaved=False,
                seqlen_offsets: Union[int, torch.Tensor] = 0):
        assert qkv.dim() == 5 and qkv.shape[2] == 3
        _rotate_q_and_k_(qkv, cos, sin, cos_k, sin_k, interleaved, seqlen_offsets, False)
        _save_offsets(ctx, (cos, sin, cos_k, sin_k), seqlen_offsets)
        ctx.interleaved = interleaved
        return qkv

    @staticmethod
    def backward(ctx, dqkv):
        (cos, sin, cos_k, sin_k), seqlen_offsets = _saved_offsets(ctx)
        _rotate_q_and_k_(dqkv, cos, sin, cos_k, sin_k, ctx.interleaved, seqlen_offsets, True)
        return dqkv, None, None, None, None, None, None


def apply_rotary_emb_qkv_(qkv, cos, sin, cos_k=None, sin_k=None, interleaved=False,
                          seqlen_offsets: Union[int, torch.Tensor] = 0):
    """qkv (batch_size, seqlen, 3, nheads, headdim); rotates q and k in place (k with cos_k / sin_k if
    given) and returns qkv."""
    return ApplyRotaryEmbQKV_.apply(qkv, cos, sin, cos_k, sin_k, interleaved, seqlen_offsets)


class ApplyRotaryEmbKV_(torch.autograd.Function):
    @staticmethod
    def forward(ctx, kv, cos, sin, interleaved=False, seqlen_offsets: Union[int, torch.Tensor] = 0):
        assert kv.dim() == 5 and kv.shape[2] == 2
        apply_rotary(kv[:, :, 0], cos, sin, seqlen_offsets=seqlen_offsets, interleaved=interleaved, inplace=True)
        _save_offsets(ctx, (cos, sin), seqlen_offsets)
        ctx.interleaved = interleaved
        return kv

    @staticmethod
    def backward(ctx, dkv):
        (cos, sin), seqlen_offsets = _saved_offsets(ctx)
        apply_rotary(dkv[:, :, 0], cos, sin, seqlen_offsets=seqlen_offsets, interleaved=ctx.interleaved,
                     inplace=True, conjugate=True)
        return dkv, None, None, None, None


def apply_rotary_emb_kv_(kv, cos, sin, interleaved=False, seqlen_offsets: Union[int, torch.Tensor] = 0):
    """kv (batch_size, seqlen, 2, nheads, headdim); rotates k in place and returns kv."""
    return ApplyRotaryEmbKV_.apply(kv, cos, sin, interleaved, seqlen_offsets)


class RotaryEmbedding(torch.nn.Module):
    """Rotary embedding layer with a lazily grown cos / sin table (RoFormer); with `scale_base` the
    XPos variant, which multiplies q's table by scale ** ((t - seqlen // 2) / scale_base) and divides
    k's by it.  Constructor arguments, buffers and forward contract follow the reference's module
    (flash_attn/layers/rotary.py:299-480)."""

    def __init__(self, dim: int, base=10000.0, interleaved=False, scale_base=None, pos_idx_in_fp32=True,
                 device=None):
        super().__init__()
        self.dim = dim
        self.base = float(base)
        self.interleaved = interleaved
        self.scale_base = scale_base
        self.pos_idx_in_fp32 = pos_idx_in_fp32
        self.register_buffer("inv_freq", self._compute_inv_freq(device), persistent=False)
        scale = None
        if scale_base is not None:
            scale = (torch.arange(0, dim, 2, device=device, dtype=torch.float32) + 0.4 * dim) / (1.4 * dim)
        self.register_buffer("scale", scale, persistent=False)
        self._seq_len_cached = 0
        self._cos_cached = self._sin_cached = None
        self._cos_k_cached = self._sin_k_cached = None

    def _compute_inv_freq(self, device=None):
        exponent = torch.arange(0, self.dim, 2, device=device, dtype=torch.float32) / self.dim
        return 1.0 / (self.base ** exponent)

    def _update_cos_sin_cache(self, seqlen, device=None, dtype=None):
        stale = (self._cos_cached is None or seqlen > self._seq_len_cached
                 or self._cos_cached.device != device or self._cos_cached.dtype != dtype
                 or (self.training and self._cos_cached.is_inference()))
        if not stale:
            return
        self._seq_len_cached = seqlen
        # positions and frequencies in fp32 unless the caller asks for the buffer's own dtype
        # (tables of models trained in pure bf16 before positions were computed in fp32)
        if self.pos_idx_in_fp32:
            t = torch.arange(seqlen, device=device, dtype=torch.float32)
            inv_freq = self.inv_freq if self.inv_freq.dtype == torch.float32 else self._compute_inv_freq(device)
        else:
            t = torch.arange(seqlen, device=device, dtype=self.inv_freq.dtype)
            inv_freq = self.inv_freq
        freqs = torch.outer(t, inv_freq)
        if self.scale is None:
            self._cos_cached = torch.cos(freqs).to(dtype)
            self._sin_cached = torch.sin(freqs).to(dtype)
            return
        power = (torch.arange(seqlen, dtype=self.scale.dtype, device=self.scale.device) - seqlen // 2) / self.scale_base
        scale = self.scale.to(device=power.device) ** power[:, None]
        self._cos_cached = (torch.cos(freqs) * scale).to(dtype)
        self._sin_cached = (torch.sin(freqs) * scale).to(dtype)
        self._cos_k_cached = (torch.cos(freqs) / scale).to(dtype)
        self._sin_k_cached = (torch.sin(freqs) / scale).to(dtype)

    def forward(self, qkv: torch.Tensor, kv: Optional[torch.Tensor] = None,
                seqlen_offset: Union[int, torch.Tensor] = 0, max_seqlen: Optional[int] = None):
        """qkv (batch, seqlen, 3, nheads, headdim) when kv is None, else q (batch, seqlen, nheads,
        headdim) with kv (batch, seqlen, 2, nheads_k, headdim).  Rotates in place; returns qkv, or
        (q, kv).  With a tensor seqlen_offset pass max_seqlen so the table covers every position."""
        seqlen = qkv.shape[1]
        if max_seqlen is not None:
            self._update_cos_sin_cache(max_seqlen, device=qkv.device, dtype=qkv.dtype)
        elif isinstance(seqlen_offset, int):
            self._update_cos_sin_cache(seqlen + seqlen_offset, device=qkv.device, dtype=qkv.dtype)
        if kv is None:
            return apply_rotary_emb_qkv_(qkv, self._cos_cached, self._sin_cached, self._cos_k_cached,
                                         self._sin_k_cached, interleaved=self.interleaved,
                                         seqlen_offsets=seqlen_offset)
        q = apply_rotary_emb_func(qkv, self._cos_cached, self._sin_cached, interleaved=self.interleaved,
                                  inplace=True, seqlen_offsets=seqlen_offset)
        cos_k = self._cos_cached if self.scale is None else self._cos_k_cached
        sin_k = self._sin_cached if self.scale is None else self._sin_k_cached
        kv = apply_rotary_emb_kv_(kv, cos_k, sin_k, interleaved=self.interleaved, seqlen_offsets=seqlen_offset)
        return q, kv
