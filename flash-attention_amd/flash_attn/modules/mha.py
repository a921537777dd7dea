"""Self-attention layer with a KV cache: the caller of `flash_attn_with_kvcache` during generation.

Covers the flash-attention wrappers `FlashSelfAttention` (:36-94) and `FlashCrossAttention` (:97-174)
and the decoding glue of the reference's flash_attn/modules/mha.py: `_update_kv_cache` (:296-322),
`MHA.allocate_inference_cache` (:422-434), `MHA._apply_rotary_update_kvcache_attention` (:442-479),
`MHA._update_kvcache_attention` (:481-507) and the self-attention branches of `MHA.forward`
(:515-653): packed QKV projection, rotary, MHA / GQA / MQA, causal mask, attention dropout, packed
variable-length input.  Not carried over (the reference's options outside the attention path):
the cross-attention projections, depthwise convolution, fused dense layers, the non-flash attention
fallbacks, activation checkpointing and the tensor-parallel variant.
"""
import math

import torch
import torch.nn as nn

from flash_attn import (flash_attn_kvpacked_func, flash_attn_qkvpacked_func, flash_attn_varlen_kvpacked_func,
                        flash_attn_varlen_qkvpacked_func, flash_attn_with_kvcache)
from flash_attn.layers.rotary import RotaryEmbedding


class FlashSelfAttention(nn.Module):
    """Softmax attention over a packed qkv tensor.  qkv (B, S, 3, H, D), or (total, 3, H, D) with
    cu_seqlens (int32, batch + 1) and max_seqlen; dropout applies in training mode only."""

    def __init__(self, causal=False, softmax_scale=None, attention_dropout=0.0, window_size=(-1, -1)):
        super().__init__()
        self.causal = causal
        self.softmax_scale = softmax_scale
        self.window_size = window_size
        self.drop = nn.Dropout(attention_dropout)

    def forward(self, qkv, causal=None, cu_seqlens=None, max_seqlen=None):
        assert qkv.dtype in [torch.float16, torch.bfloat16]
        assert qkv.is_cuda
        causal = self.causal if causal is None else causal
        p = self.drop.p if self.training else 0.0
        if cu_seqlens is not None:
            assert cu_seqlens.dtype == torch.int32
            assert isinstance(max_seqlen, int)
            return flash_attn_varlen_qkvpacked_func(qkv, cu_seqlens, max_seqlen, p, softmax_scale=self.softmax_scale,
                                                    causal=causal, window_size=self.window_size)
        return flash_attn_qkvpacked_func(qkv, p, softmax_scale=self.softmax_scale, causal=causal,
                                         window_size=self.window_size)


class FlashCrossAttention(nn.Module):
    """Softmax attention of q (B, Sq, H, D) over kv (B, Sk, 2, H_k, D), or the packed forms
    (total_q, H, D) / (total_k, 2, H_k, D) with cu_seqlens / max_seqlen for q and for k."""

    def __init__(self, causal=False, softmax_scale=None, attention_dropout=0.0, window_size=(-1, -1)):
        super().__init__()
        self.causal = causal
        self.softmax_scale = softmax_scale
        self.window_size = window_size
        self.drop = nn.Dropout(attention_dropout)

    def forward(self, q, kv, causal=None, cu_seqlens=None, max_seqlen=None, cu_seqlens_k=None, max_seqlen_k=None):
        assert q.dtype in [torch.float16, torch.bfloat16]
        assert q.is_cuda and kv.is_cuda
        causal = self.causal if causal is None else causal
        p = self.drop.p if self.training else 0.0
        if cu_seqlens is not None:
            assert cu_seqlens.dtype == torch.int32 and isinstance(max_seqlen, int)
            assert cu_seqlens_k is not None and cu_seqlens_k.dtype == torch.int32 and isinstance(max_seqlen_k, int)
            return flash_attn_varlen_kvpacked_func(q, kv, cu_seqlens, cu_seqlens_k, max_seqlen, max_seqlen_k, p,
                                                   softmax_scale=self.softmax_scale, causal=causal,
                                                   window_size=self.window_size)
        assert kv.shape[0] == q.shape[0] and kv.shape[4] == q.shape[3]
        return flash_attn_kvpacked_func(q, kv, p, softmax_scale=self.softmax_scale, causal=causal,
                                        window_size=self.window_size)


def _update_kv_cache(kv, inference_params, layer_idx):
    """Write kv (batch, seqlen, 2, nheads_kv, head_dim) at [batch_size_offset, seqlen_offset) of the
    layer's cache (allocated on first use) and return the filled part (batch, seqlen_offset + seqlen, ...)."""
    num_heads, head_dim = kv.shape[-2:]
    if layer_idx not in inference_params.key_value_memory_dict:
        inference_params.key_value_memory_dict[layer_idx] = torch.empty(
            inference_params.max_batch_size, inference_params.max_seqlen, 2, num_heads, head_dim,
            dtype=kv.dtype, device=kv.device)
    kv_cache = inference_params.key_value_memory_dict[layer_idx]
    b0 = inference_params.batch_size_offset
    b1 = b0 + kv.shape[0]
    s0 = inference_params.seqlen_offset
    s1 = s0 + kv.shape[1]
    assert b1 <= kv_cache.shape[0]
    assert s1 <= kv_cache.shape[1]
    kv_cache[b0:b1, s0:s1, ...] = kv
    return kv_cache[b0:b1, :s1, ...]


class MHA(nn.Module):
    """Multi-head self-attention on the flash attention kernels, with the reference's constructor
    arguments for the options that are supported."""

    def __init__(self, embed_dim, num_heads, num_heads_kv=None, qkv_proj_bias=True, out_proj_bias=True, dropout=0.0,
                 softmax_scale=None, causal=False, layer_idx=None, rotary_emb_dim=0, rotary_emb_base=10000.0,
                 rotary_emb_scale_base=None, rotary_emb_interleaved=False, window_size=(-1, -1), device=None,
                 dtype=None):
        factory_kwargs = {"device": device, "dtype": dtype}
        super().__init__()
        self.embed_dim = embed_dim
        self.causal = causal
        self.layer_idx = layer_idx
        self.rotary_emb_dim = rotary_emb_dim
        self.softmax_scale = softmax_scale
        self.window_size = window_size
        self.use_flash_attn = True
        self.num_heads = num_heads
        self.num_heads_kv = num_heads_kv if num_heads_kv is not None else num_heads
        assert self.num_heads % self.num_heads_kv == 0, "num_heads must be divisible by num_heads_kv"
        assert self.embed_dim % num_heads == 0, "embed_dim must be divisible by num_heads"
        self.head_dim = self.embed_dim // num_heads
        qkv_dim = self.head_dim * (self.num_heads + 2 * self.num_heads_kv)
        if self.rotary_emb_dim > 0:
            if self.rotary_emb_dim % 2 != 0 or self.rotary_emb_dim > self.head_dim:
                raise ValueError("rotary_emb_dim must be even and at most head_dim (got %d for head_dim %d)"
                                 % (self.rotary_emb_dim, self.head_dim))
            self.rotary_emb = RotaryEmbedding(self.rotary_emb_dim, base=rotary_emb_base, scale_base=rotary_emb_scale_base,
                                              interleaved=rotary_emb_interleaved, device=device)
        self.inner_attn = FlashSelfAttention(causal=causal, softmax_scale=softmax_scale, attention_dropout=dropout,
                                             window_size=window_size)
        self.inner_cross_attn = FlashCrossAttention(causal=causal, softmax_scale=softmax_scale,
                                                    attention_dropout=dropout, window_size=window_size)
        self.Wqkv = nn.Linear(embed_dim, qkv_dim, bias=qkv_proj_bias, **factory_kwargs)
        self.out_proj = nn.Linear(embed_dim, embed_dim, bias=out_proj_bias, **factory_kwargs)

    def allocate_inference_cache(self, batch_size, max_seqlen, dtype=None):
        dtype = self.out_proj.weight.dtype if dtype is None else dtype
        return torch.empty(batch_size, max_seqlen, 2, self.num_heads_kv, self.head_dim, dtype=dtype,
                           device=self.out_proj.weight.device)

    def _rotate_packed(self, x, cu_seqlens, max_seqlen):
        """Rotary on packed heads x (total, heads, head_dim), every sequence starting at position 0.
        Returns the rotated tensor.  When gradients are recorded the rotation is out of place and the
        caller must go on with the RETURNED tensor: it carries the backward (the conjugate rotation),
        which an in-place write into a view of the projection's output would bypass.  Without
        gradients x is rotated in place and returned."""
        from flash_attn.layers.rotary import apply_rotary_emb
        assert self.rotary_emb.scale is None, "packed input does not support xPos"
        self.rotary_emb._update_cos_sin_cache(max_seqlen, device=x.device, dtype=x.dtype)
        inplace = not (torch.is_grad_enabled() and x.requires_grad)
        return apply_rotary_emb(x, self.rotary_emb._cos_cached, self.rotary_emb._sin_cached,
                                interleaved=self.rotary_emb.interleaved, inplace=inplace, cu_seqlens=cu_seqlens,
                                max_seqlen=max_seqlen)

    def _update_kv_cache(self, kv, inference_params):
        assert self.layer_idx is not None, "Generation requires layer_idx in the constructor"
        return _update_kv_cache(kv, inference_params, self.layer_idx)

    def _cache_and_lengths(self, batch, inference_params):
        kv_cache = inference_params.key_value_memory_dict[self.layer_idx][:batch]
        lengths = inference_params.lengths_per_sample
        return kv_cache, (lengths[:batch] if lengths is not None else inference_params.seqlen_offset)

    def _apply_rotary_update_kvcache_attention(self, q, kv, inference_params):
        """One kernel sequence for: rotate q and the new k at each sequence's current length, append
        the new k / v to the cache, attend to the cache.  q (batch, seqlen_q, nheads, head_dim),
        kv (batch, seqlen_new, 2, nheads_kv, head_dim)."""
        assert inference_params is not None and inference_params.seqlen_offset > 0
        rotary_cos = rotary_sin = None
        if self.rotary_emb_dim > 0:
            assert self.rotary_emb.scale is None, "This code path does not support xPos"
            self.rotary_emb._update_cos_sin_cache(inference_params.max_seqlen, device=q.device, dtype=q.dtype)
            rotary_cos, rotary_sin = self.rotary_emb._cos_cached, self.rotary_emb._sin_cached
        kv_cache, cache_seqlens = self._cache_and_lengths(q.shape[0], inference_params)
        return flash_attn_with_kvcache(
            q, kv_cache[:, :, 0], kv_cache[:, :, 1], kv[:, :, 0], kv[:, :, 1], rotary_cos=rotary_cos,
            rotary_sin=rotary_sin, cache_seqlens=cache_seqlens, softmax_scale=self.softmax_scale, causal=self.causal,
            window_size=self.window_size,
            rotary_interleaved=self.rotary_emb.interleaved if self.rotary_emb_dim > 0 else False)

    def _update_kvcache_attention(self, q, kv, inference_params):
        """q and kv already rotated (or no rotary).  The prompt pass (nothing cached yet) writes the
        cache and attends within the prompt; later steps append and attend to the cache."""
        if inference_params.seqlen_offset == 0:
            kv = self._update_kv_cache(kv, inference_params)
            return self.inner_cross_attn(q, kv)
        kv_cache, cache_seqlens = self._cache_and_lengths(q.shape[0], inference_params)
        return flash_attn_with_kvcache(q, kv_cache[:, :, 0], kv_cache[:, :, 1], kv[:, :, 0], kv[:, :, 1],
                                       cache_seqlens=cache_seqlens, softmax_scale=self.softmax_scale, causal=self.causal,
                                       window_size=self.window_size)

    def forward(self, x, cu_seqlens=None, max_seqlen=None, inference_params=None):
        """x (batch, seqlen, embed_dim) -> (batch, seqlen, embed_dim); or packed (total, embed_dim) with
        cu_seqlens / max_seqlen (not together with inference_params)."""
        if cu_seqlens is not None:
            assert max_seqlen is not None and inference_params is None and x.dim() == 2
            total = x.shape[0]
            qkv = self.Wqkv(x)
            kw = dict(cu_seqlens=cu_seqlens, max_seqlen=max_seqlen)
            if self.num_heads_kv == self.num_heads:
                qkv = qkv.view(total, 3, self.num_heads, self.head_dim)
                if self.rotary_emb_dim > 0:
                    # q and k heads of a token are one run of 2 h heads: one launch rotates both
                    qk = self._rotate_packed(qkv.view(total, 3 * self.num_heads, self.head_dim)[:, : 2 * self.num_heads],
                                             cu_seqlens, max_seqlen)
                    if qk.data_ptr() != qkv.data_ptr():      # rotated out of place: rebuild the packed tensor
                        qkv = torch.cat([qk.view(total, 2, self.num_heads, self.head_dim), qkv[:, 2:]], dim=1)
                context = self.inner_attn(qkv, **kw)
            else:
                nq = self.num_heads * self.head_dim
                q = qkv[..., :nq].reshape(total, self.num_heads, self.head_dim)
                kv = qkv[..., nq:].reshape(total, 2, self.num_heads_kv, self.head_dim)
                if self.rotary_emb_dim > 0:
                    q = self._rotate_packed(q, cu_seqlens, max_seqlen)
                    k = self._rotate_packed(kv[:, 0], cu_seqlens, max_seqlen)
                    if k.data_ptr() != kv.data_ptr():
                        kv = torch.stack([k, kv[:, 1]], dim=1)
                context = self.inner_cross_attn(q, kv, cu_seqlens_k=cu_seqlens, max_seqlen_k=max_seqlen, **kw)
            return self.out_proj(context.reshape(total, self.embed_dim))
        if inference_params is None:
            seqlen_offset, rotary_max_seqlen = 0, None
        else:
            lengths = inference_params.lengths_per_sample
            seqlen_offset = lengths if lengths is not None else inference_params.seqlen_offset
            rotary_max_seqlen = inference_params.max_seqlen
        batch, seqlen = x.shape[:2]
        qkv = self.Wqkv(x)
        # The fused rotary + append path needs something cached, and a rotary dimension the KV-cache call rotates
        # (multiples of 16, as in the reference, csrc/flash_attn/flash_api.cpp:1212); other rotary dimensions are
        # rotated by the stand-alone op at each sequence's length and appended by the same call without tables.
        fused = (inference_params is not None and inference_params.seqlen_offset > 0 and self.rotary_emb_dim > 0
                 and self.rotary_emb_dim % 16 == 0)
        if self.num_heads_kv == self.num_heads:
            qkv = qkv.view(batch, seqlen, 3, self.num_heads, self.head_dim)
            if fused:
                context = self._apply_rotary_update_kvcache_attention(qkv[:, :, 0], qkv[:, :, 1:], inference_params)
            else:
                if self.rotary_emb_dim > 0:
                    qkv = self.rotary_emb(qkv, seqlen_offset=seqlen_offset, max_seqlen=rotary_max_seqlen)
                if inference_params is None:
                    context = self.inner_attn(qkv)
                else:
                    context = self._update_kvcache_attention(qkv[:, :, 0], qkv[:, :, 1:], inference_params)
        else:
            nq = self.num_heads * self.head_dim
            q = qkv[..., :nq].reshape(batch, seqlen, self.num_heads, self.head_dim)
            kv = qkv[..., nq:].reshape(batch, seqlen, 2, self.num_heads_kv, self.head_dim)
            if fused:
                context = self._apply_rotary_update_kvcache_attention(q, kv, inference_params)
            else:
                if self.rotary_emb_dim > 0:
                    q, kv = self.rotary_emb(q, kv, seqlen_offset=seqlen_offset, max_seqlen=rotary_max_seqlen)
                if inference_params is None:
                    context = self.inner_cross_attn(q, kv)
                else:
                    context = self._update_kvcache_attention(q, kv, inference_params)
        return self.out_proj(context.reshape(batch, seqlen, self.embed_dim))
