"""Packing and unpacking of padded batches for the variable-length attention API.

Same functions, arguments and return values as the reference's flash_attn/bert_padding.py
(`unpad_input` :98-122, `pad_input` :197-209, `index_first_axis` :8-38, `index_put_first_axis`
:41-64): a padded batch (batch, seqlen, ...) with a 0/1 attention mask becomes the packed
(total_tokens, ...) layout plus the int32 `cu_seqlens` that `flash_attn_varlen_func` takes, and back.
These are gathers and scatters along the first axis; they run as ordinary torch index operations on
whatever device the tensors live on and are differentiable through autograd.
"""
import torch


def index_first_axis(x, indices):
    """x[indices] for x of shape (n, ...) and integer indices (m,): returns (m, ...)."""
    return x.index_select(0, indices.to(torch.long))


def index_put_first_axis(values, indices, first_axis_dim):
    """Zero tensor (first_axis_dim, ...) with rows `indices` set to `values` (m, ...)."""
    out = torch.zeros((first_axis_dim,) + tuple(values.shape[1:]), device=values.device, dtype=values.dtype)
    return out.index_copy(0, indices.to(torch.long), values)


def unpad_input(hidden_states, attention_mask):
    """hidden_states (batch, seqlen, ...); attention_mask (batch, seqlen) bool / int, non-zero = keep.

    Returns (packed (total_nnz, ...), indices (total_nnz,), cu_seqlens (batch + 1,) int32,
    max_seqlen_in_batch int)."""
    lens = attention_mask.sum(dim=-1, dtype=torch.int32)
    indices = torch.nonzero(attention_mask.flatten(), as_tuple=False).flatten()
    max_len = int(lens.max().item()) if lens.numel() else 0
    cu_seqlens = torch.zeros(lens.numel() + 1, dtype=torch.int32, device=lens.device)
    cu_seqlens[1:] = torch.cumsum(lens, dim=0, dtype=torch.int32)
    flat = hidden_states.reshape((-1,) + tuple(hidden_states.shape[2:]))
    return index_first_axis(flat, indices), indices, cu_seqlens, max_len


def pad_input(hidden_states, indices, batch, seqlen):
    """Inverse of unpad_input: (total_nnz, ...) -> (batch, seqlen, ...) with zeros at padding."""
    out = index_put_first_axis(hidden_states, indices, batch * seqlen)
    return out.reshape((batch, seqlen) + tuple(hidden_states.shape[1:]))
