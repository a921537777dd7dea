"""Packing and unpacking of padded batches for the variable-length attention API.

Same functions, arguments and return values as the reference's flash_attn/bert_padding.py
(`unpad_input` :98-122, `unpad_input_for_concatenated_sequences` :125-194, `pad_input` :197-209,
`index_first_axis` :8-38, `index_put_first_axis` :41-64, `index_first_axis_residual` :67-95): a padded batch
(batch, seqlen, ...) with a 0/1 attention mask becomes the packed (total_tokens, ...) layout plus the int32 `cu_seqlens` that `flash_attn_varlen_func` takes, and back.
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


def index_first_axis_residual(x, indices):
    """(x[indices], x): the gathered rows together with the input itself, for layers that go on with a subset of
    the tokens and still add the full residual stream.  Differentiable through autograd: the gradient of x is the
    gradient of the second result plus the rows' gradients scattered back (what the reference's
    IndexFirstAxisResidual writes by hand, flash_attn/bert_padding.py:67-95)."""
    return x.index_select(0, indices.to(torch.long)), x


def _cu_seqlens(lens):
    cu = torch.zeros(lens.numel() + 1, dtype=torch.int32, device=lens.device)
    cu[1:] = torch.cumsum(lens, dim=0, dtype=torch.int32)
    return cu


def unpad_input_for_concatenated_sequences(hidden_states, attention_mask_in_length):
    """Rows of a padded batch that each hold SEVERAL short sequences one after the other.
    attention_mask_in_length (batch, seqlen) int: the non-zero entries of row b are the lengths of the sequences
    in row b of hidden_states, in order (their sum is the number of real tokens of the row; zeros fill the rest).
    Row [2, 3, 0, 0, 0, 0] means tokens 0-1 are one sequence and tokens 2-4 another, token 5 is padding
    (the reference's example, flash_attn/bert_padding.py:131-170).

    Returns (packed (total_nnz, ...), indices (total_nnz,), cu_seqlens (number of sequences + 1,) int32,
    max_seqlen_in_batch int), like unpad_input but with one cu_seqlens entry per short sequence."""
    batch, seqlen = attention_mask_in_length.shape
    tokens_per_row = attention_mask_in_length.sum(dim=-1)
    real = torch.arange(seqlen, device=tokens_per_row.device, dtype=tokens_per_row.dtype).expand(batch, seqlen) < tokens_per_row.unsqueeze(1)
    indices = torch.nonzero(real.flatten(), as_tuple=False).flatten()
    lens = attention_mask_in_length.flatten()
    lens = lens[torch.nonzero(lens, as_tuple=False).flatten()].to(torch.int32)       # sequence lengths, row by row
    max_len = int(lens.max().item()) if lens.numel() else 0
    flat = hidden_states.reshape((-1,) + tuple(hidden_states.shape[2:]))
    return index_first_axis(flat, indices), indices, _cu_seqlens(lens), max_len


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
