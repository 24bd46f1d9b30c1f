"""Padding bookkeeping for batches of ragged sequences stored as padded (batch, seqlen, ...) tensors.

Same functions and return conventions as the reference's flash_sparse_attn/utils/padding.py
(index_first_axis :7-15, unpad_input :18-46, pad_input :49-64, get_unpad_data :67-92, upad_input :95-167),
which the Hugging Face integration imports next to the attention operator.  They are index arithmetic on
the host side of the operator (a handful of library kernels) and never touch the attention kernels.
"""
import torch
import torch.nn.functional as F

__all__ = ["index_first_axis", "unpad_input", "pad_input", "get_unpad_data", "upad_input"]


def index_first_axis(tensor, indices):
    """Rows `indices` of `tensor` with its first two dims (batch, seqlen) merged (padding.py:7-15)."""
    return tensor.reshape(-1, *tensor.shape[2:])[indices]


def _token_index(valid):
    """(flat positions of the selected tokens, tokens per sequence as int32, cumulative lengths with a leading 0)."""
    per_seq = valid.sum(dim=-1, dtype=torch.int32)
    flat = torch.nonzero(valid.flatten(), as_tuple=False).flatten()
    cu = F.pad(torch.cumsum(per_seq, dim=0, dtype=torch.int32), (1, 0))
    return flat, per_seq, cu


def unpad_input(hidden_states, attention_mask, unused_mask=None):
    """Drop the padding of (batch, seqlen, ...) `hidden_states` (padding.py:18-46).

    `attention_mask` (batch, seqlen) marks valid tokens, `unused_mask` tokens that are allocated but unused;
    both kinds are kept.  Returns (tokens (total, ...), flat indices, cu_seqlens int32 (batch + 1),
    longest kept length as a Python int, valid tokens per sequence int32).
    """
    kept = attention_mask if unused_mask is None else attention_mask + unused_mask
    flat, per_seq, cu = _token_index(kept)
    used = attention_mask.sum(dim=-1, dtype=torch.int32)
    return index_first_axis(hidden_states, flat), flat, cu, per_seq.max().item(), used


def pad_input(hidden_states, indices, batch, seqlen):
    """Scatter (total, ...) tokens back to a zero-filled (batch, seqlen, ...) tensor (padding.py:49-64)."""
    tail = hidden_states.shape[1:]
    out = torch.zeros((batch * seqlen, *tail), device=hidden_states.device, dtype=hidden_states.dtype)
    out[indices] = hidden_states
    return out.view(batch, seqlen, *tail)


def get_unpad_data(attention_mask):
    """(flat indices of valid tokens, cu_seqlens int32 (batch + 1), longest length as int) (padding.py:67-92)."""
    flat, per_seq, cu = _token_index(attention_mask)
    return flat, cu, per_seq.max().item()


def upad_input(query_layer, key_layer, value_layer, attention_mask, query_length, unpad_input_func):
    """Unpad q, k, v with one pass over the padding mask (padding.py:95-167).

    Keys / values longer than the mask (static caches) are cut to the mask's length first.  The query is
    unpadded with the key indices when it has the key length, kept whole for single-token decoding
    (one token per sequence), and otherwise unpadded with the last `query_length` mask columns (left padding).
    Returns (q, k, v, indices_q, (cu_seqlens_q, cu_seqlens_k), (max_seqlen_q, max_seqlen_k)).
    """
    indices_k, cu_k, max_k = get_unpad_data(attention_mask)
    mask_len = attention_mask.shape[-1]
    if key_layer.shape[1] > mask_len:
        key_layer, value_layer = key_layer[:, :mask_len], value_layer[:, :mask_len]
    batch, kv_len = key_layer.shape[:2]
    key_layer = index_first_axis(key_layer, indices_k)
    value_layer = index_first_axis(value_layer, indices_k)
    if query_length == kv_len:
        query_layer = index_first_axis(query_layer, indices_k)
        indices_q, cu_q, max_q = indices_k, cu_k, max_k
    elif query_length == 1:
        max_q = 1
        cu_q = torch.arange(batch + 1, dtype=torch.int32, device=query_layer.device)
        indices_q = cu_q[:-1]
        query_layer = query_layer.squeeze(1)
    else:
        query_layer, indices_q, cu_q, max_q, *_ = unpad_input_func(query_layer, attention_mask[:, -query_length:])
    return query_layer, key_layer, value_layer, indices_q, (cu_q, cu_k), (max_q, max_k)
