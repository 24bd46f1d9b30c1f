"""Keep-mask builders that sit in front of the attention operator.

Same functions, argument meaning and error behaviour as the reference's
flash_sparse_attn/utils/mask.py (topk_indices :20-44, block_smooth :47-73, topk_mask :76-120,
relu_mask :123-160, create_mask :164-240).  They are thin host-side tensor programs: on a GPU
tensor they run as a handful of library kernels whose cost is O(rows * key_len), negligible next to
the attention they feed.
"""
from typing import Optional

import torch

__all__ = ["topk_indices", "block_smooth", "topk_mask", "relu_mask", "create_mask"]


def topk_indices(attention_bias: torch.Tensor, window_size: int, **kwargs) -> torch.Tensor:
    """Ascending positions of the `window_size` largest entries along the last dim (mask.py:20-44)."""
    picked = attention_bias.detach().topk(window_size, dim=-1, largest=True, sorted=False).indices
    return picked.sort(dim=-1).values


def block_smooth(attention_mask: torch.Tensor, key_len: int, block_size: int) -> torch.Tensor:
    """Majority vote inside aligned key blocks, in place (mask.py:47-73).

    A block of `block_size` keys becomes all-True when strictly more than half of its entries are
    True and all-False otherwise; a shorter tail block votes over its own length.
    """
    if block_size <= 0:
        raise ValueError(f"block_size must be a positive integer, got {block_size}.")
    if block_size == 1:
        return attention_mask
    n_full = key_len // block_size
    body_len = n_full * block_size
    if n_full:
        body = attention_mask[..., :body_len]
        votes = body.reshape(*body.shape[:-1], n_full, block_size).sum(dim=-1, dtype=torch.int64)
        body.copy_((2 * votes > block_size).repeat_interleave(block_size, dim=-1))
    if key_len > body_len:
        tail = attention_mask[..., body_len:]
        votes = tail.sum(dim=-1, keepdim=True, dtype=torch.int64)
        tail.copy_((2 * votes > tail.shape[-1]).expand_as(tail))
    return attention_mask


def _masked_bias(attention_bias: torch.Tensor, attention_mask: Optional[torch.Tensor], min_dtype: float):
    bias = attention_bias.detach()
    if attention_mask is not None:
        bias = bias.masked_fill(~attention_mask, min_dtype)
    return bias


def topk_mask(
    attention_bias: torch.Tensor,
    attention_mask: Optional[torch.Tensor],
    window_size: int,
    min_dtype: float,
    block_size: Optional[int] = None,
    **kwargs,
) -> torch.Tensor:
    """Keep the `window_size` largest bias entries of every row (mask.py:76-120).

    Entries already excluded by `attention_mask` are pushed to `min_dtype` first, and a selected
    entry whose value equals `min_dtype` is not kept, so a row with fewer than `window_size`
    admissible keys keeps only those.
    """
    bias = _masked_bias(attention_bias, attention_mask, min_dtype)
    values, indices = bias.topk(window_size, dim=-1, largest=True, sorted=False)
    keep = torch.zeros_like(bias, dtype=torch.bool).scatter_(-1, indices, values != min_dtype)
    if block_size is not None and block_size > 1:
        keep = block_smooth(keep, keep.shape[-1], block_size)
    return keep


def relu_mask(
    attention_bias: torch.Tensor,
    attention_mask: Optional[torch.Tensor],
    min_dtype: float,
    block_size: Optional[int] = None,
    **kwargs,
) -> torch.Tensor:
    """Keep the strictly positive bias entries (mask.py:123-160)."""
    keep = _masked_bias(attention_bias, attention_mask, min_dtype) > 0
    if block_size is not None and block_size > 1:
        keep = block_smooth(keep, keep.shape[-1], block_size)
    return keep


def create_mask(
    attention_bias: torch.Tensor,
    attention_mask: Optional[torch.Tensor],
    batch_size: int,
    query_len: int,
    key_len: int,
    window_size: int,
    min_dtype: float,
    block_size: Optional[int] = None,
    type: str = "topk",
) -> torch.Tensor:
    """Build the boolean keep-mask handed to flash_sparse_attn_func (mask.py:164-240).

    A 2-D `attention_mask` is a padding mask: (batch, key_len) is used as is; (batch, query_len) is
    taken to cover the last `query_len` keys, the `key_len - query_len` keys in front of it count as
    valid.  Any other 2-D width raises ValueError.  A 4-D mask must broadcast against the bias.
    """
    if attention_mask is not None and attention_mask.dim() == 2:
        width = attention_mask.shape[-1]
        if width == key_len:
            attention_mask = attention_mask.view(batch_size, 1, 1, key_len)
        elif width == query_len:
            attention_mask = attention_mask.view(batch_size, 1, 1, query_len)
            if key_len > query_len:
                front = attention_mask.new_ones((batch_size, 1, 1, key_len - query_len), dtype=torch.bool)
                attention_mask = torch.cat([front, attention_mask], dim=-1)
        else:
            raise ValueError(
                f"attention_mask shape {attention_mask.shape} is not compatible with key_len {key_len} or query_len {query_len}."
            )
    if type == "topk":
        return topk_mask(attention_bias, attention_mask, window_size=window_size, min_dtype=min_dtype, block_size=block_size)
    if type == "relu":
        return relu_mask(attention_bias, attention_mask, min_dtype=min_dtype, block_size=block_size, window_size=window_size)
    raise ValueError(f"Unsupported mask type: {type}. Supported types are 'topk' and 'relu'.")
