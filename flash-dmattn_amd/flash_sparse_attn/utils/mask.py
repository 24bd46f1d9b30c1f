"""Keep-mask builders that sit in front of the attention operator.

Same functions, argument meaning and error behaviour as the reference's
flash_sparse_attn/utils/mask.py (topk_indices :20-44, block_smooth :47-73, topk_mask :76-120,
relu_mask :123-160, create_mask :164-240).

For a 4-D fp16 / bf16 bias on the GPU, `topk_mask` and `relu_mask` (and so `create_mask`) run as ONE kernel of
libfdma_hip.so (`fdma_create_mask`: masked fill, radix select of the window largest values per row, exclusion of
the fill value, block smoothing) instead of masked_fill + topk + zeros + scatter (+ view / sum / copy) through
the tensor library -- on the benchmark shapes that chain costs as much as the attention it feeds.  Among entries
equal to the smallest selected value the lowest columns are kept; the reference leaves that choice to
`torch.topk`, which does not define it.  Every other input (CPU tensors, fp32, other ranks) takes the same tensor
program as the reference.
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


def _native_mask(attention_bias, attention_mask, window_size, min_dtype, block_size, kind) -> Optional[torch.Tensor]:
    """Device path; None when the inputs are not of the form the kernel takes."""
    if not (attention_bias.is_cuda and attention_bias.dim() == 4 and attention_bias.dtype in (torch.bfloat16, torch.float16)):
        return None
    if attention_mask is not None and not (attention_mask.dim() == 4 and attention_mask.dtype == torch.bool
                                           and attention_mask.device == attention_bias.device):
        return None
    from .. import _cabi

    bias = attention_bias.detach()
    shape = tuple(bias.shape) if attention_mask is None else tuple(torch.broadcast_shapes(bias.shape, attention_mask.shape))
    if kind == "topk" and window_size > shape[-1]:
        return None  # torch.topk raises for k beyond the row length; let it
    bias = bias.expand(shape)
    if shape[-1] > 1 and bias.stride(-1) != 1:
        bias = bias.contiguous()
    mask_in = None
    if attention_mask is not None:
        mask_in = attention_mask.expand(shape)
        if shape[-1] > 1 and mask_in.stride(-1) != 1:
            mask_in = mask_in.contiguous()
    out = torch.empty(shape, dtype=torch.bool, device=bias.device)
    if out.numel() == 0:
        return out
    a = _cabi.MaskArgs()
    a.bias, a.mask_out = bias.data_ptr(), out.data_ptr()
    a.mask_in = mask_in.data_ptr() if mask_in is not None else None
    a.bias_strides[:] = bias.stride()[:3]
    a.mask_in_strides[:] = mask_in.stride()[:3] if mask_in is not None else (0, 0, 0)
    a.mask_out_strides[:] = out.stride()[:3]
    a.batch, a.heads, a.rows, a.seqlen_k = shape
    a.window = int(window_size) if kind == "topk" else 0
    a.block_size = int(block_size) if block_size is not None and block_size > 1 else 0  # mask.py:112, 152
    a.type = 0 if kind == "topk" else 1
    a.dtype = _cabi.dtype_code(bias)
    a.min_value = float(min_dtype)
    # A mask that is broadcast over the queries drops whole key columns, and the attention kernels work on the list of
    # the kept ones: the kernel writes that list too, and it travels with the mask tensor (see kept_keys_of).
    kept = None
    if shape[2] == 1:
        ld = (shape[3] + 15) // 16 * 16
        rows = shape[0] * shape[1]
        kept = (torch.empty((rows, ld), dtype=torch.int32, device=bias.device),
                torch.empty((rows, ld), dtype=torch.int32, device=bias.device),
                torch.empty((rows,), dtype=torch.int32, device=bias.device), ld)
        a.kept_idx, a.kept_cnt, a.kept_count, a.kept_ld = kept[0].data_ptr(), kept[1].data_ptr(), kept[2].data_ptr(), ld
    # A mask that varies per query row is what the per-query attention kernels spend most of their memory traffic on
    # (a byte per score): the kernel also writes it packed to one bit per key, and the attention calls read that
    # instead (see mask_bits_of).
    bits = None
    if shape[2] > 1:
        row_bytes = ((shape[3] + 7) // 8 + 15) // 16 * 16
        bits = torch.empty(shape[:3] + (row_bytes,), dtype=torch.uint8, device=bias.device)
        a.bits, a.bits_row_bytes = bits.data_ptr(), row_bytes
    with _cabi.device_guard(bias.device):
        _cabi.check(_cabi.lib.fdma_create_mask(a, _cabi.current_stream(bias.device)))
    if kept is not None:
        out._fdma_kept = kept + (out._version, out.data_ptr(), tuple(out.shape))
    if bits is not None:
        out._fdma_bits = (bits, out._version, out.data_ptr(), tuple(out.shape))
    return out


def kept_keys_of(mask: Optional[torch.Tensor]):
    """(idx, cnt, count, ld) written by the device mask builder for THIS mask tensor, or None: when the tensor did not
    come from it, is not broadcast over the queries, or has been written to since."""
    kept = getattr(mask, "_fdma_kept", None)
    if kept is None:
        return None
    idx, cnt, count, ld, version, ptr, shape = kept
    if mask._version != version or mask.data_ptr() != ptr or tuple(mask.shape) != shape:
        return None
    return idx, cnt, count, ld


def mask_bits_of(mask: Optional[torch.Tensor]):
    """The uint8 tensor of bits (shape of the mask but for the last dimension; key j of a row in bit j % 8 of byte
    j // 8) written by the device mask builder for THIS mask tensor, or None: when the tensor did not come from it,
    is broadcast over the queries, or has been written to since."""
    rec = getattr(mask, "_fdma_bits", None)
    if rec is None:
        return None
    bits, version, ptr, shape = rec
    if mask._version != version or mask.data_ptr() != ptr or tuple(mask.shape) != shape:
        return None
    return bits


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
    keep = _native_mask(attention_bias, attention_mask, window_size, min_dtype, block_size, "topk")
    if keep is not None:
        return keep
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
    keep = _native_mask(attention_bias, attention_mask, 0, min_dtype, block_size, "relu")
    if keep is not None:
        return keep
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
