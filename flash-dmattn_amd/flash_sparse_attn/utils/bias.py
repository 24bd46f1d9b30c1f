"""Producer of the dynamic-mask attention bias.

`dynamic_mask_bias(value_states, dt_proj_weight, A, dt_proj_bias)` is the `A * softplus(dt_proj(V))` that the reference's
Doge caller computes in front of every attention call (examples/modeling/modeling_doge.py:217-222 of the reference: a
linear layer over the value states of all kv heads of a token, a softplus, a multiply by the per-head parameter A, a
transpose to [batch, kv heads, 1, keys] and a cast), with autograd.  The reference package itself ships no such helper:
callers that keep their own tensor program lose nothing, callers that switch get one kernel forwards (one read of V)
and two backwards instead of the chain of library kernels, and the attention's dBias -- returned in the bias's own
[batch, kv heads, 1, keys] shape -- is consumed directly.

For fp16 / bf16 tensors on the GPU the work runs in libfdma_hip.so (`fdma_dyn_bias_fwd` / `fdma_dyn_bias_bwd`; a shape
the kernels were not built for raises RuntimeError); CPU and fp32 tensors run the same tensor program as the
reference's caller.
"""
from typing import Optional

import torch
import torch.nn.functional as F

__all__ = ["dynamic_mask_bias"]


def _tensor_program(value_states, weight, a, proj_bias):
    b, l = value_states.shape[:2]
    dt = F.linear(value_states.reshape(b, l, -1), weight, proj_bias)
    return (a * F.softplus(dt)).transpose(-1, -2).unsqueeze(-2).to(value_states.dtype)


def _native_ok(value_states, weight, a, proj_bias) -> bool:
    """True when the kernels take the call.  16-bit tensors on the GPU are the kernels' business: a shape they were not
    built for is an error, not a reason to fall back quietly; CPU and fp32 tensors run the caller's tensor program."""
    if not (value_states.is_cuda and value_states.dtype in (torch.bfloat16, torch.float16)):
        return False
    if value_states.dim() != 4:
        raise RuntimeError("value_states must have shape (batch, key_len, num_kv_heads, head_dim)")
    b, l, hk, d = value_states.shape
    others = [weight, a] + ([proj_bias] if proj_bias is not None else [])
    if any(t.dtype != value_states.dtype or t.device != value_states.device for t in others):
        raise RuntimeError("dt_proj_weight, A and dt_proj_bias must have the dtype and device of value_states")
    if tuple(weight.shape) != (hk, hk * d) or a.numel() != hk or (proj_bias is not None and proj_bias.numel() != hk):
        raise RuntimeError("dt_proj_weight must be (num_kv_heads, num_kv_heads * head_dim), A and dt_proj_bias (num_kv_heads)")
    if hk > 32 or d % 8 != 0 or (hk * d) % 16 != 0:
        raise RuntimeError("the bias producer is built for up to 32 kv heads, head_dim % 8 == 0 and "
                           "(num_kv_heads * head_dim) % 16 == 0")
    return True


class _DynamicMaskBias(torch.autograd.Function):
    @staticmethod
    def forward(ctx, value_states, weight, a, proj_bias):
        from .. import _cabi

        b, l, hk, d = value_states.shape
        v = value_states if value_states.stride(-1) == 1 and all(s % 8 == 0 for s in value_states.stride()[:3]) \
            and value_states.data_ptr() % 16 == 0 else value_states.contiguous()
        w, av = weight.contiguous(), a.contiguous()
        pb = proj_bias.contiguous() if proj_bias is not None else None
        lpad = (l + 7) // 8 * 8  # rows of the bias are handed to the attention kernels' 16-byte loads
        bias_store = torch.empty((b, hk, 1, lpad), dtype=v.dtype, device=v.device)
        if lpad != l:
            bias_store[..., l:].zero_()
        dt = torch.empty((b * l, hk), dtype=torch.float32, device=v.device)
        args = _cabi.DynBiasArgs()
        args.value, args.weight, args.a = v.data_ptr(), w.data_ptr(), av.data_ptr()
        args.proj_bias = pb.data_ptr() if pb is not None else None
        args.bias, args.dt = bias_store.data_ptr(), dt.data_ptr()
        args.value_strides[:] = v.stride()[:3]
        args.bias_strides[:] = (bias_store.stride(0), bias_store.stride(1))
        args.batch, args.seqlen_k, args.num_heads_k, args.head_dim = b, l, hk, d
        args.dtype = _cabi.dtype_code(v)
        with _cabi.device_guard(v.device):
            _cabi.check(_cabi.lib.fdma_dyn_bias_fwd(args, _cabi.current_stream(v.device)))
        ctx.save_for_backward(v, w, av, pb if pb is not None else torch.empty(0, device=v.device), dt)
        ctx.has_pb = pb is not None
        return bias_store[..., :l]

    @staticmethod
    def backward(ctx, dbias):
        from .. import _cabi

        v, w, av, pb, dt = ctx.saved_tensors
        b, l, hk, d = v.shape
        g = dbias if dbias.stride(-1) == 1 else dbias.contiguous()
        dv = torch.empty((b, l, hk, d), dtype=v.dtype, device=v.device)
        dw, da = torch.empty_like(w), torch.empty_like(av)
        dpb = torch.empty_like(pb) if ctx.has_pb else None
        args = _cabi.DynBiasArgs()
        args.value, args.weight, args.a = v.data_ptr(), w.data_ptr(), av.data_ptr()
        args.proj_bias = pb.data_ptr() if ctx.has_pb else None
        args.dt = dt.data_ptr()
        args.bias = dt.data_ptr()  # unused by backward; any device pointer
        args.value_strides[:] = v.stride()[:3]
        args.batch, args.seqlen_k, args.num_heads_k, args.head_dim = b, l, hk, d
        args.dtype = _cabi.dtype_code(v)
        args.dbias = g.data_ptr()
        args.dbias_strides[:] = (g.stride(0), g.stride(1))
        args.dvalue = dv.data_ptr()
        args.dvalue_strides[:] = dv.stride()[:3]
        args.dweight, args.da = dw.data_ptr(), da.data_ptr()
        args.dproj_bias = dpb.data_ptr() if dpb is not None else None
        with _cabi.device_guard(v.device):
            nbytes = _cabi.lib.fdma_dyn_bias_bwd_workspace_bytes(args)
            ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=v.device)
            args.workspace, args.workspace_bytes = ws.data_ptr(), nbytes
            if b * l > 0:
                _cabi.check(_cabi.lib.fdma_dyn_bias_bwd(args, _cabi.current_stream(v.device)))
            else:
                dw.zero_(), da.zero_()
                if dpb is not None:
                    dpb.zero_()
        return dv, dw, da, dpb


def dynamic_mask_bias(
    value_states: torch.Tensor,
    dt_proj_weight: torch.Tensor,
    A: torch.Tensor,
    dt_proj_bias: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """attn_bias[b, j, 0, l] = A[j] * softplus(value_states[b, l].flatten() @ dt_proj_weight[j] + dt_proj_bias[j]).

    value_states: (batch, key_len, num_kv_heads, head_dim) -- the layout `flash_sparse_attn_func` takes;
    dt_proj_weight: (num_kv_heads, num_kv_heads * head_dim); A, dt_proj_bias: (num_kv_heads).
    Returns (batch, num_kv_heads, 1, key_len) in the dtype of value_states, ready to be passed as `attn_bias`
    (and to `create_mask`).  Differentiable in all four inputs.
    """
    if _native_ok(value_states, dt_proj_weight, A, dt_proj_bias) and value_states.shape[0] * value_states.shape[1] > 0:
        return _DynamicMaskBias.apply(value_states, dt_proj_weight, A, dt_proj_bias)
    return _tensor_program(value_states, dt_proj_weight, A, dt_proj_bias)
