"""The operator inside its caller (run with `-m gpu`): a dynamic-mask attention layer of the kind the reference's Doge
example builds around `flash_sparse_attn_func` (examples/modeling/modeling_doge.py:160-237 of the reference: q / k / v
projections, a bias A * softplus(dt_proj(V)) per kv head and key, a top-k keep-mask made from that bias by
`create_mask`, causal attention, output projection), with random weights.

The layer runs twice on the same weights and input: through the package (fused bias producer, device mask builder, HIP
attention, bf16) and through the caller's own tensor program for the bias plus the fp32 eager restatement of the
attention (oracle/eager.py), with the same keep-mask.  Output, input gradient
and every parameter gradient must agree -- which also checks what the hot path hands back to its caller: dBias in the
bias's own [B, Hkv, 1, Lk] shape, flowing on into A and dt_proj.
"""
import pytest
import torch
import torch.nn.functional as F
from torch import nn

from oracle import eager
from _util import rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda"


class DynamicMaskAttentionLayer(nn.Module):
    def __init__(self, hidden, heads, kv_heads, head_dim, window):
        super().__init__()
        self.heads, self.kv_heads, self.head_dim, self.window = heads, kv_heads, head_dim, window
        self.q_proj = nn.Linear(hidden, heads * head_dim, bias=False)
        self.k_proj = nn.Linear(hidden, kv_heads * head_dim, bias=False)
        self.v_proj = nn.Linear(hidden, kv_heads * head_dim, bias=False)
        self.dt_proj = nn.Linear(kv_heads * head_dim, kv_heads, bias=False)
        self.A = nn.Parameter(torch.linspace(0.5, 1.5, kv_heads))
        self.o_proj = nn.Linear(heads * head_dim, hidden, bias=False)

    def forward(self, x, native, keep=None):
        from flash_sparse_attn import flash_sparse_attn_func
        from flash_sparse_attn.utils.mask import create_mask

        B, L, _ = x.shape
        q = self.q_proj(x).view(B, L, self.heads, self.head_dim)
        k = self.k_proj(x).view(B, L, self.kv_heads, self.head_dim)
        v = self.v_proj(x).view(B, L, self.kv_heads, self.head_dim)
        if native:  # the fused producer of the package
            from flash_sparse_attn.utils.bias import dynamic_mask_bias
            bias = dynamic_mask_bias(v, self.dt_proj.weight, self.A)                 # (B, Hkv, 1, L)
        else:       # the caller's own tensor program
            dt = self.dt_proj(v.reshape(B, L, -1))                                  # (B, L, Hkv)
            bias = (self.A * F.softplus(dt)).transpose(-1, -2).unsqueeze(-2).to(x.dtype)
        if keep is None:
            keep = create_mask(bias, None, B, L, L, self.window, torch.finfo(x.dtype).min, type="topk")
        scale = self.head_dim ** -0.5
        if native:
            out = flash_sparse_attn_func(q, k, v, keep, bias, scale, True)
        else:
            out, _ = eager.attention_forward(q, k, v, keep, bias, scale, True)
            out = out.to(x.dtype)
        return self.o_proj(out.reshape(B, L, -1)), keep


@pytest.mark.parametrize("shape", [(2, 384, 256, 4, 2, 64, 96), (1, 1024, 512, 8, 2, 128, 256)])
def test_layer_forward_backward_matches_eager(shape):
    B, L, hidden, H, Hk, D, W = shape
    torch.manual_seed(5)
    layer = DynamicMaskAttentionLayer(hidden, H, Hk, D, W).to(DEV).to(torch.bfloat16)
    x = (torch.randn(B, L, hidden, generator=torch.Generator().manual_seed(6)) * 0.5).to(torch.bfloat16).to(DEV)
    results = []
    keep = None
    for native in (True, False):
        layer.zero_grad(set_to_none=True)
        xi = x.clone().requires_grad_(True)
        print(f"layer B={B} L={L} H={H} Hk={Hk} D={D} W={W} native={native}", flush=True)
        y, keep = layer(xi, native, keep)  # the second pass reuses the first pass's keep-mask
        assert keep.dtype == torch.bool and keep.shape == (B, Hk, 1, L) and int(keep.sum()) == B * Hk * W
        y.backward(torch.ones_like(y) / y.numel() ** 0.5)
        torch.cuda.synchronize()
        results.append((y.detach().float(), xi.grad.float(), {n: p.grad.float().clone() for n, p in layer.named_parameters()}))
    (y1, gx1, gp1), (y0, gx0, gp0) = results
    assert rel_err(y1, y0) <= 3e-2
    assert rel_err(gx1, gx0) <= 5e-2
    for name in gp0:
        assert torch.isfinite(gp1[name]).all()
        # dA is a sum over all tokens of terms of both signs that nearly cancel (|dA| is ~1 % of the sum of |terms|), so
        # the 16-bit rounding of dBias shows up enlarged in it, on either path
        assert rel_err(gp1[name], gp0[name]) <= (0.15 if name == "A" else 5e-2), name
