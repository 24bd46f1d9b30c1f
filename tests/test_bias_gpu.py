"""GPU tests of the fused bias producer (`fdma_dyn_bias_fwd / _bwd` behind flash_sparse_attn.utils.bias, run with `-m gpu`).

Checker: the closed form  bias[b, j, 0, l] = A[j] * softplus(V[b, l].flatten() . W[j] + pb[j])  in fp32 with torch
autograd, on the same 16-bit inputs.  Tolerances: the forward is rounded to the 16-bit output type once (relative
error <= 2^-8 of the row scale); gradients within rtol 2e-2 of their scale (sums of up to 16 Ki products rounded to 16 bits)."""
import pytest
import torch
import torch.nn.functional as F

from flash_sparse_attn.utils.bias import dynamic_mask_bias
from _util import rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda"

CASES = [
    # B, L, Hk, d, with projection bias, dtype
    (1, 8192, 8, 128, False, torch.bfloat16),
    (2, 1000, 2, 64, True, torch.bfloat16),
    (3, 77, 1, 128, True, torch.float16),
    (1, 300, 12, 32, False, torch.bfloat16),
    (2, 129, 32, 16, True, torch.bfloat16),
]


def _inputs(B, L, Hk, d, with_pb, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    v = torch.randn(B, L, Hk, d, generator=g).to(dtype)
    w = (torch.randn(Hk, Hk * d, generator=g) / (Hk * d) ** 0.5).to(dtype)
    a = torch.linspace(0.5, 1.5, Hk).to(dtype)
    pb = (0.1 * torch.randn(Hk, generator=g)).to(dtype) if with_pb else None
    gout = torch.randn(B, Hk, 1, L, generator=g).to(dtype)
    return v, w, a, pb, gout


def _reference(v, w, a, pb, gout):
    v32, w32, a32 = [t.float().requires_grad_(True) for t in (v, w, a)]
    pb32 = pb.float().requires_grad_(True) if pb is not None else None
    B, L = v.shape[:2]
    dt = F.linear(v32.reshape(B, L, -1), w32, pb32)
    bias = (a32 * F.softplus(dt)).transpose(-1, -2).unsqueeze(-2)
    (bias * gout.float()).sum().backward()
    return bias.detach(), v32.grad, w32.grad, a32.grad, (pb32.grad if pb32 is not None else None)


@pytest.mark.parametrize("case", range(len(CASES)))
def test_bias_producer_forward_backward(case):
    B, L, Hk, d, with_pb, dtype = CASES[case]
    v, w, a, pb, gout = _inputs(B, L, Hk, d, with_pb, dtype, seed=case)
    vd, wd, ad = [t.to(DEV).requires_grad_(True) for t in (v, w, a)]
    pbd = pb.to(DEV).requires_grad_(True) if pb is not None else None
    print(f"bias producer B={B} L={L} Hk={Hk} d={d} pb={with_pb} {dtype}", flush=True)
    bias = dynamic_mask_bias(vd, wd, ad, pbd)
    assert bias.shape == (B, Hk, 1, L) and bias.dtype == dtype
    bias.backward(gout.to(DEV))
    torch.cuda.synchronize()
    rb, rdv, rdw, rda, rdpb = _reference(v.to(DEV), w.to(DEV), a.to(DEV), pb.to(DEV) if pb is not None else None, gout.to(DEV))
    assert rel_err(bias, rb) <= 2.0 ** -8
    for got, ref, name in ((vd.grad, rdv, "dvalue"), (wd.grad, rdw, "dweight"), (ad.grad, rda, "dA")):
        assert torch.isfinite(got.float()).all()
        assert rel_err(got, ref) <= 2e-2, name
    if pb is not None:
        assert rel_err(pbd.grad, rdpb) <= 2e-2


def test_bias_producer_is_bit_reproducible_and_feeds_the_operator():
    """Two runs agree bit for bit (the backward folds its partial sums in a fixed order), a strided view of the value
    states gives the same result as its contiguous copy, and the bias goes straight into mask builder and operator."""
    from flash_sparse_attn import flash_sparse_attn_func
    from flash_sparse_attn.utils.mask import create_mask

    B, L, H, Hk, d = 2, 512, 4, 2, 64
    v, w, a, pb, gout = _inputs(B, L, Hk, d, True, torch.bfloat16, seed=9)
    kv = torch.randn(B, L, 2, Hk, d, generator=torch.Generator().manual_seed(10)).to(torch.bfloat16).to(DEV)
    kv[:, :, 1] = v.to(DEV)
    runs = []
    for vin in (kv[:, :, 1], kv[:, :, 1].contiguous(), kv[:, :, 1]):
        vd = vin.detach().clone().requires_grad_(True) if vin.is_contiguous() else vin.detach().requires_grad_(True)
        wd, ad, pbd = [t.to(DEV).requires_grad_(True) for t in (w, a, pb)]
        bias = dynamic_mask_bias(vd, wd, ad, pbd)
        bias.backward(gout.to(DEV))
        runs.append((bias.detach(), vd.grad, wd.grad, ad.grad, pbd.grad))
    for other in runs[1:]:
        for x, y in zip(runs[0], other):
            assert torch.equal(x, y)
    bias = runs[0][0]
    keep = create_mask(bias, None, B, L, L, 128, torch.finfo(torch.bfloat16).min, type="topk")
    q = torch.randn(B, L, H, d, device=DEV).to(torch.bfloat16)
    out = flash_sparse_attn_func(q, kv[:, :, 0], kv[:, :, 1], keep, bias, None, True)
    assert torch.isfinite(out.float()).all()


def test_bias_producer_rejects_shapes_it_was_not_built_for():
    v = torch.randn(1, 64, 2, 12, device=DEV).to(torch.bfloat16)   # head_dim not a multiple of 8
    w = torch.randn(2, 24, device=DEV).to(torch.bfloat16)
    a = torch.ones(2, device=DEV).to(torch.bfloat16)
    with pytest.raises(RuntimeError, match="head_dim % 8"):
        dynamic_mask_bias(v, w, a)
    v = torch.randn(1, 64, 2, 16, device=DEV).to(torch.bfloat16)
    with pytest.raises(RuntimeError, match="dtype and device"):
        dynamic_mask_bias(v, torch.randn(2, 32, device=DEV), a)
    # CPU tensors run the caller's tensor program
    out = dynamic_mask_bias(v.cpu(), torch.randn(2, 32).to(torch.bfloat16), a.cpu())
    assert out.shape == (1, 2, 1, 64)
