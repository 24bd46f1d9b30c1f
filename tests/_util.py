"""Shared helpers of the test suite: seeded synthetic inputs in the shapes of the benchmark
configurations, the dynamic-mask builder, and the tolerance checks.

Inputs are drawn on the CPU from a seeded generator and rounded to the compute dtype there, so the
CPU oracle and the GPU kernels see identical bits.
"""
import torch

def set_compact(mode) -> None:
    """Compaction policy of the following operator calls: "0" = tile skipping only, "2" = column compaction whenever
    the mask form allows it, None or anything else = the library's own cost rule (conftest.py resets it after
    every test)."""
    from flash_sparse_attn import _cabi
    _cabi.set_compact_mode({"0": _cabi.COMPACT_NEVER, "2": _cabi.COMPACT_ALWAYS}.get(mode, _cabi.COMPACT_AUTO))


# tolerances of the hot path (bf16): max-abs error of the output, relative error of gradients
OUT_ATOL = 2e-2
GRAD_RTOL = 5e-2


def topk_keep_mask(bias: torch.Tensor, window: int) -> torch.Tensor:
    """Boolean keep-mask with the bias's shape: per row, True on the `window` largest bias values.
    (The causal intersection is applied by is_causal=True, which gives the identical result.)"""
    w = min(window, bias.shape[-1])
    idx = bias.float().topk(w, dim=-1).indices
    return torch.zeros(bias.shape, dtype=torch.bool).scatter_(-1, idx, True)


def causal_matrix(Lq: int, Lk: int) -> torch.Tensor:
    i = torch.arange(Lq)[:, None]
    j = torch.arange(Lk)[None, :]
    return j <= i + (Lk - Lq)


def make_inputs(B, Lq, Lk, H, Hk, D, bias_shape=None, mask_shape=None, window=None, seed=0, dtype=torch.bfloat16):
    """Returns CPU tensors (q, k, v, mask, bias).  The mask is the top-`window` of the bias when the
    two shapes agree, otherwise the top-`window` of an independent N(0,1) tensor."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Lq, H, D, generator=g).to(dtype)
    k = torch.randn(B, Lk, Hk, D, generator=g).to(dtype)
    v = torch.randn(B, Lk, Hk, D, generator=g).to(dtype)
    bias = torch.randn(*bias_shape, generator=g).to(dtype) if bias_shape else None
    mask = None
    if mask_shape:
        if bias is not None and tuple(bias.shape) == tuple(mask_shape):
            src = bias
        else:
            src = torch.randn(*mask_shape, generator=g)
        mask = topk_keep_mask(src, window if window is not None else mask_shape[-1])
    return q, k, v, mask, bias


def rel_err(a: torch.Tensor, ref: torch.Tensor) -> float:
    """max |a - ref| / max |ref|"""
    return ((a.float() - ref.float()).abs().max() / ref.float().abs().max().clamp_min(1e-6)).item()


def frac_within(a: torch.Tensor, ref: torch.Tensor, tol: float) -> float:
    a, ref = a.float(), ref.float()
    return ((a - ref).abs() <= tol + tol * ref.abs()).float().mean().item()


def assert_out_close(out, ref, what="out"):
    err = (out.float() - ref.float()).abs().max().item()
    assert err <= OUT_ATOL, f"{what}: max-abs error {err:.3e} > {OUT_ATOL}"


def assert_grad_close(g, ref, what):
    """rtol 5e-2 on gradients: the worst element is within 5e-2 of the gradient's scale, and at
    least 99 % of the elements are within atol = rtol = 5e-2 of the reference."""
    assert torch.isfinite(g.float()).all(), f"{what}: non-finite gradient"
    e = rel_err(g, ref)
    assert e <= GRAD_RTOL, f"{what}: max|g - ref| / max|ref| = {e:.3e} > {GRAD_RTOL}"
    fr = frac_within(g, ref, GRAD_RTOL)
    assert fr >= 0.99, f"{what}: only {fr:.4f} of elements within {GRAD_RTOL}"
