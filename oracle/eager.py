"""TEST INFRASTRUCTURE ONLY: "safe eager" fp32 restatement of dynamic-mask attention in torch.

The formula is the reference's eager path (benchmarks/forward_equivalence.py:113-124,
benchmarks/backward_equivalence.py:118-135): GQA expand by repeat-interleave, S = Q K^T * scale + bias,
masked_fill(~mask, -inf), softmax, P V; gradients by autograd.  Two additions make it usable as a
checker for the kernels: `is_causal` is applied bottom-right aligned (csrc/flash_sparse_attn/src/mask.h:39),
and rows with no visible key give O = 0 / LSE = +inf and zero gradients
(csrc/flash_sparse_attn/src/softmax.h:210-214) instead of the NaN a softmax over an all -inf row produces.

Runs on whatever device the inputs live on (CPU, or the GPU in fp32 for sizes the C oracle cannot
finish in seconds); work is done one batch x kv-head group at a time so the score matrix fits.
"""
import torch


def _expand_heads(t, H):
    """(b, {1,Hk,H}, r, c) -> per-q-head view index helper: returns head index map"""
    h = t.shape[1]
    return None if h == H else H // h


def visible_mask(Lq, Lk, mask_bh, causal, device):
    """mask_bh: None or bool ({1,Lq}, Lk) for one (batch, head); returns bool (Lq, Lk)"""
    vis = torch.ones(Lq, Lk, dtype=torch.bool, device=device)
    if causal:
        i = torch.arange(Lq, device=device)[:, None]
        j = torch.arange(Lk, device=device)[None, :]
        vis &= j <= i + (Lk - Lq)
    if mask_bh is not None:
        vis &= mask_bh[..., :Lk].bool()
    return vis


def _slice_bh(t, b, h, H):
    """select (batch b, q-head h) of a broadcastable 4-D mask/bias -> ({1,Lq}, Lk')"""
    if t is None:
        return None
    bb = 0 if t.shape[0] == 1 else b
    hh = h if t.shape[1] == H else (0 if t.shape[1] == 1 else h // (H // t.shape[1]))
    return t[bb, hh]


def attention_forward(q, k, v, mask=None, bias=None, scale=None, causal=False):
    """fp32 safe eager forward.  q (B,Lq,H,D); k,v (B,Lk,Hk,D).  Returns (out fp32, lse fp32 (B,H,Lq)).
    Differentiable w.r.t. q, k, v, bias (empty rows contribute zero gradient)."""
    B, Lq, H, D = q.shape
    Lk, Hk = k.shape[1], k.shape[2]
    G = H // Hk
    if scale is None:
        scale = D ** -0.5
    outs = []
    lses = []
    for b in range(B):
        out_h = []
        lse_h = []
        for h in range(H):
            qh = q[b, :, h].float()
            kh = k[b, :, h // G].float()
            vh = v[b, :, h // G].float()
            s = (qh @ kh.t()) * scale
            bias_bh = _slice_bh(bias, b, h, H)
            if bias_bh is not None:
                s = s + bias_bh[..., :Lk].float()
            vis = visible_mask(Lq, Lk, _slice_bh(mask, b, h, H), causal, q.device)
            s = s.masked_fill(~vis, float("-inf"))
            empty = ~vis.any(dim=-1, keepdim=True)
            s_safe = torch.where(empty, torch.zeros_like(s), s)
            p = torch.softmax(s_safe, dim=-1)
            p = torch.where(empty, torch.zeros_like(p), p)
            out_h.append(p @ vh)
            lse = torch.logsumexp(s_safe, dim=-1)
            lse_h.append(torch.where(empty[:, 0], torch.full_like(lse, float("inf")), lse))
        outs.append(torch.stack(out_h, dim=1))
        lses.append(torch.stack(lse_h, dim=0))
    return torch.stack(outs, dim=0), torch.stack(lses, dim=0)


def attention_forward_backward(q, k, v, mask=None, bias=None, scale=None, causal=False, dout=None):
    """Returns (out, dq, dk, dv, dbias) in fp32 for loss = (out * dout).sum() (dout = 1 by default,
    i.e. the reference's loss = out.sum()).  dbias has the bias's own shape (autograd sums over
    broadcast dims)."""
    q32 = q.detach().float().requires_grad_(True)
    k32 = k.detach().float().requires_grad_(True)
    v32 = v.detach().float().requires_grad_(True)
    b32 = bias.detach().float().requires_grad_(True) if bias is not None else None
    out, _ = attention_forward(q32, k32, v32, mask, b32, scale, causal)
    loss = out.sum() if dout is None else (out * dout.float()).sum()
    loss.backward()
    return out.detach(), q32.grad, k32.grad, v32.grad, (b32.grad if b32 is not None else None)
