"""Writes tests/golden/vectors.npz: frozen input / expected-output vectors for the attention path.

The reference ships no golden vectors for this path (its checks are seeded GPU-vs-eager scripts that need a CUDA
device), and nothing of the reference is imported or run here.  The expected values are the closed form
    O = softmax(Q K^T * scale + bias  restricted to  keep-mask AND bottom-right causal) V
evaluated with plain torch in float64 (matmul / softmax / logsumexp / autograd are the library routines), on inputs
that were rounded to bf16 first, for a loss sum(O * dO).  Rows without a visible key give O = 0, LSE = +inf and
contribute no gradient (flash_sparse_attn/flash_sparse_attn_interface.py:643 and
csrc/flash_sparse_attn/src/softmax.h:210-214 of the reference).  This file deliberately shares no code with
oracle/ or with the package: the tests check the C oracle, the eager restatement and the GPU kernels against
the frozen numbers.

Run:  python tests/golden/make_vectors.py      (CPU only, a second or so; rewrites vectors.npz in place)
"""
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))

# name: B, Lq, Lk, H, Hk, D, bias shape, mask shape, keep window, causal, scale
CASES = {
    "mqa_row_bias_top32_causal": (1, 64, 64, 2, 1, 32, (1, 1, 1, 64), (1, 1, 1, 64), 32, True, 32 ** -0.5),
    "gqa_full_bias_lq_lt_lk": (2, 24, 40, 4, 2, 16, (2, 2, 24, 40), (2, 1, 24, 40), 12, True, 0.25),
    "lq_gt_lk_rows_without_keys": (1, 40, 16, 2, 2, 8, None, None, None, True, 8 ** -0.5),
    "noncausal_per_head_bias_batch_broadcast": (2, 33, 48, 4, 2, 16, (1, 4, 1, 48), (2, 2, 1, 48), 20, False, 0.3),
}
# ragged batch: lens_q, lens_k, H, Hk, D, causal, scale
RAGGED = {
    "ragged_gqa_causal": ([20, 0, 33, 7], [20, 0, 48, 3], 4, 2, 16, True, 0.25),
}


def bf16(t):
    return t.to(torch.bfloat16)


def bits(t):
    """bf16 tensor -> uint16 bit patterns (numpy has no bf16)."""
    return t.view(torch.int16).numpy().view(np.uint16)


def attend(q, k, v, keep, bias, causal, scale, dout):
    """float64 closed form for one problem.  q (B,Lq,H,D); k, v (B,Lk,Hk,D); keep bool / bias broadcastable to
    (B,H,Lq,Lk) after the head expansion below, or None.  Returns out, lse, dq, dk, dv, dbias."""
    B, Lq, H, D = q.shape
    Lk, Hk = k.shape[1], k.shape[2]
    G = H // Hk
    q64 = q.double().requires_grad_(True)
    k64 = k.double().requires_grad_(True)
    v64 = v.double().requires_grad_(True)
    b64 = bias.double().requires_grad_(True) if bias is not None else None

    def heads(t):  # (b, {1, Hk, H}, r, Lk) -> (b, H, r, Lk): query head h reads entry h // (H / heads)
        return t if t.shape[1] == H else t.repeat_interleave(H // t.shape[1], dim=1)

    s = torch.einsum("bqhd,bkhd->bhqk", q64, k64.repeat_interleave(G, dim=2)) * scale
    if b64 is not None:
        s = s + heads(b64)
    vis = torch.ones(B, H, Lq, Lk, dtype=torch.bool)
    if keep is not None:
        vis = vis & heads(keep)
    if causal:
        i = torch.arange(Lq)[:, None]
        j = torch.arange(Lk)[None, :]
        vis = vis & (j <= i + (Lk - Lq))
    s = s.masked_fill(~vis, float("-inf"))
    dead = ~vis.any(-1, keepdim=True)
    s_safe = torch.where(dead, torch.zeros_like(s), s)
    p = torch.where(dead, torch.zeros_like(s), torch.softmax(s_safe, -1))
    out = torch.einsum("bhqk,bkhd->bqhd", p, v64.repeat_interleave(G, dim=2))
    lse = torch.where(dead[..., 0], torch.full_like(s_safe[..., 0], float("inf")), torch.logsumexp(s_safe, -1))
    (out * dout.double()).sum().backward()
    return (out.detach(), lse.detach(), q64.grad, k64.grad, v64.grad, b64.grad if b64 is not None else None)


def main():
    blob = {}
    for n, (name, (B, Lq, Lk, H, Hk, D, bshape, mshape, window, causal, scale)) in enumerate(sorted(CASES.items())):
        g = torch.Generator().manual_seed(1234 + n)
        q, k, v = bf16(torch.randn(B, Lq, H, D, generator=g)), bf16(torch.randn(B, Lk, Hk, D, generator=g)), bf16(torch.randn(B, Lk, Hk, D, generator=g))
        dout = bf16(torch.randn(B, Lq, H, D, generator=g))
        bias = bf16(torch.randn(*bshape, generator=g)) if bshape else None
        keep = None
        if mshape:
            src = bias if (bias is not None and tuple(bshape) == tuple(mshape)) else torch.randn(*mshape, generator=g)
            idx = src.float().topk(window, dim=-1).indices
            keep = torch.zeros(mshape, dtype=torch.bool).scatter_(-1, idx, True)
        out, lse, dq, dk, dv, db = attend(q, k, v, keep, bias, causal, scale, dout)
        blob[f"{name}/q"], blob[f"{name}/k"], blob[f"{name}/v"], blob[f"{name}/dout"] = bits(q), bits(k), bits(v), bits(dout)
        if bias is not None:
            blob[f"{name}/bias"] = bits(bias)
            blob[f"{name}/dbias"] = db.numpy().astype(np.float32)
        if keep is not None:
            blob[f"{name}/mask"] = keep.numpy()
        blob[f"{name}/meta"] = np.array([int(causal), scale], dtype=np.float64)
        for key, t in (("out", out), ("lse", lse), ("dq", dq), ("dk", dk), ("dv", dv)):
            blob[f"{name}/{key}"] = t.numpy().astype(np.float32)
    for n, (name, (lens_q, lens_k, H, Hk, D, causal, scale)) in enumerate(sorted(RAGGED.items())):
        g = torch.Generator().manual_seed(4321 + n)
        tq, tk = sum(lens_q), sum(lens_k)
        q, k, v = bf16(torch.randn(tq, H, D, generator=g)), bf16(torch.randn(tk, Hk, D, generator=g)), bf16(torch.randn(tk, Hk, D, generator=g))
        dout = bf16(torch.randn(tq, H, D, generator=g))
        out = torch.zeros(tq, H, D, dtype=torch.float64)
        lse = torch.full((H, tq), float("inf"), dtype=torch.float64)
        dq, dk, dv = torch.zeros(tq, H, D, dtype=torch.float64), torch.zeros(tk, Hk, D, dtype=torch.float64), torch.zeros(tk, Hk, D, dtype=torch.float64)
        q0 = k0 = 0
        for lq, lk in zip(lens_q, lens_k):
            if lq and lk:
                o, l, gq, gk, gv, _ = attend(q[None, q0:q0 + lq], k[None, k0:k0 + lk], v[None, k0:k0 + lk], None, None, causal, scale,
                                             dout[None, q0:q0 + lq])
                out[q0:q0 + lq], dq[q0:q0 + lq], dk[k0:k0 + lk], dv[k0:k0 + lk] = o[0], gq[0], gk[0], gv[0]
                lse[:, q0:q0 + lq] = l[0]
            q0, k0 = q0 + lq, k0 + lk
        blob[f"{name}/q"], blob[f"{name}/k"], blob[f"{name}/v"], blob[f"{name}/dout"] = bits(q), bits(k), bits(v), bits(dout)
        blob[f"{name}/lens_q"], blob[f"{name}/lens_k"] = np.array(lens_q, dtype=np.int32), np.array(lens_k, dtype=np.int32)
        blob[f"{name}/meta"] = np.array([int(causal), scale], dtype=np.float64)
        for key, t in (("out", out), ("lse", lse), ("dq", dq), ("dk", dk), ("dv", dv)):
            blob[f"{name}/{key}"] = t.numpy().astype(np.float32)
    path = os.path.join(HERE, "vectors.npz")
    np.savez_compressed(path, **blob)
    print(path, os.path.getsize(path), "bytes,", len(blob), "arrays")


if __name__ == "__main__":
    main()
