"""Pins the CPU oracle (oracle/fdma_oracle.c and oracle/eager.py) WITHOUT the kernels.

The reference ships no golden vectors for this path (its checks are seeded GPU-vs-eager scripts), so
the oracle is pinned by what the mathematics fixes: library routines it must reduce to
(torch softmax / matmul / scaled_dot_product_attention), a brute-force per-row gather in the manner
of the reference's benchmarks/grad_equivalence.py:78-109, the literal causal matrices printed in the
reference docstring (flash_sparse_attn_interface.py:633-642), invariances of softmax attention,
torch autograd of the closed form, and fp64 finite differences.  Each check is chosen so that a
plausible mistake (dropped scale, scaled bias, wrong causal alignment, transposed operand, wrong
GQA head map, missing group/batch reduction) fails it.
"""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import c_oracle, eager
from _util import causal_matrix, make_inputs


def _rand(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed))


def test_reduces_to_sdpa_without_mask_and_bias():
    q, k, v = _rand(2, 9, 4, 16, seed=1), _rand(2, 13, 4, 16, seed=2), _rand(2, 13, 4, 16, seed=3)
    out, lse = c_oracle.forward(q, k, v)
    ref = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)).transpose(1, 2)
    assert torch.allclose(out, ref, atol=2e-6, rtol=1e-5)
    s = torch.einsum("bqhd,bkhd->bhqk", q, k) / math.sqrt(16)
    assert torch.allclose(lse, torch.logsumexp(s, -1), atol=2e-6, rtol=1e-5)
    out_e, lse_e = eager.attention_forward(q, k, v)
    assert torch.allclose(out_e, ref, atol=2e-6, rtol=1e-5)
    assert torch.allclose(lse_e, lse, atol=2e-6, rtol=1e-5)


def test_bias_is_added_after_scaling_and_not_scaled():
    # bias enters as an additive float mask of SDPA: softmax(QK^T * scale + bias)
    q, k, v = _rand(1, 7, 2, 8, seed=1), _rand(1, 11, 2, 8, seed=2), _rand(1, 11, 2, 8, seed=3)
    bias = 3.0 * _rand(1, 2, 7, 11, seed=4)
    scale = 0.37
    out, _ = c_oracle.forward(q, k, v, None, bias, scale, False)
    ref = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), attn_mask=bias, scale=scale).transpose(1, 2)
    assert torch.allclose(out, ref, atol=3e-6, rtol=1e-5)
    out_e, _ = eager.attention_forward(q, k, v, None, bias, scale, False)
    assert torch.allclose(out_e, ref, atol=3e-6, rtol=1e-5)


def test_docstring_causal_matrices():
    # flash_sparse_attn_interface.py:633-642: bottom-right aligned causal masks, literally
    m25 = torch.tensor([[1, 1, 1, 1, 0], [1, 1, 1, 1, 1]], dtype=torch.bool)
    m52 = torch.tensor([[0, 0], [0, 0], [0, 0], [1, 0], [1, 1]], dtype=torch.bool)
    assert torch.equal(causal_matrix(2, 5), m25)
    assert torch.equal(causal_matrix(5, 2), m52)
    for Lq, Lk, m in ((2, 5, m25), (5, 2, m52)):
        q, k, v = _rand(1, Lq, 1, 8, seed=5), _rand(1, Lk, 1, 8, seed=6), _rand(1, Lk, 1, 8, seed=7)
        out_c, lse_c = c_oracle.forward(q, k, v, None, None, None, True)
        out_m, lse_m = c_oracle.forward(q, k, v, m[None, None], None, None, False)
        assert torch.equal(out_c, out_m) and torch.equal(lse_c, lse_m)
        out_e, _ = eager.attention_forward(q, k, v, None, None, None, True)
        assert torch.allclose(out_e, out_c, atol=2e-6)
    # rows with no visible key: O = 0, LSE = +inf
    out_c, lse_c = c_oracle.forward(_rand(1, 5, 1, 8), _rand(1, 2, 1, 8), _rand(1, 2, 1, 8), None, None, None, True)
    assert torch.equal(out_c[0, :3], torch.zeros(3, 1, 8)) and torch.isinf(lse_c[0, 0, :3]).all() and (lse_c[0, 0, :3] > 0).all()
    assert torch.isfinite(lse_c[0, 0, 3:]).all()


def test_brute_force_row_gather():
    # per row: gather the kept keys, plain softmax over them (grad_equivalence.py:78-109 pattern)
    B, Lq, Lk, H, Hk, D = 2, 6, 10, 4, 2, 8
    q, k, v, mask, bias = make_inputs(B, Lq, Lk, H, Hk, D, (B, Hk, Lq, Lk), (B, Hk, Lq, Lk), window=4, seed=3, dtype=torch.float32)
    scale = 0.5
    out, lse = c_oracle.forward(q, k, v, mask, bias, scale, True)
    for b in range(B):
        for h in range(H):
            hk = h // (H // Hk)
            for i in range(Lq):
                keep = [j for j in range(Lk) if mask[b, hk, i, j] and j <= i + Lk - Lq]
                if not keep:
                    assert torch.equal(out[b, i, h], torch.zeros(D)) and lse[b, h, i] == float("inf")
                    continue
                s = torch.stack([(q[b, i, h] * k[b, j, hk]).sum() * scale + bias[b, hk, i, j] for j in keep])
                p = torch.softmax(s, 0)
                o = sum(p[t] * v[b, j, hk] for t, j in enumerate(keep))
                assert torch.allclose(out[b, i, h], o, atol=1e-5), (b, h, i)
                assert abs(lse[b, h, i].item() - torch.logsumexp(s, 0).item()) < 1e-5


def test_invariances():
    B, Lq, Lk, H, Hk, D = 1, 8, 12, 4, 2, 8
    q, k, v, mask, bias = make_inputs(B, Lq, Lk, H, Hk, D, (B, Hk, Lq, Lk), (B, 1, Lq, Lk), window=6, seed=9, dtype=torch.float32)
    out, lse = c_oracle.forward(q, k, v, mask, bias, None, False)
    # rows of P sum to one: V = 1 gives O = 1 on non-empty rows
    ones, _ = c_oracle.forward(q, k, torch.ones_like(v), mask, bias, None, False)
    assert torch.allclose(ones, torch.ones_like(ones), atol=1e-6)
    # adding a per-row constant to the bias changes nothing but the LSE
    shift = _rand(B, Hk, Lq, 1, seed=10)
    out2, lse2 = c_oracle.forward(q, k, v, mask, bias + shift, None, False)
    assert torch.allclose(out2, out, atol=1e-5)
    assert torch.allclose(lse2, lse + shift[:, :, :, 0].repeat_interleave(H // Hk, 1), atol=1e-5)
    # permuting keys together with their mask / bias columns leaves a non-causal output unchanged
    perm = torch.randperm(Lk, generator=torch.Generator().manual_seed(11))
    out3, _ = c_oracle.forward(q, k[:, perm], v[:, perm], mask[..., perm], bias[..., perm], None, False)
    assert torch.allclose(out3, out, atol=1e-5)


@pytest.mark.parametrize("hm,hb", [(1, 1), (2, 2), (4, 4), (1, 4), (4, 2)])
def test_gqa_head_mapping_matches_repeat_interleave(hm, hb):
    # reference: repeat_kv == repeat_interleave on the head dim (forward_equivalence.py:55-67)
    B, Lq, Lk, H, Hk, D = 2, 5, 7, 4, 2, 8
    q, k, v = _rand(B, Lq, H, D, seed=1), _rand(B, Lk, Hk, D, seed=2), _rand(B, Lk, Hk, D, seed=3)
    bias = _rand(B, hb, Lq, Lk, seed=4)
    mask = _rand(B, hm, Lq, Lk, seed=5) > -0.5
    out, _ = c_oracle.forward(q, k, v, mask, bias, None, False)
    kx, vx = k.repeat_interleave(H // Hk, 2), v.repeat_interleave(H // Hk, 2)
    bx, mx = bias.repeat_interleave(H // hb, 1), mask.repeat_interleave(H // hm, 1)
    s = torch.einsum("bqhd,bkhd->bhqk", q, kx) / math.sqrt(D) + bx
    s = s.masked_fill(~mx, float("-inf"))
    p = torch.softmax(s, -1)
    p = torch.nan_to_num(p, nan=0.0)  # empty rows
    ref = torch.einsum("bhqk,bkhd->bqhd", p, vx)
    assert torch.allclose(out, ref, atol=3e-6, rtol=1e-5)


def _autograd_reference(q, k, v, mask, bias, scale, causal, dout):
    """closed form with plain torch ops + autograd, fp64"""
    B, Lq, H, D = q.shape
    Lk, Hk = k.shape[1], k.shape[2]
    q, k, v = [t.double().requires_grad_(True) for t in (q, k, v)]
    bias = bias.double().requires_grad_(True) if bias is not None else None
    kx, vx = k.repeat_interleave(H // Hk, 2), v.repeat_interleave(H // Hk, 2)
    s = torch.einsum("bqhd,bkhd->bhqk", q, kx) * scale
    if bias is not None:
        bx = bias.expand(B, bias.shape[1], Lq, Lk).repeat_interleave(H // bias.shape[1], 1)
        s = s + bx
    vis = torch.ones(B, H, Lq, Lk, dtype=torch.bool)
    if mask is not None:
        vis = vis & mask.expand(B, mask.shape[1], Lq, Lk).repeat_interleave(H // mask.shape[1], 1)
    if causal:
        vis = vis & causal_matrix(Lq, Lk)
    empty = ~vis.any(-1, keepdim=True)
    s = s.masked_fill(~vis, float("-inf")).masked_fill(empty, 0.0)
    p = torch.softmax(s, -1).masked_fill(empty, 0.0)
    out = torch.einsum("bhqk,bkhd->bqhd", p, vx)
    (out * dout.double()).sum().backward()
    return out.detach(), q.grad, k.grad, v.grad, (bias.grad if bias is not None else None)


@pytest.mark.parametrize(
    "bias_shape,mask_shape,causal",
    [
        ((2, 2, 6, 9), (2, 2, 6, 9), True),    # per-query bias on kv heads: dbias sums over the group
        ((1, 4, 6, 9), (2, 1, 6, 9), False),   # batch-broadcast bias: dbias sums over batch
        ((2, 1, 1, 9), (2, 1, 1, 9), True),    # fully broadcast row bias: sums over heads and queries
        ((2, 2, 1, 9), None, True),
        (None, (1, 4, 6, 9), False),
    ],
)
def test_backward_matches_autograd_of_closed_form(bias_shape, mask_shape, causal):
    B, Lq, Lk, H, Hk, D = 2, 6, 9, 4, 2, 8
    q, k, v, mask, bias = make_inputs(B, Lq, Lk, H, Hk, D, bias_shape, mask_shape, window=4, seed=21, dtype=torch.float32)
    dout = _rand(B, Lq, H, D, seed=22)
    scale = 0.41
    out_r, dq_r, dk_r, dv_r, db_r = _autograd_reference(q, k, v, mask, bias, scale, causal, dout)
    dq, dk, dv, db = c_oracle.backward(q, k, v, dout, mask, bias, scale, causal)
    for a, r in ((dq, dq_r), (dk, dk_r), (dv, dv_r)):
        assert torch.allclose(a.double(), r, atol=2e-6, rtol=1e-5)
    if bias is not None:
        assert db.shape == bias.shape
        assert torch.allclose(db.double(), db_r, atol=2e-6, rtol=1e-5)
    # eager (fp32 autograd) agrees too
    _, dq_e, dk_e, dv_e, db_e = eager.attention_forward_backward(q, k, v, mask, bias, scale, causal, dout)
    for a, r in ((dq_e, dq_r), (dk_e, dk_r), (dv_e, dv_r)):
        assert torch.allclose(a.double(), r, atol=2e-5, rtol=1e-4)
    if bias is not None:
        assert torch.allclose(db_e.double(), db_r, atol=2e-5, rtol=1e-4)


def test_backward_finite_differences_fp64():
    B, Lq, Lk, H, Hk, D = 1, 3, 5, 2, 1, 4
    q, k, v, mask, bias = make_inputs(B, Lq, Lk, H, Hk, D, (1, 1, Lq, Lk), (1, 1, Lq, Lk), window=3, seed=31, dtype=torch.float32)
    dout = _rand(B, Lq, H, D, seed=32)
    scale = 0.6

    def loss(qq, kk, vv, bb):
        o, _ = c_oracle.forward(qq, kk, vv, mask, bb, scale, True)
        return (o.double() * dout.double()).sum().item()

    dq, dk, dv, db = c_oracle.backward(q, k, v, dout, mask, bias, scale, True)
    eps = 1e-2  # fp32 storage of inputs: central differences with a coarse step
    for name, t, g in (("q", q, dq), ("k", k, dk), ("v", v, dv), ("bias", bias, db)):
        flat = t.reshape(-1)
        for idx in range(0, flat.numel(), max(1, flat.numel() // 7)):
            tp, tm = t.clone(), t.clone()
            tp.reshape(-1)[idx] += eps
            tm.reshape(-1)[idx] -= eps
            args_p = [tp if n == name else x for n, x in (("q", q), ("k", k), ("v", v), ("bias", bias))]
            args_m = [tm if n == name else x for n, x in (("q", q), ("k", k), ("v", v), ("bias", bias))]
            fd = (loss(*args_p) - loss(*args_m)) / (2 * eps)
            assert abs(fd - g.reshape(-1)[idx].item()) < 2e-3 * max(1.0, abs(fd)), (name, idx, fd, g.reshape(-1)[idx].item())


def test_dbias_rows_sum_to_zero_and_empty_rows_have_zero_grads():
    # sum_k dS[q,k] = 0 for every row; rows without a visible key contribute nothing
    B, Lq, Lk, H, Hk, D = 1, 6, 4, 2, 2, 8   # Lq > Lk with causal: the first two rows are empty
    q, k, v, mask, bias = make_inputs(B, Lq, Lk, H, Hk, D, (1, 2, Lq, Lk), None, seed=41, dtype=torch.float32)
    dout = _rand(B, Lq, H, D, seed=42)
    dq, dk, dv, db = c_oracle.backward(q, k, v, dout, None, bias, None, True)
    assert torch.allclose(db.sum(-1), torch.zeros(1, 2, Lq), atol=1e-6)
    assert torch.equal(dq[:, :2], torch.zeros(1, 2, H, D))
    assert torch.equal(db[:, :, :2], torch.zeros(1, 2, 2, Lk))
    assert torch.isfinite(dk).all() and torch.isfinite(dv).all()


def test_split_combine_is_associative():
    # merging per-split (O_s, lse_s) with the LSE-weighted combine reproduces the unsplit result
    B, Lq, Lk, H, Hk, D = 2, 1, 24, 4, 2, 8
    q, k, v, mask, bias = make_inputs(B, Lq, Lk, H, Hk, D, (B, Hk, 1, Lk), (B, Hk, 1, Lk), window=6, seed=51, dtype=torch.float32)
    out, lse = c_oracle.forward(q, k, v, mask, bias)
    parts_o, parts_l = [], []
    for s in range(3):
        sl = slice(8 * s, 8 * s + 8)
        m = mask[..., sl].clone()
        if s == 1:
            m[:] = False  # an empty split: O_s = 0, lse_s = -inf by the split convention
        o_s, l_s = c_oracle.forward(q, k[:, sl], v[:, sl], m, bias[..., sl])
        l_s = torch.where(torch.isinf(l_s), torch.full_like(l_s, float("-inf")), l_s)
        parts_o.append(o_s.permute(0, 2, 1, 3).reshape(B * H, D))
        parts_l.append(l_s.reshape(B * H))
    mask2 = mask.clone()
    mask2[..., 8:16] = False
    out2, lse2 = c_oracle.forward(q, k, v, mask2, bias)
    o_c, l_c = c_oracle.combine(torch.stack(parts_o), torch.stack(parts_l))
    assert torch.allclose(o_c, out2.permute(0, 2, 1, 3).reshape(B * H, D), atol=1e-6)
    assert torch.allclose(l_c, lse2.reshape(B * H), atol=1e-6)
