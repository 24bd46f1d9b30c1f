"""GPU parity tests of the ragged-batch ("varlen") operator (run with `-m gpu` on an MI355X).

`flash_sparse_attn_varlen_func` goes through fdma_varlen_fwd / fdma_varlen_bwd of libfdma_hip.so.  The packed result
is compared sequence by sequence with the fp32 safe-eager restatement (oracle/eager.py) on the same bits; a
sequence without keys has the closed-form answer O = 0, LSE = +inf, dQ = 0, and one without queries dK = dV = 0.
Tolerances as for the fixed-length operator: out max-abs <= 2e-2, gradients rtol 5e-2 (_util.assert_grad_close).
"""
import pytest
import torch

from oracle import eager
from _util import assert_grad_close, assert_out_close

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _op():
    from flash_sparse_attn import flash_sparse_attn_varlen_func
    return flash_sparse_attn_varlen_func


def _cu(lens):
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    return torch.tensor(cu, dtype=torch.int32)


def _make(lens_q, lens_k, H, Hk, D, dtype, seed, slack_rows=0):
    """Packed q / k / v / dout of the given sequence lengths; `slack_rows` extra rows at the end belong to no sequence."""
    g = torch.Generator().manual_seed(seed)
    tq, tk = sum(lens_q) + slack_rows, sum(lens_k) + slack_rows
    q = torch.randn(tq, H, D, generator=g).to(dtype)
    k = torch.randn(tk, Hk, D, generator=g).to(dtype)
    v = torch.randn(tk, Hk, D, generator=g).to(dtype)
    do = torch.randn(tq, H, D, generator=g).to(dtype)
    return q, k, v, do


def _reference(q, k, v, do, lens_q, lens_k, causal, scale=None):
    """Per-sequence fp32 eager results packed like the inputs: out, lse (H, total_q), dq, dk, dv."""
    H = q.shape[1]
    out = torch.zeros_like(q, dtype=torch.float32)
    lse = torch.full((H, q.shape[0]), float("inf"), dtype=torch.float32, device=q.device)
    dq = torch.zeros_like(q, dtype=torch.float32)
    dk = torch.zeros_like(k, dtype=torch.float32)
    dv = torch.zeros_like(v, dtype=torch.float32)
    q0 = k0 = 0
    for lq, lk in zip(lens_q, lens_k):
        if lq > 0 and lk > 0:
            qs, ks, vs, ds = q[None, q0:q0 + lq], k[None, k0:k0 + lk], v[None, k0:k0 + lk], do[None, q0:q0 + lq]
            o, gq, gk, gv, _ = eager.attention_forward_backward(qs, ks, vs, None, None, scale, causal, dout=ds)
            _, l = eager.attention_forward(qs, ks, vs, None, None, scale, causal)
            out[q0:q0 + lq], dq[q0:q0 + lq] = o[0], gq[0]
            dk[k0:k0 + lk], dv[k0:k0 + lk] = gk[0], gv[0]
            lse[:, q0:q0 + lq] = l[0]
        q0 += lq
        k0 += lk
    return out, lse, dq, dk, dv


def _run(lens_q, lens_k, H, Hk, D, causal, dtype=torch.bfloat16, seed=0, slack_rows=0, scale=None, max_slack=0):
    q, k, v, do = _make(lens_q, lens_k, H, Hk, D, dtype, seed, slack_rows)
    qd, kd, vd, dod = [t.to(DEV) for t in (q, k, v, do)]
    cu_q, cu_k = _cu(lens_q).to(DEV), _cu(lens_k).to(DEV)
    qd, kd, vd = [t.requires_grad_(True) for t in (qd, kd, vd)]
    print(f"varlen lens_q={lens_q} lens_k={lens_k} H={H} Hk={Hk} D={D} causal={causal} {dtype}", flush=True)
    out, lse, _ = _op()(qd, kd, vd, cu_q, cu_k, max(lens_q) + max_slack, max(lens_k) + max_slack, scale, causal,
                        None, None, True)
    out.backward(dod)
    torch.cuda.synchronize()
    tq, tk = sum(lens_q), sum(lens_k)
    ro, rl, rdq, rdk, rdv = _reference(qd.detach()[:tq], kd.detach()[:tk], vd.detach()[:tk], dod[:tq], lens_q, lens_k,
                                       causal, scale)
    assert out.shape == q.shape and lse.shape == (H, q.shape[0])
    assert_out_close(out.detach()[:tq], ro)
    l = lse[:, :tq]
    assert torch.equal(torch.isinf(l), torch.isinf(rl)), "empty-row pattern of the LSE differs"
    fin = torch.isfinite(rl)
    if fin.any():
        assert (l[fin] - rl[fin]).abs().max().item() <= 1e-2
    assert (l[~fin] > 0).all()
    for g, r, n in ((qd.grad[:tq], rdq, "dq"), (kd.grad[:tk], rdk, "dk"), (vd.grad[:tk], rdv, "dv")):
        if r.numel():
            assert_grad_close(g, r, n)
    return out.detach(), lse.detach(), qd.grad, kd.grad, vd.grad


VARLEN_CASES = {
    # name: (lens_q, lens_k, H, Hk, D, dtype)
    "self_attention_ragged_gqa_d128": ([100, 1, 257, 64, 300], [100, 1, 257, 64, 300], 4, 2, 128, torch.bfloat16),
    "cross_lengths_d64": ([37, 200, 5, 129], [300, 64, 77, 129], 4, 1, 64, torch.bfloat16),
    "lq_gt_lk_rows_without_keys_fp16": ([200, 64, 130], [50, 64, 1], 2, 2, 128, torch.float16),
    "single_sequence_head_dim_96": ([333], [333], 2, 1, 96, torch.bfloat16),
    "empty_entries": ([64, 0, 130, 0], [64, 0, 200, 0], 2, 2, 64, torch.bfloat16),
    "ragged_gqa_head_dim_256": ([100, 1, 257, 64], [100, 1, 257, 64], 4, 2, 256, torch.bfloat16),
    "cross_lengths_head_dim_192_fp16": ([37, 200, 5], [300, 64, 77], 2, 1, 192, torch.float16),
}


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("name", sorted(VARLEN_CASES))
def test_varlen_vs_eager_fp32(name, causal):
    lens_q, lens_k, H, Hk, D, dtype = VARLEN_CASES[name]
    _run(lens_q, lens_k, H, Hk, D, causal, dtype, seed=len(name))


def test_varlen_sequences_without_queries_or_without_keys():
    """A sequence with keys but no queries gets dK = dV = 0, one with queries but no keys O = 0, LSE = +inf, dQ = 0
    (the reference writes O = 0 for rows whose mask row is empty, interface.py:643)."""
    _run([0, 90, 70, 0], [120, 90, 0, 33], 4, 2, 128, True, seed=3)
    _run([0, 90, 70, 0], [120, 90, 0, 33], 4, 2, 64, False, seed=4)


def test_varlen_equals_fixed_length_operator():
    """Equal lengths: the ragged-batch operator and the fixed-length operator run the same kernels on the same rows,
    so the results agree bit for bit."""
    from flash_sparse_attn import flash_sparse_attn_func
    B, L, H, Hk, D = 3, 320, 4, 2, 128
    out, lse, dq, dk, dv = _run([L] * B, [L] * B, H, Hk, D, True, seed=11)
    q, k, v, do = _make([L] * B, [L] * B, H, Hk, D, torch.bfloat16, 11)
    qf, kf, vf = [t.to(DEV).view(B, L, t.shape[1], D).requires_grad_(True) for t in (q, k, v)]
    of, lf, _ = flash_sparse_attn_func(qf, kf, vf, None, None, None, True, None, None, True)
    of.backward(do.to(DEV).view(B, L, H, D))
    torch.cuda.synchronize()
    assert torch.equal(out.view(B, L, H, D), of.detach())
    assert torch.equal(lse.view(H, B, L).transpose(0, 1), lf)
    assert torch.equal(dq.view(B, L, H, D), qf.grad)
    assert torch.equal(dk.view(B, L, Hk, D), kf.grad)
    assert torch.equal(dv.view(B, L, Hk, D), vf.grad)


def test_varlen_rows_outside_every_sequence_and_loose_max_seqlen():
    """Rows beyond cu_seqlens[-1] belong to no sequence: their gradients are not written (the operator hands back
    what `empty_like` held, so only the rows of sequences are compared), and max_seqlen_* may be loose upper bounds."""
    _run([130, 64, 200], [130, 100, 260], 4, 4, 64, True, seed=5, slack_rows=24, max_slack=100)


@pytest.mark.parametrize("causal", [True, False])
def test_varlen_large_grid_d128(causal):
    """Enough workgroups (batch * heads * ceil(max_seqlen_q / 256) >= 512) for the 256-row, 8-wave forward kernel;
    sequences of very different lengths, some shorter than one workgroup's rows."""
    lens = [1024, 700, 64, 1000, 257, 1, 512, 900]
    _run(lens, lens, 16, 4, 128, causal, seed=6)


def test_varlen_rejects_unsupported_arguments():
    f = _op()
    q, k, v, _ = _make([64], [64], 2, 2, 64, torch.bfloat16, 0)
    qd, kd, vd = [t.to(DEV) for t in (q, k, v)]
    cu = _cu([64]).to(DEV)
    with pytest.raises(RuntimeError, match="block_table"):
        f(qd, kd, vd, cu, cu, 64, 64, block_table=torch.zeros(1, 1, dtype=torch.int32, device=DEV))
    with pytest.raises(RuntimeError, match="softcap"):
        f(qd, kd, vd, cu, cu, 64, 64, softcap=1.0)
    with pytest.raises(RuntimeError, match="int32"):
        f(qd, kd, vd, cu.long(), cu, 64, 64)
    with pytest.raises(RuntimeError, match="same dtype"):
        f(qd, kd.half(), vd, cu, cu, 64, 64)
