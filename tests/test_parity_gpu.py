"""GPU parity tests of the hot path (run with `-m gpu` on an MI355X).

Every case goes through the Python operator, i.e. through the C ABI of libfdma_hip.so, and is
compared with the oracle on identical seeded inputs:
  * small shapes against the C oracle (oracle/fdma_oracle.c, IEEE double on the same bf16 bits);
  * larger shapes against the fp32 safe-eager restatement evaluated on the GPU (the C oracle would
    take minutes), which test_oracle.py ties to the C oracle.
Tolerances (bf16 compute): max-abs error of the output <= 2e-2; gradients within rtol 5e-2 as
defined in _util.assert_grad_close.
"""
import functools
import os

import pytest
import torch

from oracle import c_oracle, eager
from _util import assert_grad_close, assert_out_close, make_inputs, set_compact, topk_keep_mask

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _op():
    from flash_sparse_attn import flash_sparse_attn_func
    return flash_sparse_attn_func


def _to_dev(*ts):
    return [t.to(DEV) if t is not None else None for t in ts]


@pytest.fixture(autouse=True)
def _default_compaction_mode():
    """set_compact picks the path for query-broadcast masks ("0" = tile skipping, "2" = column compaction whenever
    the mask form allows it, None = the library's own cost rule); it is the compact_mode field of every call."""
    set_compact(None)
    yield
    set_compact(None)


def _run_fwd_bwd(q, k, v, mask, bias, causal, scale=None, dout=None, need_grad=True):
    qd, kd, vd, md, bd = _to_dev(q, k, v, mask, bias)
    if need_grad:
        qd, kd, vd = [t.requires_grad_(True) for t in (qd, kd, vd)]
        if bd is not None:
            bd.requires_grad_(True)
    out, lse, _ = _op()(qd, kd, vd, md, bd, scale, causal, None, None, True)
    grads = None
    if need_grad:
        do = torch.ones_like(out) if dout is None else dout.to(DEV)
        out.backward(do)
        grads = (qd.grad, kd.grad, vd.grad, bd.grad if bd is not None else None)
    torch.cuda.synchronize()
    return out.detach(), lse.detach(), grads


def _check_lse(lse, ref):
    ref = ref.to(lse.device)
    assert torch.equal(torch.isinf(lse), torch.isinf(ref)), "empty-row pattern of the LSE differs"
    fin = torch.isfinite(ref)
    if fin.any():
        assert (lse[fin] - ref[fin]).abs().max().item() <= 1e-2
    assert (lse[~fin] > 0).all()


SMALL_CASES = {
    # name: (B, Lq, Lk, H, Hk, D, bias_shape, mask_shape, window, causal)
    "cfg1_mqa_rowbias_topk128": (1, 256, 256, 2, 1, 64, (1, 1, 1, 256), (1, 1, 1, 256), 128, True),
    "plain_noncausal_d128": (1, 256, 256, 2, 2, 128, None, None, None, False),
    "plain_causal_ragged": (2, 300, 300, 4, 2, 128, None, None, None, True),
    "bias_only_per_head": (1, 256, 320, 4, 2, 64, (1, 4, 1, 320), None, None, True),
    "full_mask_full_bias": (2, 200, 264, 4, 2, 64, (2, 4, 200, 264), (2, 4, 200, 264), 64, True),
    "full_bias_kv_heads": (2, 200, 264, 4, 2, 64, (2, 2, 200, 264), (2, 1, 200, 264), 64, True),
    "full_bias_batch_broadcast": (2, 200, 264, 4, 2, 64, (1, 2, 200, 264), (2, 1, 200, 264), 64, True),
    "full_bias_per_head_batch_broadcast": (2, 200, 264, 4, 2, 64, (1, 4, 200, 264), (2, 4, 200, 264), 64, True),
    "row_bias_single_head": (2, 200, 264, 4, 2, 64, (2, 1, 1, 264), (2, 1, 1, 264), 64, False),
    "lq_lt_lk_bottom_right": (1, 100, 333, 2, 2, 128, (1, 2, 1, 333), (1, 1, 100, 333), 100, True),
    "lq_gt_lk_empty_rows": (1, 333, 100, 2, 2, 128, (1, 2, 1, 100), (1, 1, 333, 100), 50, True),
    "head_dim_96": (1, 256, 256, 2, 1, 96, (1, 1, 1, 256), (1, 1, 1, 256), 128, True),
    "head_dim_32": (1, 192, 256, 2, 1, 32, (1, 1, 1, 256), (1, 1, 1, 256), 128, False),
    "tiny": (1, 3, 5, 2, 1, 8, (1, 1, 3, 5), (1, 1, 3, 5), 2, True),
    # query-broadcast masks long enough for the column-compaction path (gathered K / V, scattered grads)
    "compact_gqa_bias_per_qhead": (2, 300, 300, 4, 2, 64, (2, 4, 1, 300), (2, 2, 1, 300), 77, True),
    "compact_lq_lt_lk_shared_mask": (1, 160, 400, 4, 2, 128, (1, 2, 1, 400), (1, 1, 1, 400), 90, True),
    "compact_lq_gt_lk_empty_rows": (1, 400, 200, 2, 2, 64, (1, 2, 1, 200), (1, 2, 1, 200), 50, True),
    "compact_noncausal_mask_only": (2, 257, 391, 4, 4, 128, None, (2, 4, 1, 391), 100, False),
    "compact_batch_broadcast_bias": (2, 256, 256, 4, 2, 64, (1, 2, 1, 256), (2, 2, 1, 256), 64, True),
    "compact_head_dim_96_dense_mask": (1, 200, 200, 2, 1, 96, (1, 1, 1, 200), (1, 1, 1, 200), 200, True),
    "colmask_per_query_head_gqa": (1, 256, 256, 4, 2, 64, (1, 4, 1, 256), (1, 4, 1, 256), 64, True),
    # head dims above 128 (the column-mask kernels at 256; 192 runs in the same instantiation)
    "head_dim_256_gqa_topk": (1, 300, 300, 4, 2, 256, (1, 2, 1, 300), (1, 2, 1, 300), 100, True),
    "head_dim_192_gqa_topk": (2, 200, 264, 4, 2, 192, (2, 4, 1, 264), (2, 1, 1, 264), 64, True),
    "head_dim_256_plain_noncausal": (1, 256, 320, 2, 2, 256, None, None, None, False),
    "head_dim_192_lq_lt_lk_mask_only": (1, 100, 333, 2, 1, 192, None, (1, 1, 1, 333), 120, True),
    "head_dim_256_lq_gt_lk_empty_rows": (1, 333, 100, 2, 2, 256, (1, 2, 1, 100), (1, 2, 1, 100), 50, True),
    "head_dim_136_bias_only": (1, 130, 130, 2, 2, 136, (1, 1, 1, 130), None, None, True),
    # ... and with per-query masks / biases (the general kernels at 256, 32-key tiles / 32-row steps)
    "head_dim_256_full_mask_full_bias": (2, 200, 264, 4, 2, 256, (2, 4, 200, 264), (2, 4, 200, 264), 64, True),
    "head_dim_192_full_bias_kv_heads": (1, 200, 264, 4, 2, 192, (1, 2, 200, 264), (1, 1, 200, 264), 64, True),
    "head_dim_256_full_bias_batch_broadcast": (2, 100, 160, 2, 2, 256, (1, 2, 100, 160), (2, 1, 100, 160), 40, False),
    "head_dim_192_row_bias_full_mask_lq_lt_lk": (1, 100, 333, 2, 2, 192, (1, 2, 1, 333), (1, 1, 100, 333), 100, True),
}


@functools.lru_cache(maxsize=None)
def _small_case(name):
    B, Lq, Lk, H, Hk, D, bshape, mshape, W, causal = SMALL_CASES[name]
    q, k, v, mask, bias = make_inputs(B, Lq, Lk, H, Hk, D, bshape, mshape, W, seed=0)
    dout = torch.randn(B, Lq, H, D, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16)
    fwd = c_oracle.forward(q, k, v, mask, bias, None, causal)
    bwd = c_oracle.backward(q, k, v, dout, mask, bias, None, causal)
    return (q, k, v, mask, bias, dout), fwd, bwd


def _eligible_for_compaction(name):
    mshape, Hk = SMALL_CASES[name][7], SMALL_CASES[name][4]
    bshape = SMALL_CASES[name][6]
    H = SMALL_CASES[name][3]  # (a mask row per query head over grouped kv heads: the forward alone is compacted)
    return (mshape is not None and mshape[2] == 1 and mshape[1] in (1, Hk, H) and (bshape is None or bshape[2] == 1)
            and SMALL_CASES[name][1] > 1)


@pytest.mark.parametrize("compact", ["0", "2"])
@pytest.mark.parametrize("name", list(SMALL_CASES))
def test_forward_backward_vs_c_oracle(name, compact):
    if compact == "2" and not _eligible_for_compaction(name):
        pytest.skip("mask form has no column-compaction path; covered by the other mode")
    set_compact(compact)
    B, Lq, Lk, H, Hk, D, bshape, mshape, W, causal = SMALL_CASES[name]
    (q, k, v, mask, bias, dout), (ro, rl), (rdq, rdk, rdv, rdb) = _small_case(name)
    out, lse, (dq, dk, dv, db) = _run_fwd_bwd(q, k, v, mask, bias, causal, dout=dout)
    assert out.dtype == torch.bfloat16 and out.shape == q.shape and lse.shape == (B, H, Lq)
    assert_out_close(out.cpu(), ro)
    _check_lse(lse.cpu(), rl)
    assert_grad_close(dq.cpu(), rdq, "dq")
    assert_grad_close(dk.cpu(), rdk, "dk")
    assert_grad_close(dv.cpu(), rdv, "dv")
    if bias is not None:
        assert db.shape == bias.shape and db.dtype == bias.dtype
        assert_grad_close(db.cpu(), rdb, "dbias")


@pytest.mark.parametrize("compact", ["0", "2"])
def test_fp16_inputs(compact):
    set_compact(compact)
    q, k, v, mask, bias = make_inputs(1, 256, 256, 2, 1, 64, (1, 1, 1, 256), (1, 1, 1, 256), 128, seed=0, dtype=torch.float16)
    out, lse, (dq, dk, dv, db) = _run_fwd_bwd(q, k, v, mask, bias, True)
    ro, rl = c_oracle.forward(q, k, v, mask, bias, None, True)
    assert out.dtype == torch.float16
    assert_out_close(out.cpu(), ro)
    rdq, rdk, rdv, rdb = c_oracle.backward(q, k, v, torch.ones_like(ro), mask, bias, None, True)
    for g, r, n in ((dq, rdq, "dq"), (dk, rdk, "dk"), (dv, rdv, "dv"), (db, rdb, "dbias")):
        assert_grad_close(g.cpu(), r, n)


@pytest.mark.parametrize("compact", ["0", "2"])
@pytest.mark.parametrize("kind", ["late_bias_bf16", "late_bias_noncausal_bf16", "late_keys_fp16", "huge_scores_fp16", "first_tile_tiny_bf16"])
def test_scores_that_leave_the_range_of_the_first_tile(kind, compact):
    """The column-mask forward takes the reference point of every softmax row from the first key tile it visits and
    checks later tiles against it; a workgroup in which a later score climbs out of that range (2^22 for bf16, 2^18 for
    fp16 above the first tile's maximum) starts again on its classic path.  These inputs force that: keys, or bias
    values, beyond the first tile that score tens of nats above it; fp16 scores too large for the 16-bit pieces that
    carry the reference point (beyond 4e6 in the exp2 domain); and a first tile far BELOW the rest.  (Scaled-up keys
    are tried in fp16 only: with 8-bit mantissas the rounding of the inputs alone moves such outputs by 0.1.)"""
    set_compact(compact)
    dtype = torch.float16 if kind.endswith("fp16") else torch.bfloat16
    B, L, H, Hk, D = 1, 384, 4, 2, 64
    q, k, v, mask, bias = make_inputs(B, L, L, H, Hk, D, (B, Hk, 1, L), (B, Hk, 1, L), 256, seed=41, dtype=dtype)
    causal = kind != "late_bias_noncausal_bf16"
    if kind.startswith("late_keys"):      # keys 200.. score 3x higher and carry +25 of bias: tens of nats above the first 64
        k = k.clone()
        k[:, 200:] = (k[:, 200:].float() * 3).to(dtype)
        bias = bias.clone()
        bias[..., 200:] += 25.0
    elif kind.startswith("late_bias"):
        bias = bias.clone()
        bias[..., 130:] += 60.0
    elif kind == "huge_scores_fp16":      # |q . k| * scale * log2(e) up to about 1e7
        q = (q.float().sign() * 230).to(dtype)
        k = (k.float().sign() * 230).to(dtype)
    else:                                 # the first tile scores far below every other key
        k = k.clone()
        k[:, :64] = (k[:, :64].float() * 0.01).to(dtype)
        bias = bias.clone()
        bias[..., :64] -= 50.0
    scale = 1.0 if kind == "huge_scores_fp16" else None
    out, lse, (dq, dk, dv, db) = _run_fwd_bwd(q, k, v, mask, bias, causal, scale=scale)
    ro, rl = c_oracle.forward(q, k, v, mask, bias, scale, causal)
    if kind == "huge_scores_fp16":
        # fp32 accumulators resolve scores of 4e6 to 0.5: keys that tie in q . k are told apart by their bias only
        # coarsely, so the output is held to the value range and to the LSE, not to the oracle's mixture
        assert torch.isfinite(out.float()).all() and out.float().abs().max() <= v.float().abs().max()
    else:
        assert_out_close(out.cpu(), ro)
    assert torch.equal(torch.isinf(lse.cpu()), torch.isinf(rl))
    fin = torch.isfinite(rl)
    # (the scaled queries are rounded to 16 bits before the MFMAs: the LSE of huge scores carries that relative error)
    assert ((lse.cpu()[fin] - rl[fin]).abs() <= 1e-2 + 3e-3 * rl[fin].abs()).all()
    if kind != "huge_scores_fp16":  # (gradients of 1e7-sized scores overflow the 16-bit outputs; the forward is the point)
        rdq, rdk, rdv, rdb = c_oracle.backward(q, k, v, torch.ones_like(ro), mask, bias, scale, causal)
        for g, r, n in ((dq, rdq, "dq"), (dk, rdk, "dk"), (dv, rdv, "dv"), (db, rdb, "dbias")):
            assert_grad_close(g.cpu(), r, n)


@pytest.mark.parametrize("D", [36, 100])
def test_head_dim_that_is_not_a_multiple_of_8(D):
    """FlashDMAttnFunc pads q, k, v (and dout) with zero columns up to a multiple of 8 and slices the outputs and
    gradients back (flash_sparse_attn_interface.py:415-419, 466-469, 491-493 of the reference); the default scale is
    that of the ORIGINAL head dim."""
    q, k, v, mask, bias = make_inputs(2, 200, 264, 4, 2, D, (2, 2, 1, 264), (2, 2, 1, 264), 96, seed=D)
    for compact in ("0", "2"):
        set_compact(compact)
        out, lse, (dq, dk, dv, db) = _run_fwd_bwd(q, k, v, mask, bias, True)
        assert out.shape == q.shape and dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape
        ro, rl = c_oracle.forward(q, k, v, mask, bias, None, True)
        assert_out_close(out.cpu(), ro)
        _check_lse(lse.cpu(), rl)
        rdq, rdk, rdv, rdb = c_oracle.backward(q, k, v, torch.ones_like(ro), mask, bias, None, True)
        for g, r, n in ((dq, rdq, "dq"), (dk, rdk, "dk"), (dv, rdv, "dv"), (db, rdb, "dbias")):
            assert_grad_close(g.cpu(), r, n)
    # without gradients (the call that skips the autograd node), per-query mask: the general kernels
    qd, kd, vd = _to_dev(q, k, v)
    full = mask.expand(2, 2, 200, 264).contiguous().to(DEV)
    with torch.no_grad():
        out2 = _op()(qd, kd, vd, full, bias.to(DEV), None, True)
    assert out2.shape == q.shape
    assert_out_close(out2.cpu(), ro)


def test_cfg1_reference_plumbing_config():
    """Config 1 of the benchmark: B=1, L=256, H=2, Hkv=1 (MQA), d=64, bias [B,Hkv,1,Lk], mask = top-128
    keys by bias intersected with causal (given both as a full-shape mask and as column mask +
    is_causal), scale 1/8, loss = out.sum()."""
    q, k, v, colmask, bias = make_inputs(1, 256, 256, 2, 1, 64, (1, 1, 1, 256), (1, 1, 1, 256), 128, seed=0)
    full = colmask.expand(1, 1, 256, 256) & torch.tril(torch.ones(256, 256, dtype=torch.bool))
    ro, rl = c_oracle.forward(q, k, v, full, bias, 0.125, True)
    rdq, rdk, rdv, rdb = c_oracle.backward(q, k, v, torch.ones_like(ro), full, bias, 0.125, True)
    for m, compact in ((full, "1"), (colmask, "0"), (colmask, "2")):
        set_compact(compact)
        out, lse, (dq, dk, dv, db) = _run_fwd_bwd(q, k, v, m, bias, True, scale=0.125)
        assert_out_close(out.cpu(), ro)
        _check_lse(lse.cpu(), rl)
        for g, r, n in ((dq, rdq, "dq"), (dk, rdk, "dk"), (dv, rdv, "dv"), (db, rdb, "dbias")):
            assert_grad_close(g.cpu(), r, n)
    assert int(torch.isinf(rl).sum()) > 0, "this config is expected to contain rows without a visible key"


def test_non_contiguous_views_and_mask_bias_key_dim_one():
    # q/k/v given as transposed views of (B,H,L,D) tensors (forward_equivalence.py:175-177 pattern),
    # bias with key dim 1 (expanded by the operator; dbias summed back over keys, interface.py:495-496)
    B, L, H, Hk, D = 2, 192, 4, 2, 64
    g = torch.Generator().manual_seed(3)
    q = torch.randn(B, H, L, D, generator=g).to(torch.bfloat16).transpose(1, 2)
    k = torch.randn(B, Hk, L, D, generator=g).to(torch.bfloat16).transpose(1, 2)
    v = torch.randn(B, Hk, L, D, generator=g).to(torch.bfloat16).transpose(1, 2)
    bias = torch.randn(B, Hk, L, 1, generator=g).to(torch.bfloat16)
    mask = torch.rand(B, 1, L, L, generator=g) > 0.3
    out, lse, (dq, dk, dv, db) = _run_fwd_bwd(q, k, v, mask, bias, True)
    ro, _ = c_oracle.forward(q, k, v, mask, bias.expand(B, Hk, L, L), None, True)
    assert_out_close(out.cpu(), ro)
    rdq, rdk, rdv, rdb = c_oracle.backward(q, k, v, torch.ones_like(ro), mask, bias.expand(B, Hk, L, L), None, True)
    assert db.shape == bias.shape
    assert_grad_close(dq.cpu(), rdq, "dq")
    assert_grad_close(dk.cpu(), rdk, "dk")
    assert_grad_close(dv.cpu(), rdv, "dv")
    # rows of dS sum to zero, so the exact dbias of a key-broadcast bias is 0; what the operator returns
    # is the sum over keys of bf16-rounded dS elements: rounding noise of about sqrt(L) half-ulps
    assert rdb.sum(-1, keepdim=True).abs().max() < 1e-4
    noise = 3.0 * (L ** 0.5) * 2.0 ** -9 * rdb.abs().max().item()
    worst = db.float().abs().max().item()
    assert worst <= noise, f"key-broadcast dbias {worst:.3e} exceeds rounding noise bound {noise:.3e}"


def test_fully_masked_tiles_are_skipped_and_rows_without_keys_give_zero():
    # block-structured mask: whole 64-key tiles masked out, plus a band of query rows with nothing kept
    B, L, H, Hk, D = 1, 512, 2, 2, 128
    q, k, v, _, bias = make_inputs(B, L, L, H, Hk, D, (B, Hk, 1, L), None, seed=5)
    mask = torch.zeros(B, 1, L, L, dtype=torch.bool)
    mask[..., 64:128] = True
    mask[..., 320:384] = True
    mask[:, :, 200:260, :] = False
    out, lse, (dq, dk, dv, db) = _run_fwd_bwd(q, k, v, mask, bias, False)
    ro, rl = c_oracle.forward(q, k, v, mask, bias, None, False)
    assert_out_close(out.cpu(), ro)
    _check_lse(lse.cpu(), rl)
    assert torch.equal(out[:, 200:260].cpu(), torch.zeros(B, 60, H, D, dtype=torch.bfloat16))
    rdq, rdk, rdv, rdb = c_oracle.backward(q, k, v, torch.ones_like(ro), mask, bias, None, False)
    for g, r, n in ((dq, rdq, "dq"), (dk, rdk, "dk"), (dv, rdv, "dv"), (db, rdb, "dbias")):
        assert_grad_close(g.cpu(), r, n)
    assert torch.equal(dk[:, :64].cpu(), torch.zeros(B, 64, Hk, D, dtype=torch.bfloat16))  # keys nobody keeps


def test_column_mask_with_an_all_dropped_pair_and_late_first_key():
    """Query-broadcast mask whose (batch 0, kv head 1) row keeps nothing and whose other rows keep no key
    before column 150: that pair's outputs and gradients are exactly zero, rows that see no kept key give
    O = 0 / LSE = +inf, and everything else matches the oracle."""
    set_compact("2")
    B, L, H, Hk, D = 2, 320, 4, 2, 64
    q, k, v, mask, bias = make_inputs(B, L, L, H, Hk, D, (B, Hk, 1, L), (B, Hk, 1, L), 60, seed=5)
    mask[..., :150] = False
    mask[0, 1] = False
    dout = torch.randn(B, L, H, D, generator=torch.Generator().manual_seed(6)).to(torch.bfloat16)
    out, lse, (dq, dk, dv, db) = _run_fwd_bwd(q, k, v, mask, bias, True, dout=dout)
    ro, rl = c_oracle.forward(q, k, v, mask, bias, None, True)
    assert_out_close(out.cpu(), ro)
    _check_lse(lse.cpu(), rl)
    assert torch.isinf(lse[0, 2:]).all() and torch.isinf(lse[:, :, :150]).all()
    assert not out[0, :, 2:].any() and not dq[0, :, 2:].any()
    assert not dk[0, :, 1].any() and not dv[0, :, 1].any() and not db[0, 1].any()
    assert not dk[:, :150].any() and not dv[:, :150].any() and not db[..., :150].any()
    rdq, rdk, rdv, rdb = c_oracle.backward(q, k, v, dout, mask, bias, None, True)
    for g, r, n in ((dq, rdq, "dq"), (dk, rdk, "dk"), (dv, rdv, "dv"), (db, rdb, "dbias")):
        assert_grad_close(g.cpu(), r, n)


def test_seqlen_k_zero_and_no_grad_path():
    q = torch.randn(1, 16, 2, 64, dtype=torch.bfloat16, device=DEV)
    k = torch.empty(1, 0, 2, 64, dtype=torch.bfloat16, device=DEV)
    out, lse, _ = _op()(q, k, k, None, None, None, False, None, None, True)
    assert torch.equal(out, torch.zeros_like(out)) and torch.isinf(lse).all() and (lse > 0).all()
    with torch.no_grad():
        q2 = torch.randn(1, 64, 2, 64, dtype=torch.bfloat16, device=DEV)
        o = _op()(q2, q2, q2, is_causal=True)
    assert o.shape == q2.shape and not o.requires_grad


@pytest.mark.parametrize("form", ["per_query_mask", "column_mask_compacted"])
def test_deterministic_rerun_is_bit_identical(form):
    if form == "per_query_mask":
        q, k, v, mask, bias = make_inputs(2, 384, 384, 4, 2, 64, (2, 2, 384, 384), (2, 2, 384, 384), 96, seed=7)
    else:  # dK / dV blocks split over several workgroups, partial sums folded in a fixed order
        set_compact("2")
        q, k, v, mask, bias = make_inputs(2, 640, 640, 4, 2, 64, (2, 4, 1, 640), (2, 2, 1, 640), 300, seed=7)
    a = _run_fwd_bwd(q, k, v, mask, bias, True)
    b = _run_fwd_bwd(q, k, v, mask, bias, True)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    for x, y in zip(a[2], b[2]):
        assert torch.equal(x, y)


MID_CASES = {
    # scaled-down versions of benchmark configs 2-4 (same head structure, shorter sequences),
    # checked against the fp32 eager restatement on the GPU
    "cfg2_like_gqa4_d128": (1, 2048, 2048, 8, 2, 128, (1, 2, 1, 2048), (1, 2, 1, 2048), 512, True),
    "cfg3_like_full_dbias_d64": (2, 1024, 1024, 4, 4, 64, (2, 4, 1024, 1024), (2, 4, 1024, 1024), 256, True),
    "cfg4_like_sparse_d128": (1, 4096, 4096, 4, 1, 128, (1, 1, 1, 4096), (1, 1, 1, 4096), 128, True),
}


@pytest.mark.parametrize("name", list(MID_CASES))
def test_mid_size_vs_eager_fp32(name):
    B, Lq, Lk, H, Hk, D, bshape, mshape, W, causal = MID_CASES[name]
    q, k, v, mask, bias = make_inputs(B, Lq, Lk, H, Hk, D, bshape, mshape, W, seed=11)
    out, lse, (dq, dk, dv, db) = _run_fwd_bwd(q, k, v, mask, bias, causal)
    qd, kd, vd, md, bd = _to_dev(q, k, v, mask, bias)
    ro, rdq, rdk, rdv, rdb = eager.attention_forward_backward(qd, kd, vd, md, bd, None, causal)
    assert_out_close(out, ro)
    for g, r, n in ((dq, rdq, "dq"), (dk, rdk, "dk"), (dv, rdv, "dv"), (db, rdb, "dbias")):
        assert_grad_close(g, r, n)


LARGE_GRID_CASES = {
    # name: (B, Lq, Lk, H, Hk, D, window, causal, dtype) -- batch * heads * ceil(Lq / 256) >= 512 and d = 128
    "bf16_causal_ragged": (4, 1000, 1090, 32, 8, 128, 300, True, torch.bfloat16),
    "fp16_noncausal_lq_lt_lk": (6, 520, 1090, 32, 8, 128, 200, False, torch.float16),
    "bf16_causal_lq_gt_lk_empty_rows": (4, 1024, 700, 32, 4, 128, 150, True, torch.bfloat16),
}


@pytest.mark.parametrize("compact", ["0", "2"])
@pytest.mark.parametrize("name", list(LARGE_GRID_CASES))
def test_large_grid_256_row_workgroups_vs_eager_fp32(name, compact):
    """d = 128 problems whose grid is large enough for the forward to take its 256-row, 8-wave workgroups (split
    K / V staging roles), on the original and on the compacted key axis; ragged lengths so that the last query
    block and the last key tile are partial, both dtypes, causal with empty rows and non-causal."""
    set_compact(compact)
    B, Lq, Lk, H, Hk, D, W, causal, dtype = LARGE_GRID_CASES[name]
    q, k, v, mask, bias = make_inputs(B, Lq, Lk, H, Hk, D, (B, Hk, 1, Lk), (B, Hk, 1, Lk), W, seed=5)
    q, k, v, bias = [t.to(dtype) for t in (q, k, v, bias)]
    out, lse, (dq, dk, dv, db) = _run_fwd_bwd(q, k, v, mask, bias, causal)
    qd, kd, vd, md, bd = _to_dev(q, k, v, mask, bias)
    ro, rdq, rdk, rdv, rdb = eager.attention_forward_backward(qd, kd, vd, md, bd, None, causal)
    assert_out_close(out, ro)
    _, rl = eager.attention_forward(qd, kd, vd, md, bd, None, causal)
    _check_lse(lse, rl)
    for g, r, n in ((dq, rdq, "dq"), (dk, rdk, "dk"), (dv, rdv, "dv"), (db, rdb, "dbias")):
        assert_grad_close(g, r, n)


@pytest.mark.parametrize("causal", [True, False])
def test_per_query_mask_large_grid_d128_vs_eager_fp32(causal):
    """Per-query mask and bias at d = 128 on a grid large enough (batch * heads * ceil(Lq / 256) >= 512) for the
    general forward kernel's 256-row, 8-wave workgroups; ragged lengths, GQA, bias per kv head."""
    B, Lq, Lk, H, Hk, D, W = 8, 1000, 1090, 16, 4, 128, 300
    q, k, v, mask, bias = make_inputs(B, Lq, Lk, H, Hk, D, (B, Hk, Lq, Lk), (B, H, Lq, Lk), W, seed=9)
    out, lse, (dq, dk, dv, db) = _run_fwd_bwd(q, k, v, mask, bias, causal)
    qd, kd, vd, md, bd = _to_dev(q, k, v, mask, bias)
    ro, rdq, rdk, rdv, rdb = eager.attention_forward_backward(qd, kd, vd, md, bd, None, causal)
    assert_out_close(out, ro)
    _, rl = eager.attention_forward(qd, kd, vd, md, bd, None, causal)
    _check_lse(lse, rl)
    for g, r, n in ((dq, rdq, "dq"), (dk, rdk, "dk"), (dv, rdv, "dv"), (db, rdb, "dbias")):
        assert_grad_close(g, r, n)


def test_cfg2_full_size_forward_properties():
    """Config 2 at full size (B=1, L=8192, H=32, Hkv=8, d=128, bias [1,8,1,8192], top-2048 ∩ causal).
    Checked through size-independent properties plus an eager check of one KV group:
      * V = 1  =>  O = 1 on rows with a visible key, 0 elsewhere (rows of P sum to one);
      * a per-head constant added to the bias leaves O unchanged and shifts the LSE by it;
      * the 4 query heads of KV group 0 against fp32 eager."""
    B, L, H, Hk, D, W = 1, 8192, 32, 8, 128, 2048
    q, k, v, mask, bias = make_inputs(B, L, L, H, Hk, D, (B, Hk, 1, L), (B, Hk, 1, L), W, seed=0)
    qd, kd, vd, md, bd = _to_dev(q, k, v, mask, bias)
    f = _op()
    out, lse, _ = f(qd, kd, vd, md, bd, None, True, None, None, True)
    ones, _, _ = f(qd, kd, torch.ones_like(vd), md, bd, None, True, None, None, True)
    nonempty = torch.isfinite(lse).transpose(1, 2)[..., None].expand_as(ones)  # (B, L, H, 1)
    # (the probabilities are rounded to 16 bits for the matrix pipe, their fp32 sum is not: one rounding step of slack)
    assert (ones[nonempty].float() - 1.0).abs().max().item() <= 2.0 ** -7
    assert torch.equal(ones[~nonempty], torch.zeros_like(ones[~nonempty]))
    # the shift must not itself be rounded: quantise the bias to multiples of 1/32 inside (-2, 2), so that bias and
    # bias + 2 are both exact in bf16 and the two calls see the same scores up to the constant
    bq = (torch.round(bd.float() * 32) / 32).clamp_(-1.96875, 1.96875).to(bd.dtype)
    base, lse_b, _ = f(qd, kd, vd, md, bq, None, True, None, None, True)
    shifted, lse_s, _ = f(qd, kd, vd, md, bq + 2.0, None, True, None, None, True)
    assert torch.equal((bq + 2.0).float(), bq.float() + 2.0)
    assert (shifted.float() - base.float()).abs().max().item() <= 2e-2
    fin = torch.isfinite(lse_b)
    assert (lse_s[fin] - lse_b[fin] - 2.0).abs().max().item() <= 2e-2
    ro, rl = eager.attention_forward(qd[:, :, :4], kd[:, :, :1], vd[:, :, :1], md[:, :1], bd[:, :1], None, True)
    assert_out_close(out[:, :, :4], ro)
    _check_lse(lse[:, :4], rl)


DECODE_CASES = {
    # name: (B, Lk, H, Hk, D, mask heads, bias heads, window)
    "gqa4_topk": (2, 4096, 8, 2, 128, 2, 2, 256),
    "mqa_per_head_mask": (1, 1000, 4, 1, 64, 4, 4, 100),
    "mha_no_mask": (2, 777, 4, 4, 128, None, 1, None),
    "gqa8_shared_mask": (1, 3000, 16, 2, 128, 1, 16, 64),
    "short": (3, 40, 8, 2, 64, 2, 2, 7),
    # 5000 keys per workgroup, all kept: the kept-key list (4096 entries) is worked off in two rounds
    "dense_list_overflow": (8, 20000, 8, 8, 64, None, 1, None),
    "gqa16_per_head_bias": (1, 5000, 32, 2, 128, 2, 32, 300),
    "odd_head_dim": (2, 1500, 6, 2, 40, 2, 2, 99),
    # 40 query heads on one kv head: two workgroups per split (32 + 8 columns)
    "mqa40_two_column_chunks": (1, 2000, 40, 1, 64, 1, 1, 300),
    "mqa40_per_head_mask_and_bias": (1, 1200, 40, 1, 128, 40, 40, 200),
    # head dims above 128: the split-KV kernel's instantiation at 256
    "gqa4_head_dim_256": (2, 1000, 8, 2, 256, 2, 2, 128),
    "mha_head_dim_192_no_mask": (1, 300, 2, 2, 192, None, 1, None),
    "gqa4_head_dim_256_long": (1, 9000, 8, 2, 256, 2, 8, 700),
    "mqa_head_dim_136_per_head_mask": (2, 2100, 4, 1, 136, 4, 1, 150),
}


@pytest.mark.parametrize("name", list(DECODE_CASES))
def test_decode_vs_c_oracle(name):
    B, Lk, H, Hk, D, hm, hb, W = DECODE_CASES[name]
    q, k, v, mask, bias = make_inputs(B, 1, Lk, H, Hk, D, (B, hb, 1, Lk), (B, hm, 1, Lk) if hm else None, W, seed=13)
    qd, kd, vd, md, bd = _to_dev(q, k, v, mask, bias)
    out, lse, _ = _op()(qd, kd, vd, md, bd, None, False, None, None, True)
    ro, rl = c_oracle.forward(q, k, v, mask, bias, None, False)
    assert_out_close(out.cpu(), ro)
    _check_lse(lse.cpu(), rl)
    # is_causal is a no-op for a single query token (flash_api.cpp:441)
    out_c = _op()(qd, kd, vd, md, bd, None, True)
    assert torch.equal(out_c, out)


def test_cfg5_full_size_decode():
    """Config 5: B=8, Lq=1, Lk=65536, H=32, Hkv=8, d=128, bias [8,8,1,65536], top-2048, no causal."""
    B, Lk, H, Hk, D, W = 8, 65536, 32, 8, 128, 2048
    q, k, v, mask, bias = make_inputs(B, 1, Lk, H, Hk, D, (B, Hk, 1, Lk), (B, Hk, 1, Lk), W, seed=0)
    qd, kd, vd, md, bd = _to_dev(q, k, v, mask, bias)
    out, lse, _ = _op()(qd, kd, vd, md, bd, None, False, None, None, True)
    ro, rl = eager.attention_forward(qd, kd, vd, md, bd, None, False)
    assert_out_close(out, ro)
    _check_lse(lse, rl)


SPLIT_PLAN_CASES = {
    # name: (B, Lq, Lk, H, Hk, D, window, causal) -- few 128-key blocks after compaction, so the dK/dV kernel splits
    # them over query heads and query segments; the (batch, kv head) pairs are dealt to 8 / 4 / 2 / 1 lists per pair
    "three_pairs": (3, 1500, 1500, 4, 1, 64, 700, True),
    "six_pairs_gqa2": (1, 2000, 2000, 12, 6, 128, 900, True),
    "five_pairs_mha_noncausal": (5, 1024, 1024, 1, 1, 64, 500, False),
    "two_pairs_gqa8": (1, 6000, 6000, 16, 2, 128, 1500, True),
    "short_queries": (2, 700, 3000, 8, 2, 64, 1000, True),
    "sixteen_pairs_one_block": (2, 900, 900, 16, 8, 64, 100, True),
}


@pytest.mark.parametrize("name", list(SPLIT_PLAN_CASES))
def test_compacted_backward_split_plans_vs_eager_fp32(name):
    set_compact("2")
    B, Lq, Lk, H, Hk, D, W, causal = SPLIT_PLAN_CASES[name]
    q, k, v, mask, bias = make_inputs(B, Lq, Lk, H, Hk, D, (B, Hk, 1, Lk), (B, Hk, 1, Lk), W, seed=11)
    out, lse, (dq, dk, dv, db) = _run_fwd_bwd(q, k, v, mask, bias, causal)
    qd, kd, vd, md, bd = _to_dev(q, k, v, mask, bias)
    ro, rdq, rdk, rdv, rdb = eager.attention_forward_backward(qd, kd, vd, md, bd, None, causal)
    assert_out_close(out, ro)
    for g, r, n in ((dq, rdq, "dq"), (dk, rdk, "dk"), (dv, rdv, "dv"), (db, rdb, "dbias")):
        assert_grad_close(g, r, n)
    # a second call must give the same bits (fixed-order reduction of the parts)
    out2, _, (dq2, dk2, dv2, db2) = _run_fwd_bwd(q, k, v, mask, bias, causal)
    assert torch.equal(dk, dk2) and torch.equal(dv, dv2) and torch.equal(db, db2) and torch.equal(dq, dq2)


# Numbers of kept keys around the 32-key tiles of the compacted dQ kernel at head dim 128 (one, two, three, four tiles,
# full and partial last tiles): its tiles are fetched two ahead through three LDS stages, and the first iterations
# and the tiles fetched past the last one are what a short key list exercises.
@pytest.mark.parametrize("W", [1, 2, 31, 32, 33, 63, 64, 65, 96, 97, 129])
@pytest.mark.parametrize("causal", [False, True])
def test_compacted_backward_with_few_kept_keys_d128_vs_eager_fp32(W, causal):
    set_compact("2")
    B, Lq, Lk, H, Hk, D = 2, 200, 300, 4, 2, 128
    q, k, v, mask, bias = make_inputs(B, Lq, Lk, H, Hk, D, (B, Hk, 1, Lk), (B, Hk, 1, Lk), W, seed=100 + W)
    assert int(mask[0, 0, 0].sum()) == W
    out, lse, (dq, dk, dv, db) = _run_fwd_bwd(q, k, v, mask, bias, causal)
    qd, kd, vd, md, bd = _to_dev(q, k, v, mask, bias)
    ro, rdq, rdk, rdv, rdb = eager.attention_forward_backward(qd, kd, vd, md, bd, None, causal)
    assert_out_close(out, ro)
    for g, r, n in ((dq, rdq, "dq"), (dk, rdk, "dk"), (dv, rdv, "dv"), (db, rdb, "dbias")):
        assert_grad_close(g, r, n)


def test_decode_long_splits_and_fp16():
    """One workgroup per (batch entry, kv head) walks 40 000 keys: three mask fetches of 16 384 keys each.  fp16."""
    B, Lk, H, Hk, D, W = 32, 40000, 16, 8, 64, 700
    g = torch.Generator(device=DEV).manual_seed(5)
    qd = torch.randn(B, 1, H, D, device=DEV, generator=g).to(torch.float16)
    kd = torch.randn(B, Lk, Hk, D, device=DEV, generator=g).to(torch.float16)
    vd = torch.randn(B, Lk, Hk, D, device=DEV, generator=g).to(torch.float16)
    bd = torch.randn(B, Hk, 1, Lk, device=DEV, generator=g).to(torch.float16)
    md = torch.zeros_like(bd, dtype=torch.bool).scatter_(-1, bd.float().topk(W, dim=-1).indices, True)
    out, lse, _ = _op()(qd, kd, vd, md, bd, None, False, None, None, True)
    ro, rl = eager.attention_forward(qd, kd, vd, md, bd, None, False)
    assert_out_close(out, ro)
    _check_lse(lse, rl)


def test_decode_rows_far_apart():
    """K and V rows 131 072 elements apart (views into wider buffers): the gather needs 64-bit offsets."""
    B, Lk, H, Hk, D, W = 1, 3000, 8, 2, 128, 500
    q, k, v, mask, bias = make_inputs(B, 1, Lk, H, Hk, D, (B, Hk, 1, Lk), (B, Hk, 1, Lk), W, seed=21)
    qd, kd, vd, md, bd = _to_dev(q, k, v, mask, bias)
    wide_k = torch.zeros(B, Lk, 131072, dtype=kd.dtype, device=DEV)
    wide_v = torch.zeros(B, Lk, 131072, dtype=vd.dtype, device=DEV)
    wide_k[..., : Hk * D] = kd.reshape(B, Lk, Hk * D)
    wide_v[..., : Hk * D] = vd.reshape(B, Lk, Hk * D)
    kw = wide_k[..., : Hk * D].view(B, Lk, Hk, D)
    vw = wide_v[..., : Hk * D].view(B, Lk, Hk, D)
    assert kw.stride(1) == 131072 and kw.stride(-1) == 1
    out, lse, _ = _op()(qd, kw, vw, md, bd, None, False, None, None, True)
    ref, ref_lse, _ = _op()(qd, kd, vd, md, bd, None, False, None, None, True)
    assert torch.equal(out, ref) and torch.equal(lse, ref_lse)
    ro, rl = c_oracle.forward(q, k, v, mask, bias, None, False)
    assert_out_close(out.cpu(), ro)


@pytest.mark.parametrize("name", ["gqa4_topk", "mqa40_two_column_chunks", "gqa16_per_head_bias", "gqa4_head_dim_256_long", "short"])
def test_decode_in_one_launch_equals_the_two_launch_form(name):
    """With arrival counters (fdma_fwd_args.counters) the last workgroup of a (batch entry, kv head) merges the splits in
    the decode launch itself; without them the merge is a second launch.  Same bits either way, the counters are zero
    again afterwards, and the same buffer serves the next call."""
    from flash_sparse_attn import _cabi

    B, Lk, H, Hk, D, hm, hb, W = DECODE_CASES[name]
    q, k, v, mask, bias = make_inputs(B, 1, Lk, H, Hk, D, (B, hb, 1, Lk), (B, hm, 1, Lk) if hm else None, W, seed=13)
    from flash_sparse_attn.flash_sparse_attn_interface import _pad_key_dim

    qd, kd, vd, md, bd = _to_dev(q, k, v, mask, bias)
    md, bd = _pad_key_dim(md, Lk, 16), _pad_key_dim(bd, Lk, 8)  # (rows of whole 16-byte vectors, as the operator makes them)
    stream = _cabi.current_stream(qd.device)

    def call(counters):
        out = torch.full_like(qd, float("nan"))
        lse = torch.full((B, H, 1), float("nan"), dtype=torch.float32, device=DEV)
        a = _cabi.FwdArgs()
        _cabi.fill_fwd(a, qd, kd, vd, md, bd, out, lse, D ** -0.5, False, 0.0)
        need = _cabi.lib.fdma_fwd_workspace_bytes(a)
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device=DEV)
        a.workspace, a.workspace_bytes = ws.data_ptr(), need
        if counters is not None:
            a.counters, a.counters_bytes = counters.data_ptr(), counters.numel() * 4
        assert _cabi.lib.fdma_fwd(a, stream) == 0, _cabi.last_error()
        torch.cuda.synchronize()
        return out, lse, need

    two_out, two_lse, need = call(None)
    a = _cabi.FwdArgs()
    _cabi.fill_fwd(a, qd, kd, vd, md, bd, two_out, two_lse, D ** -0.5, False, 0.0)
    cbytes = _cabi.lib.fdma_fwd_counter_bytes(a)
    if need == 0:  # a single split: nothing to merge, no counters asked for
        assert cbytes == 0
        return
    assert cbytes >= 4 * B * Hk
    counters = torch.zeros(cbytes // 4, dtype=torch.int32, device=DEV)
    for _ in range(3):
        one_out, one_lse, _ = call(counters)
        assert torch.equal(one_out, two_out) and torch.equal(one_lse, two_lse)
        assert int(counters.abs().max()) == 0
    ro, rl = c_oracle.forward(q, k, v, mask, bias, None, False)
    assert_out_close(one_out.cpu(), ro)
    _check_lse(one_lse.cpu(), rl)
    # counters that are too small are refused with a message
    a.workspace_bytes = need
    a.workspace = torch.empty(need, dtype=torch.uint8, device=DEV).data_ptr()
    a.counters, a.counters_bytes = counters.data_ptr(), 4
    if cbytes > 4:
        assert _cabi.lib.fdma_fwd(a, stream) == -3 and "arrival counters too small" in _cabi.last_error()


def test_direct_c_abi_call_without_the_python_operator():
    """Calls fdma_fwd through ctypes exactly as a foreign-language binding would."""
    from flash_sparse_attn import _cabi

    q, k, v, mask, bias = make_inputs(1, 128, 128, 2, 1, 64, (1, 1, 1, 128), (1, 1, 1, 128), 64, seed=17)
    qd, kd, vd, md, bd = _to_dev(q, k, v, mask, bias)
    out = torch.empty_like(qd)
    lse = torch.empty(1, 2, 128, dtype=torch.float32, device=DEV)
    a = _cabi.FwdArgs()
    _cabi.fill_fwd(a, qd, kd, vd, md, bd, out, lse, 0.125, True, 0.0)
    a.compact_mode = _cabi.COMPACT_NEVER
    assert _cabi.lib.fdma_fwd_workspace_bytes(a) == 0
    a.compact_mode = _cabi.COMPACT_ALWAYS
    need = _cabi.lib.fdma_fwd_workspace_bytes(a)
    assert need > 0
    if need:  # a caller that ignores the scratch request gets an error code and a message, not a fault
        assert _cabi.lib.fdma_fwd(a, _cabi.current_stream(qd.device)) == -3
        assert "workspace too small" in _cabi.last_error()
        ws = torch.empty(need, dtype=torch.uint8, device=DEV)
        a.workspace, a.workspace_bytes = ws.data_ptr(), need
    assert _cabi.lib.fdma_fwd(a, _cabi.current_stream(qd.device)) == 0, _cabi.last_error()
    torch.cuda.synchronize()
    ro, rl = c_oracle.forward(q, k, v, mask, bias, 0.125, True)
    assert_out_close(out.cpu(), ro)
    _check_lse(lse.cpu(), rl)


@pytest.mark.parametrize("form", ["column_bias_batch_broadcast", "per_query_bias_one_head"])
def test_deterministic_flag_with_shared_dbias(form):
    """dBias elements shared by several workgroups (bias broadcast over the batch, or one bias head for several kv
    heads) are summed in a fixed order when deterministic=True: reruns agree bit for bit, and the values match the
    oracle like the default (atomic) path."""
    if form == "column_bias_batch_broadcast":
        q, k, v, mask, bias = make_inputs(3, 300, 300, 4, 2, 64, (1, 2, 1, 300), (3, 2, 1, 300), 100, seed=31)
    else:
        q, k, v, mask, bias = make_inputs(2, 200, 264, 4, 2, 64, (2, 1, 200, 264), (2, 1, 200, 264), 64, seed=32)
    qd, kd, vd, md, bd = _to_dev(q, k, v, mask, bias)
    runs = []
    for _ in range(3):
        qg, kg, vg, bg = [t.clone().requires_grad_(True) for t in (qd, kd, vd, bd)]
        out = _op()(qg, kg, vg, md, bg, None, True, None, True)  # deterministic=True
        out.backward(torch.ones_like(out))
        torch.cuda.synchronize()
        runs.append((qg.grad, kg.grad, vg.grad, bg.grad))
    for other in runs[1:]:
        for a, b in zip(runs[0], other):
            assert torch.equal(a, b)
    assert runs[0][3].shape == bias.shape
    rdq, rdk, rdv, rdb = c_oracle.backward(q, k, v, torch.ones_like(q), mask, bias, None, True)
    for g, r, n in zip(runs[0], (rdq, rdk, rdv, rdb), ("dq", "dk", "dv", "dbias")):
        assert_grad_close(g.cpu(), r, n)


def test_two_host_threads_on_two_streams():
    """The library keeps no mutable state besides a thread-local error string: two host threads, each on its own
    stream (default priority), run different problems at the same time and both get the single-threaded result."""
    import threading

    cases = [make_inputs(2, 300, 300, 4, 2, 128, (2, 2, 1, 300), (2, 2, 1, 300), 100, seed=21),
             make_inputs(1, 200, 264, 4, 2, 64, (1, 4, 200, 264), (1, 4, 200, 264), 64, seed=22)]
    refs = [_run_fwd_bwd(*c, True) for c in cases]
    results, errors = [None, None], []

    def worker(n):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for _ in range(5):
                    results[n] = _run_fwd_bwd(*cases[n], True)
            stream.synchronize()
        except Exception as e:  # surfaced below: an exception in a thread would otherwise pass silently
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(n,)) for n in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for (out, lse, grads), (ro, rl, rgrads) in zip(results, refs):
        assert torch.equal(out, ro) and torch.equal(lse, rl)
        for g, r in zip(grads, rgrads):
            assert torch.equal(g, r)


@pytest.mark.skip(reason="the one attempt ended in a host-side segmentation fault inside hipStreamEndCapture "
                         "(torch.cuda.graph exit) before any replay; the cause is not established, so capture of the "
                         "operator is unsupported for now (the library refuses a capturing stream, see the next test) and this "
                         "case stays off the GPU until the cause is")
@pytest.mark.parametrize("compact", ["0", "2"])
def test_graph_capture_and_replay_matches_eager(compact):
    """Forward + backward captured into a HIP graph (the library launches only kernels: no memset nodes, no host
    synchronisation, scratch comes from torch's graph-private pool) and replayed several times with eager work in
    between; every replay must reproduce the eager result bit for bit."""
    set_compact(compact)
    q, k, v, mask, bias = make_inputs(2, 512, 512, 4, 2, 64, (2, 2, 1, 512), (2, 2, 1, 512), 100, seed=3)
    qd, kd, vd, md, bd = _to_dev(q, k, v, mask, bias)
    qd, kd, vd, bd = [t.requires_grad_(True) for t in (qd, kd, vd, bd)]
    f = _op()

    def step():
        out = f(qd, kd, vd, md, bd, None, True)
        grads = torch.autograd.grad(out, (qd, kd, vd, bd), torch.ones_like(out))
        return (out,) + grads

    ref = [t.clone() for t in step()]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    for rep in range(3):
        for t in outs:
            t.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(outs, ref):
            assert torch.equal(got, want), f"replay {rep} differs from the eager result"
        _ = (qd.detach() @ qd.detach().transpose(-1, -2)).sum().item()  # unrelated eager work between replays

def test_a_capturing_stream_is_refused_with_a_clear_error():
    """Capture of the operator is unsupported: a call on a stream that is being captured raises RuntimeError before
    anything is launched (the graph stays empty), and the operator works as before once the capture is closed."""
    q, k, v, mask, bias = make_inputs(1, 128, 128, 4, 2, 64, (1, 2, 1, 128), (1, 2, 1, 128), 64, seed=5)
    qd, kd, vd, md, bd = _to_dev(q, k, v, mask, bias)
    f = _op()
    want = f(qd, kd, vd, md, bd, None, True)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    import warnings
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")  # torch warns that the captured graph is empty
        with torch.cuda.graph(graph):
            with pytest.raises(RuntimeError, match="captured into a HIP graph"):
                f(qd, kd, vd, md, bd, None, True)
    torch.cuda.synchronize()
    assert torch.equal(f(qd, kd, vd, md, bd, None, True), want)


def test_operator_traces_under_torch_compile():
    """The custom ops carry fake implementations, so the operator can sit inside a compiled region (aot_eager
    backend: traces forward and backward with fake tensors, then runs the real kernels)."""
    q, k, v, mask, bias = make_inputs(1, 256, 256, 4, 2, 64, (1, 2, 1, 256), (1, 2, 1, 256), 64, seed=4)
    qd, kd, vd, md, bd = _to_dev(q, k, v, mask, bias)
    f = _op()

    def fn(q_, k_, v_, b_):
        return f(q_ * 1.0, k_, v_, md, b_, None, True).float().sum()

    qe, ke, ve, be = [t.clone().requires_grad_(True) for t in (qd, kd, vd, bd)]
    fn(qe, ke, ve, be).backward()
    qc, kc, vc, bc = [t.clone().requires_grad_(True) for t in (qd, kd, vd, bd)]
    torch.compile(fn, backend="aot_eager", fullgraph=True)(qc, kc, vc, bc).backward()
    for a, b_ in ((qe, qc), (ke, kc), (ve, vc), (be, bc)):
        assert torch.equal(a.grad, b_.grad)
