"""GPU tests (`-m gpu`) of the streaming form of the compacted forward (head dim 128): resident workgroups that fetch
"tile images" written by the compaction pre-pass straight into LDS (fdma_fwd_stream.hip, compact_image_kernel).

By default that form takes problems of at least 512 (256-row query block, head) items; here the threshold is lowered to
1 (fdma_set_stream_min_items) so that small problems -- which the C oracle can follow -- go through it: forward and
backward (the backward then runs on a forward workspace that holds images instead of row-major copies) against the C
oracle or the fp32 eager restatement, against the other form of the compacted forward and against tile skipping, with
lists handed over by the mask builder, and on inputs that force the redo path.
Tolerances: out max-abs <= 2e-2; gradients as in _util.assert_grad_close (rtol 5e-2).
"""
import pytest
import torch

from oracle import c_oracle, eager
from _util import OUT_ATOL, assert_grad_close, assert_out_close, make_inputs, set_compact

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(autouse=True)
def _stream_everything():
    from flash_sparse_attn import _cabi
    before = _cabi.stream_min_items(1)
    set_compact("2")
    yield
    _cabi.stream_min_items(before)
    set_compact(None)


def _run(q, k, v, mask, bias, causal, scale=None, dout=None):
    from flash_sparse_attn import flash_sparse_attn_func
    qd, kd, vd = [t.to(DEV).requires_grad_(True) for t in (q, k, v)]
    md = mask.to(DEV) if mask is not None else None
    bd = bias.to(DEV).requires_grad_(True) if bias is not None else None
    out, lse, _ = flash_sparse_attn_func(qd, kd, vd, md, bd, scale, causal, None, None, True)
    out.backward(torch.ones_like(out) if dout is None else dout.to(DEV))
    torch.cuda.synchronize()
    return out.detach(), lse.detach(), (qd.grad, kd.grad, vd.grad, bd.grad if bd is not None else None)


def _check_lse(lse, ref):
    ref = ref.to(lse.device)
    assert torch.equal(torch.isinf(lse), torch.isinf(ref)), "empty-row pattern of the LSE differs"
    fin = torch.isfinite(ref)
    if fin.any():
        assert (lse[fin] - ref[fin]).abs().max().item() <= 1e-2
    assert (lse[~fin] > 0).all()


CASES = {
    # name: (B, Lq, Lk, H, Hk, mask heads, bias heads (None = no bias), window, causal, dtype)
    "gqa4_square": (1, 512, 512, 8, 2, 2, 2, 128, True, torch.bfloat16),
    "lq_lt_lk_ragged_sizes": (2, 300, 777, 4, 2, 2, 2, 200, True, torch.bfloat16),
    "mqa_bias_per_query_head": (1, 1000, 1000, 4, 1, 1, 4, 300, True, torch.bfloat16),
    "nine_pairs_shared_mask_noncausal": (3, 260, 260, 6, 3, 1, 1, 64, False, torch.bfloat16),
    "everything_kept": (1, 1024, 1024, 8, 2, 2, 2, 1024, True, torch.bfloat16),
    "lq_gt_lk_rows_without_keys_three_kept_keys": (1, 700, 300, 4, 2, 2, 2, 3, True, torch.bfloat16),
    "many_tiles_per_item": (2, 256, 4096, 8, 4, 4, 4, 1000, True, torch.bfloat16),
    "mask_only": (2, 257, 391, 4, 4, 4, None, 100, False, torch.bfloat16),
    "fp16": (1, 640, 640, 4, 2, 2, 2, 300, True, torch.float16),
    "exactly_one_tile": (1, 300, 300, 2, 2, 2, 2, 64, True, torch.bfloat16),
    "one_key_beyond_a_tile": (1, 300, 300, 2, 2, 2, 2, 65, False, torch.bfloat16),
    "five_pairs": (5, 520, 520, 2, 1, 1, 1, 130, True, torch.bfloat16),
    # a mask row per QUERY head over grouped kv heads: compacted per query head (forward only)
    "mask_per_query_head_bias_per_kv_head": (1, 600, 600, 8, 2, 8, 2, 150, True, torch.bfloat16),
    "mask_per_query_head_bias_per_query_head": (2, 300, 500, 4, 2, 4, 4, 100, True, torch.bfloat16),
    "mask_per_query_head_shared_bias_noncausal": (1, 512, 512, 6, 3, 6, 1, 99, False, torch.bfloat16),
    # ... many rows over few keys and one bias row for sixteen heads: four members whose dK / dV / dBias are summed
    # (in fp32, rounded once), with sums of thousands of terms per dBias element
    "mask_per_query_head_shared_bias_many_rows_few_keys": (2, 549, 33, 16, 4, 16, 1, 8, True, torch.bfloat16),
}


@pytest.mark.parametrize("name", list(CASES))
def test_streaming_forward_and_its_backward_vs_oracle(name):
    B, Lq, Lk, H, Hk, hm, hb, W, causal, dtype = CASES[name]
    q, k, v, mask, bias = make_inputs(B, Lq, Lk, H, Hk, 128, (B, hb, 1, Lk) if hb else None, (B, hm, 1, Lk), W, seed=5, dtype=dtype)
    dout = torch.randn(B, Lq, H, 128, generator=torch.Generator().manual_seed(6)).to(dtype)
    out, lse, grads = _run(q, k, v, mask, bias, causal, dout=dout)
    if B * H * Lq * Lk <= 1 << 23:
        ro, rl = c_oracle.forward(q, k, v, mask, bias, None, causal)
        refs = c_oracle.backward(q, k, v, dout, mask, bias, None, causal)
    else:
        dev = [t.to(DEV) if t is not None else None for t in (q, k, v, mask, bias)]
        ro, rl = eager.attention_forward(*dev, None, causal)
        _, *refs = eager.attention_forward_backward(*dev, None, causal, dout=dout.to(DEV))
    assert_out_close(out.cpu(), ro.cpu())
    _check_lse(lse.cpu(), rl.cpu())
    for g, r, n in zip(grads, refs, ("dq", "dk", "dv", "dbias")):
        if g is not None:
            assert_grad_close(g.cpu(), r.cpu(), n)
    # the same problem through the other form of the compacted forward (row-major copies, a workgroup per query block)
    # and through tile skipping: the forward agrees to rounding, and the backward -- which reads none of the images --
    # bit for bit between the two compacted forms when fed the same output
    from flash_sparse_attn import _cabi
    _cabi.stream_min_items(1 << 30)
    out2, lse2, grads2 = _run(q, k, v, mask, bias, causal, dout=dout)
    _cabi.stream_min_items(1)
    assert (out.float() - out2.float()).abs().max().item() <= 2e-2
    fin = torch.isfinite(lse2)
    # (the streaming form reads K pre-multiplied by the softmax scale and rounded to 16 bits, the other one rounds the
    # scaled Q: scores differ by the rounding of one operand, and so does the LSE of a row with few keys)
    assert torch.equal(torch.isfinite(lse), fin) and (lse[fin] - lse2[fin]).abs().max().item() <= 1e-2
    # a second run gives the same bits
    out3, lse3, grads3 = _run(q, k, v, mask, bias, causal, dout=dout)
    assert torch.equal(out, out3) and torch.equal(lse, lse3)
    for a, b in zip(grads, grads3):
        if a is not None:
            assert torch.equal(a, b)


def test_pairs_without_a_kept_key_and_a_late_first_key():
    """One (batch, kv head) pair keeps nothing at all (its rows come out as zeros with LSE = +inf, its gradients as
    zeros), another keeps only keys in the last quarter (under the causal rule most of its rows see nothing)."""
    B, L, H, Hk = 2, 600, 4, 2
    q, k, v, mask, bias = make_inputs(B, L, L, H, Hk, 128, (B, Hk, 1, L), (B, Hk, 1, L), 150, seed=12)
    mask[0, 1] = False
    mask[1, 0, :, : 3 * L // 4] = False
    out, lse, grads = _run(q, k, v, mask, bias, True)
    ro, rl = c_oracle.forward(q, k, v, mask, bias, None, True)
    refs = c_oracle.backward(q, k, v, torch.ones_like(ro), mask, bias, None, True)
    assert_out_close(out.cpu(), ro)
    _check_lse(lse.cpu(), rl)
    assert float(out[0, :, 2:].abs().max()) == 0.0 and bool(torch.isinf(lse[0, 2:]).all())
    for g, r, n in zip(grads, refs, ("dq", "dk", "dv", "dbias")):
        assert_grad_close(g.cpu(), r, n)


@pytest.mark.parametrize("bias_heads", ["kv", "query"])
def test_streaming_forward_with_lists_from_the_mask_builder(bias_heads):
    """Kept-key lists handed over by the device mask builder: the image pre-pass numbers nothing and copies the lists;
    results equal those of the same mask as a plain tensor, bit for bit.  ("query": a bias row, hence a mask row and a
    list, per query head over grouped kv heads -- compacted per query head.)"""
    from flash_sparse_attn.utils import mask as M
    B, Lq, Lk, H, Hk, W = 2, 520, 777, 4, 2, 250
    q, k, v, _, bias = make_inputs(B, Lq, Lk, H, Hk, 128, (B, Hk if bias_heads == "kv" else H, 1, Lk), None, None, seed=9)
    bd = bias.to(DEV)
    mask = M.topk_mask(bd, None, W, torch.finfo(bd.dtype).min)
    assert M.kept_keys_of(mask) is not None
    a = _run(q, k, v, mask, bias, True)
    b = _run(q, k, v, mask.clone(), bias, True)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    for x, y in zip(a[2], b[2]):
        assert torch.equal(x, y)
    ro, rl = c_oracle.forward(q, k, v, mask.cpu(), bias, None, True)
    assert_out_close(a[0].cpu(), ro)


@pytest.mark.parametrize("kind", ["late_bias_bf16", "late_bias_noncausal_bf16", "late_keys_fp16", "huge_scores_fp16", "first_tile_tiny_bf16"])
def test_items_that_leave_the_common_path_are_redone(kind):
    """Scores that climb out of the range the first tile's reference point allows (or a reference the 16-bit pieces
    cannot express): the item is noted and redone with the classic softmax at the end of its workgroup's life."""
    dtype = torch.float16 if kind.endswith("fp16") else torch.bfloat16
    B, L, H, Hk, D = 1, 640, 4, 2, 128
    q, k, v, mask, bias = make_inputs(B, L, L, H, Hk, D, (B, Hk, 1, L), (B, Hk, 1, L), 400, seed=41, dtype=dtype)
    causal = kind != "late_bias_noncausal_bf16"
    if kind.startswith("late_keys"):
        k = k.clone()
        k[:, 300:] = (k[:, 300:].float() * 3).to(dtype)
        bias = bias.clone()
        bias[..., 300:] += 25.0
    elif kind.startswith("late_bias"):
        bias = bias.clone()
        bias[..., 230:] += 60.0
    elif kind == "huge_scores_fp16":
        q = (q.float().sign() * 160).to(dtype)
        k = (k.float().sign() * 160).to(dtype)
    else:
        k = k.clone()
        k[:, :100] = (k[:, :100].float() * 0.01).to(dtype)
        bias = bias.clone()
        bias[..., :100] -= 50.0
    scale = 1.0 if kind == "huge_scores_fp16" else None
    out, lse, grads = _run(q, k, v, mask, bias, causal, scale=scale)
    ro, rl = c_oracle.forward(q, k, v, mask, bias, scale, causal)
    if kind == "huge_scores_fp16":
        assert torch.isfinite(out.float()).all() and out.float().abs().max() <= v.float().abs().max()
    else:
        assert_out_close(out.cpu(), ro)
    assert torch.equal(torch.isinf(lse.cpu()), torch.isinf(rl))
    fin = torch.isfinite(rl)
    assert ((lse.cpu()[fin] - rl[fin]).abs() <= 1e-2 + 3e-3 * rl[fin].abs()).all()
    if kind != "huge_scores_fp16":
        refs = c_oracle.backward(q, k, v, torch.ones_like(ro), mask, bias, scale, causal)
        for g, r, n in zip(grads, refs, ("dq", "dk", "dv", "dbias")):
            assert_grad_close(g.cpu(), r, n)


def test_default_threshold_takes_the_headline_shape_and_not_a_small_one():
    """The rule is a pure function of the problem: the workspace sizes of both forms differ, which shows which one a
    problem gets."""
    from flash_sparse_attn import _cabi
    _cabi.stream_min_items(512)

    def need(B, L, H, Hk):
        q = torch.empty(B, L, H, 128, dtype=torch.bfloat16, device=DEV)
        k = torch.empty(B, L, Hk, 128, dtype=torch.bfloat16, device=DEV)
        m = torch.ones(B, Hk, 1, L, dtype=torch.bool, device=DEV)
        a = _cabi.FwdArgs()
        _cabi.fill_fwd(a, q, k, k, m, None, q, torch.empty(B, H, L, device=DEV), 0.1, True, 0.0)
        a.compact_mode = _cabi.COMPACT_ALWAYS
        return _cabi.lib.fdma_fwd_workspace_bytes(a)

    lists = lambda B, L, Hk: 2 * (B * Hk * L * 4) + 256 + B * Hk * L * 4  # idx, cnt, count, fb (rounded sizes aside)
    big = need(1, 8192, 32, 8)    # 1024 items: tile images (35840 + 2048 bytes per 64 keys)
    small = need(1, 1024, 8, 2)   # 32 items: row-major copies (2 * 64 * 256 bytes per 64 keys)
    assert abs(big - (lists(1, 8192, 8) + 8 * 128 * (35840 + 2048))) <= 4096
    assert abs(small - (lists(1, 1024, 2) + 2 * 16 * 2 * 64 * 256)) <= 4096


def _draw_streamed(it):
    import random
    rng = random.Random(9100 + it)
    Hk = rng.choice([1, 2, 3, 4])
    H = Hk * rng.choice([1, 2, 4])
    B = rng.choice([1, 2, 3])
    Lq, Lk = rng.randint(2, 900), rng.randint(1, 1500)
    hm = rng.choice([1, Hk, Hk, H])
    hb = rng.choice([None, 1, Hk, H])
    W = max(2, int(Lk * rng.choice([0.02, 0.1, 0.25, 0.6, 1.0])))  # (one kept key: P = 1, dS = 0, nothing to compare dQ with)
    return dict(B=B, Lq=Lq, Lk=Lk, H=H, Hk=Hk, hm=hm, hb=hb, W=W, causal=rng.random() < 0.7,
                dtype=rng.choice([torch.bfloat16, torch.bfloat16, torch.float16]), qscale=rng.choice([1.0, 1.0, 2.5]))


@pytest.mark.parametrize("it", range(24))
def test_streamed_random_case_vs_eager_fp32(it):
    """Seeded random shapes through the streaming forward (every compacted call at head dim 128 takes it here): ragged
    row and key counts, 1 to 12 (batch, kv head) pairs, mask rows per pair, per kv head or per query head, every bias
    head count, both dtypes, larger score scales."""
    c = _draw_streamed(it)
    print({k: str(v) for k, v in c.items()}, flush=True)
    q, k, v, mask, bias = make_inputs(c["B"], c["Lq"], c["Lk"], c["H"], c["Hk"], 128,
                                      (c["B"], c["hb"], 1, c["Lk"]) if c["hb"] else None, (c["B"], c["hm"], 1, c["Lk"]), c["W"],
                                      seed=2000 + it, dtype=c["dtype"])
    q = (q.float() * c["qscale"]).to(c["dtype"])
    dout = torch.randn(q.shape, generator=torch.Generator().manual_seed(3000 + it)).to(c["dtype"])
    out, lse, grads = _run(q, k, v, mask, bias, c["causal"], dout=dout)
    dev = [t.to(DEV) if t is not None else None for t in (q, k, v, mask, bias)]
    ro, rl = eager.attention_forward(*dev, None, c["causal"])
    _, *refs = eager.attention_forward_backward(*dev, None, c["causal"], dout=dout.to(DEV))
    # (scores 2.5 times larger carry 2.5 times the rounding of their 16-bit operands: twice the bound, as in the sweep
    # of the operator's other paths)
    assert (out.float() - ro.float()).abs().max().item() <= OUT_ATOL * (2 if c["qscale"] > 1 else 1)
    assert torch.equal(torch.isinf(lse), torch.isinf(rl))
    fin = torch.isfinite(rl)
    if fin.any():
        assert (lse[fin] - rl[fin]).abs().max().item() <= 1e-2 * c["qscale"]
    for g, r, n in zip(grads, refs, ("dq", "dk", "dv", "dbias")):
        if g is not None:
            assert_grad_close(g.cpu(), r.cpu(), n)
