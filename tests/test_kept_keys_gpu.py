"""GPU tests (`-m gpu`) of the two hand-overs around the column-compaction path:

  * the device keep-mask builder writes, next to the bool mask, the kept columns of every query-broadcast row as an
    ordered list with prefix counts (`fdma_kept_keys`), and the attention calls take the lists instead of scanning
    the mask again;
  * the backward of an autograd node reuses the workspace of its forward call (index lists, compacted K / V copies)
    instead of scanning and gathering a second time (`fdma_bwd_args.fwd_workspace`).
Neither changes what is computed: every comparison here is bit for bit against the same call without the hand-over.
"""
import pytest
import torch

from _util import set_compact
from flash_sparse_attn import flash_sparse_attn_func
from flash_sparse_attn import flash_sparse_attn_interface as iface
from flash_sparse_attn.utils import mask as M

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _inputs(B, Lq, Lk, H, Hk, D, Hm, seed, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Lq, H, D, generator=g).to(dtype).to(DEV)
    k = torch.randn(B, Lk, Hk, D, generator=g).to(dtype).to(DEV)
    v = torch.randn(B, Lk, Hk, D, generator=g).to(dtype).to(DEV)
    bias = torch.randn(B, Hm, 1, Lk, generator=g).to(dtype).to(DEV)
    return q, k, v, bias


@pytest.mark.parametrize("shape,window,block", [((2, 3, 1, 1000), 100, None), ((1, 8, 1, 8192), 2048, None),
                                                ((2, 2, 1, 777), 300, 64), ((3, 1, 1, 50), 50, None),
                                                ((1, 2, 1, 40000), 1000, None)])
def test_mask_builder_writes_the_kept_columns_as_lists(shape, window, block):
    bias = torch.randn(shape, generator=torch.Generator().manual_seed(shape[-1])).to(torch.bfloat16).to(DEV)
    mask = M.topk_mask(bias, None, window, torch.finfo(torch.bfloat16).min, block_size=block)
    kept = M.kept_keys_of(mask)
    assert kept is not None
    idx, cnt, count, ld = kept
    torch.cuda.synchronize()
    rows = mask.reshape(-1, shape[-1])
    assert ld % 16 == 0 and ld >= shape[-1] and idx.shape == cnt.shape == (rows.shape[0], ld)
    assert torch.equal(count.long(), rows.sum(-1))
    assert torch.equal(cnt[:, :shape[-1]].long(), rows.long().cumsum(-1))
    for r in range(rows.shape[0]):
        n = int(count[r])
        assert torch.equal(idx[r, :n].long(), rows[r].nonzero().flatten())
    # a mask that has been written to since no longer carries its lists
    mask[..., 0] = True
    assert M.kept_keys_of(mask) is None
    # a per-query mask has none to begin with
    per_query = M.topk_mask(bias.expand(-1, -1, 4, -1), None, window, torch.finfo(torch.bfloat16).min)
    assert M.kept_keys_of(per_query) is None


def _run(q, k, v, mask, bias, causal=True):
    qg, kg, vg, bg = [t.detach().clone().requires_grad_(True) for t in (q, k, v, bias)]
    out, lse, _ = flash_sparse_attn_func(qg, kg, vg, mask, bg, None, causal, None, None, True)
    out.backward(torch.ones_like(out))
    torch.cuda.synchronize()
    return [out.detach(), lse.detach(), qg.grad, kg.grad, vg.grad, bg.grad]


CASES = [
    # B, Lq, Lk, H, Hk, D, mask heads, window
    (1, 512, 512, 8, 2, 128, 2, 128),
    (2, 300, 777, 4, 2, 64, 2, 200),     # key length that is no multiple of 16: the mask is padded on the way in
    (2, 256, 640, 4, 4, 128, 1, 96),     # one mask head for all kv heads
    (1, 1024, 1024, 8, 2, 128, 2, 1024), # everything kept
    (1, 384, 384, 2, 1, 32, 1, 1),       # a single kept key per row
]


@pytest.mark.parametrize("case", range(len(CASES)))
@pytest.mark.parametrize("mode", ["2", "auto"])
def test_attention_with_handed_over_lists_is_bit_identical(case, mode):
    B, Lq, Lk, H, Hk, D, Hm, W = CASES[case]
    q, k, v, bias = _inputs(B, Lq, Lk, H, Hk, D, Hm, seed=case)
    set_compact(mode)
    try:
        mask = M.topk_mask(bias, None, W, torch.finfo(bias.dtype).min)
        assert M.kept_keys_of(mask) is not None
        with_lists = _run(q, k, v, mask, bias)
        plain = mask.clone()  # same values, no lists: the attention call scans it
        assert M.kept_keys_of(plain) is None
        scanned = _run(q, k, v, plain, bias)
    finally:
        set_compact("auto")
    for a, b in zip(with_lists, scanned):
        assert torch.equal(a, b)


@pytest.mark.parametrize("Lk", [1, 15, 16, 17, 255, 256, 257, 511, 512, 513, 1000, 1281])
@pytest.mark.parametrize("pattern", ["random", "all", "last_only", "first_segments_empty", "every_256th"])
def test_forward_scan_and_gather_in_one_launch_at_segment_boundaries(Lk, pattern):
    """The forward numbers and gathers the kept columns in one launch, 256 original columns per workgroup: key lengths
    and masks around those boundaries, forward and backward against the same call on the tile-skipping kernels (other
    order of summation: tolerances), and the backward on the forward's workspace against the backward that scans and
    gathers for itself (bit for bit)."""
    B, Lq, H, Hk, D = 2, 130, 4, 2, 64
    q, k, v, bias = _inputs(B, Lq, Lk, H, Hk, D, Hk, seed=Lk)
    g = torch.Generator().manual_seed(1000 + Lk)
    if pattern == "random":
        mask = torch.rand(B, Hk, 1, Lk, generator=g) < 0.3
        mask[..., 0] = True
    elif pattern == "all":
        mask = torch.ones(B, Hk, 1, Lk, dtype=torch.bool)
    elif pattern == "last_only":
        mask = torch.zeros(B, Hk, 1, Lk, dtype=torch.bool)
        mask[..., Lk - 1] = True
    elif pattern == "first_segments_empty":
        mask = torch.rand(B, Hk, 1, Lk, generator=g) < 0.5
        mask[..., :min(Lk - 1, 512)] = False
        mask[..., Lk - 1] = True
    else:
        mask = torch.zeros(B, Hk, 1, Lk, dtype=torch.bool)
        mask[..., ::256] = True
    mask = mask.to(DEV)
    try:
        set_compact("2")
        got = _run(q, k, v, mask, bias, causal=False)
        mpad, bpad = iface._pad_key_dim(mask, Lk, 16), iface._pad_key_dim(bias, Lk, 8)
        out, lse, _ = iface._wrapped_flash_sparse_attn_forward(q, k, v, mpad, bpad, D ** -0.5, False, 0.0, False)
        dq, dk, dv, dbp = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v), torch.empty_like(bpad)
        iface._wrapped_flash_sparse_attn_backward(torch.ones_like(out), q, k, v, mpad, bpad, out, lse, dq, dk, dv, dbp,
                                                  D ** -0.5, False, 0.0, False)
        torch.cuda.synchronize()
        set_compact("0")
        ref = _run(q, k, v, mask, bias, causal=False)
    finally:
        set_compact("auto")
    for a, b in zip(got, [out, lse, dq, dk, dv, dbp[..., :Lk]]):
        assert torch.equal(a, b)
    assert (got[0].float() - ref[0].float()).abs().max().item() <= 2e-2
    assert (got[1] - ref[1]).abs().max().item() <= 1e-3
    for a, b, name in zip(got[2:], ref[2:], ("dq", "dk", "dv", "dbias")):
        err = (a.float() - b.float()).abs().max().item()
        assert err <= 5e-2 * max(1.0, b.float().abs().max().item()), (name, err)


@pytest.mark.parametrize("Lk", [65536, 65537, 70000])
def test_long_key_axes_take_the_two_launch_pre_pass_above_65536_keys(Lk):
    """Up to 65536 keys the forward numbers and gathers in one launch, above that in two (the one-launch form recounts
    the mask in front of every 256-key segment): the same results on both sides of the limit, against tile skipping."""
    B, Lq, H, Hk, D = 1, 160, 2, 1, 64
    q, k, v, bias = _inputs(B, Lq, Lk, H, Hk, D, Hk, seed=7)
    mask = (torch.rand(B, Hk, 1, Lk, generator=torch.Generator().manual_seed(Lk)) < 0.02).to(DEV)
    mask[..., Lk - 1] = True
    try:
        set_compact("2")
        got = _run(q, k, v, mask, bias, causal=True)
        set_compact("0")
        ref = _run(q, k, v, mask, bias, causal=True)
    finally:
        set_compact("auto")
    assert (got[0].float() - ref[0].float()).abs().max().item() <= 2e-2
    assert (got[1] - ref[1]).abs().max().item() <= 1e-3
    for a, b, name in zip(got[2:], ref[2:], ("dq", "dk", "dv", "dbias")):
        err = (a.float() - b.float()).abs().max().item()
        assert err <= 5e-2 * max(1.0, b.float().abs().max().item()), (name, err)


def test_more_pairs_than_a_grid_dimension_holds_fall_back_to_tile_skipping():
    """65536 (batch, kv head) pairs: the pre-pass launches could not carry the pair in the grid's y dimension, so the
    call takes the tile-skipping kernels even when compaction is asked for -- same bits as with compaction off."""
    B, Lq, Lk, H, Hk, D = 65536, 2, 16, 1, 1, 32
    q, k, v, bias = _inputs(B, Lq, Lk, H, Hk, D, Hk, seed=3)
    mask = (torch.rand(B, Hk, 1, Lk, generator=torch.Generator().manual_seed(3)) < 0.5).to(DEV)
    mask[..., 0] = True
    try:
        set_compact("2")
        got = _run(q, k, v, mask, bias, causal=True)
        set_compact("0")
        ref = _run(q, k, v, mask, bias, causal=True)
    finally:
        set_compact("auto")
    for a, b in zip(got, ref):
        assert torch.equal(a, b)


@pytest.mark.parametrize("case", range(len(CASES)))
def test_backward_on_the_forward_workspace_is_bit_identical(case):
    B, Lq, Lk, H, Hk, D, Hm, W = CASES[case]
    q, k, v, bias = _inputs(B, Lq, Lk, H, Hk, D, Hm, seed=10 + case)
    mask = M.topk_mask(bias, None, W, torch.finfo(bias.dtype).min).clone()
    set_compact("2")
    try:
        reused = _run(q, k, v, mask, bias)
        # the same operator calls by hand, outside an autograd node: the backward then has no forward workspace
        mpad, bpad = iface._pad_key_dim(mask, Lk, 16), iface._pad_key_dim(bias, Lk, 8)
        out, lse, _ = iface._wrapped_flash_sparse_attn_forward(q, k, v, mpad, bpad, D ** -0.5, True, 0.0, False)
        dq, dk, dv, dbp = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v), torch.empty_like(bpad)
        iface._wrapped_flash_sparse_attn_backward(torch.ones_like(out), q, k, v, mpad, bpad, out, lse, dq, dk, dv, dbp,
                                                  D ** -0.5, True, 0.0, False)
        torch.cuda.synchronize()
    finally:
        set_compact("auto")
    for a, b in zip(reused, [out, lse, dq, dk, dv, dbp[..., :Lk]]):
        assert torch.equal(a, b)


def test_deterministic_backward_with_shared_bias_does_not_take_the_forward_workspace():
    """deterministic=True expands a batch-broadcast bias for the backward: another problem than the forward's, whose
    workspace must then be left alone (results against the plain operator on the expanded bias)."""
    B, Lq, Lk, H, Hk, D = 2, 256, 512, 4, 2, 64
    q, k, v, _ = _inputs(B, Lq, Lk, H, Hk, D, Hk, seed=5)
    bias = torch.randn(1, Hk, 1, Lk, generator=torch.Generator().manual_seed(6)).to(torch.bfloat16).to(DEV)
    mask = M.topk_mask(bias, None, 128, torch.finfo(bias.dtype).min)
    set_compact("2")
    try:
        qg, kg, vg, bg = [t.detach().clone().requires_grad_(True) for t in (q, k, v, bias)]
        out = flash_sparse_attn_func(qg, kg, vg, mask, bg, None, True, None, True)
        out.backward(torch.ones_like(out))
        q2, k2, v2 = [t.detach().clone().requires_grad_(True) for t in (q, k, v)]
        b2 = bias.expand(B, -1, -1, -1).contiguous().requires_grad_(True)
        out2 = flash_sparse_attn_func(q2, k2, v2, mask.expand(B, -1, -1, -1).contiguous(), b2, None, True, None, True)
        out2.backward(torch.ones_like(out2))
        torch.cuda.synchronize()
    finally:
        set_compact("auto")
    assert torch.equal(out, out2) and torch.equal(qg.grad, q2.grad) and torch.equal(kg.grad, k2.grad)
    ref_db = b2.grad.float().sum(0, keepdim=True)
    assert (bg.grad.float() - ref_db).abs().max().item() <= 2e-2 * ref_db.abs().max().item()


def test_per_query_mask_of_column_causal_form_takes_the_column_mask_kernels():
    """Under the compaction policy "always" a [B, Hk, Lq, Lk] mask whose rows are one column mask cut off at the causal
    limit is recognised and runs like that column mask with is_causal=True (bit for bit); a mask that differs from the
    form in a single element is not, and goes through the per-query kernels.  Both against the C oracle."""
    from _util import assert_grad_close, assert_out_close, make_inputs
    from oracle import c_oracle

    B, Lq, Lk, H, Hk, D, W = 2, 200, 264, 4, 2, 64, 80
    q, k, v, colmask, bias = make_inputs(B, Lq, Lk, H, Hk, D, (B, Hk, 1, Lk), (B, Hk, 1, Lk), W, seed=3)
    causal = torch.arange(Lk)[None, :] <= torch.arange(Lq)[:, None] + (Lk - Lq)
    full = colmask & causal                       # (B, Hk, Lq, Lk)
    broken = full.clone()
    broken[1, 0, 50, 3] = ~broken[1, 0, 50, 3]   # one element off the form
    dout = torch.randn(B, Lq, H, D, generator=torch.Generator().manual_seed(4)).to(torch.bfloat16)

    def run(mask, is_causal):
        qg, kg, vg, bg = [t.to(DEV).requires_grad_(True) for t in (q, k, v, bias)]
        out, lse, _ = flash_sparse_attn_func(qg, kg, vg, mask.to(DEV), bg, None, is_causal, None, None, True)
        out.backward(dout.to(DEV))
        torch.cuda.synchronize()
        return [out.detach(), lse.detach(), qg.grad, kg.grad, vg.grad, bg.grad]

    set_compact("2")
    try:
        as_columns = run(colmask, True)
        recognised = run(full, False)            # (the mask carries the causal rule itself)
        recognised_c = run(full, True)
        fallback = run(broken, False)
    finally:
        set_compact("auto")
    for a, b, c in zip(as_columns, recognised, recognised_c):
        assert torch.equal(a, b) and torch.equal(a, c)
    for got, mask in ((recognised, full), (fallback, broken)):
        ro, rl = c_oracle.forward(q, k, v, mask, bias, None, False)
        rdq, rdk, rdv, rdb = c_oracle.backward(q, k, v, dout, mask, bias, None, False)
        assert_out_close(got[0].cpu(), ro)
        for g, r, name in ((got[2], rdq, "dq"), (got[3], rdk, "dk"), (got[4], rdv, "dv"), (got[5], rdb, "dbias")):
            assert_grad_close(g.cpu(), r, name)
    assert not torch.equal(recognised[0], fallback[0])


@pytest.mark.parametrize("mode", ["2", "auto"])
def test_builder_mask_wider_than_the_keys_is_scanned_not_trusted(mode):
    """A mask from the device builder whose key length is the keys' rounded up to 128 (a caller that pads mask and bias
    first): its lists number the columns of the WIDE row, kept columns beyond the keys included, so the attention call
    must not take them.  Results equal those of the same values as a plain tensor (bit for bit) and the C oracle on the
    first Lk columns."""
    from _util import assert_grad_close, assert_out_close
    from oracle import c_oracle

    B, Lq, Lk, H, Hk, D, W = 2, 200, 300, 4, 2, 64, 120
    Lw = 384
    q, k, v, _ = _inputs(B, Lq, Lk, H, Hk, D, Hk, seed=21)
    bias = torch.randn(B, Hk, 1, Lw, generator=torch.Generator().manual_seed(22)).to(torch.bfloat16).to(DEV)
    set_compact(mode)
    try:
        mask = M.topk_mask(bias, None, W, torch.finfo(bias.dtype).min)
        assert M.kept_keys_of(mask) is not None and mask.shape[-1] == Lw
        assert int(mask[..., Lk:].sum()) > 0  # (kept columns beyond the keys exist: the lists would point past K)
        with_lists = _run(q, k, v, mask, bias[..., :Lk])
        scanned = _run(q, k, v, mask.clone(), bias[..., :Lk])
    finally:
        set_compact("auto")
    for a, b in zip(with_lists, scanned):
        assert torch.equal(a, b)
    qc, kc, vc, mc, bc = [t.cpu() for t in (q, k, v, mask[..., :Lk], bias[..., :Lk])]
    ro, _ = c_oracle.forward(qc, kc, vc, mc, bc, None, True)
    rdq, rdk, rdv, rdb = c_oracle.backward(qc, kc, vc, torch.ones_like(ro), mc, bc, None, True)
    assert_out_close(with_lists[0].cpu(), ro)
    for g, r, name in ((with_lists[2], rdq, "dq"), (with_lists[3], rdk, "dk"), (with_lists[4], rdv, "dv")):
        assert_grad_close(g.cpu(), r, name)
    assert_grad_close(with_lists[5].cpu(), rdb, "dbias")


@pytest.mark.parametrize("mode", ["2", "auto"])
def test_builder_mask_with_key_dim_one_is_expanded_not_trusted(mode):
    """A builder-made mask with a key dimension of 1 (one keep decision for every key) carries lists for a row of one
    column; the operator expands the mask over the keys and must scan it instead."""
    B, Lq, Lk, H, Hk, D = 1, 128, 256, 4, 2, 64
    q, k, v, _ = _inputs(B, Lq, Lk, H, Hk, D, Hk, seed=23)
    bias1 = torch.randn(B, Hk, 1, 1, generator=torch.Generator().manual_seed(24)).to(torch.bfloat16).to(DEV)
    set_compact(mode)
    try:
        mask = M.topk_mask(bias1, None, 1, torch.finfo(bias1.dtype).min)
        assert mask.shape[-1] == 1 and bool(mask.all())
        qg, kg, vg = [t.detach().clone().requires_grad_(True) for t in (q, k, v)]
        out = flash_sparse_attn_func(qg, kg, vg, mask, None, None, True)
        out.backward(torch.ones_like(out))
        q2, k2, v2 = [t.detach().clone().requires_grad_(True) for t in (q, k, v)]
        out2 = flash_sparse_attn_func(q2, k2, v2, None, None, None, True)
        out2.backward(torch.ones_like(out2))
        torch.cuda.synchronize()
    finally:
        set_compact("auto")
    assert (out.float() - out2.float()).abs().max().item() <= 2e-2
    for a, b in ((qg.grad, q2.grad), (kg.grad, k2.grad), (vg.grad, v2.grad)):
        assert (a.float() - b.float()).abs().max().item() <= 5e-2 * b.float().abs().max().item()
