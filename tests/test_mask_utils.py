"""Keep-mask builders (flash_sparse_attn/utils/mask.py) against brute-force loops on small inputs.

The expected values are computed element by element in plain Python from the definitions (k largest
entries of a row, majority vote per block), not with the tensor routines the functions themselves use.
Ties in top-k are avoided by construction (distinct values): which of two equal entries torch.topk
returns is not fixed by the reference either.
"""
import itertools

import pytest
import torch

from flash_sparse_attn.utils.mask import block_smooth, create_mask, relu_mask, topk_indices, topk_mask

MIN = torch.finfo(torch.float32).min


def distinct_bias(shape, seed):
    g = torch.Generator().manual_seed(seed)
    n = 1
    for s in shape:
        n *= s
    return (torch.randperm(n, generator=g).float() - n / 2 + 0.5).reshape(shape)


def rows_of(t):
    return itertools.product(*[range(s) for s in t.shape[:-1]])


def loop_topk(bias, keep_in, k):
    out = torch.zeros(bias.shape, dtype=torch.bool)
    for idx in rows_of(bias):
        row = [(MIN if (keep_in is not None and not bool(keep_in[idx][j])) else float(bias[idx][j]), j)
               for j in range(bias.shape[-1])]
        row.sort(reverse=True)
        for v, j in row[:k]:
            if v != MIN:
                out[idx][j] = True
    return out


def loop_smooth(mask, block):
    out = mask.clone()
    L = mask.shape[-1]
    for idx in rows_of(mask):
        for s in range(0, L, block):
            e = min(s + block, L)
            cnt = sum(bool(mask[idx][j]) for j in range(s, e))
            for j in range(s, e):
                out[idx][j] = 2 * cnt > (e - s)
    return out


def test_topk_indices_sorted_positions():
    bias = distinct_bias((2, 3, 17), 0)
    got = topk_indices(bias, 5)
    assert got.shape == (2, 3, 5)
    for b, h in itertools.product(range(2), range(3)):
        want = sorted(sorted(range(17), key=lambda j: -float(bias[b, h, j]))[:5])
        assert got[b, h].tolist() == want


@pytest.mark.parametrize("shape", [(2, 2, 1, 19), (1, 3, 4, 16)])
@pytest.mark.parametrize("with_mask", [False, True])
def test_topk_mask_matches_loops(shape, with_mask):
    bias = distinct_bias(shape, 1)
    keep_in = None
    if with_mask:
        keep_in = torch.rand(shape, generator=torch.Generator().manual_seed(2)) > 0.6
        keep_in[..., 0, :] = False
        keep_in[..., 0, :3] = True  # a row with fewer admissible keys than the window
    got = topk_mask(bias, keep_in, window_size=6, min_dtype=MIN)
    assert torch.equal(got, loop_topk(bias, keep_in, 6))
    assert int(got.sum(-1).max()) <= 6
    if with_mask:
        assert not bool((got & ~keep_in).any())
        assert int(got[..., 0, :].sum(-1).max()) == 3


@pytest.mark.parametrize("key_len,block", [(16, 4), (19, 4), (7, 8), (12, 1), (9, 2)])
def test_block_smooth_matches_loops(key_len, block):
    m = torch.rand((2, 2, 3, key_len), generator=torch.Generator().manual_seed(key_len * 31 + block)) > 0.5
    want = loop_smooth(m, block)
    got = block_smooth(m.clone(), key_len, block)
    assert torch.equal(got, want)


def test_block_smooth_is_in_place_and_idempotent_and_rejects_bad_block():
    m = torch.rand((1, 1, 2, 24), generator=torch.Generator().manual_seed(5)) > 0.5
    r = block_smooth(m, 24, 8)
    assert r.data_ptr() == m.data_ptr()
    assert torch.equal(block_smooth(r.clone(), 24, 8), r)
    with pytest.raises(ValueError, match="block_size must be a positive integer"):
        block_smooth(m, 24, 0)


def test_exact_half_is_dropped():
    m = torch.tensor([[True, True, False, False, True, True, True, False]])
    assert block_smooth(m.clone(), 8, 4).tolist() == [[False] * 4 + [True] * 4]


def test_relu_mask():
    bias = distinct_bias((2, 2, 3, 11), 3)
    keep_in = torch.rand(bias.shape, generator=torch.Generator().manual_seed(4)) > 0.3
    got = relu_mask(bias, keep_in, MIN)
    assert torch.equal(got, (bias > 0) & keep_in)
    assert torch.equal(relu_mask(bias, None, MIN), bias > 0)
    assert torch.equal(relu_mask(bias, None, MIN, block_size=4), loop_smooth(bias > 0, 4))


def test_create_mask_padding_forms():
    B, Lq, Lk, k = 2, 4, 10, 3
    bias = distinct_bias((B, 2, 1, Lk), 6)
    pad_k = torch.ones(B, Lk, dtype=torch.bool)
    pad_k[0, :4] = False
    got = create_mask(bias, pad_k, B, Lq, Lk, k, MIN)
    assert torch.equal(got, loop_topk(bias, pad_k.view(B, 1, 1, Lk).expand_as(bias), k))
    # a (batch, query_len) padding mask covers the last query_len keys
    pad_q = torch.ones(B, Lq, dtype=torch.bool)
    pad_q[1, 0] = False
    full = torch.ones(B, Lk, dtype=torch.bool)
    full[1, Lk - Lq] = False
    got_q = create_mask(bias, pad_q, B, Lq, Lk, k, MIN)
    assert torch.equal(got_q, loop_topk(bias, full.view(B, 1, 1, Lk).expand_as(bias), k))
    # no padding mask, relu type, block smoothing
    got_r = create_mask(bias, None, B, Lq, Lk, k, MIN, block_size=2, type="relu")
    assert torch.equal(got_r, loop_smooth(bias > 0, 2))
    with pytest.raises(ValueError, match="not compatible with key_len"):
        create_mask(bias, torch.ones(B, 7, dtype=torch.bool), B, Lq, Lk, k, MIN)
    with pytest.raises(ValueError, match="Unsupported mask type"):
        create_mask(bias, None, B, Lq, Lk, k, MIN, type="other")


def test_bias_is_detached():
    bias = distinct_bias((1, 1, 2, 9), 7).requires_grad_()
    assert not topk_mask(bias, None, 3, MIN).requires_grad
