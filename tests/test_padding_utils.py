"""Padding helpers (flash_sparse_attn/utils/padding.py) against per-sequence Python loops."""
import torch

from flash_sparse_attn.utils.padding import get_unpad_data, index_first_axis, pad_input, unpad_input, upad_input


def _case(seed=0, B=3, L=7, H=2, D=4):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, L, H, D, generator=g)
    lens = [7, 3, 5]
    mask = torch.zeros(B, L, dtype=torch.bool)
    for b, n in enumerate(lens):
        mask[b, L - n:] = True  # left padding
    return x, mask, lens


def test_unpad_matches_loops_and_pad_inverts_it():
    x, mask, lens = _case()
    B, L = mask.shape
    tokens, idx, cu, mx, used = unpad_input(x, mask)
    want = torch.cat([x[b, L - n:] for b, n in enumerate(lens)])
    assert torch.equal(tokens, want)
    assert idx.tolist() == [b * L + t for b, n in enumerate(lens) for t in range(L - n, L)]
    assert cu.dtype == torch.int32 and cu.tolist() == [0, 7, 10, 15]
    assert mx == 7 and isinstance(mx, int)
    assert used.dtype == torch.int32 and used.tolist() == lens
    back = pad_input(tokens, idx, B, L)
    assert torch.equal(back, x * mask[:, :, None, None])
    i2, cu2, mx2 = get_unpad_data(mask)
    assert torch.equal(i2, idx) and torch.equal(cu2, cu) and mx2 == mx
    assert torch.equal(index_first_axis(x, idx), tokens)


def test_unused_mask_tokens_are_kept_but_not_counted_as_used():
    x, mask, lens = _case(1)
    unused = torch.zeros_like(mask)
    unused[1, 0] = True
    tokens, idx, cu, mx, used = unpad_input(x, mask.int(), unused.int())
    assert tokens.shape[0] == sum(lens) + 1 and cu.tolist() == [0, 7, 11, 16] and used.tolist() == lens


def test_upad_input_three_query_forms():
    x, mask, lens = _case(2)
    B, L, H, D = x.shape
    k, v = x + 1, x + 2
    q, kk, vv, iq, (cq, ck), (mq, mk) = upad_input(x, k, v, mask, L, unpad_input)
    assert torch.equal(kk, unpad_input(k, mask)[0]) and torch.equal(vv, unpad_input(v, mask)[0])
    assert torch.equal(q, unpad_input(x, mask)[0]) and torch.equal(cq, ck) and mq == mk == 7
    # single-token decoding: every sequence contributes its one query
    q1 = x[:, -1:]
    q, kk, vv, iq, (cq, ck), (mq, mk) = upad_input(q1, k, v, mask, 1, unpad_input)
    assert q.shape == (B, H, D) and cq.tolist() == [0, 1, 2, 3] and iq.tolist() == [0, 1, 2] and mq == 1 and mk == 7
    # shorter query block: the last query_length mask columns decide; static cache longer than the mask is cut
    klong = torch.cat([k, k[:, :2]], dim=1)
    q, kk, vv, iq, (cq, ck), (mq, mk) = upad_input(x[:, -4:], klong, torch.cat([v, v[:, :2]], dim=1), mask, 4, unpad_input)
    assert torch.equal(kk, unpad_input(k, mask)[0])
    assert cq.tolist() == [0, 4, 7, 11] and mq == 4
    assert torch.equal(q, torch.cat([x[b, L - min(n, 4):] for b, n in enumerate(lens)]))
