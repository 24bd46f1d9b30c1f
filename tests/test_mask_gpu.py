"""GPU tests of the device keep-mask builder (`fdma_create_mask` behind flash_sparse_attn.utils.mask, run with `-m gpu`).

The checker is the tensor-program form of the same functions evaluated on CPU copies of the inputs (the path
tests/test_mask_utils.py ties to plain loops).  Where all values of a row differ the two must agree bit for bit;
where values tie at the selection threshold the reference leaves the choice to torch.topk, so the test checks
what is defined: the number of kept entries, the multiset of kept values, and this build's own rule (lowest
columns first among equal values).
"""
import pytest
import torch

from flash_sparse_attn.utils import mask as M

pytestmark = pytest.mark.gpu
DEV = "cuda"


def distinct_bias(shape, seed, dtype=torch.bfloat16):
    """Rows of pairwise different finite values (distinct 16-bit patterns, both signs)."""
    g = torch.Generator().manual_seed(seed)
    n = shape[-1]
    rows = 1
    for s in shape[:-1]:
        rows *= s
    # finite, non-zero magnitudes: bf16 exponents 0x30..0x47 / fp16 exponents 0x04..0x1b, any mantissa
    lo, hi = (0x3000, 0x4800) if dtype == torch.bfloat16 else (0x1000, 0x7000)
    out = torch.empty(rows, n, dtype=torch.int32)
    for r in range(rows):
        mags = torch.randperm(hi - lo, generator=g)[: (n + 1) // 2 + 1] + lo
        vals = torch.cat([mags, mags | 0x8000])[torch.randperm(2 * mags.numel(), generator=g)][:n]
        out[r] = vals.to(torch.int32)
    return out.to(torch.uint16).view(dtype).reshape(shape)


CASES = [
    # bias shape, mask shape or None, window, block_size, dtype
    ((2, 3, 1, 1000), None, 100, None, torch.bfloat16),
    ((1, 2, 37, 129), (1, 2, 37, 129), 40, None, torch.bfloat16),
    ((1, 8, 1, 8192), None, 2048, None, torch.bfloat16),
    ((2, 2, 1, 777), (2, 1, 1, 777), 300, 64, torch.bfloat16),
    ((1, 2, 5, 300), (3, 1, 1, 300), 300, None, torch.float16),
    ((2, 1, 1, 64), (2, 1, 1, 64), 48, 16, torch.float16),
    ((1, 1, 3, 5000), None, 1, None, torch.bfloat16),
]


@pytest.mark.parametrize("case", range(len(CASES)))
def test_topk_mask_distinct_values_equals_tensor_program(case):
    bshape, mshape, window, block, dtype = CASES[case]
    bias = distinct_bias(bshape, seed=case, dtype=dtype)
    mask_in = None
    if mshape is not None:
        mask_in = torch.rand(mshape, generator=torch.Generator().manual_seed(100 + case)) < 0.6
    min_dtype = torch.finfo(dtype).min
    ref = M.topk_mask(bias, mask_in, window, min_dtype, block_size=block)
    got = M.topk_mask(bias.to(DEV), mask_in.to(DEV) if mask_in is not None else None, window, min_dtype, block_size=block)
    torch.cuda.synchronize()
    assert got.dtype == torch.bool and got.shape == ref.shape
    assert torch.equal(got.cpu(), ref)


def test_topk_mask_fewer_admissible_entries_than_window():
    """A row whose incoming mask admits fewer than `window` keys keeps exactly those (mask.py:101-108)."""
    bias = distinct_bias((2, 2, 1, 200), seed=3)
    mask_in = torch.zeros(2, 1, 1, 200, dtype=torch.bool)
    mask_in[0, ..., 10:40] = True
    min_dtype = torch.finfo(torch.bfloat16).min
    got = M.topk_mask(bias.to(DEV), mask_in.to(DEV), 64, min_dtype).cpu()
    assert torch.equal(got, mask_in.expand(2, 2, 1, 200))
    assert torch.equal(got, M.topk_mask(bias, mask_in, 64, min_dtype))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_topk_mask_with_ties(dtype):
    """N(0,1) in 16 bits repeats values: the count and the kept values are what torch.topk gives; among entries
    equal to the smallest kept value the lowest columns are kept."""
    g = torch.Generator().manual_seed(5)
    bias = torch.randn(2, 4, 1, 8192, generator=g).to(dtype)
    bias[0, 0, 0, :4000] = 0.5  # a long run of equal values across the threshold
    window = 2048
    got = M.topk_mask(bias.to(DEV), None, window, torch.finfo(dtype).min).cpu()
    assert (got.sum(-1) == window).all()
    ref_vals = bias.float().topk(window, dim=-1).values.sort(dim=-1).values
    for idx in [(0, 0, 0), (0, 3, 0), (1, 2, 0)]:
        row, keep = bias[idx].float(), got[idx]
        assert torch.equal(row[keep].sort().values, ref_vals[idx])
        t = row[keep].min()
        ties = (row == t).nonzero()[:, 0]
        kept_ties = keep[ties]
        n = int(kept_ties.sum())
        assert kept_ties[:n].all() and not kept_ties[n:].any()


@pytest.mark.parametrize("block", [None, 32])
def test_relu_mask_equals_tensor_program(block):
    g = torch.Generator().manual_seed(7)
    bias = torch.randn(2, 3, 4, 333, generator=g).to(torch.bfloat16)
    bias[0, 0, 0, :7] = 0.0
    bias[0, 0, 0, 7] = -0.0
    mask_in = torch.rand(2, 1, 4, 333, generator=g) < 0.7
    min_dtype = torch.finfo(torch.bfloat16).min
    for m in (None, mask_in):
        ref = M.relu_mask(bias, m, min_dtype, block_size=block)
        got = M.relu_mask(bias.to(DEV), m.to(DEV) if m is not None else None, min_dtype, block_size=block).cpu()
        assert torch.equal(got, ref)


def test_create_mask_padding_mask_and_attention():
    """create_mask on the device from a 2-D padding mask, fed to the attention operator: same output as with the
    mask built by the tensor program on the host."""
    from flash_sparse_attn import flash_sparse_attn_func

    B, L, H, Hk, D, W = 2, 512, 4, 2, 64, 128
    g = torch.Generator().manual_seed(9)
    q, k, v = [torch.randn(B, L, n, D, generator=g).to(torch.bfloat16) for n in (H, Hk, Hk)]
    bias = distinct_bias((B, Hk, 1, L), seed=11)
    pad = torch.ones(B, L, dtype=torch.bool)
    pad[1, :100] = False
    min_dtype = torch.finfo(torch.bfloat16).min
    ref_mask = M.create_mask(bias, pad, B, L, L, W, min_dtype, block_size=None, type="topk")
    got_mask = M.create_mask(bias.to(DEV), pad.to(DEV), B, L, L, W, min_dtype, block_size=None, type="topk")
    assert torch.equal(got_mask.cpu(), ref_mask)
    qd, kd, vd, bd = [t.to(DEV) for t in (q, k, v, bias)]
    o1 = flash_sparse_attn_func(qd, kd, vd, got_mask, bd, None, True)
    o2 = flash_sparse_attn_func(qd, kd, vd, ref_mask.to(DEV), bd, None, True)
    torch.cuda.synchronize()
    assert torch.equal(o1, o2)
