"""GPU tests (`-m gpu`) of the bit-packed hand-over of a per-query keep-mask: the device mask builder writes, next to
the bool mask, every row packed to one bit per key (`fdma_mask_bits`), and the per-query attention kernels read that
instead of a byte per score.  It does not change what is computed: every comparison here is bit for bit against the
same call with the mask as a plain bool tensor.
"""
import numpy as np
import pytest
import torch

from flash_sparse_attn import flash_sparse_attn_func
from flash_sparse_attn.utils import mask as M

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.mark.parametrize("shape,window,block", [((2, 3, 5, 1000), 100, None), ((1, 2, 300, 777), 300, 64),
                                                ((3, 1, 7, 50), 20, None), ((1, 2, 130, 4096), 1024, None),
                                                ((1, 1, 3, 33), 5, None), ((2, 2, 2, 8), 3, None)])
def test_mask_builder_writes_the_rows_packed_to_bits(shape, window, block):
    bias = torch.randn(shape, generator=torch.Generator().manual_seed(shape[-1])).to(torch.bfloat16).to(DEV)
    mask = M.topk_mask(bias, None, window, torch.finfo(torch.bfloat16).min, block_size=block)
    bits = M.mask_bits_of(mask)
    assert bits is not None and bits.dtype == torch.uint8 and tuple(bits.shape[:3]) == shape[:3]
    torch.cuda.synchronize()
    n_bytes = (shape[-1] + 7) // 8
    assert bits.shape[-1] >= n_bytes and bits.shape[-1] % 4 == 0
    want = np.packbits(mask.cpu().numpy().astype(np.uint8), axis=-1, bitorder="little")
    assert want.shape[-1] == n_bytes
    assert np.array_equal(bits[..., :n_bytes].cpu().numpy(), want)
    # a mask that has been written to since no longer carries its bits
    mask[..., 0] = True
    assert M.mask_bits_of(mask) is None
    # a query-broadcast mask has none to begin with (it carries index lists instead)
    col = M.topk_mask(bias[:, :, :1], None, window, torch.finfo(torch.bfloat16).min)
    assert M.mask_bits_of(col) is None and M.kept_keys_of(col) is not None


def _run(q, k, v, mask, bias, causal):
    qg, kg, vg, bg = [t.detach().clone().requires_grad_(True) for t in (q, k, v, bias)]
    out, lse, _ = flash_sparse_attn_func(qg, kg, vg, mask, bg, None, causal, None, None, True)
    g = torch.Generator().manual_seed(5)
    out.backward(torch.randn(out.shape, generator=g).to(out.dtype).to(DEV))
    torch.cuda.synchronize()
    return out.detach(), lse.detach(), qg.grad, kg.grad, vg.grad, bg.grad


CASES = {
    # name: (B, Lq, Lk, H, Hk, Hm, D, window, causal, dtype)
    "d64_mha": (2, 300, 300, 4, 4, 4, 64, 100, True, torch.bfloat16),
    "d128_gqa_mask_per_kv_head": (1, 257, 391, 8, 2, 2, 128, 150, True, torch.bfloat16),
    "d128_one_mask_head_noncausal": (2, 130, 777, 4, 2, 1, 128, 300, False, torch.float16),
    "d256_lk_not_a_multiple_of_8": (1, 100, 333, 2, 1, 1, 256, 120, True, torch.bfloat16),
    "d32_lq_gt_lk": (1, 500, 100, 2, 2, 2, 32, 40, True, torch.bfloat16),
    "d96_short_rows": (3, 33, 13, 2, 2, 2, 96, 5, False, torch.bfloat16),
    "d128_large_grid": (1, 2048, 2048, 8, 8, 8, 128, 512, True, torch.bfloat16),
}


@pytest.mark.parametrize("name", list(CASES))
def test_attention_with_and_without_the_bits_is_bit_identical(name):
    B, Lq, Lk, H, Hk, Hm, D, W, causal, dt = CASES[name]
    g = torch.Generator().manual_seed(len(name))
    q = torch.randn(B, Lq, H, D, generator=g).to(dt).to(DEV)
    k = torch.randn(B, Lk, Hk, D, generator=g).to(dt).to(DEV)
    v = torch.randn(B, Lk, Hk, D, generator=g).to(dt).to(DEV)
    bias = torch.randn(B, Hm, Lq, Lk, generator=g).to(dt).to(DEV)
    mask = M.topk_mask(bias, None, W, torch.finfo(dt).min)
    assert M.mask_bits_of(mask) is not None
    plain = mask.clone()
    assert M.mask_bits_of(plain) is None
    with_bits = _run(q, k, v, mask, bias, causal)
    without = _run(q, k, v, plain, bias, causal)
    for a, b, n in zip(with_bits, without, ("out", "lse", "dq", "dk", "dv", "dbias")):
        assert torch.equal(a, b), n
    assert all(torch.isfinite(t.float()).all() for t in with_bits[2:])


def test_wrong_bits_change_the_result():
    """The kernels really read the bits: with the bits of another mask attached, the output follows the bits."""
    B, Lq, Lk, H, D = 1, 128, 256, 2, 64
    g = torch.Generator().manual_seed(9)
    q = torch.randn(B, Lq, H, D, generator=g).to(torch.bfloat16).to(DEV)
    k = torch.randn(B, Lk, H, D, generator=g).to(torch.bfloat16).to(DEV)
    v = torch.randn(B, Lk, H, D, generator=g).to(torch.bfloat16).to(DEV)
    bias = torch.randn(B, H, Lq, Lk, generator=g).to(torch.bfloat16).to(DEV)
    other = torch.randn(B, H, Lq, Lk, generator=g).to(torch.bfloat16).to(DEV)
    lowest = torch.finfo(torch.bfloat16).min
    mask_a = M.topk_mask(bias, None, 64, lowest)
    mask_b = M.topk_mask(other, None, 64, lowest)
    ref_b = flash_sparse_attn_func(q, k, v, mask_b.clone(), bias, None, False)
    # the bool mask of A with the bits of B attached
    rec = mask_b._fdma_bits
    mask_a._fdma_bits = (rec[0], mask_a._version, mask_a.data_ptr(), tuple(mask_a.shape))
    out = flash_sparse_attn_func(q, k, v, mask_a, bias, None, False)
    torch.cuda.synchronize()
    assert torch.equal(out, ref_b)
