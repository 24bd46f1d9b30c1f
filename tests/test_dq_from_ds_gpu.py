"""GPU tests (`-m gpu`) of the backward for a per-query bias with a row per query head and batch entry: dBias is then dS
itself, and dQ is made from the dS tiles the dK/dV kernel has written (fdma_bwd_dq_ds.hip) instead of from a second pass
over Q, K, V, dO, mask and bias.  Shapes chosen for that kernel's edges: key counts that end inside a 16-byte chunk,
inside a tile and on a tile boundary, fewer rows than a workgroup covers, rows without a visible key (Lq > Lk), every
head-dim instantiation, both dtypes, causal and not, grouped kv heads.  Checked against the C oracle (fp64), to the
path's tolerances."""
import pytest
import torch

from oracle import c_oracle
from _util import assert_grad_close, assert_out_close, make_inputs

pytestmark = pytest.mark.gpu
DEV = "cuda"

CASES = {
    # name: (B, Lq, Lk, H, Hk, D, window, causal, dtype)
    "keys_end_inside_a_chunk": (1, 130, 203, 2, 2, 64, 60, True, torch.bfloat16),
    "keys_end_on_a_tile": (2, 256, 128, 2, 1, 64, 40, False, torch.bfloat16),
    "three_keys": (1, 70, 3, 2, 2, 64, 3, False, torch.bfloat16),
    "few_rows": (2, 5, 300, 4, 2, 32, 100, True, torch.bfloat16),
    "rows_without_keys": (1, 300, 90, 2, 2, 64, 30, True, torch.bfloat16),
    "head_dim_128_gqa": (1, 260, 330, 4, 2, 128, 100, True, torch.bfloat16),
    "head_dim_96_fp16": (1, 200, 264, 2, 1, 96, 64, True, torch.float16),
    "head_dim_256": (1, 140, 200, 2, 2, 256, 50, False, torch.bfloat16),
    "many_tiles": (1, 128, 1100, 2, 2, 64, 300, False, torch.bfloat16),
}


@pytest.mark.parametrize("name", list(CASES))
def test_backward_with_bias_per_query_and_head_vs_c_oracle(name):
    from flash_sparse_attn import flash_sparse_attn_func

    B, Lq, Lk, H, Hk, D, W, causal, dtype = CASES[name]
    q, k, v, mask, bias = make_inputs(B, Lq, Lk, H, Hk, D, (B, H, Lq, Lk), (B, Hk, Lq, Lk), W, seed=11, dtype=dtype)
    dout = torch.randn(B, Lq, H, D, generator=torch.Generator().manual_seed(12)).to(dtype)
    qd, kd, vd = [t.to(DEV).requires_grad_(True) for t in (q, k, v)]
    bd = bias.to(DEV).requires_grad_(True)
    out, lse, _ = flash_sparse_attn_func(qd, kd, vd, mask.to(DEV), bd, None, causal, None, None, True)
    out.backward(dout.to(DEV))
    torch.cuda.synchronize()
    ro, _ = c_oracle.forward(q, k, v, mask, bias, None, causal)
    rdq, rdk, rdv, rdb = c_oracle.backward(q, k, v, dout, mask, bias, None, causal)
    assert_out_close(out.detach().cpu(), ro)
    for g, r, n in ((qd.grad, rdq, "dq"), (kd.grad, rdk, "dk"), (vd.grad, rdv, "dv"), (bd.grad, rdb, "dbias")):
        assert_grad_close(g.cpu(), r, n)
    # a second run gives the same bits
    qd.grad = None
    out2, _, _ = flash_sparse_attn_func(qd, kd, vd, mask.to(DEV), bd, None, causal, None, None, True)
    dq1 = torch.autograd.grad(out2, qd, dout.to(DEV))[0]
    dq2 = torch.autograd.grad(flash_sparse_attn_func(qd, kd, vd, mask.to(DEV), bd, None, causal), qd, dout.to(DEV))[0]
    assert torch.equal(dq1, dq2)
