"""Seeded random-shape sweep of the operator against the fp32 eager restatement (run with `-m gpu`): ragged lengths from 1
to 900, every mask / bias form the operator takes (absent, per key column with 1 / Hkv / H heads, per query), causal
and not, bf16 and fp16, GQA ratios 1 / 2 / 4, head dims 32 to 128 (and, in a second block of cases, 136 to 256), larger score scales (they exercise the lazy rescale
of the running maximum), both paths for query-broadcast masks (tile skipping, column compaction) and a few grids large
enough for the 8-wave kernels.  The shapes are drawn from a fixed seed, so a failure names a reproducible case."""
import os
import random

import pytest
import torch

from oracle import eager
from _util import GRAD_RTOL, OUT_ATOL, make_inputs, set_compact

pytestmark = pytest.mark.gpu
DEV = "cuda"
N_CASES = 48
N_WIDE = 16  # further cases, numbered from N_CASES on, with head dims above 128


def _draw(it):
    rng = random.Random(7000 + it)
    D = rng.choice([32, 64, 96, 128, 128, 128])
    if it >= N_CASES:
        D = rng.choice([136, 160, 192, 256, 256])
    Hk = rng.choice([1, 2, 4])
    H = Hk * rng.choice([1, 2, 4])
    big = it % 8 == 7 and it < N_CASES
    B = rng.choice([1, 2, 3])
    Lq, Lk = rng.randint(1, 700), rng.randint(1, 900)
    form = rng.choice(["col", "col", "col_h", "full", "none", "bias_only", "mask_only"])
    if big:  # enough 256-row blocks for the 8-wave forward / dQ kernels
        B, H, Hk, D = 8, 16, rng.choice([4, 16]), 128
        Lq, Lk = rng.choice([1000, 1024]), rng.choice([1024, 1090, 777])
    causal = rng.random() < 0.7
    hm = {"col": Hk, "col_h": H, "full": rng.choice([1, Hk, H]), "none": 0, "bias_only": 0, "mask_only": rng.choice([1, Hk])}[form]
    hb = {"col": rng.choice([1, Hk, H]), "col_h": H, "full": rng.choice([1, Hk, H]), "none": 0, "bias_only": rng.choice([1, Hk, H]),
          "mask_only": 0}[form]
    rows = Lq if form == "full" else 1
    W = max(2, int(Lk * rng.choice([0.05, 0.25, 0.5, 1.0])))
    return dict(B=B, Lq=Lq, Lk=Lk, H=H, Hk=Hk, D=D, causal=causal, form=form,
                bias_shape=(B, hb, rows, Lk) if hb else None, mask_shape=(B, hm, rows, Lk) if hm else None, W=W,
                dtype=rng.choice([torch.bfloat16, torch.bfloat16, torch.float16]), qscale=rng.choice([1.0, 1.0, 3.0]),
                compact=rng.choice(["0", "1", "2"]))


@pytest.mark.parametrize("it", range(N_CASES + N_WIDE))
def test_random_case_vs_eager_fp32(it, monkeypatch):
    from flash_sparse_attn import flash_sparse_attn_func

    c = _draw(it)
    set_compact(c["compact"])
    print({k: (str(v) if k == "dtype" else v) for k, v in c.items()}, flush=True)
    q, k, v, mask, bias = make_inputs(c["B"], c["Lq"], c["Lk"], c["H"], c["Hk"], c["D"], c["bias_shape"], c["mask_shape"], c["W"],
                                      seed=1000 + it, dtype=c["dtype"])
    q = (q.float() * c["qscale"]).to(c["dtype"])
    qd, kd, vd = [t.to(DEV).requires_grad_(True) for t in (q, k, v)]
    md = mask.to(DEV) if mask is not None else None
    bd = bias.to(DEV).requires_grad_(True) if bias is not None else None
    out, lse, _ = flash_sparse_attn_func(qd, kd, vd, md, bd, None, c["causal"], None, None, True)
    do = torch.randn(out.shape, generator=torch.Generator().manual_seed(7 + it)).to(c["dtype"]).to(DEV)
    out.backward(do)
    torch.cuda.synchronize()
    bref = bd.detach() if bd is not None else None
    ro, rdq, rdk, rdv, rdb = eager.attention_forward_backward(qd.detach(), kd.detach(), vd.detach(), md, bref, None, c["causal"], dout=do)
    _, rl = eager.attention_forward(qd.detach(), kd.detach(), vd.detach(), md, bref, None, c["causal"])
    assert (out.float() - ro).abs().max().item() <= OUT_ATOL * (2 if c["qscale"] > 1 else 1)
    assert torch.equal(torch.isinf(lse), torch.isinf(rl))
    fin = torch.isfinite(rl)
    if fin.any():
        assert (lse[fin] - rl[fin]).abs().max().item() <= 2e-2 * c["qscale"]
    for name, g, r in (("dq", qd.grad, rdq), ("dk", kd.grad, rdk), ("dv", vd.grad, rdv), ("dbias", bd.grad if bd is not None else None, rdb)):
        if g is None:
            continue
        assert torch.isfinite(g.float()).all(), name
        # relative to the gradient's scale; a gradient that is (nearly) zero everywhere -- e.g. rows that see one key
        # only -- is held to an absolute bound instead
        scale = max(r.abs().max().item(), 2e-2)
        assert (g.float() - r).abs().max().item() <= GRAD_RTOL * scale, name
