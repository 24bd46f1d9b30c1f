"""Frozen vectors (tests/golden/vectors.npz, written by tests/golden/make_vectors.py from the float64 closed form of
masked, biased softmax attention; the reference itself ships none for this path).

CPU: the C oracle and the fp32 eager restatement must reproduce them, so a regression of either checker is caught
without a GPU.  GPU (`-m gpu`): the operator, through the C ABI, must match them within the path's tolerances
(out max-abs <= 2e-2; gradients rtol 5e-2 as defined in _util.assert_grad_close)."""
import os

import numpy as np
import pytest
import torch

from oracle import c_oracle, eager
from _util import assert_grad_close, assert_out_close, set_compact

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "vectors.npz")
VEC = np.load(PATH)  # allow_pickle stays False
NAMES = sorted({k.split("/")[0] for k in VEC.files})
FIXED = [n for n in NAMES if f"{n}/lens_q" not in VEC.files]
RAGGED = [n for n in NAMES if f"{n}/lens_q" in VEC.files]


def _bf16(name, key):
    a = VEC[f"{name}/{key}"]
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


def _opt(name, key, conv):
    return conv(name, key) if f"{name}/{key}" in VEC.files else None


def _f32(name, key):
    return torch.from_numpy(VEC[f"{name}/{key}"].astype(np.float32))


def _load(name):
    causal, scale = VEC[f"{name}/meta"]
    mask = _opt(name, "mask", lambda n, k: torch.from_numpy(VEC[f"{n}/{k}"].copy()))
    return (_bf16(name, "q"), _bf16(name, "k"), _bf16(name, "v"), _bf16(name, "dout"), mask, _opt(name, "bias", _bf16),
            bool(causal), float(scale))


def _close(a, ref, tol, what):
    a, ref = a.float(), ref.float()
    fin = torch.isfinite(ref)
    assert torch.equal(torch.isfinite(a), fin), f"{what}: pattern of infinities differs"
    err = (a[fin] - ref[fin]).abs().max().item() if fin.any() else 0.0
    scale = max(1.0, ref[fin].abs().max().item()) if fin.any() else 1.0
    assert err <= tol * scale, f"{what}: {err:.3e} > {tol * scale:.3e}"


def test_fixture_inventory():
    assert len(FIXED) == 4 and len(RAGGED) == 1
    for n in NAMES:
        for key in ("q", "k", "v", "dout", "out", "lse", "dq", "dk", "dv", "meta"):
            assert f"{n}/{key}" in VEC.files


@pytest.mark.parametrize("name", FIXED)
def test_c_oracle_reproduces_golden_vectors(name):
    q, k, v, do, mask, bias, causal, scale = _load(name)
    out, lse = c_oracle.forward(q, k, v, mask, bias, scale, causal)
    dq, dk, dv, db = c_oracle.backward(q, k, v, do, mask, bias, scale, causal)
    for got, key in ((out, "out"), (lse, "lse"), (dq, "dq"), (dk, "dk"), (dv, "dv")):
        _close(got, _f32(name, key), 2e-6, f"{name}/{key}")
    if bias is not None:
        _close(db, _f32(name, "dbias"), 2e-6, f"{name}/dbias")


@pytest.mark.parametrize("name", FIXED)
def test_eager_restatement_reproduces_golden_vectors(name):
    q, k, v, do, mask, bias, causal, scale = _load(name)
    out, dq, dk, dv, db = eager.attention_forward_backward(q, k, v, mask, bias, scale, causal, dout=do)
    _, lse = eager.attention_forward(q, k, v, mask, bias, scale, causal)
    for got, key in ((out, "out"), (lse, "lse"), (dq, "dq"), (dk, "dk"), (dv, "dv")):
        _close(got, _f32(name, key), 2e-5, f"{name}/{key}")
    if bias is not None:
        _close(db, _f32(name, "dbias"), 2e-5, f"{name}/dbias")


@pytest.mark.parametrize("name", RAGGED)
def test_c_oracle_reproduces_ragged_golden_vectors(name):
    """The oracle has no ragged entry point: it is run per sequence, which is what the ragged layout means."""
    q, k, v, do, _, _, causal, scale = _load(name)
    q0 = k0 = 0
    for lq, lk in zip(VEC[f"{name}/lens_q"].tolist(), VEC[f"{name}/lens_k"].tolist()):
        if lq and lk:
            sq, sk = slice(q0, q0 + lq), slice(k0, k0 + lk)
            out, lse = c_oracle.forward(q[None, sq], k[None, sk], v[None, sk], None, None, scale, causal)
            dq, dk, dv, _ = c_oracle.backward(q[None, sq], k[None, sk], v[None, sk], do[None, sq], None, None, scale, causal)
            _close(out[0], _f32(name, "out")[sq], 2e-6, "out")
            _close(lse[0], _f32(name, "lse")[:, sq], 2e-6, "lse")
            _close(dq[0], _f32(name, "dq")[sq], 2e-6, "dq")
            _close(dk[0], _f32(name, "dk")[sk], 2e-6, "dk")
            _close(dv[0], _f32(name, "dv")[sk], 2e-6, "dv")
        q0, k0 = q0 + lq, k0 + lk


def _check_lse(lse, ref):
    assert torch.equal(torch.isinf(lse), torch.isinf(ref)), "empty-row pattern of the LSE differs"
    fin = torch.isfinite(ref)
    assert (lse[fin] - ref[fin]).abs().max().item() <= 1e-2
    assert (lse[~fin] > 0).all()


@pytest.mark.gpu
@pytest.mark.parametrize("compact", ["0", "2"])
@pytest.mark.parametrize("name", FIXED)
def test_operator_matches_golden_vectors(name, compact, monkeypatch):
    from flash_sparse_attn import flash_sparse_attn_func

    set_compact(compact)  # tile skipping / column compaction where the mask form allows it
    q, k, v, do, mask, bias, causal, scale = _load(name)
    dev = "cuda"
    qd, kd, vd = [t.to(dev).requires_grad_(True) for t in (q, k, v)]
    md = mask.to(dev) if mask is not None else None
    bd = bias.to(dev).requires_grad_(True) if bias is not None else None
    print(f"golden {name} compact={compact}", flush=True)
    out, lse, _ = flash_sparse_attn_func(qd, kd, vd, md, bd, scale, causal, None, None, True)
    out.backward(do.to(dev))
    torch.cuda.synchronize()
    assert_out_close(out.detach().cpu(), _f32(name, "out"))
    _check_lse(lse.cpu(), _f32(name, "lse"))
    for g, key in ((qd.grad, "dq"), (kd.grad, "dk"), (vd.grad, "dv")):
        assert_grad_close(g.cpu(), _f32(name, key), key)
    if bias is not None:
        assert_grad_close(bd.grad.cpu(), _f32(name, "dbias"), "dbias")


@pytest.mark.gpu
@pytest.mark.parametrize("name", RAGGED)
def test_ragged_operator_matches_golden_vectors(name):
    from flash_sparse_attn import flash_sparse_attn_varlen_func

    q, k, v, do, _, _, causal, scale = _load(name)
    lens_q, lens_k = VEC[f"{name}/lens_q"].tolist(), VEC[f"{name}/lens_k"].tolist()
    dev = "cuda"
    cu_q = torch.tensor([0] + np.cumsum(lens_q).tolist(), dtype=torch.int32, device=dev)
    cu_k = torch.tensor([0] + np.cumsum(lens_k).tolist(), dtype=torch.int32, device=dev)
    qd, kd, vd = [t.to(dev).requires_grad_(True) for t in (q, k, v)]
    print(f"golden {name}", flush=True)
    out, lse, _ = flash_sparse_attn_varlen_func(qd, kd, vd, cu_q, cu_k, max(lens_q), max(lens_k), scale, causal,
                                                None, None, True)
    out.backward(do.to(dev))
    torch.cuda.synchronize()
    assert_out_close(out.detach().cpu(), _f32(name, "out"))
    _check_lse(lse.cpu(), _f32(name, "lse"))
    for g, key in ((qd.grad, "dq"), (kd.grad, "dk"), (vd.grad, "dv")):
        assert_grad_close(g.cpu(), _f32(name, key), key)
