"""ctypes wrapper around libfdma_oracle.so (built from fdma_oracle.c by `make -C oracle`).

TEST INFRASTRUCTURE ONLY.  Inputs are torch CPU tensors in the operator's layouts
(q (B,Lq,H,D); k,v (B,Lk,Hk,D); mask bool / bias 4-D with broadcastable dims); they are converted
to fp32 (bf16 / fp16 values are exactly representable) and the arithmetic is IEEE double.
"""
import ctypes
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "libfdma_oracle.so")


class _Shape(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in ("b", "lq", "lk", "h", "hk", "d", "mb", "mh", "mq", "mk", "bb", "bh", "bq", "bk")] + [
        ("scale", ctypes.c_float), ("causal", ctypes.c_int32)]


def build() -> str:
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)
    return _LIB


def _lib():
    if not os.path.exists(_LIB):
        build()
    lib = ctypes.CDLL(_LIB)
    fp = ctypes.c_void_p
    lib.fdma_oracle_fwd.argtypes = [ctypes.POINTER(_Shape)] + [fp] * 7
    lib.fdma_oracle_fwd.restype = ctypes.c_int
    lib.fdma_oracle_bwd.argtypes = [ctypes.POINTER(_Shape)] + [fp] * 10
    lib.fdma_oracle_bwd.restype = ctypes.c_int
    lib.fdma_oracle_combine.argtypes = [ctypes.c_int, ctypes.c_long, ctypes.c_int] + [fp] * 4
    lib.fdma_oracle_combine.restype = ctypes.c_int
    return lib


_cached = None


def lib():
    global _cached
    if _cached is None:
        _cached = _lib()
    return _cached


def _f32(t):
    return None if t is None else np.ascontiguousarray(t.detach().to(torch.float32).cpu().numpy())


def _u8(t):
    return None if t is None else np.ascontiguousarray(t.detach().cpu().numpy().astype(np.uint8))


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _shape(q, k, mask, bias, scale, causal):
    s = _Shape()
    s.b, s.lq, s.h, s.d = q.shape
    s.lk, s.hk = k.shape[1], k.shape[2]
    s.mb, s.mh, s.mq, s.mk = mask.shape if mask is not None else (0, 0, 0, 0)
    s.bb, s.bh, s.bq, s.bk = bias.shape if bias is not None else (0, 0, 0, 0)
    s.scale = float(scale)
    s.causal = int(bool(causal))
    return s


def forward(q, k, v, mask=None, bias=None, scale=None, causal=False):
    """returns (out fp32 (B,Lq,H,D), lse fp32 (B,H,Lq))"""
    if scale is None:
        scale = q.shape[-1] ** -0.5
    qa, ka, va, ma, ba = _f32(q), _f32(k), _f32(v), _u8(mask), _f32(bias)
    s = _shape(qa, ka, ma, ba, scale, causal)
    out = np.empty(qa.shape, np.float32)
    lse = np.empty((s.b, s.h, s.lq), np.float32)
    rc = lib().fdma_oracle_fwd(ctypes.byref(s), _p(qa), _p(ka), _p(va), _p(ma), _p(ba), _p(out), _p(lse))
    assert rc == 0
    return torch.from_numpy(out), torch.from_numpy(lse)


def backward(q, k, v, dout, mask=None, bias=None, scale=None, causal=False):
    """returns (dq, dk, dv, dbias or None), fp32, dbias at the bias's own (broadcast) shape"""
    if scale is None:
        scale = q.shape[-1] ** -0.5
    qa, ka, va, ma, ba, da = _f32(q), _f32(k), _f32(v), _u8(mask), _f32(bias), _f32(dout)
    s = _shape(qa, ka, ma, ba, scale, causal)
    dq, dk, dv = np.empty(qa.shape, np.float32), np.empty(ka.shape, np.float32), np.empty(va.shape, np.float32)
    db = np.empty(ba.shape, np.float32) if ba is not None else None
    rc = lib().fdma_oracle_bwd(ctypes.byref(s), _p(qa), _p(ka), _p(va), _p(ma), _p(ba), _p(da), _p(dq), _p(dk), _p(dv), _p(db))
    assert rc == 0
    return torch.from_numpy(dq), torch.from_numpy(dk), torch.from_numpy(dv), (torch.from_numpy(db) if db is not None else None)


def combine(o_part, lse_part):
    """o_part (S, R, D), lse_part (S, R) -> (o (R, D), lse (R,))"""
    oa, la = _f32(o_part), _f32(lse_part)
    S, R, D = oa.shape
    o, lse = np.empty((R, D), np.float32), np.empty((R,), np.float32)
    rc = lib().fdma_oracle_combine(S, R, D, _p(oa), _p(la), _p(o), _p(lse))
    assert rc == 0
    return torch.from_numpy(o), torch.from_numpy(lse)
