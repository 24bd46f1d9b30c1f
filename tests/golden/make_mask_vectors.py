"""Writes tests/golden/mask_vectors.npz: inputs and outputs of the REFERENCE's keep-mask builders.

Run in the build container only (`python tests/golden/make_mask_vectors.py`): it loads
/root/reference/flash_sparse_attn/utils/mask.py by file path (the module needs nothing but torch) and calls
topk_mask / relu_mask / block_smooth / create_mask on small inputs.  What these functions return is not fixed by a
closed form in two places -- which of several EQUAL values torch.topk selects, and the in-place block vote -- so the
outputs are frozen here as data.  The fixture holds inputs and expected masks only; the GPU box never sees the reference.

Bias values are small integers, exact in bf16 / fp16 / fp32, so the same fixture serves the fp32 tensor program on
the CPU and the 16-bit device kernel.  Cases named *_distinct have pairwise different values in every row (the
result is then fully determined and must be matched bit for bit); cases named *_ties repeat values, and only what
every valid top-k choice shares is comparable: the number of kept entries per row and the multiset of kept values.
"""
import importlib.util
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
REF = "/root/reference/flash_sparse_attn/utils/mask.py"


def load_reference():
    spec = importlib.util.spec_from_file_location("reference_mask", REF)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def distinct_rows(gen, shape):
    """Integers, pairwise different inside every row of the last dim, centred on zero."""
    L = shape[-1]
    rows = int(np.prod(shape[:-1]))
    out = torch.stack([torch.randperm(L, generator=gen) for _ in range(rows)]).reshape(shape)
    return (out - L // 2).float()


def main():
    ref = load_reference()
    g = torch.Generator().manual_seed(2024)
    MIN = float(torch.finfo(torch.bfloat16).min)
    cases = {}

    def add(name, fn, bias, mask, **kw):
        """fn: 'topk' | 'relu' | 'create'; stores inputs and the reference's output."""
        if fn == "topk":
            out = ref.topk_mask(bias.clone(), None if mask is None else mask.clone(), kw["window"], MIN, kw.get("block"))
        elif fn == "relu":
            out = ref.relu_mask(bias.clone(), None if mask is None else mask.clone(), MIN, kw.get("block"))
        else:
            out = ref.create_mask(bias.clone(), None if mask is None else mask.clone(), kw["batch"], kw["query_len"],
                                  kw["key_len"], kw["window"], MIN, kw.get("block"), kw["type"])
        cases[name] = dict(fn=fn, bias=bias, mask=mask, out=out, **kw)

    # top-k on distinct values: plain, with a 4-D mask, window >= admissible keys, window == row length, block smoothing
    b = distinct_rows(g, (2, 3, 5, 64))
    add("topk_distinct_plain", "topk", b, None, window=17)
    m = torch.rand(2, 3, 5, 64, generator=g) > 0.4
    add("topk_distinct_masked", "topk", b, m, window=17)
    add("topk_distinct_window_exceeds_admissible", "topk", b, torch.rand(2, 3, 5, 64, generator=g) > 0.85, window=30)
    add("topk_distinct_full_window", "topk", b, None, window=64)
    add("topk_distinct_broadcast_mask", "topk", distinct_rows(g, (2, 4, 1, 100)), torch.rand(2, 1, 1, 100, generator=g) > 0.3, window=40)
    for blk in (2, 8, 16, 64):
        add(f"topk_distinct_block{blk}", "topk", distinct_rows(g, (1, 2, 3, 100)), None, window=45, block=blk)  # 100 keys: tails of 0, 4, 4, 36
    add("topk_distinct_block_masked", "topk", distinct_rows(g, (2, 2, 1, 256)), torch.rand(2, 2, 1, 256, generator=g) > 0.5, window=100, block=32)
    # relu
    br = distinct_rows(g, (2, 2, 4, 100))
    add("relu_distinct_plain", "relu", br, None)
    add("relu_distinct_masked", "relu", br, torch.rand(2, 2, 4, 100, generator=g) > 0.5)
    add("relu_distinct_block8", "relu", br, None, block=8)
    add("relu_distinct_block7_masked", "relu", br, torch.rand(2, 1, 4, 100, generator=g) > 0.3, block=7)
    # create_mask: 2-D padding masks of both widths, 4-D masks, both types
    bc = distinct_rows(g, (3, 2, 1, 96))
    pad_k = torch.ones(3, 96, dtype=torch.bool)
    pad_k[0, :10] = False
    pad_k[2, 50:] = False
    add("create_topk_2d_key_width", "create", bc, pad_k, batch=3, query_len=40, key_len=96, window=32, type="topk")
    pad_q = torch.ones(3, 40, dtype=torch.bool)
    pad_q[1, :7] = False
    add("create_topk_2d_query_width", "create", bc, pad_q, batch=3, query_len=40, key_len=96, window=32, type="topk")
    add("create_topk_2d_query_width_block", "create", bc, pad_q, batch=3, query_len=40, key_len=96, window=32, type="topk", block=16)
    add("create_relu_2d_key_width", "create", bc, pad_k, batch=3, query_len=40, key_len=96, window=32, type="relu")
    bq = distinct_rows(g, (2, 2, 6, 48))
    causal = torch.tril(torch.ones(6, 48, dtype=torch.bool), diagonal=42).view(1, 1, 6, 48)
    add("create_topk_4d_causal", "create", bq, causal, batch=2, query_len=6, key_len=48, window=12, type="topk")
    add("create_topk_equal_lengths_2d", "create", distinct_rows(g, (2, 1, 1, 32)), torch.rand(2, 32, generator=g) > 0.2,
        batch=2, query_len=32, key_len=32, window=8, type="topk")
    # ties: few distinct values per row
    bt = torch.randint(-3, 4, (2, 2, 3, 64), generator=g).float()
    add("topk_ties_plain", "topk", bt, None, window=20)
    add("topk_ties_masked", "topk", bt, torch.rand(2, 2, 3, 64, generator=g) > 0.4, window=20)
    # block_smooth on its own (in place on a clone), including a tail
    raw = torch.rand(2, 3, 4, 50, generator=g) > 0.5
    for blk in (1, 4, 16, 50, 64):
        cases[f"block_smooth_{blk}"] = dict(fn="smooth", mask_in=raw, out=ref.block_smooth(raw.clone(), 50, blk), block=blk, key_len=50)

    flat = {}
    meta = []
    for name, c in cases.items():
        for k, v in c.items():
            if torch.is_tensor(v):
                flat[f"{name}/{k}"] = v.numpy().astype(np.uint8 if v.dtype == torch.bool else np.float32)
        meta.append(";".join([name] + [f"{k}={v}" for k, v in c.items() if not torch.is_tensor(v) and v is not None]))
    flat["__meta__"] = np.array(meta)
    flat["__min_dtype__"] = np.array([MIN], dtype=np.float64)
    path = os.path.join(HERE, "mask_vectors.npz")
    np.savez_compressed(path, **flat)
    print(f"{len(cases)} cases -> {path} ({os.path.getsize(path)} bytes)")


if __name__ == "__main__":
    main()
