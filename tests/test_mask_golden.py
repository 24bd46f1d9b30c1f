"""The keep-mask builders against outputs of the reference's own utils/mask.py, frozen in tests/golden/mask_vectors.npz.

The fixture (inputs and expected masks, written by tests/golden/make_mask_vectors.py from
flash_sparse_attn/utils/mask.py:47-240 of the reference) pins what a restatement cannot: the block vote with a tail
block, the exclusion of the fill value when the window exceeds the admissible keys, and the 2-D padding-mask
handling of both widths.  Cases with pairwise different values per row must match bit for bit, on the CPU tensor
program here and on the device kernel (`-m gpu`).  In the *_ties cases the reference's result depends on which of
several equal values torch.topk picks, which torch does not define: only the number of kept entries per row and
the multiset of kept values are compared.
"""
import os

import numpy as np
import pytest
import torch

from flash_sparse_attn.utils import mask as M

FIXTURE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "mask_vectors.npz")


def load_cases():
    z = np.load(FIXTURE)
    cases = {}
    for line in z["__meta__"]:
        name, *kv = str(line).split(";")
        c = dict(p.split("=", 1) for p in kv)
        for k in ("window", "block", "batch", "query_len", "key_len"):
            if k in c:
                c[k] = int(c[k])
        for k in ("bias", "mask", "mask_in", "out"):
            if f"{name}/{k}" in z.files:
                a = torch.from_numpy(z[f"{name}/{k}"])
                c[k] = a.bool() if a.dtype == torch.uint8 else a
        cases[name] = c
    return cases, float(z["__min_dtype__"][0])


CASES, FILL = load_cases()
BUILDER_CASES = sorted(n for n, c in CASES.items() if c["fn"] != "smooth")
SMOOTH_CASES = sorted(n for n, c in CASES.items() if c["fn"] == "smooth")


def run_case(c, device, dtype):
    bias = c["bias"].to(dtype).to(device)
    mask = c.get("mask")
    mask = None if mask is None else mask.to(device)
    # the fill value only has to lie below every bias value; each 16-bit type gets its own most negative number,
    # as a caller of that type would pass it
    MIN = FILL if dtype == torch.float32 else torch.finfo(dtype).min
    if c["fn"] == "topk":
        return M.topk_mask(bias, mask, c["window"], MIN, c.get("block"))
    if c["fn"] == "relu":
        return M.relu_mask(bias, mask, MIN, c.get("block"))
    return M.create_mask(bias, mask, c["batch"], c["query_len"], c["key_len"], c["window"], MIN, c.get("block"), c["type"])


def check(name, c, got):
    want = c["out"]
    assert got.dtype == torch.bool and tuple(got.shape) == tuple(want.shape), name
    if "ties" not in name:
        assert torch.equal(got, want), f"{name}: {(got != want).sum().item()} entries differ"
        return
    assert torch.equal(got.sum(-1), want.sum(-1)), name
    bias = c["bias"].expand(want.shape)
    big = torch.finfo(torch.float32).max
    kept_got = torch.where(got, bias, big).sort(-1).values
    kept_want = torch.where(want, bias, big).sort(-1).values
    assert torch.equal(kept_got, kept_want), name


def test_fixture_covers_what_it_claims():
    """The fixture is only worth its cases: tails, windows beyond the admissible keys, both 2-D widths, both types."""
    assert len(BUILDER_CASES) >= 20 and len(SMOOTH_CASES) >= 5
    c = CASES["topk_distinct_window_exceeds_admissible"]
    admissible = c["mask"].sum(-1)
    assert (admissible < c["window"]).any() and torch.equal(c["out"].sum(-1)[admissible < c["window"]], admissible[admissible < c["window"]])
    assert CASES["create_topk_2d_key_width"]["mask"].shape[-1] == CASES["create_topk_2d_key_width"]["key_len"]
    assert CASES["create_topk_2d_query_width"]["mask"].shape[-1] == CASES["create_topk_2d_query_width"]["query_len"]
    assert any(CASES[n]["key_len"] % CASES[n]["block"] for n in SMOOTH_CASES)
    for n in BUILDER_CASES:
        if "distinct" in n:  # every row's values differ, so the expected mask is the only valid one
            b = CASES[n]["bias"]
            assert (b.sort(-1).values.diff(dim=-1) != 0).all(), n


@pytest.mark.parametrize("name", SMOOTH_CASES)
def test_block_smooth_equals_reference_output(name):
    c = CASES[name]
    got = M.block_smooth(c["mask_in"].clone(), c["key_len"], c["block"])
    assert torch.equal(got, c["out"])


@pytest.mark.parametrize("name", BUILDER_CASES)
def test_tensor_program_equals_reference_output(name):
    check(name, CASES[name], run_case(CASES[name], "cpu", torch.float32))


@pytest.mark.parametrize("name", BUILDER_CASES)
def test_tensor_program_in_16_bits_equals_reference_output(name):
    """The fixture's values are small integers, so the 16-bit forms of the inputs select the same entries."""
    check(name, CASES[name], run_case(CASES[name], "cpu", torch.bfloat16))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("name", BUILDER_CASES)
def test_device_kernel_equals_reference_output(name, dtype):
    c = CASES[name]
    assert c["bias"].abs().max() <= 256  # exact in both 16-bit types
    got = run_case(c, "cuda", dtype)
    torch.cuda.synchronize()
    check(name, c, got.cpu())
