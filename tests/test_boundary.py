"""CPU-only checks of the drop-in boundary: the C-ABI library loads and exports every symbol that
include/fdma.h declares, the ctypes mirrors match the compiled structs, argument validation
reproduces the reference's error rules (csrc/flash_sparse_attn/flash_api.cpp:371-438, 824-898 of the
reference) without touching a GPU, and the Python surface has the reference's names and signatures
(flash_sparse_attn/__init__.py:87-97, flash_sparse_attn_interface.py:610-621)."""
import ctypes
import inspect
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    from flash_sparse_attn import _cabi

    header = open(os.path.join(ROOT, "include", "fdma.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(fdma_[a-z_0-9]+)\s*\(", header))
    assert declared == set(_cabi.EXPORTS), declared ^ set(_cabi.EXPORTS)
    lib = ctypes.CDLL(_cabi.lib_path())
    for name in declared:
        assert hasattr(lib, name), f"{name} not exported"
    assert lib.fdma_abi_version() == 6


def test_struct_mirrors_match_compiled_sizes():
    from flash_sparse_attn import _cabi

    assert _cabi.lib.fdma_sizeof_fwd_args() == ctypes.sizeof(_cabi.FwdArgs)
    assert _cabi.lib.fdma_sizeof_bwd_args() == ctypes.sizeof(_cabi.BwdArgs)
    assert _cabi.lib.fdma_sizeof_varlen_fwd_args() == ctypes.sizeof(_cabi.VarlenFwdArgs)
    assert _cabi.lib.fdma_sizeof_varlen_bwd_args() == ctypes.sizeof(_cabi.VarlenBwdArgs)
    assert _cabi.lib.fdma_sizeof_mask_args() == ctypes.sizeof(_cabi.MaskArgs)
    assert _cabi.lib.fdma_sizeof_dyn_bias_args() == ctypes.sizeof(_cabi.DynBiasArgs)


def _valid_fwd():
    from flash_sparse_attn import _cabi

    a = _cabi.FwdArgs()
    for name in ("q", "k", "v", "out", "lse"):
        setattr(a, name, 0x1000)
    a.batch, a.seqlen_q, a.seqlen_k = 2, 128, 256
    a.num_heads, a.num_heads_k, a.num_heads_mask, a.num_heads_bias = 8, 2, 1, 1
    a.head_dim, a.dtype, a.is_causal, a.softmax_scale, a.softcap = 64, 0, 1, 0.125, 0.0
    for s, v in (("q_strides", (128 * 8 * 64, 8 * 64, 64)), ("k_strides", (256 * 2 * 64, 2 * 64, 64)),
                 ("v_strides", (256 * 2 * 64, 2 * 64, 64)), ("o_strides", (128 * 8 * 64, 8 * 64, 64))):
        getattr(a, s)[:] = v
    return a


def test_validation_accepts_a_good_call_and_needs_no_gpu():
    from flash_sparse_attn import _cabi

    a = _valid_fwd()
    assert _cabi.lib.fdma_fwd_validate(a) == 0, _cabi.last_error()
    assert _cabi.lib.fdma_fwd_workspace_bytes(a) == 0


@pytest.mark.parametrize(
    "mutate,needle",
    [
        (lambda a: setattr(a, "dtype", 7), "only support fp16 and bf16"),
        (lambda a: setattr(a, "batch", 0), "batch size must be positive"),
        (lambda a: setattr(a, "head_dim", 264), "at most 256"),
        (lambda a: setattr(a, "head_dim", 60), "multiple of 8"),
        (lambda a: setattr(a, "num_heads_k", 3), "must divide number of heads in query"),
        (lambda a: (setattr(a, "mask", 0x2000), setattr(a, "num_heads_mask", 3)), "Number of heads in mask must be 1, h_k or h"),
        (lambda a: (setattr(a, "bias", 0x2000), setattr(a, "num_heads_bias", 5)), "Number of heads in bias must be 1, h_k or h"),
        (lambda a: setattr(a, "q", 0x1004), "16-byte aligned"),
        (lambda a: setattr(a, "softcap", 30.0), "softcap"),
        (lambda a: a.k_strides.__setitem__(1, 1 << 24), "row strides of 2^24 elements or more"),
    ],
)
def test_validation_errors(mutate, needle):
    from flash_sparse_attn import _cabi

    a = _valid_fwd()
    mutate(a)
    rc = _cabi.lib.fdma_fwd_validate(a)
    assert rc < 0
    assert needle in _cabi.last_error(), _cabi.last_error()
    with pytest.raises(RuntimeError, match=re.escape(needle)):
        _cabi.check(rc)


def _with_per_query_mask(a):
    a.mask = 0x2000
    a.num_heads_mask = 2
    a.mask_strides[:] = (2 * 128 * 256, 128 * 256, 256)
    a.mask_bits.bits = 0x4000
    a.mask_bits.strides[:] = (2 * 128 * 32, 128 * 32, 32)
    return a


def test_mask_bits_validation():
    from flash_sparse_attn import _cabi

    a = _with_per_query_mask(_valid_fwd())
    assert _cabi.lib.fdma_fwd_validate(a) == 0, _cabi.last_error()
    for mutate, needle in (
        (lambda x: setattr(x, "mask", 0), "mask_bits without a mask"),
        (lambda x: x.mask_bits.strides.__setitem__(0, 0), "broadcast over the same dimensions"),
        (lambda x: x.mask_bits.strides.__setitem__(2, 24), "rounded up to 8"),
        (lambda x: setattr(x.mask_bits, "bits", 0x4004), "multiples of 8 bytes"),
        (lambda x: x.mask_bits.strides.__setitem__(1, 128 * 32 + 4), "multiples of 8 bytes"),
    ):
        a = _with_per_query_mask(_valid_fwd())
        mutate(a)
        assert _cabi.lib.fdma_fwd_validate(a) < 0
        assert needle in _cabi.last_error(), _cabi.last_error()


def test_backward_validation():
    from flash_sparse_attn import _cabi

    b = _cabi.BwdArgs()
    ctypes.memmove(ctypes.byref(b.f), ctypes.byref(_valid_fwd()), ctypes.sizeof(_cabi.FwdArgs))
    for name in ("dout", "dq", "dk", "dv", "softmax_d"):
        setattr(b, name, 0x3000)
    for s, src in (("do_strides", b.f.q_strides), ("dq_strides", b.f.q_strides), ("dk_strides", b.f.k_strides), ("dv_strides", b.f.k_strides)):
        getattr(b, s)[:] = list(src)
    assert _cabi.lib.fdma_bwd_validate(b) == 0, _cabi.last_error()
    b.f.bias = 0x4000  # bias without dbias
    assert _cabi.lib.fdma_bwd_validate(b) < 0 and "dbias" in _cabi.last_error()
    b.dbias = 0x5000
    b.f.bias_strides[:] = (512, 256, 0)
    b.dbias_strides[:] = (512, 256, 256)  # broadcast pattern differs from the bias
    assert _cabi.lib.fdma_bwd_validate(b) < 0 and "broadcast pattern" in _cabi.last_error()
    b.dbias_strides[:] = (512, 256, 0)
    assert _cabi.lib.fdma_bwd_validate(b) == 0, _cabi.last_error()
    # bias broadcast over kv groups (1 head, Hk = 2): shared dbias elements need fp32 scratch
    assert _cabi.lib.fdma_bwd_workspace_bytes(b) == 2 * 1 * 1 * 256 * 4
    b.f.num_heads_bias = 2
    assert _cabi.lib.fdma_bwd_workspace_bytes(b) == 0
    b.f.bias_strides[0] = b.dbias_strides[0] = 0  # batch-broadcast bias with batch 2: shared again
    assert _cabi.lib.fdma_bwd_workspace_bytes(b) == 1 * 2 * 1 * 256 * 4


def test_decode_workspace_size():
    from flash_sparse_attn import _cabi

    a = _valid_fwd()
    a.batch, a.seqlen_q, a.seqlen_k, a.num_heads, a.num_heads_k, a.head_dim = 8, 1, 65536, 32, 8, 128
    n = _cabi.lib.fdma_fwd_workspace_bytes(a)
    assert n > 0 and n % ((128 + 1) * 4 * 8 * 32) == 0  # splits * B * H rows of (d + 1) floats


def test_python_surface_matches_reference_names():
    import flash_sparse_attn as fsa
    from flash_sparse_attn import flash_sparse_attn_interface as itf

    assert fsa.__version__ == "1.2.3"
    assert set(fsa.__all__) == {
        "CUDA_AVAILABLE", "TRITON_AVAILABLE", "FLEX_AVAILABLE", "flash_sparse_attn_func", "flash_sparse_attn_varlen_func",
        "triton_sparse_attn_func", "flex_sparse_attn_func", "get_available_backends", "flash_sparse_attn_func_auto"}
    assert fsa.CUDA_AVAILABLE and fsa.get_available_backends() == ["cuda"]
    assert fsa.flash_sparse_attn_func_auto() is fsa.flash_sparse_attn_func
    assert fsa.flash_sparse_attn_func_auto(backend="cuda") is itf.flash_sparse_attn_func
    with pytest.raises(RuntimeError, match="Triton backend is not available"):
        fsa.flash_sparse_attn_func_auto(backend="triton")
    with pytest.raises(RuntimeError, match="Flex backend is not available"):
        fsa.flash_sparse_attn_func_auto(backend="flex")
    with pytest.raises(ValueError, match="Unknown backend"):
        fsa.flash_sparse_attn_func_auto(backend="nope")
    sig = inspect.signature(itf.flash_sparse_attn_func)
    assert list(sig.parameters) == ["query", "key", "value", "attn_mask", "attn_bias", "softmax_scale", "is_causal",
                                    "softcap", "deterministic", "return_attn_probs"]
    assert all(p.default is None for n, p in sig.parameters.items() if n not in ("query", "key", "value"))
    for name in ("FlashDMAttnFunc", "_flash_sparse_attn_forward", "_flash_sparse_attn_backward", "maybe_contiguous",
                 "round_multiple", "flash_sparse_attn_varlen_func"):
        assert hasattr(itf, name)
    # the custom ops are registered under the reference's names
    assert hasattr(torch.ops.flash_sparse_attn, "_flash_sparse_attn_forward")
    assert hasattr(torch.ops.flash_sparse_attn, "_flash_sparse_attn_backward")


def test_cpu_tensors_are_rejected_loudly():
    """No CPU fallback: the operator only exists for device tensors (device_types="cuda")."""
    from flash_sparse_attn import flash_sparse_attn_func

    q = torch.randn(1, 8, 2, 64, dtype=torch.bfloat16)
    with pytest.raises((RuntimeError, NotImplementedError)):
        flash_sparse_attn_func(q, q, q)


def test_dispatch_modes_and_functorch_see_the_registered_operators():
    """In plain eager mode the operator bodies run directly (the dispatcher costs more than a small kernel), but a
    TorchDispatchMode / TorchFunctionMode (FLOP counters, profilers) and functorch transforms must get the registered
    operators, as with the reference (flash_sparse_attn_interface.py:73, 126, 432)."""
    from torch.overrides import TorchFunctionMode
    from torch.utils._python_dispatch import TorchDispatchMode

    from flash_sparse_attn import flash_sparse_attn_func, flash_sparse_attn_varlen_func
    from flash_sparse_attn import flash_sparse_attn_interface as itf

    seen = []

    class Recorder(TorchDispatchMode):
        def __torch_dispatch__(self, func, types, args=(), kwargs=None):
            seen.append(str(func))
            if "_flash_sparse_attn_forward" in str(func):  # (stands in for the device: shapes of the fake kernel)
                q = args[0]
                return (torch.empty_like(q), torch.empty(q.shape[0], q.shape[2], q.shape[1]), torch.empty(0, dtype=q.dtype))
            if "_flash_sparse_attn_varlen_forward" in str(func):
                q = args[0]
                return (torch.empty_like(q), torch.empty(q.shape[1], q.shape[0]), torch.empty(0, dtype=q.dtype))
            return func(*args, **(kwargs or {}))

    q = torch.randn(1, 8, 2, 64, dtype=torch.bfloat16)
    assert itf._plain_eager(q, q, q)
    with Recorder():
        assert not itf._plain_eager(q, q, q)
        out = flash_sparse_attn_func(q, q, q)
        assert out.shape == q.shape
        cu = torch.tensor([0, 8], dtype=torch.int32)
        flash_sparse_attn_varlen_func(q[0], q[0], q[0], cu, cu, 8, 8)
    assert any("flash_sparse_attn._flash_sparse_attn_forward" in f for f in seen)
    assert any("flash_sparse_attn._flash_sparse_attn_varlen_forward" in f for f in seen)

    class Passive(TorchFunctionMode):
        def __torch_function__(self, func, types, args=(), kwargs=None):
            return func(*args, **(kwargs or {}))

    with Passive():
        assert not itf._plain_eager(q)

    wrapped = []

    def probe(x):
        wrapped.append(itf._plain_eager(x))
        return x.float().sum()

    torch.func.grad(probe)(torch.randn(4))
    assert wrapped == [False]
    assert not itf._nothing_to_differentiate(True, q.requires_grad_(True))
    assert itf._nothing_to_differentiate(False, q)


def test_product_package_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "flash-dmattn_amd")
    for dirpath, _, files in os.walk(pkg):
        for fn in files:
            if fn.endswith((".py", ".cpp", ".hip", ".h")):
                text = open(os.path.join(dirpath, fn)).read()
                assert "oracle" not in text.lower(), f"{fn} mentions the oracle"


def test_compaction_workspace_rule():
    """fdma_*_workspace_bytes is pure host arithmetic: the column-compaction path asks for scratch exactly when the
    mask is query-broadcast and the call's compact_mode allows it; a mask with a row per QUERY head over grouped kv heads
    is compacted per query head in the forward (G copies of the kept K / V rows) and not at all in the backward."""
    import torch
    from flash_sparse_attn import _cabi

    def args(Lq, Lk, H, Hk, Hm, mask_rows):
        B, D = 1, 64
        q = torch.empty(B, Lq, H, D, dtype=torch.bfloat16)
        k = torch.empty(B, Lk, Hk, D, dtype=torch.bfloat16)
        mask = torch.empty(B, Hm, mask_rows, Lk, dtype=torch.bool)
        bias = torch.empty(B, Hk, 1, Lk, dtype=torch.bfloat16)
        lse = torch.empty(B, H, Lq, dtype=torch.float32)
        a = _cabi.FwdArgs()
        _cabi.fill_fwd(a, q, k, k, mask, bias, torch.empty_like(q), lse, 0.125, True, 0.0)
        return a

    small = args(256, 256, 4, 2, 2, 1)
    big = args(4096, 4096, 4, 2, 2, 1)
    per_query = args(4096, 4096, 4, 2, 2, 4096)
    per_qhead = args(4096, 4096, 4, 2, 4, 1)
    assert small.compact_mode == _cabi.COMPACT_AUTO == 0   # (the default of a freshly filled block)
    big.compact_mode = _cabi.COMPACT_NEVER
    assert _cabi.lib.fdma_fwd_workspace_bytes(big) == 0
    for a in (small, per_query, per_qhead):
        a.compact_mode = _cabi.COMPACT_ALWAYS
    assert _cabi.lib.fdma_fwd_workspace_bytes(small) > 0
    assert _cabi.lib.fdma_fwd_workspace_bytes(per_query) == 0
    per_qhead_need = _cabi.lib.fdma_fwd_workspace_bytes(per_qhead)
    big.compact_mode = _cabi.COMPACT_ALWAYS
    assert per_qhead_need > 1.5 * _cabi.lib.fdma_fwd_workspace_bytes(big)   # a copy per query head, not per kv head
    import ctypes
    b = _cabi.BwdArgs()  # (the backward of that form takes the tile-skipping kernels: no compaction scratch)
    ctypes.memmove(ctypes.byref(b.f), ctypes.byref(per_qhead), ctypes.sizeof(per_qhead))
    assert _cabi.lib.fdma_bwd_workspace_bytes(b) == 0
    small.compact_mode = big.compact_mode = _cabi.COMPACT_AUTO
    assert _cabi.lib.fdma_fwd_workspace_bytes(small) == 0       # too small for the pre-pass to pay
    need = _cabi.lib.fdma_fwd_workspace_bytes(big)
    kv_bytes = 2 * 4096 * 2 * 64 * 2
    assert kv_bytes <= need <= 2 * kv_bytes                      # dense K / V copies plus index lists


def _valid_varlen_fwd():
    from flash_sparse_attn import _cabi

    a = _cabi.VarlenFwdArgs()
    for name in ("q", "k", "v", "out", "lse", "cu_seqlens_q", "cu_seqlens_k"):
        setattr(a, name, 0x1000)
    a.batch, a.total_q, a.total_k, a.max_seqlen_q, a.max_seqlen_k = 3, 300, 500, 128, 256
    a.num_heads, a.num_heads_k, a.head_dim, a.dtype, a.is_causal = 8, 2, 64, 0, 1
    a.softmax_scale, a.softcap = 0.125, 0.0
    for s, v in (("q_strides", (8 * 64, 64)), ("k_strides", (2 * 64, 64)), ("v_strides", (2 * 64, 64)),
                 ("o_strides", (8 * 64, 64))):
        getattr(a, s)[:] = v
    return a


@pytest.mark.parametrize(
    "field,value,message",
    [
        ("dtype", 7, "only support fp16 and bf16"),
        ("batch", 0, "batch size must be positive"),
        ("head_dim", 260, "head dimension at most 256"),
        ("head_dim", 60, "multiple of 8"),
        ("num_heads_k", 3, "must divide number of heads in query"),
        ("cu_seqlens_q", 0, "cu_seqlens_q and cu_seqlens_k must be device pointers"),
        ("cu_seqlens_k", 0x1002, "4-byte aligned"),
        ("softcap", 1.0, "softcap is not supported"),
        ("q", 0x1008, "16-byte aligned"),
    ],
)
def test_varlen_validation_rejects(field, value, message):
    """Ragged-batch argument rules (csrc/flash_sparse_attn/flash_api.cpp:583-660 of the reference), checked
    without a GPU."""
    from flash_sparse_attn import _cabi

    a = _valid_varlen_fwd()
    assert _cabi.lib.fdma_varlen_fwd_validate(a) == 0, _cabi.last_error()
    setattr(a, field, value)
    assert _cabi.lib.fdma_varlen_fwd_validate(a) < 0
    assert message in _cabi.last_error()


def test_varlen_backward_validation():
    from flash_sparse_attn import _cabi

    b = _cabi.VarlenBwdArgs()
    b.f = _valid_varlen_fwd()
    for name in ("dout", "dq", "dk", "dv", "softmax_d"):
        setattr(b, name, 0x2000)
    for s, v in (("do_strides", (8 * 64, 64)), ("dq_strides", (8 * 64, 64)), ("dk_strides", (2 * 64, 64)),
                 ("dv_strides", (2 * 64, 64))):
        getattr(b, s)[:] = v
    assert _cabi.lib.fdma_varlen_bwd_validate(b) == 0, _cabi.last_error()
    b.dk = 0
    assert _cabi.lib.fdma_varlen_bwd_validate(b) < 0
    assert "dout, dq, dk, dv must be device pointers" in _cabi.last_error()
    b.dk = 0x2000
    b.dq_strides[0] = 8 * 64 + 4
    assert _cabi.lib.fdma_varlen_bwd_validate(b) < 0
    assert "multiples of 8" in _cabi.last_error()


def test_varlen_operator_signature_matches_reference():
    """flash_sparse_attn_interface.py:687-701 of the reference."""
    from flash_sparse_attn import flash_sparse_attn_varlen_func

    names = list(inspect.signature(flash_sparse_attn_varlen_func).parameters)
    assert names == ["query", "key", "value", "cu_seqlens_q", "cu_seqlens_k", "max_seqlen_q", "max_seqlen_k",
                     "softmax_scale", "is_causal", "softcap", "deterministic", "return_attn_probs", "block_table"]


def test_mask_builder_validation():
    """Argument rules of fdma_create_mask (the builder behind flash_sparse_attn.utils.mask), checked without a GPU."""
    from flash_sparse_attn import _cabi

    def good():
        a = _cabi.MaskArgs()
        a.bias, a.mask_out = 0x1000, 0x2000
        a.batch, a.heads, a.rows, a.seqlen_k = 2, 4, 1, 512
        a.bias_strides[:] = (4 * 512, 512, 0)
        a.mask_out_strides[:] = (4 * 512, 512, 512)
        a.window, a.block_size, a.type, a.dtype, a.min_value = 128, 0, 0, 0, -3.0e38
        return a

    assert _cabi.lib.fdma_create_mask_validate(good()) == 0, _cabi.last_error()
    for field, value, message in (("dtype", 3, "fp16 or bf16"), ("type", 2, "Unsupported mask type"),
                                  ("window", -1, "window_size must be non-negative"),
                                  ("block_size", -2, "block_size must be a positive integer"),
                                  ("bias", 0, "device pointers"), ("bias", 0x1001, "2-byte aligned"),
                                  ("min_value", float("nan"), "must not be NaN")):
        a = good()
        setattr(a, field, value)
        assert _cabi.lib.fdma_create_mask_validate(a) < 0, field
        assert message in _cabi.last_error()
    # the optional bit-packed output: 8-byte aligned rows of at least ceil(seqlen_k / 8) bytes rounded up to 8
    a = good()
    a.bits, a.bits_row_bytes = 0x3000, 64
    assert _cabi.lib.fdma_create_mask_validate(a) == 0, _cabi.last_error()
    for bits, row_bytes, message in ((0x3000, 60, "multiple of 8"), (0x3000, 56, "multiple of 8"), (0x3004, 64, "8-byte aligned")):
        a = good()
        a.bits, a.bits_row_bytes = bits, row_bytes
        assert _cabi.lib.fdma_create_mask_validate(a) < 0
        assert message in _cabi.last_error(), _cabi.last_error()


def test_bias_producer_validation_and_workspace():
    """Argument rules of fdma_dyn_bias_* (the producer behind flash_sparse_attn.utils.bias), checked without a GPU."""
    from flash_sparse_attn import _cabi

    def good():
        a = _cabi.DynBiasArgs()
        for name in ("value", "weight", "a", "bias", "dt", "dbias", "dvalue", "dweight", "da"):
            setattr(a, name, 0x1000)
        a.batch, a.seqlen_k, a.num_heads_k, a.head_dim, a.dtype = 2, 1000, 8, 128, 0
        a.value_strides[:] = (1000 * 1024, 1024, 128)
        a.dvalue_strides[:] = (1000 * 1024, 1024, 128)
        a.bias_strides[:] = (8 * 1000, 1000)
        a.dbias_strides[:] = (8 * 1000, 1000)
        return a

    assert _cabi.lib.fdma_dyn_bias_validate(good(), 0) == 0, _cabi.last_error()
    assert _cabi.lib.fdma_dyn_bias_validate(good(), 1) == 0, _cabi.last_error()
    # 2000 tokens -> 63 workgroups of 32 tokens, each with Hk * Hk * d + 2 * Hk fp32 partial sums
    assert _cabi.lib.fdma_dyn_bias_bwd_workspace_bytes(good()) == 63 * (8 * 8 * 128 + 16) * 4
    for field, value, backward, message in (("dtype", 5, 0, "fp16 or bf16"), ("num_heads_k", 33, 0, "1 to 32 kv heads"),
                                            ("head_dim", 12, 0, "multiple of 8"), ("weight", 0, 0, "device pointers"),
                                            ("value", 0x1008, 0, "16-byte aligned"), ("dweight", 0, 1, "device pointers"),
                                            ("dproj_bias", 0x1000, 1, "exactly when proj_bias"),
                                            ("dvalue", 0x1004, 1, "8-byte aligned")):
        a = good()
        setattr(a, field, value)
        assert _cabi.lib.fdma_dyn_bias_validate(a, backward) < 0, field
        assert message in _cabi.last_error(), (field, _cabi.last_error())


def test_missing_library_fails_loudly():
    """Without libfdma_hip.so there is nothing to fall back to: the operator module refuses to import, the package reports
    no backend (as the reference does without its extension), and asking for one raises."""
    import subprocess
    import sys

    code = r'''
import importlib, sys
sys.path.insert(0, sys.argv[1])
try:
    importlib.import_module("flash_sparse_attn.flash_sparse_attn_interface")
    print("IMPORTED")
except ImportError as e:
    print("ImportError:", e)
import flash_sparse_attn as pkg
print("CUDA_AVAILABLE", pkg.CUDA_AVAILABLE, pkg.flash_sparse_attn_func, pkg.get_available_backends())
try:
    pkg.flash_sparse_attn_func_auto()
    print("RETURNED")
except RuntimeError as e:
    print("RuntimeError:", e)
'''
    env = dict(os.environ, FDMA_LIB="/nonexistent/libfdma_hip.so")
    out = subprocess.run([sys.executable, "-c", code, os.path.join(ROOT, "flash-dmattn_amd")], env=env, capture_output=True,
                         text=True, timeout=300).stdout
    assert "ImportError:" in out and "no fallback" in out and "IMPORTED" not in out, out
    assert "CUDA_AVAILABLE False None []" in out, out
    assert "RuntimeError: No flash attention backend is available" in out and "RETURNED" not in out, out
