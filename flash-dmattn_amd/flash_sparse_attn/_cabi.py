"""ctypes binding of libfdma_hip.so (declared in include/fdma.h).

This is the only place the Python operator touches native code.  It plays the part of the
reference's ``import flash_sparse_attn_cuda`` (flash_sparse_attn/flash_sparse_attn_interface.py:7):
importing this module raises ImportError when the HIP library has not been built, and there is no
CPU or eager fallback behind it.
"""
import contextlib
import ctypes
import os
import struct
from typing import Optional, Sequence

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_DEFAULT_LIB = os.path.normpath(os.path.join(_HERE, "..", "lib", "libfdma_hip.so"))


class KeptKeys(ctypes.Structure):
    """fdma_kept_keys: the kept columns of a query-broadcast keep-mask as lists."""
    _fields_ = [("idx", ctypes.c_void_p), ("cnt", ctypes.c_void_p), ("count", ctypes.c_void_p), ("ld", ctypes.c_int32)]


class MaskBits(ctypes.Structure):
    """fdma_mask_bits: a per-query keep-mask packed to one bit per key (strides in bytes: batch, head, row)."""
    _fields_ = [("bits", ctypes.c_void_p), ("strides", ctypes.c_int64 * 3)]


class FwdArgs(ctypes.Structure):
    _fields_ = [
        ("q", ctypes.c_void_p), ("k", ctypes.c_void_p), ("v", ctypes.c_void_p),
        ("mask", ctypes.c_void_p), ("bias", ctypes.c_void_p),
        ("out", ctypes.c_void_p), ("lse", ctypes.c_void_p),
        ("q_strides", ctypes.c_int64 * 3), ("k_strides", ctypes.c_int64 * 3),
        ("v_strides", ctypes.c_int64 * 3), ("o_strides", ctypes.c_int64 * 3),
        ("mask_strides", ctypes.c_int64 * 3), ("bias_strides", ctypes.c_int64 * 3),
        ("batch", ctypes.c_int32), ("seqlen_q", ctypes.c_int32), ("seqlen_k", ctypes.c_int32),
        ("num_heads", ctypes.c_int32), ("num_heads_k", ctypes.c_int32),
        ("num_heads_mask", ctypes.c_int32), ("num_heads_bias", ctypes.c_int32),
        ("head_dim", ctypes.c_int32), ("dtype", ctypes.c_int32), ("is_causal", ctypes.c_int32),
        ("softmax_scale", ctypes.c_float), ("softcap", ctypes.c_float),
        ("compact_mode", ctypes.c_int32),
        ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_size_t),
        ("kept", KeptKeys),
        ("mask_bits", MaskBits),
        ("counters", ctypes.c_void_p), ("counters_bytes", ctypes.c_size_t),
    ]


class BwdArgs(ctypes.Structure):
    _fields_ = [
        ("f", FwdArgs),
        ("dout", ctypes.c_void_p),
        ("dq", ctypes.c_void_p), ("dk", ctypes.c_void_p), ("dv", ctypes.c_void_p),
        ("dbias", ctypes.c_void_p),
        ("do_strides", ctypes.c_int64 * 3), ("dq_strides", ctypes.c_int64 * 3),
        ("dk_strides", ctypes.c_int64 * 3), ("dv_strides", ctypes.c_int64 * 3),
        ("dbias_strides", ctypes.c_int64 * 3),
        ("softmax_d", ctypes.c_void_p),
        ("deterministic", ctypes.c_int32),
        ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_size_t),
        ("fwd_workspace", ctypes.c_void_p), ("fwd_workspace_bytes", ctypes.c_size_t),
    ]


class VarlenFwdArgs(ctypes.Structure):
    _fields_ = [
        ("q", ctypes.c_void_p), ("k", ctypes.c_void_p), ("v", ctypes.c_void_p),
        ("out", ctypes.c_void_p), ("lse", ctypes.c_void_p),
        ("cu_seqlens_q", ctypes.c_void_p), ("cu_seqlens_k", ctypes.c_void_p),
        ("q_strides", ctypes.c_int64 * 2), ("k_strides", ctypes.c_int64 * 2),
        ("v_strides", ctypes.c_int64 * 2), ("o_strides", ctypes.c_int64 * 2),
        ("batch", ctypes.c_int32), ("total_q", ctypes.c_int32), ("total_k", ctypes.c_int32),
        ("max_seqlen_q", ctypes.c_int32), ("max_seqlen_k", ctypes.c_int32),
        ("num_heads", ctypes.c_int32), ("num_heads_k", ctypes.c_int32), ("head_dim", ctypes.c_int32),
        ("dtype", ctypes.c_int32), ("is_causal", ctypes.c_int32),
        ("softmax_scale", ctypes.c_float), ("softcap", ctypes.c_float),
    ]


class VarlenBwdArgs(ctypes.Structure):
    _fields_ = [
        ("f", VarlenFwdArgs),
        ("dout", ctypes.c_void_p),
        ("dq", ctypes.c_void_p), ("dk", ctypes.c_void_p), ("dv", ctypes.c_void_p),
        ("do_strides", ctypes.c_int64 * 2), ("dq_strides", ctypes.c_int64 * 2),
        ("dk_strides", ctypes.c_int64 * 2), ("dv_strides", ctypes.c_int64 * 2),
        ("softmax_d", ctypes.c_void_p),
        ("deterministic", ctypes.c_int32),
    ]


class MaskArgs(ctypes.Structure):
    _fields_ = [
        ("bias", ctypes.c_void_p), ("mask_in", ctypes.c_void_p), ("mask_out", ctypes.c_void_p),
        ("bias_strides", ctypes.c_int64 * 3), ("mask_in_strides", ctypes.c_int64 * 3),
        ("mask_out_strides", ctypes.c_int64 * 3),
        ("batch", ctypes.c_int32), ("heads", ctypes.c_int32), ("rows", ctypes.c_int32), ("seqlen_k", ctypes.c_int32),
        ("window", ctypes.c_int32), ("block_size", ctypes.c_int32), ("type", ctypes.c_int32), ("dtype", ctypes.c_int32),
        ("min_value", ctypes.c_float),
        ("kept_idx", ctypes.c_void_p), ("kept_cnt", ctypes.c_void_p), ("kept_count", ctypes.c_void_p),
        ("kept_ld", ctypes.c_int32),
        ("bits", ctypes.c_void_p), ("bits_row_bytes", ctypes.c_int64),
    ]


class DynBiasArgs(ctypes.Structure):
    _fields_ = [
        ("value", ctypes.c_void_p), ("weight", ctypes.c_void_p), ("proj_bias", ctypes.c_void_p), ("a", ctypes.c_void_p),
        ("bias", ctypes.c_void_p), ("dt", ctypes.c_void_p),
        ("value_strides", ctypes.c_int64 * 3), ("bias_strides", ctypes.c_int64 * 2),
        ("batch", ctypes.c_int32), ("seqlen_k", ctypes.c_int32), ("num_heads_k", ctypes.c_int32), ("head_dim", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
        ("dbias", ctypes.c_void_p), ("dbias_strides", ctypes.c_int64 * 2),
        ("dvalue", ctypes.c_void_p), ("dvalue_strides", ctypes.c_int64 * 3),
        ("dweight", ctypes.c_void_p), ("da", ctypes.c_void_p), ("dproj_bias", ctypes.c_void_p),
        ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_size_t),
    ]


EXPORTS = (
    "fdma_fwd", "fdma_fwd_noalloc", "fdma_bwd", "fdma_fwd_workspace_bytes", "fdma_fwd_counter_bytes", "fdma_bwd_workspace_bytes",
    "fdma_set_stream_min_items",
    "fdma_fwd_validate", "fdma_bwd_validate", "fdma_last_error", "fdma_abi_version",
    "fdma_sizeof_fwd_args", "fdma_sizeof_bwd_args",
    "fdma_varlen_fwd", "fdma_varlen_bwd", "fdma_varlen_fwd_validate", "fdma_varlen_bwd_validate",
    "fdma_sizeof_varlen_fwd_args", "fdma_sizeof_varlen_bwd_args",
    "fdma_create_mask", "fdma_create_mask_validate", "fdma_sizeof_mask_args",
    "fdma_dyn_bias_fwd", "fdma_dyn_bias_bwd", "fdma_dyn_bias_bwd_workspace_bytes", "fdma_dyn_bias_validate",
    "fdma_sizeof_dyn_bias_args",
)


# Column compaction policy handed to every attention call (fdma_fwd_args.compact_mode): 0 = the library decides
# from the problem, 1 = never (tile skipping only), 2 = whenever the mask form allows it.  The environment variable
# FDMA_COMPACT is read ONCE, here, as the default ("0" = never, "2" = always); set_compact_mode() changes it for
# the process, compact_mode() for a with-block.
NOALLOC_SCRATCH_BYTES = (8 << 20) - (64 << 10)  # FDMA_NOALLOC_SCRATCH_BYTES - FDMA_NOALLOC_COUNTER_BYTES: what a problem may need
COMPACT_AUTO, COMPACT_NEVER, COMPACT_ALWAYS = 0, 1, 2
_compact_mode = {"0": COMPACT_NEVER, "2": COMPACT_ALWAYS}.get(os.environ.get("FDMA_COMPACT", "")[:1], COMPACT_AUTO)


def get_compact_mode() -> int:
    return _compact_mode


def set_compact_mode(mode: int) -> int:
    """Set the compaction policy of later calls; returns the previous one."""
    global _compact_mode
    if mode not in (COMPACT_AUTO, COMPACT_NEVER, COMPACT_ALWAYS):
        raise ValueError("compact mode must be COMPACT_AUTO, COMPACT_NEVER or COMPACT_ALWAYS")
    previous, _compact_mode = _compact_mode, mode
    return previous


@contextlib.contextmanager
def compact_mode(mode: int):
    previous = set_compact_mode(mode)
    try:
        yield
    finally:
        set_compact_mode(previous)


def stream_min_items(n: int = 0) -> int:
    """Threshold (in 256-row query block x head items) from which the compacted forward at head dim 128 streams tile
    images (fdma_set_stream_min_items); n <= 0 only queries.  Returns the value before the call."""
    return lib.fdma_set_stream_min_items(int(n))


def lib_path() -> str:
    return os.environ.get("FDMA_LIB", _DEFAULT_LIB)


def _load() -> ctypes.CDLL:
    path = lib_path()
    if not os.path.exists(path):
        raise ImportError(
            f"libfdma_hip.so not found at {path}: build it with `make -C flash-dmattn_amd/csrc` "
            "(or __graft_entry__.build()); there is no fallback implementation"
        )
    try:
        lib = ctypes.CDLL(path)
    except OSError as e:  # missing HIP runtime etc.
        raise ImportError(f"cannot load {path}: {e}") from e
    lib.fdma_fwd.argtypes = [ctypes.POINTER(FwdArgs), ctypes.c_void_p]
    lib.fdma_fwd.restype = ctypes.c_int
    lib.fdma_fwd_noalloc.argtypes = [ctypes.POINTER(FwdArgs), ctypes.c_void_p]
    lib.fdma_fwd_noalloc.restype = ctypes.c_int
    lib.fdma_bwd.argtypes = [ctypes.POINTER(BwdArgs), ctypes.c_void_p]
    lib.fdma_bwd.restype = ctypes.c_int
    lib.fdma_fwd_validate.argtypes = [ctypes.POINTER(FwdArgs)]
    lib.fdma_fwd_validate.restype = ctypes.c_int
    lib.fdma_bwd_validate.argtypes = [ctypes.POINTER(BwdArgs)]
    lib.fdma_bwd_validate.restype = ctypes.c_int
    lib.fdma_fwd_workspace_bytes.argtypes = [ctypes.POINTER(FwdArgs)]
    lib.fdma_fwd_workspace_bytes.restype = ctypes.c_size_t
    lib.fdma_fwd_counter_bytes.argtypes = [ctypes.POINTER(FwdArgs)]
    lib.fdma_fwd_counter_bytes.restype = ctypes.c_size_t
    lib.fdma_set_stream_min_items.argtypes = [ctypes.c_int]
    lib.fdma_set_stream_min_items.restype = ctypes.c_int
    lib.fdma_bwd_workspace_bytes.argtypes = [ctypes.POINTER(BwdArgs)]
    lib.fdma_bwd_workspace_bytes.restype = ctypes.c_size_t
    lib.fdma_last_error.argtypes = []
    lib.fdma_last_error.restype = ctypes.c_char_p
    lib.fdma_abi_version.restype = ctypes.c_int
    lib.fdma_sizeof_fwd_args.restype = ctypes.c_size_t
    lib.fdma_sizeof_bwd_args.restype = ctypes.c_size_t
    if lib.fdma_abi_version() != 6:
        raise ImportError(f"{path}: ABI version {lib.fdma_abi_version()} != 6")
    lib.fdma_varlen_fwd.argtypes = [ctypes.POINTER(VarlenFwdArgs), ctypes.c_void_p]
    lib.fdma_varlen_fwd.restype = ctypes.c_int
    lib.fdma_varlen_bwd.argtypes = [ctypes.POINTER(VarlenBwdArgs), ctypes.c_void_p]
    lib.fdma_varlen_bwd.restype = ctypes.c_int
    lib.fdma_varlen_fwd_validate.argtypes = [ctypes.POINTER(VarlenFwdArgs)]
    lib.fdma_varlen_fwd_validate.restype = ctypes.c_int
    lib.fdma_varlen_bwd_validate.argtypes = [ctypes.POINTER(VarlenBwdArgs)]
    lib.fdma_varlen_bwd_validate.restype = ctypes.c_int
    lib.fdma_sizeof_varlen_fwd_args.restype = ctypes.c_size_t
    lib.fdma_sizeof_varlen_bwd_args.restype = ctypes.c_size_t
    lib.fdma_create_mask.argtypes = [ctypes.POINTER(MaskArgs), ctypes.c_void_p]
    lib.fdma_create_mask.restype = ctypes.c_int
    lib.fdma_create_mask_validate.argtypes = [ctypes.POINTER(MaskArgs)]
    lib.fdma_create_mask_validate.restype = ctypes.c_int
    lib.fdma_sizeof_mask_args.restype = ctypes.c_size_t
    lib.fdma_dyn_bias_fwd.argtypes = [ctypes.POINTER(DynBiasArgs), ctypes.c_void_p]
    lib.fdma_dyn_bias_fwd.restype = ctypes.c_int
    lib.fdma_dyn_bias_bwd.argtypes = [ctypes.POINTER(DynBiasArgs), ctypes.c_void_p]
    lib.fdma_dyn_bias_bwd.restype = ctypes.c_int
    lib.fdma_dyn_bias_bwd_workspace_bytes.argtypes = [ctypes.POINTER(DynBiasArgs)]
    lib.fdma_dyn_bias_bwd_workspace_bytes.restype = ctypes.c_size_t
    lib.fdma_dyn_bias_validate.argtypes = [ctypes.POINTER(DynBiasArgs), ctypes.c_int]
    lib.fdma_dyn_bias_validate.restype = ctypes.c_int
    lib.fdma_sizeof_dyn_bias_args.restype = ctypes.c_size_t
    sizes = ((lib.fdma_sizeof_dyn_bias_args(), DynBiasArgs), (lib.fdma_sizeof_mask_args(), MaskArgs), (lib.fdma_sizeof_fwd_args(), FwdArgs), (lib.fdma_sizeof_bwd_args(), BwdArgs),
             (lib.fdma_sizeof_varlen_fwd_args(), VarlenFwdArgs), (lib.fdma_sizeof_varlen_bwd_args(), VarlenBwdArgs))
    if any(n != ctypes.sizeof(t) for n, t in sizes):
        raise ImportError(f"{path}: argument block size differs from the Python mirror")
    return lib


lib = _load()


def last_error() -> str:
    return lib.fdma_last_error().decode()


def check(rc: int) -> None:
    """Every failure of the native layer surfaces as RuntimeError, as TORCH_CHECK does."""
    if rc != 0:
        raise RuntimeError(last_error() or f"libfdma_hip error {rc}")


_DTYPES = {torch.bfloat16: 0, torch.float16: 1}


def dtype_code(t: torch.Tensor) -> int:
    if t.dtype not in _DTYPES:
        raise RuntimeError("FlashSparseAttention only support fp16 and bf16 data type")
    return _DTYPES[t.dtype]


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _s3(t: torch.Tensor) -> Sequence[int]:
    """(batch, row, head) strides of a (B, L, H, D) tensor."""
    return (t.stride(0), t.stride(1), t.stride(2))


def _bcast3(t: torch.Tensor) -> Sequence[int]:
    """(batch, head, row) strides of a 4-D mask / bias, 0 for size-1 (broadcast) dims."""
    sh, st = t.shape, t.stride()
    return (0 if sh[0] == 1 else st[0], 0 if sh[1] == 1 else st[1], 0 if sh[2] == 1 else st[2])


_FWD_STRUCT = struct.Struct("@7P18q10i2fiPN3Pi4xP3qPN")
assert _FWD_STRUCT.size == ctypes.sizeof(FwdArgs)


def fill_fwd(a: FwdArgs, q, k, v, mask, bias, out, lse, softmax_scale, is_causal, softcap, kept=None, bits=None) -> None:
    """Fill the argument block in one struct.pack (ctypes field-by-field assignment costs ~10 us a call).
    `kept`: None, or (idx, cnt, count, ld) -- the mask's kept columns as int32 tensors (fdma_kept_keys).
    `bits`: None, or the mask packed to one bit per key, a uint8 tensor of the mask's shape but for the last
    dimension (fdma_mask_bits)."""
    bt = _bcast3(bits) if bits is not None else (0, 0, 0)
    ms = _bcast3(mask) if mask is not None else (0, 0, 0)
    bs = _bcast3(bias) if bias is not None else (0, 0, 0)
    batch, seqlen_q, num_heads, head_dim = q.shape
    qs, ks, vs, os_ = q.stride(), k.stride(), v.stride(), out.stride()
    _FWD_STRUCT.pack_into(
        _as_buffer(a), 0,
        q.data_ptr(), k.data_ptr(), v.data_ptr(),
        mask.data_ptr() if mask is not None else 0, bias.data_ptr() if bias is not None else 0,
        out.data_ptr(), lse.data_ptr(),
        qs[0], qs[1], qs[2], ks[0], ks[1], ks[2],
        vs[0], vs[1], vs[2], os_[0], os_[1], os_[2],
        ms[0], ms[1], ms[2], bs[0], bs[1], bs[2],
        batch, seqlen_q, k.shape[1], num_heads, k.shape[2],
        mask.shape[1] if mask is not None else 1, bias.shape[1] if bias is not None else 1,
        head_dim, dtype_code(q), int(bool(is_causal)),
        float(softmax_scale), float(softcap), _compact_mode, 0, 0,
        kept[0].data_ptr() if kept else 0, kept[1].data_ptr() if kept else 0, kept[2].data_ptr() if kept else 0,
        kept[3] if kept else 0,
        bits.data_ptr() if bits is not None else 0, bt[0], bt[1], bt[2],
        0, 0,
    )


def fill_varlen_fwd(a: VarlenFwdArgs, q, k, v, out, lse, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
                    softmax_scale, is_causal, softcap) -> None:
    a.q, a.k, a.v = q.data_ptr(), k.data_ptr(), v.data_ptr()
    a.out, a.lse = out.data_ptr(), lse.data_ptr()
    a.cu_seqlens_q, a.cu_seqlens_k = cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr()
    a.q_strides[:] = (q.stride(0), q.stride(1))
    a.k_strides[:] = (k.stride(0), k.stride(1))
    a.v_strides[:] = (v.stride(0), v.stride(1))
    a.o_strides[:] = (out.stride(0), out.stride(1))
    a.batch = cu_seqlens_q.numel() - 1
    a.total_q, a.total_k = q.shape[0], k.shape[0]
    a.max_seqlen_q, a.max_seqlen_k = int(max_seqlen_q), int(max_seqlen_k)
    a.num_heads, a.num_heads_k, a.head_dim = q.shape[1], k.shape[1], q.shape[2]
    a.dtype = dtype_code(q)
    a.is_causal = int(bool(is_causal))
    a.softmax_scale, a.softcap = float(softmax_scale), float(softcap)


def _as_buffer(a):
    return (ctypes.c_char * ctypes.sizeof(a)).from_address(ctypes.addressof(a))


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_NO_GUARD = contextlib.nullcontext()


def current_stream(device: torch.device) -> int:
    """Handle of torch's current stream on `device` (the raw getter skips building a Stream object: 0.3 vs 4 us)."""
    if _raw_stream is not None:
        return _raw_stream(device.index if device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(device).cuda_stream


def device_guard(device: torch.device):
    """Context that makes `device` current for the launch; free when it already is."""
    if device.index is None or device.index == torch.cuda.current_device():
        return _NO_GUARD
    return torch.cuda.device(device)
