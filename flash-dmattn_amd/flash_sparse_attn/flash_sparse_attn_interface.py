"""Python operator of Flash Dynamic Mask Attention on MI355X.

Host-side mirror of the reference's flash_sparse_attn/flash_sparse_attn_interface.py: the same public
functions, argument meaning, defaults, return conventions and error behaviour
(`flash_sparse_attn_func` :610-684, `FlashDMAttnFunc` :382-498, the custom ops
`flash_sparse_attn::_flash_sparse_attn_forward/_backward` :73-123, 206-285), but the compiled
extension behind it is libfdma_hip.so (hand-written gfx950 kernels behind a C ABI) instead of
`flash_sparse_attn_cuda`.  PyTorch is used for device memory, streams and autograd only.

Differences that are visible only in cost, not in results:
  * gradients are allocated with ``empty_like`` (the kernels write every element exactly once)
    instead of ``zeros_like`` (:463-464);
  * mask / bias are padded along the key dimension only when the kernels' 16-byte row alignment
    needs it, not always to a multiple of 128 (:420-430);
  * dK / dV / dBias come out of the kernels at their final shapes; there are no expanded
    temporaries or host-side reductions (flash_api.cpp:970-983, 1027-1047).
"""
import threading
from typing import Any, Optional, Tuple

import torch

from . import _cabi
from .utils.mask import kept_keys_of, mask_bits_of


def maybe_contiguous(x: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    return x.contiguous() if x is not None and x.stride(-1) != 1 else x


def round_multiple(x, m):
    return (x + m - 1) // m * m


def _aligned(x: Optional[torch.Tensor], elems: int) -> Optional[torch.Tensor]:
    """Make x usable by the kernels' 16-byte vector accesses: last dim contiguous, base pointer
    16-byte aligned, every other stride a multiple of `elems` elements."""
    if x is None:
        return None
    if x.is_contiguous() and x.shape[-1] % elems == 0 and x.data_ptr() % 16 == 0:
        return x  # fast path: every stride of a contiguous tensor is a multiple of its last dim
    x = maybe_contiguous(x)
    ok = x.data_ptr() % 16 == 0 and all(x.size(i) == 1 or x.stride(i) % elems == 0 for i in range(x.dim() - 1))
    return x if ok else x.contiguous().clone(memory_format=torch.contiguous_format)


_len_dispatch_stack = getattr(torch._C, "_len_torch_dispatch_stack", None)
_len_function_stack = getattr(torch._C, "_len_torch_function_stack", None)
_is_functorch_wrapped = getattr(getattr(torch._C, "_functorch", None), "is_functorch_wrapped_tensor", None)


def _plain_eager(*tensors) -> bool:
    """True when nothing but the device would see a call on these tensors: eager mode, no TorchDispatchMode /
    TorchFunctionMode active (FLOP counters, profilers, fake-tensor tracing install such modes and must see the
    registered operators), and every tensor an ordinary torch.Tensor that no functorch transform (torch.func.grad /
    vmap / jvp) has wrapped.  Where torch lacks one of the probes the answer is False: the dispatcher is always right."""
    if torch.compiler.is_compiling():
        return False
    if _len_dispatch_stack is None or _len_function_stack is None or _is_functorch_wrapped is None:
        return False
    if _len_dispatch_stack() > 0 or _len_function_stack() > 0:
        return False
    for t in tensors:
        if t is not None and (type(t) is not torch.Tensor or _is_functorch_wrapped(t)):
            return False
    return True


def _direct_when_eager(op, body):
    """Callable for one of the operators below.  On plain tensors in eager mode it runs the operator's Python
    body directly: the dispatch of a torch.library operator costs about 20 us per call, more than a small
    attention call takes on the device.  Under torch.compile, under an active dispatch / function mode, and for
    fake tensors, tensor subclasses or functorch-wrapped tensors the registered operator is called, as the reference
    always does (flash_sparse_attn_interface.py:126, 432)."""
    def call(*args, **kwargs):
        if _plain_eager(*[a for a in args[:5] if a is None or isinstance(a, torch.Tensor)]):
            return body(*args, **kwargs)
        return op(*args, **kwargs)

    return call


_HALF_TYPES = (torch.float16, torch.bfloat16)


def _inputs_plainly_ok(q, k, v, mask, bias) -> bool:
    """One pass over what _check_inputs checks, without messages: True means every rule holds (the usual case, and the
    one that matters for calls that take a few microseconds on the device); False sends the call through _check_inputs,
    which finds the rule that failed and raises the reference's message for it."""
    dt = q.dtype
    if not (dt in _HALF_TYPES and k.dtype is dt and v.dtype is dt and q.is_cuda and k.is_cuda and v.is_cuda):
        return False
    qs, ks = q.shape, k.shape
    if not (len(qs) == 4 and len(ks) == 4 and ks == v.shape):
        return False
    batch, seqlen_q, num_heads, head_size = qs
    seqlen_k, num_heads_k = ks[1], ks[2]
    if not (batch > 0 and head_size <= 256 and head_size % 8 == 0 and num_heads_k > 0 and num_heads % num_heads_k == 0
            and ks[0] == batch and ks[3] == head_size):
        return False
    for t, want in ((mask, torch.bool), (bias, dt)):
        if t is None:
            continue
        ts = t.shape
        if not (t.dtype is want and t.is_cuda and len(ts) == 4 and (ts[0] == batch or ts[0] == 1)
                and (ts[1] == 1 or ts[1] == num_heads_k or ts[1] == num_heads) and (ts[2] == 1 or ts[2] == seqlen_q)
                and ts[3] >= seqlen_k):
            return False
    return True


def _check_inputs(q, k, v, mask, bias) -> None:
    """Device / dtype / rank / shape checks of mha_fwd (flash_api.cpp:371-438, 477-479)."""
    if _inputs_plainly_ok(q, k, v, mask, bias):
        return
    if q.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError("FlashSparseAttention only support fp16 and bf16 data type")
    if k.dtype != q.dtype:
        raise RuntimeError("query and key must have the same dtype")
    if v.dtype != q.dtype:
        raise RuntimeError("query and value must have the same dtype")
    for name, t in (("q", q), ("k", k), ("v", v), ("mask", mask), ("bias", bias)):
        if t is not None and not t.is_cuda:
            raise RuntimeError(f"{name} must be on CUDA")
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise RuntimeError("q, k, v must have shape (batch_size, seqlen, nheads, headdim)")
    batch, seqlen_q, num_heads, head_size = q.shape
    seqlen_k, num_heads_k = k.shape[1], k.shape[2]
    if batch <= 0:
        raise RuntimeError("batch size must be positive")
    if head_size > 256:
        raise RuntimeError("FlashSparseAttention forward only supports head dimension at most 256")
    if head_size % 8 != 0:
        raise RuntimeError("query, key, value, and out_ must have a head_size that is a multiple of 8")
    if num_heads_k <= 0 or num_heads % num_heads_k != 0:
        raise RuntimeError("Number of heads in key/value must divide number of heads in query")
    if tuple(k.shape) != (batch, seqlen_k, num_heads_k, head_size):
        raise RuntimeError(f"k must have shape ({batch}, {seqlen_k}, {num_heads_k}, {head_size})")
    if tuple(v.shape) != (batch, seqlen_k, num_heads_k, head_size):
        raise RuntimeError(f"v must have shape ({batch}, {seqlen_k}, {num_heads_k}, {head_size})")
    for name, t in (("mask", mask), ("bias", bias)):
        if t is None:
            continue
        if name == "mask" and t.dtype != torch.bool:
            raise RuntimeError("mask must have dtype bool")
        if name == "bias" and t.dtype != q.dtype:
            raise RuntimeError("bias must have the same dtype as inputs")
        if t.dim() != 4:
            raise RuntimeError(f"{name} must have 4 dimensions with shape (batch_size, nheads, seqlen_q, seqlen_k_rounded)")
        if t.size(0) not in (batch, 1):
            raise RuntimeError(f"Batch dimension in {name} must be 1 or equal to batch size")
        if t.size(1) not in (1, num_heads_k, num_heads):
            raise RuntimeError(f"Number of heads in {name} must be 1, h_k or h")
        if t.size(2) not in (1, seqlen_q):
            raise RuntimeError(f"Query length dimension in {name} must be 1 or equal to seqlen_q")
        if t.size(3) < seqlen_k:
            raise RuntimeError(f"Key length dimension in {name} must be seqlen_k_rounded")


# Side inputs of the two operator bodies that are not part of the reference's operator signatures: the kept-key
# lists (query-broadcast mask) or the bit-packed form (per-query mask) of a mask made by the device mask builder, and
# the forward call's workspace (index lists and compacted K / V
# copies), which the backward of the same autograd node reuses.  FlashDMAttnFunc sets them around its calls; a body
# that is called without them (torch.compile, direct operator calls) takes the ordinary path.
_tls = threading.local()


class _handoff:
    def __init__(self, **items):
        self.items = items

    def __enter__(self):
        self.prev = getattr(_tls, "items", None)
        _tls.items = self.items
        return self.items

    def __exit__(self, *exc):
        _tls.items = self.prev


def _lists_for(lists, mask, k, exact):
    """The mask builder's second output (kept-key lists, or bit rows) for `mask`, if it describes the key axis of this
    call: the lists number the kept columns of the WHOLE mask row, so a mask that is wider than K (already padded) or
    has a key dimension of 1 (expanded later) is scanned by the kernels instead.  Bit rows may be wider than K."""
    if lists is None or mask is None:
        return None
    width, seqlen_k = mask.shape[-1], k.shape[1]
    return lists if (width == seqlen_k or (not exact and width > seqlen_k)) else None


def _handoff_get(name):
    items = getattr(_tls, "items", None)
    return items.get(name) if items else None


# Per-(device, stream) scratch of the decode path (seqlen_q == 1), where a call takes about as long on the device as
# three tensor allocations take on the host.  Calls on one stream run one after the other, so they can share the
# split-KV workspace; calls on different streams may overlap on the device and get buffers of their own.  The arrival
# counters of the one-launch decode (fdma_fwd_args.counters) are zero before a call and zero after it: they are
# cleared when the buffer is made and then serve every later call on that stream.
_decode_scratch = {}
_decode_sizes = {}   # (batch, heads, kv heads, keys, head dim) -> (workspace bytes, counter bytes): pure functions of the shape
_empty_probs = {}    # the empty S_dmask tensor per (dtype, device)


def _decode_buffers(device: torch.device, stream: int, nbytes: int, cbytes: int):
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream)
    ws, counters = _decode_scratch.get(key, (None, None))
    if ws is None or ws.numel() < nbytes or counters.numel() * 4 < cbytes:
        ws = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        counters = torch.zeros(max(1024, (cbytes + 3) // 4), dtype=torch.int32, device=device)
        _decode_scratch[key] = (ws, counters)
    return ws, counters


def _flash_sparse_attn_forward_body(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, mask: Optional[torch.Tensor], bias: Optional[torch.Tensor],
    softmax_scale: float, is_causal: bool, softcap: float, return_softmax: bool,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    _check_inputs(q, k, v, mask, bias)
    kept = _handoff_get("kept") or _lists_for(kept_keys_of(mask), mask, k, exact=True)
    bits = _handoff_get("bits")
    if bits is None:
        bits = _lists_for(mask_bits_of(mask), mask, k, exact=False)
    q, k, v = [_aligned(x, 8) for x in (q, k, v)]
    mask = _aligned(mask, 16)
    bias = _aligned(bias, 8)
    batch, seqlen_q, num_heads, _ = q.shape
    out = torch.empty_like(q, memory_format=torch.contiguous_format)
    softmax_lse = torch.empty((batch, num_heads, seqlen_q), dtype=torch.float32, device=q.device)
    # The attention-probability dump is a debugging aid of the reference ("for testing only",
    # interface.py:661-663); it is not produced here.
    pkey = (q.dtype, q.device)
    p = _empty_probs.get(pkey)
    if p is None:
        p = _empty_probs[pkey] = torch.empty((0,), dtype=q.dtype, device=q.device)
    if seqlen_q == 0:
        return out, softmax_lse, p
    args = _cabi.FwdArgs()
    _cabi.fill_fwd(args, q, k, v, mask, bias, out, softmax_lse, softmax_scale, is_causal, softcap, kept, bits)
    with _cabi.device_guard(q.device):
        stream = _cabi.current_stream(q.device)
        workspace = None
        if seqlen_q == 1:
            # split-KV decode: workspace and arrival counters (with them the splits are merged by the same launch)
            skey = (batch, num_heads, k.shape[2], k.shape[1], q.shape[3])
            sizes = _decode_sizes.get(skey)
            if sizes is None:
                sizes = _decode_sizes[skey] = (_cabi.lib.fdma_fwd_workspace_bytes(args), _cabi.lib.fdma_fwd_counter_bytes(args))
            if sizes[0]:
                ws, counters = _decode_buffers(q.device, stream, sizes[0], sizes[1])
                args.workspace, args.workspace_bytes = ws.data_ptr(), ws.numel()
                if sizes[1]:
                    args.counters, args.counters_bytes = counters.data_ptr(), counters.numel() * 4
        else:
            nbytes = _cabi.lib.fdma_fwd_workspace_bytes(args)
            if nbytes:
                workspace = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
                args.workspace, args.workspace_bytes = workspace.data_ptr(), nbytes
        _cabi.check(_cabi.lib.fdma_fwd(args, stream))
    items = getattr(_tls, "items", None)
    per_query_head = mask is not None and mask.shape[1] == num_heads and num_heads != k.shape[2]
    if items is not None and workspace is not None and seqlen_q > 1 and not per_query_head:
        # (the compaction path's lists and copies; what identifies the problem they belong to goes with them.  A mask with
        # a row per query head over grouped kv heads is compacted in the forward only: nothing for the backward to reuse)
        items["fwd_ws_out"] = (workspace, (_cabi.get_compact_mode(), _cabi.stream_min_items()), None if bias is None else tuple(bias.shape))
    return out, softmax_lse, p


_flash_sparse_attn_forward = torch.library.custom_op("flash_sparse_attn::_flash_sparse_attn_forward", mutates_args=(), device_types="cuda")(_flash_sparse_attn_forward_body)


@torch.library.register_fake("flash_sparse_attn::_flash_sparse_attn_forward")
def _flash_sparse_attn_forward_fake(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, mask: Optional[torch.Tensor], bias: Optional[torch.Tensor],
    softmax_scale: float, is_causal: bool, softcap: float, return_softmax: bool,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    batch_size, seqlen_q, num_heads, _ = q.shape
    out = torch.empty_like(q, memory_format=torch.contiguous_format)
    softmax_lse = torch.empty((batch_size, num_heads, seqlen_q), dtype=torch.float32, device=q.device)
    p = torch.empty((0,), dtype=q.dtype, device=q.device)
    return out, softmax_lse, p


_wrapped_flash_sparse_attn_forward = _direct_when_eager(_flash_sparse_attn_forward, _flash_sparse_attn_forward_body)


def _per_query_head_groups(q, k, mask, bias) -> int:
    """Query heads per kv head when the backward of this call is to be taken apart by group member (see
    _backward_per_query_head), else 1: a query-broadcast mask with a row per QUERY head over grouped kv heads, next to
    no bias or a query-broadcast one, on a problem for which the library would compact a mask with a row per kv head
    (fdma_compact.hip: use_compact -- the same rule, on what one group member sees)."""
    if mask is None or mask.shape[2] != 1 or (bias is not None and bias.shape[2] != 1):
        return 1
    num_heads, num_heads_k = q.shape[2], k.shape[2]
    if mask.shape[1] != num_heads or num_heads == num_heads_k:
        return 1
    mode = _cabi.get_compact_mode()
    seqlen_q, seqlen_k = q.shape[1], k.shape[1]
    if mode == _cabi.COMPACT_NEVER or seqlen_q < 2 or seqlen_k < 1 or q.shape[0] * num_heads_k > 65535:
        return 1
    if mode != _cabi.COMPACT_ALWAYS and not (seqlen_q >= 128 and seqlen_k >= 128 and seqlen_q * seqlen_k >= 1 << 21):
        return 1
    return num_heads // num_heads_k


def _backward_per_query_head(dout, q, k, v, mask, bias, out, softmax_lse, dq, dk, dv, dbias, softmax_scale, is_causal,
                             softcap, deterministic):
    """Backward for a query-broadcast mask with a row per QUERY head over grouped kv heads.  The heads of a kv group keep
    different keys, so the library's compacted backward -- one list of kept keys per kv head, dK / dV summed over the
    group in registers -- does not apply to the call as a whole, and its tile-skipping kernels find hardly a tile to
    skip.  Group member g of every kv head (query heads g, g + G, ...: strided views, no copies) together with its mask
    rows IS a problem of the compacted form, without grouping: the call is taken apart into G of them.  dQ (and dBias
    with a row per query head) of the members are disjoint; dK, dV (and a dBias shared by the group) are summed."""
    G = q.shape[2] // k.shape[2]
    batch, seqlen_q, num_heads, _ = q.shape
    softmax_d = torch.empty((batch, num_heads, round_multiple(seqlen_q, 128)), device=q.device, dtype=torch.float32)
    bias_per_head = bias is not None and bias.shape[1] == num_heads
    # The members' dK, dV (and shared dBias) are summed in fp32 and rounded once, as the reference sums its per-head
    # dK / dV over a group (flash_api.cpp:1027-1047); summed in the 16-bit type they would be rounded G times.
    dk_t, dv_t = torch.empty_like(dk), torch.empty_like(dv)
    dk_sum = torch.zeros(dk.shape, device=dk.device, dtype=torch.float32)
    dv_sum = torch.zeros(dv.shape, device=dv.device, dtype=torch.float32)
    dbias_t = dbias_sum = None
    if bias is not None and not bias_per_head:
        dbias_t = torch.empty_like(dbias)
        dbias_sum = torch.zeros(dbias.shape, device=dbias.device, dtype=torch.float32)
    with _handoff():  # (lists, bit rows and forward workspaces belong to the whole call, not to a member)
        for g in range(G):
            member = slice(g, None, G)
            bias_g = bias[:, member] if bias_per_head else bias
            dbias_g = None if bias is None else (dbias[:, member] if bias_per_head else dbias_t)
            d = _flash_sparse_attn_backward_body(
                dout[:, :, member], q[:, :, member], k, v, mask[:, member], bias_g, out[:, :, member],
                softmax_lse[:, member], dq[:, :, member], dk_t, dv_t, dbias_g,
                softmax_scale, is_causal, softcap, deterministic)
            softmax_d[:, member] = d
            dk_sum.add_(dk_t)
            dv_sum.add_(dv_t)
            if dbias_sum is not None:
                dbias_sum.add_(dbias_t)
    dk.copy_(dk_sum)
    dv.copy_(dv_sum)
    if dbias_sum is not None:
        dbias.copy_(dbias_sum)
    return softmax_d


def _flash_sparse_attn_backward_body(
    dout: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, mask: Optional[torch.Tensor], bias:
    Optional[torch.Tensor], out: torch.Tensor, softmax_lse: torch.Tensor, dq: Optional[torch.Tensor], dk:
    Optional[torch.Tensor], dv: Optional[torch.Tensor], dbias: Optional[torch.Tensor], softmax_scale: float,
    is_causal: bool, softcap: float, deterministic: bool,
) -> torch.Tensor:
    _check_inputs(q, k, v, mask, bias)
    if out.dtype != q.dtype:
        raise RuntimeError("query and out must have the same dtype")
    if dout.dtype != q.dtype:
        raise RuntimeError("query and dout must have the same dtype")
    if tuple(out.shape) != tuple(q.shape) or tuple(dout.shape) != tuple(q.shape):
        raise RuntimeError("out and dout must have the shape of q")
    if _per_query_head_groups(q, k, mask, bias) > 1 and all(t is not None for t in (dq, dk, dv)):
        return _backward_per_query_head(dout, q, k, v, mask, bias, out, softmax_lse, dq, dk, dv, dbias, softmax_scale,
                                        is_causal, softcap, deterministic)
    dout, q, k, v, out = [_aligned(x, 8) for x in (dout, q, k, v, out)]
    mask = _aligned(mask, 16)
    bias = _aligned(bias, 8)
    softmax_lse = softmax_lse.contiguous()
    batch, seqlen_q, num_heads, _ = q.shape
    softmax_d = torch.empty((batch, num_heads, round_multiple(seqlen_q, 128)), device=q.device, dtype=torch.float32)

    # Outputs handed in by the caller are written in place when their layout allows the kernels'
    # vector stores; otherwise a staging tensor is filled and copied back.
    def staging(t, like, name):
        if t is None:
            raise RuntimeError(f"{name} must be provided")
        if t.dtype != q.dtype:
            raise RuntimeError(f"{name} must have the same dtype as q")
        if tuple(t.shape) != tuple(like.shape):
            raise RuntimeError(f"{name} must have the shape of its input")
        ok = t.stride(-1) == 1 and t.data_ptr() % 16 == 0 and all(
            t.size(i) == 1 or t.stride(i) % 8 == 0 for i in range(t.dim() - 1))
        return t if ok else torch.empty_like(t, memory_format=torch.contiguous_format)

    dq_w, dk_w, dv_w = staging(dq, q, "dq"), staging(dk, k, "dk"), staging(dv, v, "dv")
    dbias_w = staging(dbias, bias, "dbias") if bias is not None else None

    # A bias that is broadcast over the batch (batch > 1) or has one head for several kv heads makes several
    # workgroups add into the same dbias element; the kernels do that with fp32 atomics, whose order is not fixed.
    # With deterministic=True every (batch entry, kv head) gets its own slice instead and the slices are summed in
    # a fixed order afterwards, which is what the reference always does (flash_api.cpp:970-983, 1027-1047).
    dbias_sum_dims = ()
    if deterministic and bias is not None:
        dbias_sum_dims = tuple(d for d, full in ((0, batch), (1, k.size(2))) if bias.size(d) == 1 and full > 1)
    if dbias_sum_dims:
        bias = bias.expand(batch if 0 in dbias_sum_dims else bias.size(0), k.size(2) if 1 in dbias_sum_dims else bias.size(1),
                           -1, -1).contiguous()
        dbias_final, dbias_w = dbias_w, torch.empty_like(bias)

    args = _cabi.BwdArgs()
    _cabi.fill_fwd(args.f, q, k, v, mask, bias, out, softmax_lse, softmax_scale, is_causal, softcap, _handoff_get("kept"),
                   _handoff_get("bits"))
    fwd_ws = _handoff_get("fwd_ws")
    if (fwd_ws is not None and fwd_ws[1] == (_cabi.get_compact_mode(), _cabi.stream_min_items())
            and fwd_ws[2] == (None if bias is None else tuple(bias.shape))):
        args.fwd_workspace, args.fwd_workspace_bytes = fwd_ws[0].data_ptr(), fwd_ws[0].numel()
    args.dout = dout.data_ptr()
    args.dq, args.dk, args.dv = dq_w.data_ptr(), dk_w.data_ptr(), dv_w.data_ptr()
    args.dbias = dbias_w.data_ptr() if dbias_w is not None else None
    args.do_strides[:] = _cabi._s3(dout)
    args.dq_strides[:] = _cabi._s3(dq_w)
    args.dk_strides[:] = _cabi._s3(dk_w)
    args.dv_strides[:] = _cabi._s3(dv_w)
    args.dbias_strides[:] = _cabi._bcast3(dbias_w) if dbias_w is not None else (0, 0, 0)
    args.softmax_d = softmax_d.data_ptr()
    args.deterministic = int(bool(deterministic))
    with _cabi.device_guard(q.device):
        nbytes = _cabi.lib.fdma_bwd_workspace_bytes(args)
        workspace = None
        if nbytes:
            workspace = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
            args.workspace, args.workspace_bytes = workspace.data_ptr(), nbytes
        else:
            args.workspace, args.workspace_bytes = None, 0
        if seqlen_q > 0:
            _cabi.check(_cabi.lib.fdma_bwd(args, _cabi.current_stream(q.device)))
        else:  # empty query: gradients are zero (flash_api.cpp:1019-1025)
            for t in (dk_w, dv_w, dbias_w, softmax_d):
                if t is not None:
                    t.zero_()
    if dbias_sum_dims:
        dbias_final.copy_(dbias_w.sum(dim=dbias_sum_dims, keepdim=True, dtype=torch.float32))
        dbias_w = dbias_final
    for given, work in ((dq, dq_w), (dk, dk_w), (dv, dv_w), (dbias, dbias_w)):
        if given is not None and work is not given:
            given.copy_(work)
    return softmax_d


_flash_sparse_attn_backward = torch.library.custom_op(
    "flash_sparse_attn::_flash_sparse_attn_backward", mutates_args=("dq", "dk", "dv", "dbias"), device_types="cuda"
)(_flash_sparse_attn_backward_body)


@torch.library.register_fake("flash_sparse_attn::_flash_sparse_attn_backward")
def _flash_sparse_attn_backward_fake(
    dout: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, mask: Optional[torch.Tensor], bias:
    Optional[torch.Tensor], out: torch.Tensor, softmax_lse: torch.Tensor, dq: Optional[torch.Tensor], dk:
    Optional[torch.Tensor], dv: Optional[torch.Tensor], dbias: Optional[torch.Tensor], softmax_scale: float,
    is_causal: bool, softcap: float, deterministic: bool,
) -> torch.Tensor:
    batch_size, seqlen_q, num_heads, _ = q.shape
    return torch.empty((batch_size, num_heads, round_multiple(seqlen_q, 128)), device=q.device, dtype=torch.float32)


_wrapped_flash_sparse_attn_backward = _direct_when_eager(_flash_sparse_attn_backward, _flash_sparse_attn_backward_body)


def _pad_key_dim(t: Optional[torch.Tensor], seqlen_k: int, elems: int) -> Optional[torch.Tensor]:
    """Key-dimension rule of FlashDMAttnFunc.forward (interface.py:420-430): a size-1 key dim is
    expanded, any other length is padded.  The reference pads to a multiple of 128 always; the
    kernels here only need rows of a whole number of 16-byte vectors."""
    if t is None:
        return None
    if t.shape[-1] == 1 and seqlen_k != 1:
        return t.expand(*t.shape[:-1], round_multiple(seqlen_k, 128))
    if t.shape[-1] % elems != 0:
        return torch.nn.functional.pad(t, [0, round_multiple(max(seqlen_k, t.shape[-1]), 128) - t.shape[-1]])
    return t


def _nothing_to_differentiate(grad_enabled: bool, *tensors: Optional[torch.Tensor]) -> bool:
    """True for an eager call on plain tensors none of which asks for a gradient: the autograd node would record
    nothing, and going through it costs about 10 us per call -- as much as a decode-sized kernel takes."""
    if not _plain_eager(*tensors):
        return False
    for t in tensors:
        if t is not None and grad_enabled and t.requires_grad:
            return False
    return True


class _NoGradContext:
    """Stands in for the autograd context when FlashDMAttnFunc.forward is called directly (nothing to differentiate)."""

    def save_for_backward(self, *tensors):
        pass


class FlashDMAttnFunc(torch.autograd.Function):

    @staticmethod
    def forward(
        ctx: torch.autograd.function.FunctionCtx, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, mask:
        Optional[torch.Tensor], bias: Optional[torch.Tensor], softmax_scale: Optional[float], is_causal:
        Optional[bool], softcap: Optional[float], deterministic: Optional[bool], return_softmax: Optional[bool],
        is_grad_enabled: bool = True,
    ):
        is_grad = is_grad_enabled and any(x.requires_grad for x in [q, k, v])
        if softmax_scale is None:
            softmax_scale = q.shape[-1] ** (-0.5)
        if is_causal is None:
            is_causal = False
        if softcap is None:
            softcap = 0.0
        if deterministic is None:
            deterministic = False
        if return_softmax is None:
            return_softmax = False
        seqlen_k_bias_og = bias.shape[-1] if bias is not None else 0

        # Padding to multiple of 8 for 16-bit memory allocations
        head_size_og = q.size(3)
        if head_size_og % 8 != 0:
            q = torch.nn.functional.pad(q, [0, 8 - head_size_og % 8])
            k = torch.nn.functional.pad(k, [0, 8 - head_size_og % 8])
            v = torch.nn.functional.pad(v, [0, 8 - head_size_og % 8])
        # (the hand-overs are eager-mode business: a traced graph calls the operators as they are)
        eager = not torch.compiler.is_compiling()
        # (taken before the mask may be replaced by a padded copy; only for a mask over exactly the keys of this call)
        kept = _lists_for(kept_keys_of(mask), mask, k, exact=True) if eager else None
        bits = _lists_for(mask_bits_of(mask), mask, k, exact=False) if eager else None
        mask = _pad_key_dim(mask, k.shape[1], 16)
        bias = _pad_key_dim(bias, k.shape[1], 8)

        if eager and (is_grad or kept is not None or bits is not None):
            with _handoff(kept=kept, bits=bits) as side:
                out_padded, softmax_lse, S_dmask = _wrapped_flash_sparse_attn_forward(
                    q, k, v, mask, bias, softmax_scale, is_causal=is_causal, softcap=softcap, return_softmax=return_softmax,
                )
        else:  # (a traced graph, or nothing to hand over and no backward to keep the workspace for)
            side = {}
            out_padded, softmax_lse, S_dmask = _wrapped_flash_sparse_attn_forward(
                q, k, v, mask, bias, softmax_scale, is_causal=is_causal, softcap=softcap, return_softmax=return_softmax,
            )

        if is_grad:
            ctx.save_for_backward(q, k, v, mask, bias, out_padded, softmax_lse)
            if eager:
                ctx.kept = kept
                ctx.bits = bits
                ctx.fwd_ws = side.get("fwd_ws_out")
            ctx.softmax_scale = softmax_scale
            ctx.is_causal = is_causal
            ctx.softcap = softcap
            ctx.deterministic = deterministic
            ctx.seqlen_k_bias_og = seqlen_k_bias_og

        # (the slice is a tensor-library call of its own: skipped when nothing was padded and no graph is traced)
        out = out_padded if (eager and out_padded.shape[-1] == head_size_og) else out_padded[..., :head_size_og]

        return out if not return_softmax else (out, softmax_lse, S_dmask)

    @staticmethod
    def backward(
        ctx: torch.autograd.function.FunctionCtx,
        dout: torch.Tensor,
        *args: Any,
    ):
        q, k, v, mask, bias, out, softmax_lse = ctx.saved_tensors
        # every element of the gradients is written by the kernels: no zero fill
        dq = torch.empty_like(q, memory_format=torch.contiguous_format)
        dk = torch.empty_like(k, memory_format=torch.contiguous_format)
        dv = torch.empty_like(v, memory_format=torch.contiguous_format)
        dbias = torch.empty(bias.shape, dtype=bias.dtype, device=bias.device) if bias is not None else None

        head_size_og = dout.size(3)
        dout_padded = dout
        if head_size_og % 8 != 0:
            dout_padded = torch.nn.functional.pad(dout, [0, 8 - head_size_og % 8])

        if torch.compiler.is_compiling():
            _wrapped_flash_sparse_attn_backward(
                dout_padded, q, k, v, mask, bias, out, softmax_lse, dq, dk, dv, dbias, ctx.softmax_scale, ctx.is_causal,
                ctx.softcap, ctx.deterministic,
            )
        else:
            with _handoff(kept=getattr(ctx, "kept", None), bits=getattr(ctx, "bits", None), fwd_ws=getattr(ctx, "fwd_ws", None)):
                _wrapped_flash_sparse_attn_backward(
                    dout_padded, q, k, v, mask, bias, out, softmax_lse, dq, dk, dv, dbias, ctx.softmax_scale, ctx.is_causal,
                    ctx.softcap, ctx.deterministic,
                )

        # We could have padded the head dimension
        dq = dq[..., : dout.shape[-1]]
        dk = dk[..., : dout.shape[-1]]
        dv = dv[..., : dout.shape[-1]]

        if dbias is not None:
            dbias = (
                dbias[..., : k.shape[1]].sum(dim=-1, keepdim=True)
                if ctx.seqlen_k_bias_og == 1
                else dbias[..., : k.shape[1]]
            )

        return dq, dk, dv, None, dbias, None, None, None, None, None, None


def _column_causal_form(mask, bias, query, key, is_causal):
    """A keep-mask that arrives with one row per query but is really a column mask under the causal rule -- every row
    equals the last row cut off at the row's causal limit -- can run through the column-mask kernels (tile skipping,
    column compaction) instead of the kernels that stream a mask tile per score tile.  Finding that out takes a pass
    over the whole mask and a host synchronisation, so it is done only under the compaction policy "always"
    (`_cabi.set_compact_mode(COMPACT_ALWAYS)` / `FDMA_COMPACT=2`).  Returns (mask, is_causal) to call the operator with:
    the last row and True when the mask has that form, the arguments unchanged otherwise."""
    if (mask is None or _cabi.get_compact_mode() != _cabi.COMPACT_ALWAYS or torch.compiler.is_compiling()
            or type(mask) is not torch.Tensor or mask.dim() != 4 or mask.dtype != torch.bool):
        return mask, is_causal
    Lq, Lk = query.size(1), key.size(1)
    if (mask.size(2) != Lq or Lq < 2 or mask.size(3) < Lk or mask.size(1) not in (1, key.size(2))
            or (bias is not None and bias.size(2) != 1)):
        return mask, is_causal
    m = mask[..., :Lk]
    rows = torch.arange(Lq, device=mask.device)[:, None]
    cols = torch.arange(Lk, device=mask.device)[None, :]
    causal = cols <= rows + (Lk - Lq)  # bottom-right aligned
    col = m[:, :, -1:, :]              # the last row may see every key
    if not torch.equal(m & causal if is_causal else m, col & causal):
        return mask, is_causal
    return col.contiguous(), True


def flash_sparse_attn_func(
    query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, attn_mask: Optional[torch.Tensor] = None, attn_bias:
    Optional[torch.Tensor] = None, softmax_scale: Optional[float] = None, is_causal: Optional[bool] = None, softcap:
    Optional[float] = None, deterministic: Optional[bool] = None, return_attn_probs: Optional[bool] = None,
):
    """Dynamic-mask attention with MQA/GQA: K, V may have fewer heads than Q (the number of Q heads
    must be divisible by the number of KV heads; Q head h attends to KV head h // (H // Hkv)).

    attn_mask and attn_bias may have a head dimension of 1, nheads_k or nheads, a batch dimension
    of 1 or batch_size, and a query dimension of 1 or seqlen_q; size-1 dimensions broadcast.

    If is_causal=True, the causal mask is aligned to the bottom right corner of the attention
    matrix.  For seqlen_q = 2 and seqlen_k = 5 the causal mask (1 = keep, 0 = masked out) is:
        1 1 1 1 0
        1 1 1 1 1
    and for seqlen_q = 5 and seqlen_k = 2:
        0 0
        0 0
        0 0
        1 0
        1 1
    If a row of the mask is all zero, the output row is zero.

    Arguments:
        query: (batch_size, seqlen, nheads, headdim)
        key: (batch_size, seqlen_k, nheads_k, headdim)
        value: (batch_size, seqlen_k, nheads_k, headdim)
        attn_mask: optional bool tensor ({batch_size|1}, {nheads|nheads_k|1}, {seqlen_q|1}, {seqlen_k|1});
            True keeps a score, False masks it out.
        attn_bias: optional tensor of query's dtype, same shape rules, added to the scaled scores.
        softmax_scale: scaling of QK^T before the bias is added. Default 1 / sqrt(headdim).
        is_causal: apply the (bottom-right aligned) causal mask.
        softcap: must be None or 0 (soft-capping is not built).
        deterministic: dQ, dK and dV never go through atomics and are bit-reproducible regardless.  dBias of a
            bias that is broadcast over the batch (batch > 1) or shared by several kv heads is accumulated with
            fp32 atomics unless this flag is set; with it, one slice per (batch entry, kv head) is written and
            the slices are summed in a fixed order.
        return_attn_probs: also return (softmax_lse, S_dmask); S_dmask is an empty tensor.
    Return:
        out: (batch_size, seqlen, nheads, headdim).
        softmax_lse [optional]: (batch_size, nheads, seqlen), fp32 logsumexp of each score row
            (+inf for rows with no visible key).
    """
    grad_enabled = torch.is_grad_enabled()
    attn_mask, is_causal = _column_causal_form(attn_mask, attn_bias, query, key, is_causal)
    args = (query, key, value, attn_mask, attn_bias, softmax_scale, is_causal, softcap, deterministic, return_attn_probs,
            grad_enabled)
    if _nothing_to_differentiate(grad_enabled, query, key, value, attn_bias):
        return FlashDMAttnFunc.forward(_NoGradContext(), *args)
    return FlashDMAttnFunc.apply(*args)


def _check_varlen_inputs(q, k, v, cu_seqlens_q, cu_seqlens_k) -> None:
    """Checks of mha_varlen_fwd (flash_api.cpp:583-660) that concern torch tensors."""
    if q.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError("FlashSparseAttention only support fp16 and bf16 data type")
    if k.dtype != q.dtype:
        raise RuntimeError("query and key must have the same dtype")
    if v.dtype != q.dtype:
        raise RuntimeError("query and value must have the same dtype")
    for name, t in (("cu_seqlens_q", cu_seqlens_q), ("cu_seqlens_k", cu_seqlens_k)):
        if t.dtype != torch.int32:
            raise RuntimeError(f"{name} must have dtype int32")
        if t.device != q.device:
            raise RuntimeError(f"{name} must be on the device of q")
        if not t.is_contiguous():
            raise RuntimeError(f"{name} must be contiguous")
    if q.dim() != 3 or k.dim() != 3 or v.dim() != 3:
        raise RuntimeError("q, k, v must have shape (total, nheads, headdim)")
    if tuple(k.shape) != tuple(v.shape) or k.shape[2] != q.shape[2]:
        raise RuntimeError("k and v must have shape (total_k, num_heads_k, head_size)")
    batch = cu_seqlens_q.numel() - 1
    if batch <= 0:
        raise RuntimeError("batch size must be positive")
    if cu_seqlens_k.numel() != batch + 1:
        raise RuntimeError("cu_seqlens_k must have shape (batch_size + 1)")


def _flash_sparse_attn_varlen_forward_body(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu_seqlens_q: torch.Tensor, cu_seqlens_k: torch.Tensor,
    max_seqlen_q: int, max_seqlen_k: int, softmax_scale: float, is_causal: bool, softcap: float = 0.0, return_softmax:
    bool = False, block_table: Optional[torch.Tensor] = None, leftpad_k: Optional[torch.Tensor] = None, seqused_k:
    Optional[torch.Tensor] = None, zero_tensors: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Ragged-batch forward (interface.py:129-167 of the reference).  Rows of `out` / `softmax_lse` that belong to
    no sequence (beyond cu_seqlens_q[-1]) are zero-filled when `zero_tensors` is set and left unwritten otherwise."""
    if block_table is not None or leftpad_k is not None or seqused_k is not None:
        raise RuntimeError("paged KV (block_table), leftpad_k and seqused_k are not supported by this build")
    _check_varlen_inputs(q, k, v, cu_seqlens_q, cu_seqlens_k)
    q, k, v = [_aligned(x, 8) for x in (q, k, v)]
    total_q, num_heads, _ = q.shape
    out = torch.zeros_like(q, memory_format=torch.contiguous_format) if zero_tensors else torch.empty_like(q, memory_format=torch.contiguous_format)
    softmax_lse = torch.empty((num_heads, total_q), dtype=torch.float32, device=q.device)
    if zero_tensors:
        softmax_lse.fill_(float("-inf"))  # flash_api.cpp:699-702
    p = torch.empty((0,), dtype=q.dtype, device=q.device)
    if total_q == 0:
        return out, softmax_lse, p
    args = _cabi.VarlenFwdArgs()
    _cabi.fill_varlen_fwd(args, q, k, v, out, softmax_lse, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
                          softmax_scale, is_causal, softcap)
    with _cabi.device_guard(q.device):
        _cabi.check(_cabi.lib.fdma_varlen_fwd(args, _cabi.current_stream(q.device)))
    return out, softmax_lse, p


_flash_sparse_attn_varlen_forward = torch.library.custom_op("flash_sparse_attn::_flash_sparse_attn_varlen_forward", mutates_args=(), device_types="cuda")(_flash_sparse_attn_varlen_forward_body)


@torch.library.register_fake("flash_sparse_attn::_flash_sparse_attn_varlen_forward")
def _flash_sparse_attn_varlen_forward_fake(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu_seqlens_q: torch.Tensor, cu_seqlens_k: torch.Tensor,
    max_seqlen_q: int, max_seqlen_k: int, softmax_scale: float, is_causal: bool, softcap: float = 0.0, return_softmax:
    bool = False, block_table: Optional[torch.Tensor] = None, leftpad_k: Optional[torch.Tensor] = None, seqused_k:
    Optional[torch.Tensor] = None, zero_tensors: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    total_q, num_heads, _ = q.shape
    out = torch.empty_like(q, memory_format=torch.contiguous_format)
    softmax_lse = torch.empty((num_heads, total_q), dtype=torch.float32, device=q.device)
    p = torch.empty((0,), dtype=q.dtype, device=q.device)
    return out, softmax_lse, p


_wrapped_flash_sparse_attn_varlen_forward = _direct_when_eager(_flash_sparse_attn_varlen_forward, _flash_sparse_attn_varlen_forward_body)


def _flash_sparse_attn_varlen_backward_body(
    dout: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, out: torch.Tensor, softmax_lse:
    torch.Tensor, dq: Optional[torch.Tensor], dk: Optional[torch.Tensor], dv: Optional[torch.Tensor], cu_seqlens_q:
    torch.Tensor, cu_seqlens_k: torch.Tensor, max_seqlen_q: int, max_seqlen_k: int, softmax_scale: float, is_causal:
    bool, softcap: float, deterministic: bool, zero_tensors: bool = False,
) -> torch.Tensor:
    """Ragged-batch backward (interface.py:291-339 of the reference).  Gradient rows that belong to no sequence are
    zero-filled when `zero_tensors` is set and left unwritten otherwise (flash_api.cpp:1209-1214)."""
    _check_varlen_inputs(q, k, v, cu_seqlens_q, cu_seqlens_k)
    if out.dtype != q.dtype:
        raise RuntimeError("query and out must have the same dtype")
    if dout.dtype != q.dtype:
        raise RuntimeError("query and dout must have the same dtype")
    if tuple(out.shape) != tuple(q.shape) or tuple(dout.shape) != tuple(q.shape):
        raise RuntimeError("out and dout must have the shape of q")
    dout, q, k, v, out = [_aligned(x, 8) for x in (dout, q, k, v, out)]
    softmax_lse = softmax_lse.contiguous()
    total_q, num_heads, _ = q.shape
    softmax_d = torch.empty((num_heads, total_q), device=q.device, dtype=torch.float32)

    def staging(t, like, name):
        if t is None:
            raise RuntimeError(f"{name} must be provided")
        if t.dtype != q.dtype:
            raise RuntimeError(f"{name} must have the same dtype as q")
        if tuple(t.shape) != tuple(like.shape):
            raise RuntimeError(f"{name} must have the shape of its input")
        ok = t.stride(-1) == 1 and t.data_ptr() % 16 == 0 and all(
            t.size(i) == 1 or t.stride(i) % 8 == 0 for i in range(t.dim() - 1))
        return t if ok else torch.empty_like(t, memory_format=torch.contiguous_format)

    dq_w, dk_w, dv_w = staging(dq, q, "dq"), staging(dk, k, "dk"), staging(dv, v, "dv")
    if zero_tensors:
        for t in (dq_w, dk_w, dv_w, softmax_d):
            t.zero_()
    args = _cabi.VarlenBwdArgs()
    _cabi.fill_varlen_fwd(args.f, q, k, v, out, softmax_lse, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
                          softmax_scale, is_causal, softcap)
    args.dout = dout.data_ptr()
    args.dq, args.dk, args.dv = dq_w.data_ptr(), dk_w.data_ptr(), dv_w.data_ptr()
    args.do_strides[:] = (dout.stride(0), dout.stride(1))
    args.dq_strides[:] = (dq_w.stride(0), dq_w.stride(1))
    args.dk_strides[:] = (dk_w.stride(0), dk_w.stride(1))
    args.dv_strides[:] = (dv_w.stride(0), dv_w.stride(1))
    args.softmax_d = softmax_d.data_ptr()
    args.deterministic = int(bool(deterministic))
    with _cabi.device_guard(q.device):
        _cabi.check(_cabi.lib.fdma_varlen_bwd(args, _cabi.current_stream(q.device)))
    for given, work in ((dq, dq_w), (dk, dk_w), (dv, dv_w)):
        if given is not None and work is not given:
            given.copy_(work)
    return softmax_d


_flash_sparse_attn_varlen_backward = torch.library.custom_op(
    "flash_sparse_attn::_flash_sparse_attn_varlen_backward", mutates_args=("dq", "dk", "dv"), device_types="cuda"
)(_flash_sparse_attn_varlen_backward_body)


@torch.library.register_fake("flash_sparse_attn::_flash_sparse_attn_varlen_backward")
def _flash_sparse_attn_varlen_backward_fake(
    dout: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, out: torch.Tensor, softmax_lse:
    torch.Tensor, dq: Optional[torch.Tensor], dk: Optional[torch.Tensor], dv: Optional[torch.Tensor], cu_seqlens_q:
    torch.Tensor, cu_seqlens_k: torch.Tensor, max_seqlen_q: int, max_seqlen_k: int, softmax_scale: float, is_causal:
    bool, softcap: float, deterministic: bool, zero_tensors: bool = False,
) -> torch.Tensor:
    total_q, num_heads, _ = q.shape
    return torch.empty((num_heads, total_q), device=q.device, dtype=torch.float32)


_wrapped_flash_sparse_attn_varlen_backward = _direct_when_eager(_flash_sparse_attn_varlen_backward, _flash_sparse_attn_varlen_backward_body)


class FlashAttnVarlenFunc(torch.autograd.Function):
    """Autograd node of the ragged-batch path (interface.py:500-608 of the reference): argument defaults, head
    dimension padded to a multiple of 8, saved tensors, slicing of the padded gradients."""

    @staticmethod
    def forward(
        ctx, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu_seqlens_q: torch.Tensor, cu_seqlens_k:
        torch.Tensor, max_seqlen_q: int, max_seqlen_k: int, softmax_scale: Optional[float], is_causal: Optional[bool],
        softcap: Optional[float], deterministic: Optional[bool], return_softmax: Optional[bool], block_table:
        Optional[torch.Tensor], is_grad_enabled: bool = True,
    ):
        is_grad = is_grad_enabled and any(x.requires_grad for x in [q, k, v])
        if softmax_scale is None:
            softmax_scale = q.shape[-1] ** (-0.5)
        is_causal = False if is_causal is None else is_causal
        softcap = 0.0 if softcap is None else softcap
        deterministic = False if deterministic is None else deterministic
        return_softmax = False if return_softmax is None else return_softmax

        head_size_og = q.size(2)
        if head_size_og % 8 != 0:
            pad = [0, 8 - head_size_og % 8]
            q, k, v = (torch.nn.functional.pad(t, pad) for t in (q, k, v))

        out_padded, softmax_lse, S_dmask = _wrapped_flash_sparse_attn_varlen_forward(
            q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, softmax_scale,
            is_causal=is_causal, softcap=softcap, return_softmax=return_softmax, block_table=block_table,
        )
        if is_grad:
            ctx.save_for_backward(q, k, v, out_padded, softmax_lse, cu_seqlens_q, cu_seqlens_k)
            ctx.max_seqlen_q = max_seqlen_q
            ctx.max_seqlen_k = max_seqlen_k
            ctx.softmax_scale = softmax_scale
            ctx.is_causal = is_causal
            ctx.softcap = softcap
            ctx.deterministic = deterministic
        out = out_padded[..., :head_size_og]
        return out if not return_softmax else (out, softmax_lse, S_dmask)

    @staticmethod
    def backward(ctx, dout, *args):
        q, k, v, out, softmax_lse, cu_seqlens_q, cu_seqlens_k = ctx.saved_tensors
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        head_size_og = dout.size(2)
        dout_padded = dout
        if head_size_og % 8 != 0:
            dout_padded = torch.nn.functional.pad(dout, [0, 8 - head_size_og % 8])
        _wrapped_flash_sparse_attn_varlen_backward(
            dout_padded, q, k, v, out, softmax_lse, dq, dk, dv, cu_seqlens_q, cu_seqlens_k,
            ctx.max_seqlen_q, ctx.max_seqlen_k, ctx.softmax_scale, ctx.is_causal, ctx.softcap, ctx.deterministic,
        )
        dq = dq[..., : dout.shape[-1]]
        dk = dk[..., : dout.shape[-1]]
        dv = dv[..., : dout.shape[-1]]
        return dq, dk, dv, None, None, None, None, None, None, None, None, None, None, None


def flash_sparse_attn_varlen_func(
    query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, cu_seqlens_q: torch.Tensor, cu_seqlens_k:
    torch.Tensor, max_seqlen_q: int, max_seqlen_k: int, softmax_scale: Optional[float] = None, is_causal:
    Optional[bool] = None, softcap: Optional[float] = None, deterministic: Optional[bool] = None, return_attn_probs:
    Optional[bool] = None, block_table: Optional[torch.Tensor] = None,
):
    """Ragged-batch ("varlen") attention without mask or bias, signature and semantics of the reference's
    `flash_sparse_attn_varlen_func` (interface.py:687-760).

    query: (total_q, nheads, headdim); key, value: (total_k, nheads_k, headdim); the sequences of the batch lie
    back to back and `cu_seqlens_q` / `cu_seqlens_k` (int32, batch + 1, on the device) hold their first rows.
    MQA / GQA through nheads_k < nheads (query head h uses kv head h // (nheads / nheads_k)).  With
    `is_causal` the mask is aligned to the bottom right corner of every sequence's attention matrix; a row
    without visible keys gives a zero output.  `max_seqlen_q` / `max_seqlen_k` are upper bounds of the
    sequence lengths.  The lengths are read on the device only: the call never synchronises.

    Returns out (total_q, nheads, headdim), or (out, softmax_lse (nheads, total_q), S_dmask (empty)) when
    `return_attn_probs` is set.  Paged KV (`block_table`) and softcapping raise RuntimeError.
    """
    grad_enabled = torch.is_grad_enabled()
    args = (query, key, value, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, softmax_scale, is_causal, softcap,
            deterministic, return_attn_probs, block_table, grad_enabled)
    if _nothing_to_differentiate(grad_enabled, query, key, value):
        return FlashAttnVarlenFunc.forward(None, *args)
    return FlashAttnVarlenFunc.apply(*args)
