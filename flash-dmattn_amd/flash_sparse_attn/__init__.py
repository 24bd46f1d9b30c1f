"""flash_sparse_attn for MI355X: the package surface of SmallDoges/flash-dmattn
(flash_sparse_attn/__init__.py:5-97 of the reference) served by one native backend, the gfx950 HIP
library libfdma_hip.so.  The backend keeps the reference's name "cuda" so that
``flash_sparse_attn_func_auto(backend="cuda")`` and callers that test ``CUDA_AVAILABLE`` work
unchanged; the Triton and Flex backends of the reference do not exist here and report as unavailable.
"""
from typing import Callable, Dict, List, Optional, Tuple

__version__ = "1.2.3"

try:  # the native library is the only implementation: without it the backend is simply absent
    from flash_sparse_attn.flash_sparse_attn_interface import flash_sparse_attn_func, flash_sparse_attn_varlen_func
except ImportError:
    flash_sparse_attn_func = flash_sparse_attn_varlen_func = None

triton_sparse_attn_func = flex_sparse_attn_func = None
CUDA_AVAILABLE = flash_sparse_attn_func is not None
TRITON_AVAILABLE = FLEX_AVAILABLE = False

# backend name -> (callable or None, what the reference tells the user when that backend is missing);
# the order is the order of preference when no backend is asked for
_BACKENDS: Dict[str, Tuple[Optional[Callable], str]] = {
    "cuda": (flash_sparse_attn_func, "CUDA backend is not available. Please build the CUDA extension."),
    "triton": (triton_sparse_attn_func, "Triton backend is not available. Please install triton: pip install triton"),
    "flex": (flex_sparse_attn_func, "Flex backend is not available. Please install transformers: pip install transformers"),
}


def get_available_backends() -> List[str]:
    """Names of the backends that can be used, in order of preference."""
    return [name for name, (fn, _) in _BACKENDS.items() if fn is not None]


def flash_sparse_attn_func_auto(backend: Optional[str] = None, **kwargs):
    """The attention function of the requested backend ('cuda', 'triton', 'flex'), or of the first available one when
    `backend` is None.  As in the reference, the callable is returned, not called; keyword arguments are ignored."""
    if backend is None:
        available = get_available_backends()
        if not available:
            raise RuntimeError("No flash attention backend is available. Please install at least one of: triton, "
                               "transformers, or build the CUDA extension.")
        backend = available[0]
    if backend not in _BACKENDS:
        raise ValueError(f"Unknown backend: {backend}. Available backends: {get_available_backends()}")
    fn, missing = _BACKENDS[backend]
    if fn is None:
        raise RuntimeError(missing)
    return fn


__all__ = ["CUDA_AVAILABLE", "TRITON_AVAILABLE", "FLEX_AVAILABLE", "flash_sparse_attn_func", "flash_sparse_attn_varlen_func",
           "triton_sparse_attn_func", "flex_sparse_attn_func", "get_available_backends", "flash_sparse_attn_func_auto"]
