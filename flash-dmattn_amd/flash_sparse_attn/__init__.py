"""flash_sparse_attn for MI355X: the package surface of SmallDoges/flash-dmattn
(flash_sparse_attn/__init__.py:5-97 of the reference) served by one native backend, the gfx950 HIP
library libfdma_hip.so.  The backend keeps the reference's name "cuda" so that
``flash_sparse_attn_func_auto(backend="cuda")`` and callers that test ``CUDA_AVAILABLE`` work
unchanged; the Triton and Flex backends of the reference do not exist here and report as unavailable.
"""
from typing import Optional

__version__ = "1.2.3"

try:
    from flash_sparse_attn.flash_sparse_attn_interface import flash_sparse_attn_func, flash_sparse_attn_varlen_func
    CUDA_AVAILABLE = True
except ImportError:
    CUDA_AVAILABLE = False
    flash_sparse_attn_func, flash_sparse_attn_varlen_func = None, None

TRITON_AVAILABLE = False
triton_sparse_attn_func = None

FLEX_AVAILABLE = False
flex_sparse_attn_func = None


def get_available_backends():
    """Return a list of available backends."""
    backends = []
    if CUDA_AVAILABLE:
        backends.append("cuda")
    if TRITON_AVAILABLE:
        backends.append("triton")
    if FLEX_AVAILABLE:
        backends.append("flex")
    return backends


def flash_sparse_attn_func_auto(backend: Optional[str] = None, **kwargs):
    """Return the attention function of the requested backend ('cuda', 'triton', 'flex'), or of the
    first available one when `backend` is None.  Note that, as in the reference, this returns the
    callable and does not call it."""
    if backend is None:
        if CUDA_AVAILABLE:
            backend = "cuda"
        elif TRITON_AVAILABLE:
            backend = "triton"
        elif FLEX_AVAILABLE:
            backend = "flex"
        else:
            raise RuntimeError("No flash attention backend is available. Please install at least one of: triton, transformers, or build the CUDA extension.")

    if backend == "cuda":
        if not CUDA_AVAILABLE:
            raise RuntimeError("CUDA backend is not available. Please build the CUDA extension.")
        return flash_sparse_attn_func

    elif backend == "triton":
        if not TRITON_AVAILABLE:
            raise RuntimeError("Triton backend is not available. Please install triton: pip install triton")
        return triton_sparse_attn_func

    elif backend == "flex":
        if not FLEX_AVAILABLE:
            raise RuntimeError("Flex backend is not available. Please install transformers: pip install transformers")
        return flex_sparse_attn_func

    else:
        raise ValueError(f"Unknown backend: {backend}. Available backends: {get_available_backends()}")


__all__ = [
    "CUDA_AVAILABLE",
    "TRITON_AVAILABLE",
    "FLEX_AVAILABLE",
    "flash_sparse_attn_func",
    "flash_sparse_attn_varlen_func",
    "triton_sparse_attn_func",
    "flex_sparse_attn_func",
    "get_available_backends",
    "flash_sparse_attn_func_auto",
]
