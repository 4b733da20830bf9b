"""Loader of the C++ list-gathering helper (``csrc/tensor_rows.cpp``).

``native`` is the extension module, or None when it has not been built: then the same rows are made
by the Python loops in ``fused_adam_hip.py`` / ``optim/adam.py`` (several passes over every tensor per
step instead of one).  The helper only reads pointers and metadata; the kernels are in
``libfsadam.so`` either way.
"""
from __future__ import annotations

import torch  # the helper links against torch's libraries: they must be mapped first

try:
    from .csrc import _tensor_rows as native
except ImportError:  # not built
    native = None

__all__ = ["native", "dtype_code", "describe"]


def dtype_code(dtype: torch.dtype) -> int:
    """0 for float32, 1 for float16: the only element types the step knows."""
    return 1 if dtype == torch.float16 else 0


def describe(status: int) -> str:
    """Name of a negative status of ``fill_rows`` / ``gather`` (for messages and tests)."""
    if native is None:
        return str(status)
    for name in ("NOT_TENSOR", "NOT_CONTIGUOUS", "NOT_CUDA", "NUMEL", "DTYPE", "DEVICE", "LENGTH", "NO_GRAD", "SPARSE",
                 "NO_STATE", "STALE", "ERROR"):
        if getattr(native, name, None) == status:
            return name
    return str(status)
