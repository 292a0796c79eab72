"""Small torch-side helpers (dtype mapping, device facts)."""

from __future__ import annotations

import numpy as np
import torch


def torch_to_oeq_dtype(torch_dtype):
    """torch dtype -> numpy scalar type (reference: core/utils.py:120-134)."""
    if torch_dtype == torch.float32:
        return np.float32
    if torch_dtype == torch.float64:
        return np.float64
    raise ValueError("Unsupported torch dtype!")


def oeq_to_torch_dtype(np_dtype):
    dt = np.dtype(np_dtype)
    if dt == np.float32:
        return torch.float32
    if dt == np.float64:
        return torch.float64
    raise ValueError(f"Unsupported dtype {np_dtype}")


_cu_cache = [None]


def compute_units() -> int:
    """CU count of the current GPU (256 on MI355X; also the default with no GPU,
    so kernels can be generated and compiled on a host without one)."""
    if _cu_cache[0] is None:
        n = 256
        if torch.cuda.is_available():
            from .. import runtime as rt
            n = int(rt.device_props(torch.cuda.current_device()).compute_units)
        _cu_cache[0] = n
    return _cu_cache[0]
