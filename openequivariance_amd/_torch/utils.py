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


def transpose_irreps(array: torch.Tensor, irreps, src_layout: str, dst_layout: str) -> torch.Tensor:
    r"""Re-lay-out the trailing (feature) dimension of an irrep-packed tensor between
    ``"mul_ir"`` (blocks stored ``[mul, 2l+1]``) and ``"ir_mul"`` (``[2l+1, mul]``); same
    contract as the reference function
    (openequivariance/openequivariance/_torch/utils.py:80-147): leading dimensions
    are kept, the result is a new tensor (a clone when both layouts agree) and the
    operation is differentiable (one ``index_select``).

    :raises TypeError: if ``array`` is not a tensor.
    :raises ValueError: for layouts other than ``"mul_ir"`` / ``"ir_mul"``.
    """
    from ..core.layout import check_layouts, layout_permutation

    check_layouts(src_layout, dst_layout)
    if not isinstance(array, torch.Tensor):
        raise TypeError(f"Expected torch.Tensor, got {type(array)}")
    if src_layout == dst_layout:
        return array.clone()
    index = torch.from_numpy(layout_permutation(irreps, src_layout, dst_layout).copy()).to(array.device)
    return array.index_select(-1, index)
