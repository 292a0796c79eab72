"""Row layouts of irrep-packed feature arrays.

``mul_ir``: each irrep block of a row is stored ``[mul, 2l+1]`` (e3nn's layout);
``ir_mul``: ``[2l+1, mul]``. Converting between them is a fixed permutation of the
trailing axis (cf. openequivariance/openequivariance/core/utils.py:212-259).
"""

from __future__ import annotations

from functools import lru_cache

import numpy as np

from .spec import Irreps

LAYOUTS = ("mul_ir", "ir_mul")


def check_layouts(src_layout: str, dst_layout: str) -> None:
    if src_layout not in LAYOUTS:
        raise ValueError(f"Unsupported src_layout: {src_layout}")
    if dst_layout not in LAYOUTS:
        raise ValueError(f"Unsupported dst_layout: {dst_layout}")


@lru_cache(maxsize=256)
def _gather_index(irreps_str: str, to_ir_mul: bool) -> np.ndarray:
    """``dst[..., t] = src[..., index[t]]``."""
    irreps = Irreps(irreps_str)
    parts, off = [], 0
    for mul, ir in irreps:
        d = ir.dim
        block = off + np.arange(mul * d, dtype=np.int64)
        # source viewed as [mul, d] (mul_ir) or [d, mul] (ir_mul); the destination is its transpose
        shape = (mul, d) if to_ir_mul else (d, mul)
        parts.append(block.reshape(shape).T.reshape(-1))
        off += mul * d
    index = np.concatenate(parts) if parts else np.zeros(0, dtype=np.int64)
    index.setflags(write=False)
    return index


def layout_permutation(irreps, src_layout: str, dst_layout: str) -> np.ndarray:
    """Gather index that takes a row from ``src_layout`` to ``dst_layout``."""
    check_layouts(src_layout, dst_layout)
    irreps = Irreps(irreps)
    if src_layout == dst_layout:
        return np.arange(irreps.dim, dtype=np.int64)
    return _gather_index(str(irreps), dst_layout == "ir_mul")


def transpose_irrep_layout(array: np.ndarray, irreps, src_layout: str, dst_layout: str) -> np.ndarray:
    """numpy version: returns a new array with the trailing axis re-laid-out."""
    index = layout_permutation(irreps, src_layout, dst_layout)
    array = np.asarray(array)
    assert array.shape[-1] == len(index), f"trailing dimension {array.shape[-1]} != irreps.dim {len(index)}"
    return np.ascontiguousarray(array[..., index])
