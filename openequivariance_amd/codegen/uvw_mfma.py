"""MFMA kernels for shared-weight 'uvw' products (dense channel mixing)."""

from __future__ import annotations

from .lower import Lowered


def supported(low: Lowered) -> bool:
    return False
