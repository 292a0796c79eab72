"""Real spherical harmonics (component normalisation) for making Y inputs."""

from __future__ import annotations

import math

import numpy as np

from .cg import wigner_3j


def spherical_harmonics(lmax: int, vectors: np.ndarray) -> np.ndarray:
    """``[n, (lmax+1)^2]`` harmonics of the directions of ``vectors`` with
    ``|Y^l|^2 = 2l+1``; ``Y^1 = sqrt(3) (x, y, z)`` and higher degrees by the
    CG recursion ``Y^{l+1} ~ C(l,1,l+1) (Y^l (x) Y^1)``."""
    v = np.asarray(vectors, dtype=np.float64)
    v = v / np.linalg.norm(v, axis=1, keepdims=True)
    ys = [np.ones((v.shape[0], 1)), math.sqrt(3.0) * v]
    for l in range(1, lmax):
        nxt = np.einsum("ijk,zi,zj->zk", wigner_3j(l, 1, l + 1), ys[l], ys[1])
        nxt *= math.sqrt(2 * l + 3) / np.linalg.norm(nxt, axis=1, keepdims=True)
        ys.append(nxt)
    return np.concatenate(ys[: lmax + 1], axis=1)
