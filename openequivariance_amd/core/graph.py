"""Graph containers and synthetic graphs for the fused convolution."""

from __future__ import annotations

import numpy as np


class CoordGraph:
    """Edge list sorted row-major by (receiver, sender) plus the permutation
    that lists the sorted edges in sender-major order. Same attributes as the
    reference container (openequivariance/openequivariance/core/ConvolutionBase.py:57-82)."""

    def __init__(self, coords, rows, cols, name: str = ""):
        rows, cols = np.asarray(rows), np.asarray(cols)
        assert len(rows) == len(cols)
        self.nnz = len(rows)
        self.node_count = coords.shape[0]
        self.coords = coords
        self.name = name
        order = np.lexsort((cols, rows))
        self.order = order
        self.rows = rows[order]
        self.cols = cols[order]
        self.transpose_perm = np.lexsort((self.rows, self.cols)).astype(self.rows.dtype)


def periodic_radius_graph(n_nodes: int, mean_degree: float = 32.0, cutoff: float = 5.0, seed: int = 0):
    """Uniform points in a periodic cube sized so that the expected number of
    neighbours within ``cutoff`` is ``mean_degree``; directed edges both ways.
    Returns (coords [N,3], rows, cols, edge_vectors [E,3]) with minimum-image
    vectors pointing from sender to receiver."""
    from scipy.spatial import cKDTree

    rng = np.random.default_rng(seed)
    side = (4.0 / 3.0 * np.pi * cutoff**3 * n_nodes / mean_degree) ** (1.0 / 3.0)
    assert side > 2 * cutoff, "box too small for the minimum-image convention"
    coords = rng.uniform(0.0, side, size=(n_nodes, 3))
    tree = cKDTree(coords, boxsize=side)
    pairs = tree.query_pairs(cutoff, output_type="ndarray")
    rows = np.concatenate([pairs[:, 0], pairs[:, 1]]).astype(np.int64)
    cols = np.concatenate([pairs[:, 1], pairs[:, 0]]).astype(np.int64)
    vec = coords[rows] - coords[cols]
    vec -= side * np.round(vec / side)
    return coords, rows, cols, vec
