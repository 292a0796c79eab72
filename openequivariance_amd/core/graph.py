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

    def save_npz(self, path) -> None:
        """Write ``coords``, ``row``, ``col`` (the keys of the reference's graph files,
        openequivariance/openequivariance/benchmark/ConvBenchmarkSuite.py:21-32) as an ``.npz`` archive."""
        np.savez(path, coords=self.coords, row=self.rows, col=self.cols)

    @classmethod
    def from_npz(cls, path, name: str = "") -> "CoordGraph":
        """Read a graph written by :meth:`save_npz` (plain arrays only: nothing is unpickled)."""
        with np.load(path, allow_pickle=False) as z:
            return cls(z["coords"], z["row"].astype(np.int64), z["col"].astype(np.int64), name)


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


def spatial_order(coords: np.ndarray, bits: int = 10) -> np.ndarray:
    """Permutation that lists the nodes along a Z-order (Morton) curve through
    their coordinates. Numbering the nodes of a graph this way keeps the
    neighbours of consecutive receivers close in memory, which is what lets the
    gathered sender rows of the fused convolution hit in L2."""
    c = np.asarray(coords, dtype=np.float64)
    lo, hi = c.min(axis=0), c.max(axis=0)
    q = np.minimum(((c - lo) / np.maximum(hi - lo, 1e-300) * (1 << bits)).astype(np.uint64), (1 << bits) - 1)
    code = np.zeros(len(c), dtype=np.uint64)
    for b in range(bits):
        for d in range(c.shape[1]):
            code |= ((q[:, d] >> np.uint64(b)) & np.uint64(1)) << np.uint64(b * c.shape[1] + d)
    return np.argsort(code, kind="stable")


def relabel_nodes(order: np.ndarray, rows: np.ndarray, cols: np.ndarray):
    """Node ``order[i]`` becomes node ``i``. Returns the relabelled (rows, cols);
    node feature arrays must be permuted with ``X[order]``."""
    inv = np.empty_like(order)
    inv[order] = np.arange(len(order), dtype=order.dtype)
    return inv[rows], inv[cols]
