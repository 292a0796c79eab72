"""Pins the CPU oracle (oracle/e3nn_ref.py) and the package's own CG generator:
golden vectors dumped from the reference's numpy modules, closed forms,
invariants, brute force on tiny problems, finite differences."""

import json
import math
import os

import numpy as np
import pytest

from openequivariance_amd.core import problems as P
from openequivariance_amd.core.cg import sparse_cg, wigner_3j
from openequivariance_amd.core.spec import TPProblem
from oracle import e3nn_ref as R


def _triples(lmax):
    return [(a, b, c) for a in range(lmax + 1) for b in range(lmax + 1)
            for c in range(abs(a - b), min(lmax, a + b) + 1)]


# ---------------------------------------------------------------- CG tensors

def test_cg_matches_golden(golden_dir):
    gold = np.load(os.path.join(golden_dir, "wigner_3j.npz"))
    assert len(gold.files) == 69
    for key in gold.files:
        l1, l2, l3 = (int(t) for t in key.split("_"))
        np.testing.assert_allclose(wigner_3j(l1, l2, l3), gold[key], atol=1e-14, rtol=0)
        if max(l1, l2, l3) <= 4:  # sympy route is slow for large l
            np.testing.assert_allclose(R.wigner_3j_ref(l1, l2, l3), gold[key], atol=1e-13, rtol=0)


@pytest.mark.parametrize("l", [(5, 3, 4), (6, 6, 6)])
def test_cg_oracle_high_l(golden_dir, l):
    gold = np.load(os.path.join(golden_dir, "wigner_3j.npz"))
    np.testing.assert_allclose(R.wigner_3j_ref(*l), gold["%d_%d_%d" % l], atol=1e-13, rtol=0)


def test_cg_closed_forms():
    eps = np.zeros((3, 3, 3))
    for i, j, k in [(0, 1, 2), (1, 2, 0), (2, 0, 1)]:
        eps[i, j, k], eps[i, k, j] = 1.0, -1.0
    for f in (wigner_3j, R.wigner_3j_ref):
        np.testing.assert_allclose(f(1, 1, 1), eps / math.sqrt(6), atol=1e-15)
        np.testing.assert_allclose(f(1, 1, 0)[:, :, 0], np.eye(3) / math.sqrt(3), atol=1e-15)
        for l in range(5):
            np.testing.assert_allclose(f(0, l, l)[0], np.eye(2 * l + 1) / math.sqrt(2 * l + 1), atol=1e-15)
            np.testing.assert_allclose(f(l, 0, l)[:, 0, :], np.eye(2 * l + 1) / math.sqrt(2 * l + 1), atol=1e-15)


def test_cg_norm_and_symmetry():
    for (a, b, c) in _triples(3):
        C = wigner_3j(a, b, c)
        assert abs((C * C).sum() - 1.0) < 1e-14
        sign = (-1) ** (a + b + c)
        np.testing.assert_allclose(wigner_3j(b, a, c), sign * C.transpose(1, 0, 2), atol=1e-14)
        np.testing.assert_allclose(wigner_3j(c, b, a), sign * C.transpose(2, 1, 0), atol=1e-14)


def test_cg_nonzero_counts():
    expect = {(1, 1, 1): 6, (1, 1, 2): 11, (1, 2, 2): 16, (1, 2, 3): 21, (1, 3, 3): 26, (2, 2, 2): 25,
              (2, 2, 3): 28, (2, 3, 3): 41, (3, 3, 3): 42, (2, 3, 2): 28}
    for l, n in expect.items():
        assert len(sparse_cg(*l)) == n
    for l in range(4):
        assert len(sparse_cg(0, l, l)) == len(sparse_cg(l, l, 0)) == 2 * l + 1


def _wigner_D_from_sh(l, Rm, rng):
    """D^l(R) fitted from Y^l(R r) = D^l Y^l(r) on random directions."""
    pts = rng.normal(size=(200, 3))
    Y = R.spherical_harmonics(l, pts)[:, l * l:(l + 1) ** 2]
    Yr = R.spherical_harmonics(l, pts @ Rm.T)[:, l * l:(l + 1) ** 2]
    D, *_ = np.linalg.lstsq(Y, Yr, rcond=None)
    return D.T


def test_cg_equivariance():
    rng = np.random.default_rng(1)
    q, _ = np.linalg.qr(rng.normal(size=(3, 3)))
    if np.linalg.det(q) < 0:
        q[:, 0] *= -1
    D = [_wigner_D_from_sh(l, q, rng) for l in range(4)]
    np.testing.assert_allclose(D[1], q, atol=1e-10)
    for l in range(4):
        np.testing.assert_allclose(D[l] @ D[l].T, np.eye(2 * l + 1), atol=1e-9)
    for (a, b, c) in _triples(3):
        C = wigner_3j(a, b, c)
        rotated = np.einsum("ijk,ia,jb,kc->abc", C, D[a], D[b], D[c])
        np.testing.assert_allclose(rotated, C, atol=1e-9)


def test_spherical_harmonics_norms():
    rng = np.random.default_rng(2)
    Y = R.spherical_harmonics(3, rng.normal(size=(50, 3)))
    np.testing.assert_allclose(Y[:, 0], 1.0)
    for l in range(4):
        np.testing.assert_allclose((Y[:, l * l:(l + 1) ** 2] ** 2).sum(1), 2 * l + 1, rtol=1e-12)
    from openequivariance_amd.core.sh import spherical_harmonics
    np.testing.assert_allclose(spherical_harmonics(3, rng.normal(size=(5, 3))).shape, (5, 16))


# ------------------------------------------------------- problem conventions

_MAKERS = {
    "cfg1": P.config1_single_uvu, "cfg2": P.config2_nequip_uvu, "cfg3": P.config3_mace_uvu,
    "cfg4": P.config4_uvw_shared, "mace_large": lambda: P.mace_problems()[0],
    "nequip_lips": lambda: P.nequip_problems()[0],
    "mixed_norm": lambda: TPProblem(
        "3x1o+2x2e", "2x1o+1x0e", "3x1o+2x2e+4x0e",
        [(0, 0, 2, "uvw", True, 0.5), (0, 1, 0, "uvw", True), (1, 0, 0, "uvw", True, 2.0), (1, 1, 1, "uvw", True)],
        irrep_normalization="norm", path_normalization="path", in1_var=[1.0, 2.0], in2_var=[0.5, 1.0],
        out_var=[1.0, 3.0, 2.0], shared_weights=False, internal_weights=False),
}


@pytest.mark.parametrize("name", sorted(_MAKERS))
def test_problem_conventions_match_golden(golden_dir, name):
    gold = json.load(open(os.path.join(golden_dir, "problems.json")))[name]
    p = _MAKERS[name]()
    assert str(p.irreps_in1) == gold["irreps_in1"]
    assert str(p.irreps_in2) == gold["irreps_in2"]
    assert str(p.irreps_out) == gold["irreps_out"]
    assert p.weight_numel == gold["weight_numel"]
    assert p.shared_weights == gold["shared_weights"]
    assert len(p.instructions) == len(gold["instructions"])
    ref = R.Problem.from_spec(p)
    for n, (ins, g, rp) in enumerate(zip(p.instructions, gold["instructions"], ref.paths)):
        assert [ins.i_in1, ins.i_in2, ins.i_out, ins.connection_mode, ins.has_weight] == g[:5]
        assert abs(ins.path_weight - g[5]) < 1e-15
        assert list(ins.path_shape) == g[6]
        lo, hi, _ = p.weight_range_and_shape_for_instruction(n)
        assert [lo, hi] == gold["weight_ranges"][n]
        # the oracle recomputes the normalisation independently from the raw instructions
        assert abs(rp["coeff"] - g[5]) < 1e-15 and rp["woff"] == lo


def test_config_dimension_table():
    rows = {"cfg1": (1, 5, 7, 5, 1, 28), "cfg2": (13, 288, 16, 1376, 416, 125),
            "cfg3": (23, 2048, 16, 12672, 2944, 353), "cfg4": (11, 576, 9, 576, 45056, 83)}
    for name, (npaths, l1, l2, l3, wn, nnz) in rows.items():
        p = _MAKERS[name]()
        got_nnz = sum(len(sparse_cg(p.irreps_in1[i.i_in1].ir.l, p.irreps_in2[i.i_in2].ir.l,
                                    p.irreps_out[i.i_out].ir.l)) for i in p.instructions)
        assert (len(p.instructions), p.irreps_in1.dim, p.irreps_in2.dim, p.irreps_out.dim, p.weight_numel,
                got_nnz) == (npaths, l1, l2, l3, wn, nnz)


def test_normalisation_closed_forms():
    p = P.config3_mace_uvu()
    for ins in p.instructions:
        assert abs(ins.path_weight - math.sqrt(p.irreps_out[ins.i_out].ir.dim)) < 1e-15
    p4 = P.config4_uvw_shared()
    fan = {0: 3, 1: 4, 2: 4}
    for ins in p4.instructions:
        l3 = p4.irreps_out[ins.i_out].ir.l
        assert abs(ins.path_weight - math.sqrt((2 * l3 + 1) / (64 * fan[ins.i_out]))) < 1e-15


# ------------------------------------------------------------ forward oracle

def _rand(prob, B, rng, shared=None):
    shared = prob.shared_weights if shared is None else shared
    x = rng.normal(size=(B, prob.dims[0]))
    y = rng.normal(size=(B, prob.dims[1]))
    w = rng.normal(size=(prob.weight_numel,) if shared else (B, prob.weight_numel))
    return x, y, w


TINY = [
    ("2x1o+1x2e", "1x1o+2x0e", "2x1o+2x2e+1x2e", [(0, 0, 1, "uvu", True), (0, 1, 0, "uvu", True), (1, 1, 2, "uvu", True),
                                                    (0, 1, 0, "uvu", True, 0.7)], False),
    ("2x1o+1x2e", "1x1o+2x0e", "3x1o+2x2e", [(0, 0, 1, "uvw", True), (0, 1, 0, "uvw", True), (1, 1, 1, "uvw", True),
                                               (1, 0, 0, "uvw", True)], True),
    ("2x1o+1x2e", "1x1o+2x0e", "3x1o+2x2e", [(0, 0, 1, "uvw", True), (1, 0, 0, "uvw", True)], False),
]


@pytest.mark.parametrize("case", TINY)
def test_einsum_oracle_matches_loops(case):
    a, b, o, ins, shared = case
    prob = R.Problem(a, b, o, ins, shared)
    rng = np.random.default_rng(3)
    x, y, w = _rand(prob, 3, rng)
    np.testing.assert_allclose(R.tp_forward(prob, x, y, w), R.tp_forward_loops(prob, x, y, w), atol=1e-13)


def test_forward_special_cases():
    rng = np.random.default_rng(4)
    B = 5
    x3, y3, w = rng.normal(size=(B, 3)), rng.normal(size=(B, 3)), rng.normal(size=(B, 1))
    dot = R.Problem("1x1o", "1x1o", "1x0e", [(0, 0, 0, "uvu", True)], False)
    np.testing.assert_allclose(R.tp_forward(dot, x3, y3, w)[:, 0], w[:, 0] * (x3 * y3).sum(1) / math.sqrt(3), atol=1e-14)
    cross = R.Problem("1x1o", "1x1o", "1x1e", [(0, 0, 0, "uvu", True)], False)
    np.testing.assert_allclose(R.tp_forward(cross, x3, y3, w), w * np.cross(x3, y3) / math.sqrt(2), atol=1e-14)
    x5, y1 = rng.normal(size=(B, 5)), rng.normal(size=(B, 1))
    scal = R.Problem("1x2e", "1x0e", "1x2e", [(0, 0, 0, "uvu", True)], False)
    np.testing.assert_allclose(R.tp_forward(scal, x5, y1, w), w * y1 * x5, atol=1e-14)
    one = R.Problem("1x0e", "1x0e", "1x0e", [(0, 0, 0, "uvu", True)], False)
    np.testing.assert_allclose(R.tp_forward(one, y1, y1 * 2, w), w * y1 * y1 * 2, atol=1e-14)


@pytest.mark.parametrize("case", TINY)
def test_backward_oracle_finite_differences(case):
    a, b, o, ins, shared = case
    prob = R.Problem(a, b, o, ins, shared)
    rng = np.random.default_rng(5)
    x, y, w = _rand(prob, 2, rng)
    g = rng.normal(size=(2, prob.dims[2]))
    dx, dy, dw = R.tp_backward(prob, x, y, w, g)

    def S(xx, yy, ww):
        return (R.tp_forward(prob, xx, yy, ww) * g).sum()

    h = 1e-6
    for arr, grad in ((x, dx), (y, dy), (w, dw)):
        flat = arr.reshape(-1)
        for idx in rng.choice(flat.size, size=min(6, flat.size), replace=False):
            old = flat[idx]
            flat[idx] = old + h
            up = S(x, y, w)
            flat[idx] = old - h
            dn = S(x, y, w)
            flat[idx] = old
            assert abs((up - dn) / (2 * h) - grad.reshape(-1)[idx]) < 1e-6
    # adjoint identity <g, J dx> = <J^T g, dx> for a random direction (exact: the map is linear in x)
    delta = rng.normal(size=x.shape)
    lhs = (g * (R.tp_forward(prob, x + delta, y, w) - R.tp_forward(prob, x, y, w))).sum()
    assert abs(lhs - (dx * delta).sum()) < 1e-9


def test_conv_oracle_small_graphs():
    rng = np.random.default_rng(6)
    prob = R.Problem.from_spec(P.config1_single_uvu())
    # the reference's toy graph: receivers [0,1,1,2], senders [1,0,2,1] (tests/example_test.py:46-56)
    rows, cols = np.array([0, 1, 1, 2]), np.array([1, 0, 2, 1])
    X, Y, W = rng.normal(size=(3, 5)), rng.normal(size=(4, 7)), rng.normal(size=(4, 1))
    Z = R.conv_forward(prob, X, Y, W, rows, cols)
    msg = R.tp_forward(prob, X[cols], Y, W)
    np.testing.assert_allclose(Z[0], msg[0], atol=1e-14)
    np.testing.assert_allclose(Z[1], msg[1] + msg[2], atol=1e-14)
    np.testing.assert_allclose(Z[2], msg[3], atol=1e-14)
    # edge order does not matter; isolated node gives a zero row
    perm = np.array([2, 0, 3, 1])
    np.testing.assert_allclose(R.conv_forward(prob, X, Y[perm], W[perm], rows[perm], cols[perm]), Z, atol=1e-14)
    Z4 = R.conv_forward(prob, np.vstack([X, X[:1]]), Y, W, rows, cols)
    assert np.all(Z4[3] == 0)
    # backward against finite differences on X
    G = rng.normal(size=Z.shape)
    dX, dY, dW = R.conv_backward(prob, X, Y, W, G, rows, cols)
    delta = rng.normal(size=X.shape)
    lhs = (G * (R.conv_forward(prob, X + delta, Y, W, rows, cols) - Z)).sum()
    assert abs(lhs - (dX * delta).sum()) < 1e-10
    dlt = rng.normal(size=W.shape)
    lhs = (G * (R.conv_forward(prob, X, Y, W + dlt, rows, cols) - Z)).sum()
    assert abs(lhs - (dW * dlt).sum()) < 1e-10
    dlt = rng.normal(size=Y.shape)
    lhs = (G * (R.conv_forward(prob, X, Y + dlt, W, rows, cols) - Z)).sum()
    assert abs(lhs - (dY * dlt).sum()) < 1e-10


def test_sorted_graph_matches_coordgraph():
    from openequivariance_amd.core.graph import CoordGraph, periodic_radius_graph
    coords, rows, cols, vec = periodic_radius_graph(200, 10.0, 5.0, seed=3)
    rng = np.random.default_rng(0)
    sh = rng.permutation(len(rows))
    g = CoordGraph(coords, rows[sh], cols[sh])
    r, c, order, tperm = R.sorted_graph(rows[sh], cols[sh])
    assert np.array_equal(g.rows, r) and np.array_equal(g.cols, c) and np.array_equal(g.transpose_perm, tperm)
    assert np.all(np.diff(g.rows) >= 0)
    assert np.all(np.diff(g.cols[g.transpose_perm]) >= 0)
    # both directions present, no self loops, minimum-image vectors within the cutoff
    assert set(zip(rows.tolist(), cols.tolist())) == set(zip(cols.tolist(), rows.tolist()))
    assert np.all(rows != cols) and np.all(np.linalg.norm(vec, axis=1) < 5.0)


# ------------------------------------------------------------ torch restatement (second-order checker, CPU baseline)

@pytest.mark.parametrize("case", TINY)
def test_torch_restatement_matches_numpy_oracle(case):
    """oracle/torch_ref.py is the checker of every second/third-derivative test and what bench.py times as
    the CPU baseline: its forward equals the brute-force loops, its autograd gradients equal the hand-written
    backward of the numpy oracle, for per-row and shared weights, 'uvu' and 'uvw'."""
    import torch
    from oracle.torch_ref import TorchTP

    a, b, o, ins, shared = case
    prob = R.Problem(a, b, o, ins, shared)
    rng = np.random.default_rng(11)
    x, y, w = _rand(prob, 4, rng)
    g = rng.normal(size=(4, prob.dims[2]))
    tx, ty, tw = (torch.tensor(v, dtype=torch.float64, requires_grad=True) for v in (x, y, w))
    z = TorchTP(prob, torch.float64)(tx, ty, tw)
    np.testing.assert_allclose(z.detach().numpy(), R.tp_forward_loops(prob, x, y, w), atol=1e-13)
    z.backward(torch.tensor(g))
    for got, want in zip((tx.grad, ty.grad, tw.grad), R.tp_backward(prob, x, y, w, g)):
        np.testing.assert_allclose(got.numpy(), want, atol=1e-12)


@pytest.mark.parametrize("make", [P.config1_single_uvu, P.config2_nequip_uvu, P.config4_uvw_shared])
def test_torch_restatement_conv_matches_numpy_oracle(make):
    import torch
    from oracle.torch_ref import TorchConv

    prob = R.Problem.from_spec(make())
    rng = np.random.default_rng(12)
    n, E = 7, 19
    rows, cols = rng.integers(0, n, size=E), rng.integers(0, n, size=E)
    X, Y = rng.normal(size=(n, prob.dims[0])), rng.normal(size=(E, prob.dims[1]))
    W = rng.normal(size=(prob.weight_numel,) if prob.shared_weights else (E, prob.weight_numel))
    G = rng.normal(size=(n, prob.dims[2]))
    tX, tY, tW = (torch.tensor(v, dtype=torch.float64, requires_grad=True) for v in (X, Y, W))
    Z = TorchConv(prob, torch.float64)(tX, tY, tW, torch.tensor(rows), torch.tensor(cols))
    np.testing.assert_allclose(Z.detach().numpy(), R.conv_forward(prob, X, Y, W, rows, cols), atol=1e-12)
    Z.backward(torch.tensor(G))
    for got, want in zip((tX.grad, tY.grad, tW.grad), R.conv_backward(prob, X, Y, W, G, rows, cols)):
        np.testing.assert_allclose(got.numpy(), want, atol=1e-11)
