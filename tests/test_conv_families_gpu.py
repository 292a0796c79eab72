"""Convolution over the problem families the reference's conv suite covers
(tests/conv_test.py:173-292): production models (MACE, DiffDock, e3tools), the
single-instruction grids for 'uvu' and 'uvw', and shared weights in atomic mode;
forward and backward in both modes against the CPU oracle."""

import numpy as np
import pytest
import torch

import openequivariance_amd as oeq
from openequivariance_amd.core import problems as P
from openequivariance_amd.core.graph import CoordGraph, periodic_radius_graph
from oracle import e3nn_ref as R
from gpu_util import err, tol_of

pytestmark = pytest.mark.gpu

UVU_MULS = [(1, 1, 1), (8, 1, 8), (16, 1, 16), (32, 1, 32), (5, 1, 5), (13, 1, 13), (19, 1, 19), (33, 1, 33),
            (49, 1, 49), (128, 1, 128), (1, 2, 1), (1, 16, 1), (1, 32, 1), (16, 3, 16)]
UVU_IRS = [(0, 0, 0), (1, 1, 1), (1, 0, 1), (1, 2, 1), (2, 0, 2), (5, 3, 5), (7, 2, 5)]
UVW_MULS = [(1, 1, 1), (4, 1, 4), (8, 1, 8), (16, 1, 16), (32, 1, 32), (5, 1, 5), (13, 1, 13), (33, 1, 33),
            (49, 1, 49), (64, 1, 64), (1, 2, 1), (1, 4, 1), (1, 16, 1), (1, 32, 1), (16, 3, 16)]
UVW_IRS = [(0, 0, 0), (1, 1, 1), (1, 0, 1), (1, 2, 1), (5, 3, 5), (7, 2, 5)]


def _single(mode, m, i, dtype):
    return oeq.TPProblem(f"{m[0]}x{i[0]}e", f"{m[1]}x{i[1]}e", f"{m[2]}x{i[2]}e", [(0, 0, 0, mode, True)],
                         shared_weights=False, internal_weights=False, irrep_dtype=dtype, weight_dtype=dtype,
                         label=f"{mode}-{m[0]}x{i[0]}e__x__{m[1]}x{i[1]}e---{m[2]}x{i[2]}e")


def _cases():
    out = []
    for mode, muls, irs in (("uvu", UVU_MULS, UVU_IRS), ("uvw", UVW_MULS, UVW_IRS)):
        for n, m in enumerate(muls):  # two irrep triples per multiplicity, in rotation
            for q in range(2):
                dtype = np.float64 if (n + q) % 4 == 3 else np.float32
                out.append(_single(mode, m, irs[(2 * n + q) % len(irs)], dtype))
    out += P.mace_problems() + P.diffdock_problems() + P.e3tools_problems()
    out += P.nequix_problems() + P.seven_net_problems()  # a different multiplicity per irrep
    # ... with an input block no instruction reads and an output block no instruction writes
    out.append(oeq.TPProblem("100x0e+70x1o+40x2e+96x1e", "1x0e+2x1o", "100x0e+70x1o+100x1o+40x1o+33x2e",
                             [(0, 0, 0, "uvu", True), (1, 0, 1, "uvu", True), (0, 1, 2, "uvu", True),
                              (2, 1, 3, "uvu", True, 0.7)], shared_weights=False, internal_weights=False,
                             label="folded-gaps"))
    # wider than four waves and ragged: chunk waves with bodies specialised per chunk
    out.append(oeq.TPProblem("300x0e+70x1o+20x2e", "1x0e+1x1o", "300x0e+70x1o+300x1o+20x1o",
                             [(0, 0, 0, "uvu", True), (1, 0, 1, "uvu", True), (0, 1, 2, "uvu", True),
                              (2, 1, 3, "uvu", True)], shared_weights=False, internal_weights=False,
                             label="very-wide-ragged"))
    shared = P.mace_problems()[0].clone()
    shared.shared_weights = True
    shared.label = "mace-large-shared"
    out.append(shared)
    return out


CASES = _cases()
GRAPH = {}


def _graph():
    if not GRAPH:
        coords, rows, cols, _ = periodic_radius_graph(24, 5, 5.0, 3)
        keep = (rows != 4) & (cols != 7)  # node 4 receives nothing, node 7 sends nothing
        GRAPH["g"] = (coords, rows[keep], cols[keep])
    return GRAPH["g"]


@pytest.mark.parametrize("problem", CASES, ids=[p.label for p in CASES])
def test_conv_family(problem):
    tol = tol_of(problem)
    coords, rows, cols = _graph()
    n, E = coords.shape[0], len(rows)
    rng = np.random.default_rng(12345)
    dt = np.dtype(problem.irrep_dtype)
    X = rng.uniform(size=(n, problem.irreps_in1.dim)).astype(dt)
    Y = rng.uniform(size=(E, problem.irreps_in2.dim)).astype(dt)
    W = rng.uniform(size=(problem.weight_numel,) if problem.shared_weights else (E, problem.weight_numel)).astype(dt)
    G = rng.uniform(size=(n, problem.irreps_out.dim)).astype(dt)
    ref = R.Problem.from_spec(problem)
    z_ref = R.conv_forward(ref, X, Y, W, rows, cols)
    dx_ref, dy_ref, dw_ref = R.conv_backward(ref, X, Y, W, G, rows, cols)
    for det in ([False] if problem.shared_weights else [True, False]):
        if det:
            g = CoordGraph(coords, rows, cols)
            order, r_, c_, perm = g.order, g.rows, g.cols, g.transpose_perm
        else:
            order = rng.permutation(E)
            r_, c_, perm = rows[order], cols[order], None
        conv = oeq.TensorProductConv(problem, deterministic=det)
        tX = torch.tensor(X, device="cuda", requires_grad=True)
        tY = torch.tensor(Y[order], device="cuda", requires_grad=True)
        tW = torch.tensor(W if problem.shared_weights else W[order], device="cuda", requires_grad=True)
        tperm = torch.tensor(perm, device="cuda") if perm is not None else None
        z = conv(tX, tY, tW, torch.tensor(r_, device="cuda"), torch.tensor(c_, device="cuda"), tperm)
        z.backward(torch.tensor(G, device="cuda"))
        assert err(z, z_ref) <= tol, det
        assert err(tX.grad, dx_ref) <= tol, det
        dy = np.empty_like(Y)
        dy[order] = tY.grad.cpu().numpy()
        assert err(dy, dy_ref) <= tol, det
        dw = tW.grad.cpu().numpy()
        if not problem.shared_weights:
            full = np.empty_like(W)
            full[order] = dw
            dw = full
        assert err(dw, dw_ref) <= tol, det
