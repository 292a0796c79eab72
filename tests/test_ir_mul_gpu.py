"""`layout="ir_mul"` kernels against the CPU oracle (which works in `mul_ir`:
inputs are converted on the way in, results on the way out) and against the
`mul_ir` kernels wrapped in layout conversions, as the reference tests do
(tests/batch_test.py:309-380, tests/conv_test.py:325-355)."""

import numpy as np
import pytest
import torch

import openequivariance_amd as oeq
from openequivariance_amd.core import problems as P
from openequivariance_amd.core.graph import CoordGraph, periodic_radius_graph
from openequivariance_amd.core.layout import transpose_irrep_layout as tr
from oracle import e3nn_ref as R
from gpu_util import err, tol_of, tp_inputs

pytestmark = pytest.mark.gpu


def _single(mul):
    return oeq.TPProblem(f"{mul}x5e", "1x3e", f"{mul}x5e", [(0, 0, 0, "uvu", True)], shared_weights=False,
                         internal_weights=False, label=f"ir_mul_repr_{mul}x1x{mul}_l535")


def _multi_v(shared):
    return oeq.TPProblem("5x1e+3x2e", "2x1e+1x0e", "5x1e+3x2e+5x0e",
                         [(0, 0, 0, "uvu", True), (0, 1, 0, "uvu", True), (1, 0, 1, "uvu", True),
                          (0, 0, 2, "uvu", True)], shared_weights=shared, internal_weights=False, label="odd-uvu")


PROBLEMS = [
    ("mace-large", lambda: P.mace_problems()[0]),
    ("mace-medium", lambda: P.mace_problems()[1]),
    ("cfg3-f64", lambda: P.config3_mace_uvu(np.float64)),
    ("cfg2", P.config2_nequip_uvu),
    ("5x5e", lambda: _single(5)),
    ("13x5e", lambda: _single(13)),
    ("multi-v", lambda: _multi_v(False)),
    ("multi-v-shared", lambda: _multi_v(True)),
    # wide rows with a different multiplicity per irrep: folded into 64-channel pieces whose components
    # stay a whole block's multiplicity apart
    ("nequix-first", lambda: P.nequix_problems()[0]),
    ("sevennet-main", lambda: P.seven_net_problems()[1]),
    ("folded-gaps", lambda: oeq.TPProblem(
        "100x0e+70x1o+40x2e+96x1e", "1x0e+2x1o", "100x0e+70x1o+100x1o+40x1o+33x2e",
        [(0, 0, 0, "uvu", True), (1, 0, 1, "uvu", True), (0, 1, 2, "uvu", True), (2, 1, 3, "uvu", True, 0.7)],
        shared_weights=False, internal_weights=False, label="folded-gaps")),
    # every piece exactly 64 channels wide (the shape the convolution's staged operand loads accept), one block
    # folded into two of them: the staged loads must step a whole block's multiplicity between components
    ("folded-64s", lambda: oeq.TPProblem(
        "64x4e+128x3e", "1x1e+1x0e", "64x4e+128x2e+128x3e+128x4e+128x3e",
        [(0, 1, 0, "uvu", True), (1, 0, 1, "uvu", True), (1, 0, 2, "uvu", True), (1, 0, 3, "uvu", True),
         (1, 1, 4, "uvu", True)], shared_weights=False, internal_weights=False, label="folded-64s")),
    # a block of more than 1024 channels: pieces of 1024 whose components stay the block's multiplicity apart
    ("uvu-1100", lambda: oeq.TPProblem("1100x1o", "1x1o", "1100x2e+1100x0e",
                                       [(0, 0, 0, "uvu", True), (0, 0, 1, "uvu", True)], shared_weights=False,
                                       internal_weights=False, label="uvu-1100")),
]


def _ir_mul(problem):
    q = problem.clone()
    q.layout = "ir_mul"
    return q


@pytest.mark.parametrize("name,make", PROBLEMS, ids=[c[0] for c in PROBLEMS])
def test_batch_ir_mul(name, make):
    problem = make()
    tol = tol_of(problem)
    B = 67
    x, y, w, g = tp_inputs(problem, B, seed=3)  # mul_ir data
    ref = R.Problem.from_spec(problem)
    z_ref = R.tp_forward(ref, x, y, w)
    dx_ref, dy_ref, dw_ref = R.tp_backward(ref, x, y, w, g)
    i1, i2, io = problem.irreps_in1, problem.irreps_in2, problem.irreps_out
    tx = torch.tensor(tr(x, i1, "mul_ir", "ir_mul"), device="cuda", requires_grad=True)
    ty = torch.tensor(tr(y, i2, "mul_ir", "ir_mul"), device="cuda", requires_grad=True)
    tw = torch.tensor(w, device="cuda", requires_grad=True)
    tg = torch.tensor(tr(g, io, "mul_ir", "ir_mul"), device="cuda")
    tp = oeq.TensorProduct(_ir_mul(problem))
    z = tp(tx, ty, tw)
    z.backward(tg)
    assert err(tr(z.detach().cpu().numpy(), io, "ir_mul", "mul_ir"), z_ref) <= tol
    assert err(tr(tx.grad.cpu().numpy(), i1, "ir_mul", "mul_ir"), dx_ref) <= tol
    assert err(tr(ty.grad.cpu().numpy(), i2, "ir_mul", "mul_ir"), dy_ref) <= tol
    assert err(tw.grad, dw_ref) <= tol

    # the mul_ir kernels behind layout conversions agree with the native ir_mul kernels
    tp_m = oeq.TensorProduct(problem)
    z_w = oeq.transpose_irreps(
        tp_m(oeq.transpose_irreps(tx.detach(), i1, "ir_mul", "mul_ir"),
             oeq.transpose_irreps(ty.detach(), i2, "ir_mul", "mul_ir"), tw.detach()), io, "mul_ir", "ir_mul")
    assert err(z.detach(), z_w.cpu().numpy()) <= tol


CONV = [c for c in PROBLEMS if c[0] in ("mace-large", "cfg3-f64", "cfg2", "13x5e", "multi-v", "multi-v-shared",
                                        "nequix-first", "sevennet-main", "folded-gaps", "folded-64s")]


@pytest.mark.parametrize("hub", [256, 2], ids=["whole-segments", "chunks-of-2"])
@pytest.mark.parametrize("name,make", CONV, ids=[c[0] for c in CONV])
def test_conv_ir_mul(name, make, hub, monkeypatch):
    # (second run: every edge segment cut into chunks of two edges, so that extra walk positions, the rows they
    # write and the chunked sender-side sums are exercised in this layout as well)
    if hub != 256:
        monkeypatch.setenv("OEQ_AMD_TUNE", f"conv_hub={hub}")
    problem = make()
    tol = tol_of(problem)
    n_nodes = 40
    coords, rows, cols, _ = periodic_radius_graph(n_nodes, 6, 5.0, 1)
    keep = (rows != 3) & (cols != 3) & (rows != 5)
    rows, cols = rows[keep], cols[keep]
    E = len(rows)
    rng = np.random.default_rng(5)
    dt = np.dtype(problem.irrep_dtype)
    i1, i2, io = problem.irreps_in1, problem.irreps_in2, problem.irreps_out
    X = rng.uniform(size=(n_nodes, i1.dim)).astype(dt)
    Y = rng.uniform(size=(E, i2.dim)).astype(dt)
    W = rng.uniform(size=(problem.weight_numel,) if problem.shared_weights else (E, problem.weight_numel)).astype(dt)
    G = rng.uniform(size=(n_nodes, io.dim)).astype(dt)
    ref = R.Problem.from_spec(problem)
    z_ref = R.conv_forward(ref, X, Y, W, rows, cols)
    dx_ref, dy_ref, dw_ref = R.conv_backward(ref, X, Y, W, G, rows, cols)
    for det in ([False] if problem.shared_weights else [False, True]):
        if det:
            gr = CoordGraph(coords, rows, cols)
            order, r_, c_, perm = gr.order, gr.rows, gr.cols, gr.transpose_perm
        else:
            order = rng.permutation(E)
            r_, c_, perm = rows[order], cols[order], None
        conv = oeq.TensorProductConv(_ir_mul(problem), deterministic=det)
        tX = torch.tensor(tr(X, i1, "mul_ir", "ir_mul"), device="cuda", requires_grad=True)
        tY = torch.tensor(tr(Y[order], i2, "mul_ir", "ir_mul"), device="cuda", requires_grad=True)
        tW = torch.tensor(W if problem.shared_weights else W[order], device="cuda", requires_grad=True)
        tr_, tc_ = torch.tensor(r_, device="cuda"), torch.tensor(c_, device="cuda")
        tperm = torch.tensor(perm, device="cuda") if perm is not None else None
        z = conv(tX, tY, tW, tr_, tc_, tperm)
        z.backward(torch.tensor(tr(G, io, "mul_ir", "ir_mul"), device="cuda"))
        assert err(tr(z.detach().cpu().numpy(), io, "ir_mul", "mul_ir"), z_ref) <= tol, (name, det)
        assert err(tr(tX.grad.cpu().numpy(), i1, "ir_mul", "mul_ir"), dx_ref) <= tol, (name, det)
        dy = tr(tY.grad.cpu().numpy(), i2, "ir_mul", "mul_ir")
        dy_back = np.empty_like(dy)
        dy_back[order] = dy
        assert err(dy_back, dy_ref) <= tol, (name, det)
        dw = tW.grad.cpu().numpy()
        if not problem.shared_weights:
            dw_back = np.empty_like(dw)
            dw_back[order] = dw
            dw = dw_back
        assert err(dw, dw_ref) <= tol, (name, det)
