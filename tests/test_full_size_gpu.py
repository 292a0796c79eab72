"""Benchmark-size runs, where the float64 oracle is too slow to evaluate everything: agreement of a
sample with the oracle plus size-independent properties (exact scaling laws, edge-order invariance,
atomic vs deterministic agreement, bitwise reproducibility)."""

import numpy as np
import pytest
import torch

import openequivariance_amd as oeq
from openequivariance_amd.core import problems as P
from openequivariance_amd.core.graph import CoordGraph, periodic_radius_graph
from openequivariance_amd.core.sh import spherical_harmonics
from oracle import e3nn_ref as R
from gpu_util import err

pytestmark = pytest.mark.gpu


def _rel(a, b):
    return float((a - b).abs().max() / b.abs().max())


def test_cfg2_full_batch():
    problem = P.config2_nequip_uvu()
    B = 200000
    gen = torch.Generator(device="cuda").manual_seed(0)
    x = torch.randn(B, 288, device="cuda", generator=gen, requires_grad=True)
    v = torch.randn(B, 3, device="cuda", generator=gen)
    y = torch.tensor(spherical_harmonics(3, v.cpu().numpy()).astype(np.float32), device="cuda").requires_grad_(True)
    w = torch.randn(B, 416, device="cuda", generator=gen, requires_grad=True)
    g = torch.randn(B, 1376, device="cuda", generator=gen)
    tp = oeq.TensorProduct(problem)
    z = tp(x, y, w)
    z.backward(g)
    idx = torch.tensor([0, 1, 2, 31, 32, 33, 65535, 65536, B - 3, B - 2, B - 1], device="cuda")
    ref = R.Problem.from_spec(problem)
    xs, ys, ws, gs = (t[idx].detach().cpu().numpy() for t in (x, y, w, g))
    assert err(z[idx], R.tp_forward(ref, xs, ys, ws)) <= 1e-5
    dx, dy, dw = R.tp_backward(ref, xs, ys, ws, gs)
    assert err(x.grad[idx], dx) <= 1e-5 and err(y.grad[idx], dy) <= 1e-5 and err(w.grad[idx], dw) <= 1e-5
    assert torch.equal(tp(4.0 * x, y, 0.5 * w), 2.0 * z)  # powers of two scale exactly
    assert torch.isfinite(z).all() and torch.isfinite(x.grad).all()


def test_cfg1_full_batch():
    """Config 1 at its scaled-up size: 100 000 rows, uniform[0,1) inputs from seed 0, every row against the
    oracle (the problem is small enough for that)."""
    problem = P.config1_single_uvu()
    B = 100000
    rng = np.random.default_rng(0)
    x, y, w, g = (rng.uniform(size=(B, d)).astype(np.float32) for d in (5, 7, 1, 5))
    tx, ty, tw = (torch.tensor(a, device="cuda", requires_grad=True) for a in (x, y, w))
    tp = oeq.TensorProduct(problem)
    z = tp(tx, ty, tw)
    z.backward(torch.tensor(g, device="cuda"))
    ref = R.Problem.from_spec(problem)
    assert err(z, R.tp_forward(ref, x, y, w)) <= 1e-5
    for got, want in zip((tx.grad, ty.grad, tw.grad), R.tp_backward(ref, x, y, w, g)):
        assert err(got, want) <= 1e-5
    assert torch.equal(tp(2.0 * tx, ty, 0.25 * tw), 0.5 * z)


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
def test_cfg3_full_batch(dtype):
    """Config 3 at its full size, 500 000 rows, in both precisions: a sample of rows (first, last, both sides
    of the boundaries between the blocks of a grid-sized sweep) against the oracle, exact scaling by powers of
    two, linearity in the output gradient, same bits on a second run."""
    problem = P.config3_mace_uvu(dtype)
    tdt = torch.float32 if dtype == np.float32 else torch.float64
    tol = 1e-5 if dtype == np.float32 else 1e-12
    B = 500000
    gen = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randn(B, 2048, device="cuda", generator=gen, dtype=tdt)
    v = torch.randn(B, 3, device="cuda", generator=gen, dtype=torch.float64)
    y = torch.tensor(spherical_harmonics(3, v.cpu().numpy()).astype(dtype), device="cuda")
    w = torch.randn(B, 2944, device="cuda", generator=gen, dtype=tdt)
    g = torch.randn(B, 12672, device="cuda", generator=gen, dtype=tdt)
    tp = oeq.TensorProduct(problem)
    ops = torch.ops.oeq_amd
    z = ops.tp_forward(x, y, w, tp.kid)
    idx = torch.tensor([0, 1, 2, 2047, 2048, 2049, 250000, 499998, B - 1], device="cuda")
    ref = R.Problem.from_spec(problem)
    xs, ys, ws, gs = (t[idx].cpu().numpy() for t in (x, y, w, g))
    assert err(z[idx], R.tp_forward(ref, xs, ys, ws)) <= tol
    assert torch.isfinite(z).all()
    assert torch.equal(ops.tp_forward(4.0 * x, y, 0.5 * w, tp.kid), 2.0 * z)
    del z
    dx, dy, dw = ops.tp_backward(x, y, w, g, tp.kid)
    rx, ry, rw = R.tp_backward(ref, xs, ys, ws, gs)
    assert err(dx[idx], rx) <= tol and err(dy[idx], ry) <= tol and err(dw[idx], rw) <= tol
    dx2, dy2, dw2 = ops.tp_backward(x, y, w, g, tp.kid)
    assert torch.equal(dx, dx2) and torch.equal(dy, dy2) and torch.equal(dw, dw2)
    del dx2, dy2, dw2
    # linear in the output gradient (a power of two scales exactly)
    sx, sy, sw = ops.tp_backward(x, y, w, 2.0 * g, tp.kid)
    assert torch.equal(sx, 2.0 * dx) and torch.equal(sy, 2.0 * dy) and torch.equal(sw, 2.0 * dw)


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
def test_cfg4_full_batch_mfma(dtype):
    problem = P.config4_uvw_shared(dtype)
    tol = 1e-5 if dtype == np.float32 else 1e-12
    td = torch.float32 if dtype == np.float32 else torch.float64
    B = 262144 if dtype == np.float32 else 65536
    gen = torch.Generator(device="cuda").manual_seed(1)
    x = torch.randn(B, 576, device="cuda", generator=gen, dtype=td, requires_grad=True)
    v = torch.randn(B, 3, device="cuda", generator=gen)
    y = torch.tensor(spherical_harmonics(2, v.cpu().numpy()).astype(dtype), device="cuda").requires_grad_(True)
    w = (torch.randn(45056, device="cuda", generator=gen, dtype=td) / np.sqrt(64 * 11)).requires_grad_(True)
    g = torch.randn(B, 576, device="cuda", generator=gen, dtype=td)
    tp = oeq.TensorProduct(problem)
    z = tp(x, y, w)
    z.backward(g)
    idx = torch.tensor([0, 1, 15, 16, 17, 4095, 4096, B - 17, B - 16, B - 1], device="cuda")
    ref = R.Problem.from_spec(problem)
    xs, ys, gs = (t[idx].detach().cpu().numpy() for t in (x, y, g))
    wn = w.detach().cpu().numpy()
    assert err(z[idx], R.tp_forward(ref, xs, ys, wn)) <= tol
    dx, dy, _ = R.tp_backward(ref, xs, ys, wn, gs)
    assert err(x.grad[idx], dx) <= tol and err(y.grad[idx], dy) <= tol
    # weight gradient: linear in the output gradient; a sum over disjoint row sets adds up
    half = B // 2
    _, _, dw1 = torch.ops.oeq_amd.tp_backward(x[:half].detach(), y[:half].detach(), w.detach(), g[:half], tp.kid)
    _, _, dw2 = torch.ops.oeq_amd.tp_backward(x[half:].detach(), y[half:].detach(), w.detach(), g[half:], tp.kid)
    assert _rel(dw1 + dw2, w.grad) <= tol
    # and it matches the oracle on a slice small enough to evaluate (first 2048 rows)
    n = 2048
    _, _, dws = torch.ops.oeq_amd.tp_backward(x[:n].detach(), y[:n].detach(), w.detach(), g[:n], tp.kid)
    _, _, dw_ref = R.tp_backward(ref, x[:n].detach().cpu().numpy(), y[:n].detach().cpu().numpy(), wn,
                                 g[:n].cpu().numpy())
    assert err(dws, dw_ref) <= tol
    # deterministic reduction: bitwise equal on a second run
    _, _, dw_again = torch.ops.oeq_amd.tp_backward(x.detach(), y.detach(), w.detach(), g, tp.kid)
    assert torch.equal(dw_again, w.grad)


@pytest.mark.parametrize("name", ["diffdock-shared", "mul2-f64"])
def test_padded_matrix_core_tiles_full_batch(name):
    """Shared weights with multiplicities that are no multiples of 16 (tiles padded with zero weights; second case:
    a two-channel second operand, fp64) at 262 144 / 65 536 rows: rows at tile and grid boundaries against the oracle,
    the weight gradient as a sum over disjoint row sets and against the oracle on a slice, same bits on a second run."""
    from openequivariance_amd.codegen import uvw_mfma
    from openequivariance_amd.codegen.lower import lower
    if name == "diffdock-shared":
        problem = P.diffdock_problems()[0].clone()
        problem.shared_weights = True
        B, dtype = 262144, np.float32
    else:
        problem = P.FullyConnectedTPProblem("40x0e+30x1o", "2x0e+1x1o", "25x0e+10x1o+5x2e", shared_weights=True,
                                            internal_weights=False, irrep_dtype=np.float64, weight_dtype=np.float64)
        B, dtype = 65536, np.float64
    low = lower(problem)
    assert uvw_mfma.supported(low)
    tol = 1e-5 if dtype == np.float32 else 1e-12
    td = torch.float32 if dtype == np.float32 else torch.float64
    gen = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn(B, low.L1, device="cuda", generator=gen, dtype=td)
    y = torch.randn(B, low.L2, device="cuda", generator=gen, dtype=td)
    w = torch.randn(low.WN, device="cuda", generator=gen, dtype=td) / 8
    g = torch.randn(B, low.L3, device="cuda", generator=gen, dtype=td)
    tp = oeq.TensorProduct(problem)
    ops = torch.ops.oeq_amd
    z = ops.tp_forward(x, y, w, tp.kid)
    dx, dy, dw = ops.tp_backward(x, y, w, g, tp.kid)
    assert all(torch.isfinite(t).all() for t in (z, dx, dy, dw))
    idx = torch.tensor([0, 1, 15, 16, 17, 8191, 8192, B - 17, B - 16, B - 1], device="cuda")
    ref = R.Problem.from_spec(problem)
    xs, ys, gs = (t[idx].cpu().numpy() for t in (x, y, g))
    wn = w.cpu().numpy()
    assert err(z[idx], R.tp_forward(ref, xs, ys, wn)) <= tol
    rx, ry, _ = R.tp_backward(ref, xs, ys, wn, gs)
    assert err(dx[idx], rx) <= tol and err(dy[idx], ry) <= tol
    half = B // 2
    _, _, dw1 = ops.tp_backward(x[:half], y[:half], w, g[:half], tp.kid)
    _, _, dw2 = ops.tp_backward(x[half:], y[half:], w, g[half:], tp.kid)
    assert _rel(dw1 + dw2, dw) <= tol
    n = 2048
    _, _, dws = ops.tp_backward(x[:n], y[:n], w, g[:n], tp.kid)
    _, _, dw_ref = R.tp_backward(ref, x[:n].cpu().numpy(), y[:n].cpu().numpy(), wn, g[:n].cpu().numpy())
    assert err(dws, dw_ref) <= tol
    again = ops.tp_backward(x, y, w, g, tp.kid)
    assert torch.equal(again[0], dx) and torch.equal(again[1], dy) and torch.equal(again[2], dw)
    assert torch.equal(ops.tp_forward(2.0 * x, y, 0.25 * w, tp.kid), 0.5 * z)


def test_cfg5_full_graph():
    problem = P.config5_mace_conv()
    N = 50000
    coords, rows, cols, vec = periodic_radius_graph(N, 32.0, 5.0, seed=0)
    g = CoordGraph(coords, rows, cols)
    E = g.nnz
    assert 1.5e6 < E < 1.7e6
    Y = torch.tensor(spherical_harmonics(3, vec).astype(np.float32)[g.order], device="cuda")
    gen = torch.Generator(device="cuda").manual_seed(0)
    X = torch.randn(N, 2048, device="cuda", generator=gen)
    W = torch.randn(E, 2944, device="cuda", generator=gen)
    G = torch.randn(N, 12672, device="cuda", generator=gen)
    tr, tc, tp = (torch.tensor(a, device="cuda") for a in (g.rows, g.cols, g.transpose_perm))
    det = oeq.TensorProductConv(problem, deterministic=True)
    ops = torch.ops.oeq_amd
    z = ops.conv_forward(X, Y, W, tr, tc, tp, det.kid)
    dx, dy, dw = ops.conv_backward(X, Y, W, G, tr, tc, tp, det.kid)
    # bitwise reproducible
    z2 = ops.conv_forward(X, Y, W, tr, tc, tp, det.kid)
    dx2, dy2, dw2 = ops.conv_backward(X, Y, W, G, tr, tc, tp, det.kid)
    assert torch.equal(z, z2) and torch.equal(dx, dx2) and torch.equal(dy, dy2) and torch.equal(dw, dw2)
    # Oracle on the sub-graphs of 64 receivers (forward, dY, dW of their edges) and of 64 senders (dX): the
    # highest-degree node on either side, the first and the last node of every XCD's range of the walk order
    # (read from the index the ops built), and a seeded random draw.
    from openequivariance_amd._torch import ops as O
    ks = O.get_entry(det.kid).kernels()
    index, side = O._conv_index(ks, N, E, tr, tc, tp, True)
    off, n_order = ks.conv_index_piece(N, E, side, "order")
    order = index[off:off + 8 * n_order].view(torch.int64).cpu().numpy()
    assert n_order == N and np.array_equal(np.sort(order), np.arange(N))
    per = (N + 7) // 8
    edge_nodes = [int(order[min(N - 1, v)]) for x in range(8) for v in (x * per, (x + 1) * per - 1)]
    rng = np.random.default_rng(0)
    in_deg, out_deg = np.bincount(g.rows, minlength=N), np.bincount(g.cols, minlength=N)
    recv = sorted(set(edge_nodes + [int(in_deg.argmax()), 0, N - 1] + rng.integers(0, N, 64).tolist()))[:80]
    send = sorted(set(edge_nodes + [int(out_deg.argmax()), 0, N - 1] + rng.integers(0, N, 64).tolist()))[:80]
    assert len(recv) >= 64 and len(send) >= 64
    ref = R.Problem.from_spec(problem)
    scale = {"z": float(z.abs().max()), "dy": float(dy.abs().max()), "dw": float(dw.abs().max()),
             "dx": float(dx.abs().max())}
    worst = {key: 0.0 for key in scale}
    for r in recv:
        e0, e1 = np.searchsorted(g.rows, [r, r + 1])
        sl = slice(e0, e1)
        xs, ys, ws = X[tc[sl]].cpu().numpy(), Y[sl].cpu().numpy(), W[sl].cpu().numpy()
        msg = R.tp_forward(ref, xs, ys, ws)
        gx, gy, gw = R.tp_backward(ref, xs, ys, ws, G[r:r + 1].expand(e1 - e0, -1).cpu().numpy())
        worst["z"] = max(worst["z"], float(np.abs(z[r].cpu().numpy() - msg.sum(0)).max()))
        worst["dy"] = max(worst["dy"], float(np.abs(dy[sl].cpu().numpy() - gy).max()))
        worst["dw"] = max(worst["dw"], float(np.abs(dw[sl].cpu().numpy() - gw).max()))
    for s in send:  # sum of the dX terms of the sender's out-edges
        te = torch.tensor(np.nonzero(g.cols == s)[0], device="cuda")
        gx, _, _ = R.tp_backward(ref, X[tc[te]].cpu().numpy(), Y[te].cpu().numpy(), W[te].cpu().numpy(),
                                 G[tr[te]].cpu().numpy())
        worst["dx"] = max(worst["dx"], float(np.abs(dx[s].cpu().numpy() - gx.sum(0)).max()))
    # max normalised error (fp32 bar: 1e-5), normalised by the largest magnitude of the whole result
    for key in worst:
        assert worst[key] / scale[key] <= 1e-5, (key, worst[key], scale[key])
    # deterministic=False: on the sorted list the device-side grouping reproduces the caller's order (same
    # bits for the output and the per-edge gradients; the sender gradient is accumulated with float atomics
    # and agrees to tolerance); on shuffled edges it agrees to tolerance and the forward is reproducible
    perm = torch.randperm(E, device="cuda", generator=gen)
    at = oeq.TensorProductConv(problem, deterministic=False)
    dummy = torch.zeros(1, dtype=torch.int64, device="cuda")
    assert torch.equal(ops.conv_forward(X, Y, W, tr, tc, dummy, at.kid), z)
    dxs, dys, dws = ops.conv_backward(X, Y, W, G, tr, tc, dummy, at.kid)
    assert _rel(dxs, dx) <= 1e-5 and torch.equal(dys, dy) and torch.equal(dws, dw)
    del dxs, dys, dws
    Yp, Wp, rp, cp = Y[perm].contiguous(), W[perm].contiguous(), tr[perm].contiguous(), tc[perm].contiguous()
    za = ops.conv_forward(X, Yp, Wp, rp, cp, dummy, at.kid)
    assert _rel(za, z) <= 1e-5
    dxa, dya, dwa = ops.conv_backward(X, Yp, Wp, G, rp, cp, dummy, at.kid)
    assert _rel(dxa, dx) <= 1e-5 and _rel(dya, dy[perm]) <= 1e-5 and _rel(dwa, dw[perm]) <= 1e-5
    assert torch.equal(ops.conv_forward(X, Yp, Wp, rp, cp, dummy, at.kid), za)
    # exact scaling laws
    assert torch.equal(ops.conv_forward(2.0 * X, Y, W, tr, tc, tp, det.kid), 2.0 * z)
    assert torch.isfinite(z).all() and torch.isfinite(dx).all()
