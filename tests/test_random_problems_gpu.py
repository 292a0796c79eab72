"""Seeded random problems against the CPU restatement: irreps of either parity with l <= 3, multiplicities from
1 to 130 (packed rows, single waves, rows wider than a wave), several paths into one output block, output blocks
no path writes, path weights, 'uvu' and 'uvw', per-row and shared weights, fp32 and fp64. For each problem: batch
forward / backward, the fused second-order pair where the kernel set has one, and the convolution (caller-sorted
and device-grouped edge lists; with and without compensated summation) forward / backward / second order. The
fixed problem zoo of the other test files covers the shapes models use; this sweep looks for generator corner
cases between them. A second generator draws shared-weight fully connected problems for the matrix-core kernels
with multiplicities that are no multiples of 16."""

import numpy as np
import pytest
import torch

import openequivariance_amd as oeq
from openequivariance_amd._torch import ops
from openequivariance_amd.core.graph import CoordGraph, periodic_radius_graph
from oracle import e3nn_ref as R

pytestmark = pytest.mark.gpu

MULS1 = [1, 2, 3, 5, 8, 16, 17, 32, 40, 64, 70, 96, 128, 130]
MULS2 = [1, 1, 1, 1, 2, 3]
MULSO = [1, 2, 4, 6, 16, 24]


def _irreps(blocks):
    return "+".join(f"{m}x{l}{'e' if p == 1 else 'o'}" for m, l, p in blocks)


def random_problem(rng):
    """None when the draw selected no path."""
    mode = "uvu" if rng.random() < 0.6 else "uvw"
    wide = rng.random() < 0.5
    in1 = [(int(rng.choice(MULS1 if wide else MULS1[:8])), int(rng.integers(0, 4)), int(rng.choice([1, -1])))
           for _ in range(rng.integers(1, 5))]
    if mode == "uvw":
        in1 = [(min(m, 48), l, p) for m, l, p in in1]
    in2 = [(int(rng.choice(MULS2)), int(rng.integers(0, 4)), int(rng.choice([1, -1]))) for _ in range(rng.integers(1, 4))]
    out, paths = [], []
    for i1, (m1, l1, p1) in enumerate(in1):
        for i2, (m2, l2, p2) in enumerate(in2):
            if rng.random() < 0.35:
                continue
            for l3 in range(abs(l1 - l2), min(l1 + l2, 3) + 1):
                if rng.random() < 0.4:
                    continue
                mo = m1 if mode == "uvu" else int(rng.choice(MULSO))
                same = [k for k, b in enumerate(out) if b == (mo, l3, p1 * p2)]
                if same and rng.random() < 0.4:
                    io = int(rng.choice(same))
                else:
                    out.append((mo, l3, p1 * p2))
                    io = len(out) - 1
                paths.append((i1, i2, io, mode, True, 1.0 if rng.random() < 0.7 else float(rng.uniform(0.3, 2.0))))
    if not paths:
        return None
    if rng.random() < 0.3:
        out.append((int(rng.choice([3, 16])), int(rng.integers(0, 3)), 1))  # a block no path writes
    dt = np.float64 if rng.random() < 0.3 else np.float32
    return oeq.TPProblem(_irreps(in1), _irreps(in2), _irreps(out), paths, shared_weights=bool(rng.random() < 0.3),
                         internal_weights=False, irrep_dtype=dt, weight_dtype=dt)


def _second_order(fn, x, y, w, g, a, b, c):
    """Gradients of <a, dx> + <b, dy> + <c, dw> w.r.t. (x, y, w, g); float64 autograd on the host."""
    t = [torch.tensor(v.double().cpu().numpy(), requires_grad=True) for v in (x, y, w, g)]
    cot = [torch.tensor(v.double().cpu().numpy()) for v in (a, b, c)]
    first = torch.autograd.grad(fn(*t[:3]), t[:3], t[3], create_graph=True)
    s = sum((p * q).sum() for p, q in zip(cot, first))
    return [None if v is None else v.numpy() for v in torch.autograd.grad(s, t, allow_unused=True)]


def _rand(rng, shape, dt):
    return torch.tensor(rng.uniform(-1, 1, size=shape).astype(dt), device="cuda")


def _compare(tag, got, want, tol):
    for n, (a, b) in enumerate(zip(got, want)):
        if b is None:
            continue
        e = R.normalized_error(a.detach().cpu().numpy(), b)
        assert e <= tol, (tag, n, e)


def random_shared_fully_connected_problem(rng):
    """Shared weights, multiplicities from 3 to 130 of which few are multiples of 16, one to three channels in the
    second operand: the matrix-core kernels on tiles padded with zero weights (pieces of 64 channels plus a narrow
    rest, k-steps and output tiles that end inside a group of 4 or 16 channels, one sub-path per channel of the
    second operand). None when the draw selected no path."""
    muls = [3, 5, 10, 12, 17, 20, 24, 33, 40, 48, 50, 64, 70, 100, 130]
    in1 = [(int(rng.choice(muls)), int(rng.integers(0, 4)), int(rng.choice([1, -1]))) for _ in range(rng.integers(1, 4))]
    in2 = [(int(rng.choice([1, 1, 1, 2, 3])), int(rng.integers(0, 4)), int(rng.choice([1, -1])))
           for _ in range(rng.integers(1, 4))]
    out = [(int(rng.choice(muls)), int(rng.integers(0, 4)), int(rng.choice([1, -1]))) for _ in range(rng.integers(1, 4))]
    paths = [(i1, i2, io, "uvw", True, 1.0 if rng.random() < 0.7 else float(rng.uniform(0.3, 2.0)))
             for i1, (_, l1, p1) in enumerate(in1) for i2, (_, l2, p2) in enumerate(in2)
             for io, (_, lo, po) in enumerate(out)
             if abs(l1 - l2) <= lo <= l1 + l2 and po == p1 * p2 and rng.random() < 0.85]
    if not paths:
        return None
    dt = np.float64 if rng.random() < 0.4 else np.float32
    return oeq.TPProblem(_irreps(in1), _irreps(in2), _irreps(out), paths, shared_weights=True, internal_weights=False,
                         irrep_dtype=dt, weight_dtype=dt)


@pytest.mark.parametrize("seed", range(2000, 2030))
def test_random_problem(seed):
    rng = np.random.default_rng(seed)
    problem = random_problem(rng)
    if problem is None:
        pytest.skip("the draw selected no path")
    _check_every_op(problem, rng)


@pytest.mark.parametrize("seed", range(2100, 2116))
def test_random_shared_weight_problem_on_padded_tiles(seed):
    rng = np.random.default_rng(seed)
    problem = random_shared_fully_connected_problem(rng)
    if problem is None:
        pytest.skip("the draw selected no path")
    _check_every_op(problem, rng)


def _check_every_op(problem, rng):
    from oracle.torch_ref import TorchConv, TorchTP
    dt = np.dtype(problem.irrep_dtype)
    tol = 1e-5 if dt == np.float32 else 1e-12
    ref = R.Problem.from_spec(problem)
    tp = oeq.TensorProduct(problem)
    e = ops.get_entry(tp.kid)
    B = 37
    wshape = (e.WN,) if problem.shared_weights else (B, e.WN)
    x, a = (_rand(rng, (B, e.L1), dt) for _ in range(2))
    y, b = (_rand(rng, (B, e.L2), dt) for _ in range(2))
    w, c = (_rand(rng, wshape, dt) for _ in range(2))
    g = _rand(rng, (B, e.L3), dt)
    xn, yn, wn, gn = (t.cpu().numpy() for t in (x, y, w, g))
    _compare("tp forward", [ops.tp_forward(x, y, w, tp.kid)], [R.tp_forward(ref, xn, yn, wn)], tol)
    _compare("tp backward", ops.tp_backward(x, y, w, g, tp.kid), R.tp_backward(ref, xn, yn, wn, gn), tol)
    if e.kernels().has_double_backward():
        _compare("tp second order", ops.tp_double_backward(x, y, w, g, a, b, c, tp.kid),
                 _second_order(TorchTP(ref, torch.float64), x, y, w, g, a, b, c), tol)

    coords, rows, cols, _ = periodic_radius_graph(30, 6.0, 3.0, seed=1)
    gph = CoordGraph(coords, rows, cols)
    N, E = 30, gph.nnz
    for det in ([True, False] if not problem.shared_weights else [False]):
        conv = oeq.TensorProductConv(problem, deterministic=det, kahan=bool(det and rng.random() < 0.5))
        ec = ops.get_entry(conv.kid)
        if det:
            r_, c_, p_ = gph.rows, gph.cols, gph.transpose_perm
        else:
            order = rng.permutation(E)
            r_, c_, p_ = gph.rows[order], gph.cols[order], np.zeros(0, np.int64)
        tr, tc, tpm = (torch.tensor(v, device="cuda") for v in (r_, c_, p_))
        wsh = (e.WN,) if problem.shared_weights else (E, e.WN)
        X, A = (_rand(rng, (N, e.L1), dt) for _ in range(2))
        Y, Bc = (_rand(rng, (E, e.L2), dt) for _ in range(2))
        W, C = (_rand(rng, wsh, dt) for _ in range(2))
        G = _rand(rng, (N, e.L3), dt)
        Xn, Yn, Wn, Gn = (t.cpu().numpy() for t in (X, Y, W, G))
        _compare(f"conv forward det={det}", [ops.conv_forward(X, Y, W, tr, tc, tpm, conv.kid)],
                 [R.conv_forward(ref, Xn, Yn, Wn, r_, c_)], tol)
        _compare(f"conv backward det={det}", ops.conv_backward(X, Y, W, G, tr, tc, tpm, conv.kid),
                 R.conv_backward(ref, Xn, Yn, Wn, Gn, r_, c_), tol)
        if ec.kernels().has_double_backward():
            oracle = TorchConv(ref, torch.float64)
            want = _second_order(lambda p, q, s: oracle(p, q, s, torch.tensor(r_), torch.tensor(c_)), X, Y, W, G, A, Bc, C)
            _compare(f"conv second order det={det}", ops.conv_double_backward(X, Y, W, G, A, Bc, C, tr, tc, tpm, conv.kid),
                     want, tol)


def test_weight_gradient_stores_of_partial_blocks_inside_the_path_chain():
    """A row of mixed multiplicity (5, 96, 8 channels) with a second operand too long for the weight gradients
    to wait in registers until the end of the row: their stores sit inside the chain of paths, and only the lanes
    with a channel may store. As branches these stores once made the compiler spill, from inside a block that runs
    with part of the lanes switched off, values that are used after it; dX and dY of fp32 and fp64 rows came out
    wrong (found by a random draw of the generator above). The idle lanes now store to a scratch array instead."""
    ins = [(0, 0, 0), (0, 0, 1), (1, 0, 2), (1, 0, 3), (1, 0, 4), (1, 1, 5), (1, 1, 6, 1.4141618459745515), (1, 1, 7),
           (1, 1, 8), (1, 2, 9), (1, 2, 4), (2, 0, 10), (2, 0, 11, 0.6803777663418822), (2, 0, 12), (2, 1, 13), (2, 1, 14),
           (2, 1, 15, 0.7911603214136989), (2, 1, 16), (2, 2, 10), (2, 2, 17), (2, 2, 18, 0.3223124028973989)]
    ins = [(t[0], t[1], t[2], "uvu", True, t[3] if len(t) > 3 else 1.0) for t in ins]
    out = ("5x1e+5x2e+96x0o+96x2o+96x3o+96x0e+96x1e+96x2e+96x3e+96x1o+8x0e+8x1e+8x3e+8x0o+8x1o+8x2o+8x3o+8x2e+8x3e")
    for dt in (np.float32, np.float64):
        problem = oeq.TPProblem("5x2e+96x3o+8x3e+16x0o", "3x3e+1x3o+1x3e", out, ins, shared_weights=False,
                                internal_weights=False, irrep_dtype=dt, weight_dtype=dt)
        ref = R.Problem.from_spec(problem)
        tp = oeq.TensorProduct(problem)
        e = ops.get_entry(tp.kid)
        rng = np.random.default_rng(1)
        B = 19
        x, y, w, g = (_rand(rng, (B, n), dt) for n in (e.L1, e.L2, e.WN, e.L3))
        a, b, c = (_rand(rng, (B, n), dt) for n in (e.L1, e.L2, e.WN))
        tol = 1e-5 if dt == np.float32 else 1e-12
        xn, yn, wn, gn = (t.cpu().numpy() for t in (x, y, w, g))
        _compare("backward", ops.tp_backward(x, y, w, g, tp.kid), R.tp_backward(ref, xn, yn, wn, gn), tol)
        from oracle.torch_ref import TorchTP
        _compare("second order", ops.tp_double_backward(x, y, w, g, a, b, c, tp.kid),
                 _second_order(TorchTP(ref, torch.float64), x, y, w, g, a, b, c), tol)
