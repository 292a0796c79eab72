"""GPU parity of the fused convolution against the CPU oracle (tensor product
on gathered sender rows + scatter-add), atomic and deterministic modes."""

import numpy as np
import pytest
import torch

import openequivariance_amd as oeq
from openequivariance_amd.core import problems as P
from openequivariance_amd.core.graph import CoordGraph, periodic_radius_graph
from oracle import e3nn_ref as R
from gpu_util import err, tol_of

pytestmark = pytest.mark.gpu


def _graph(n_nodes, deg, seed, punch_holes=True):
    coords, rows, cols, vec = periodic_radius_graph(n_nodes, deg, 5.0, seed)
    if punch_holes:  # node 3 fully isolated, node 5 receives nothing, edges no longer symmetric
        keep = (rows != 3) & (cols != 3) & (rows != 5)
        rows, cols = rows[keep], cols[keep]
    return coords, rows, cols


def _buffers(problem, n_nodes, E, seed):
    rng = np.random.default_rng(seed)
    dt = np.dtype(problem.irrep_dtype)
    X = rng.uniform(size=(n_nodes, problem.irreps_in1.dim)).astype(dt)
    Y = rng.uniform(size=(E, problem.irreps_in2.dim)).astype(dt)
    W = rng.uniform(size=(problem.weight_numel,) if problem.shared_weights else (E, problem.weight_numel)).astype(dt)
    G = rng.uniform(size=(n_nodes, problem.irreps_out.dim)).astype(dt)
    return X, Y, W, G


def _odd(shared):
    return oeq.TPProblem("5x1e+3x2e", "2x1e+1x0e", "5x1e+3x2e+5x0e",
                         [(0, 0, 0, "uvu", True), (0, 1, 0, "uvu", True), (1, 0, 1, "uvu", True),
                          (0, 0, 2, "uvu", True)], shared_weights=shared, internal_weights=False, label="odd-uvu")


def _ragged():
    # one row per wave, lanes without a channel in every block
    return oeq.TPProblem("40x1e+17x2e", "2x1e+1x0e", "40x1e+17x2e+40x0e",
                         [(0, 0, 0, "uvu", True), (0, 1, 0, "uvu", True), (1, 0, 1, "uvu", True),
                          (0, 0, 2, "uvu", True)], shared_weights=False, internal_weights=False, label="ragged-uvu")


def _fc(shared):
    return P.FullyConnectedTPProblem("4x0e+3x1o", "1x0e+2x1o", "5x0e+2x1o+1x2e", shared_weights=shared,
                                     internal_weights=False, label="fc-uvw")


def _as_f64(problem):
    out = problem.clone()
    out.irrep_dtype = out.weight_dtype = np.float64
    return out


CASES = [
    ("cfg1", P.config1_single_uvu, 40, 6),
    ("cfg2", P.config2_nequip_uvu, 60, 8),
    ("cfg5-f32", P.config5_mace_conv, 50, 8),
    ("cfg5-f64", lambda: P.config5_mace_conv(np.float64), 30, 6),
    ("mace-large", lambda: P.mace_problems()[0], 40, 6),
    ("odd", lambda: _odd(False), 40, 6),
    ("odd-shared", lambda: _odd(True), 40, 6),
    # 'uvw' problems: fused kernels (receiver walk forward, per-edge backward + ordered sender-side sum; shared
    # weights: partial weight-gradient rows per wave, summed in order); shared weights on the matrix cores: batch
    # kernels on gathered rows + ordered segment sum
    ("uvw", lambda: _fc(False), 40, 6),
    ("uvw-diffdock", lambda: P.diffdock_problems()[0], 40, 6),
    ("uvw-diffdock-f64", lambda: _as_f64(P.diffdock_problems()[1]), 30, 5),
    ("uvw-e3tools-conv", lambda: P.e3tools_problems()[0], 40, 6),
    ("uvw-shared", lambda: _fc(True), 40, 6),
    # (second operands of more than 64 values keep a problem off the matrix cores: the general kernels' weight
    # gradient in an LDS copy per wave, with 20 and with 70 channels, and in partial rows in global memory)
    ("uvw-shared-lds", lambda: P.FullyConnectedTPProblem(
        "20x0e+10x1o", "40x0e+10x1o", "12x0e+6x1o", shared_weights=True, internal_weights=False,
        label="uvw-shared-lds"), 40, 6),
    ("uvw-shared-lds-wide", lambda: P.FullyConnectedTPProblem(
        "70x0e+3x1o", "1x0e+1x1o+1x2e+1x3o+1x4e+1x5o+1x6e+1x7o+1x8e", "3x0e+2x1o", shared_weights=True, internal_weights=False,
        label="uvw-shared-lds-wide"), 40, 6),
    ("uvw-shared-global-f64", lambda: _as_f64(P.FullyConnectedTPProblem(
        "20x0e+10x1o", "40x0e+10x1o", "40x0e+20x1o", shared_weights=True, internal_weights=False,
        label="uvw-shared-global")), 30, 5),
    ("uvw-shared-mfma-mul2", lambda: P.FullyConnectedTPProblem(
        "40x0e+30x1o", "2x0e+1x1o", "25x0e+10x1o+5x2e", shared_weights=True, internal_weights=False,
        label="uvw-shared-mfma-mul2"), 40, 6),
    ("uvw-shared-mfma-padded", lambda: P.FullyConnectedTPProblem(
        "40x0e+30x1o", "1x0e+1x1o", "50x0e+20x1o+10x2e", shared_weights=True, internal_weights=False,
        label="uvw-shared-mfma-padded"), 40, 6),
    ("uvw-shared-tetris", lambda: P.tetris_poly_problems()[0], 40, 6),
    ("uvw-cfg4-mfma", P.config4_uvw_shared, 30, 5),
    # output gradient too large for one wave: forward shares the output segments, backward the output
    # blocks, between several waves of a node (64 channels: one chunk; 128: two)
    # an irrep block of 2048 channels: two pieces of 1024, sixteen chunk waves per node
    ("uvu-2048", lambda: oeq.TPProblem("2048x1o", "1x1o", "2048x0e+2048x2e",
                                       [(0, 0, 0, "uvu", True), (0, 0, 1, "uvu", True)], shared_weights=False,
                                       internal_weights=False, label="uvu-2048"), 24, 4),
    ("nequip-benzene", lambda: P.nequip_problems()[3], 30, 5),
    ("benzene-128", lambda: P.ChannelwiseTPP(
        "128x0o + 128x0e + 128x1o + 128x1e + 128x2o + 128x2e + 128x3o + 128x3e", "0e + 1o + 2e + 3o",
        "128x0o + 128x0e + 128x1o + 128x1e + 128x2o + 128x2e + 128x3o + 128x3e", "benzene-128"), 24, 4),
    # the backward kernel that shares a node between waves, with a single owner (135 gradient words: more than the
    # ordinary kernel keeps in registers, few enough for one wave), with two (SevenNet main layer) and with four
    # (benzene above); and the forward kernel regenerated with one wave per node because its shared form spills
    ("one-owner", lambda: P.ChannelwiseTPP("64x0e+64x1o+64x2e+64x3o", "0e+1o+2e+3o", "0e+1o+2e+3o+4e", "one-owner"), 30, 5),
    ("one-owner-128", lambda: P.ChannelwiseTPP("128x0e+128x1o+128x2e+128x3o", "0e+1o+2e+3o", "0e+1o+2e+3o+4e",
                                               "one-owner-128"), 24, 4),
    ("sevennet-main", lambda: P.seven_net_problems()[1], 30, 5),
    ("four-irreps-even", lambda: P.ChannelwiseTPP("64x0e+64x1e+64x2e+64x3e", "1x0e+1x1e+1x2e+1x3e", "0e+1e+2e+3e",
                                                  "four-irreps-even"), 30, 5),
    # eight waves share a node in the backward kernel: no smaller count brings a wave's share under the register limit
    ("benzene-f64", lambda: _as_f64(P.nequip_problems()[3]), 24, 4),
    # the forward kernel held to a third of a SIMD's registers (it fits them without scratch memory)
    ("96-channels", lambda: P.ChannelwiseTPP("96x0e+96x1o+96x2e+96x3o", "1x0e+1x1o+1x2e+1x3o", "0e+1o+2e+3o",
                                             "96-channels"), 30, 5),
]


@pytest.mark.parametrize("name,make,n_nodes,deg", CASES, ids=[c[0] for c in CASES])
def test_conv_matches_oracle(name, make, n_nodes, deg):
    problem = make()
    tol = tol_of(problem)
    coords, rows, cols = _graph(n_nodes, deg, seed=0)
    E = len(rows)
    X, Y, W, G = _buffers(problem, n_nodes, E, seed=12345)
    ref = R.Problem.from_spec(problem)
    z_ref = R.conv_forward(ref, X, Y, W, rows, cols)
    dx_ref, dy_ref, dw_ref = R.conv_backward(ref, X, Y, W, G, rows, cols)
    assert np.all(z_ref[3] == 0) and np.all(z_ref[5] == 0) and np.all(dx_ref[3] == 0)
    rng = np.random.default_rng(1)
    modes = [False] if problem.shared_weights else [False, True]
    for det in modes:
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
        tr, tc = torch.tensor(r_, device="cuda"), torch.tensor(c_, device="cuda")
        tp = torch.tensor(perm, device="cuda") if perm is not None else None
        z = conv(tX, tY, tW, tr, tc, tp)
        assert err(z, z_ref) <= tol, (name, det)
        z.backward(torch.tensor(G, device="cuda"))
        assert err(tX.grad, dx_ref) <= tol, (name, det)
        assert err(tY.grad, dy_ref[order]) <= tol, (name, det)
        assert err(tW.grad, dw_ref if problem.shared_weights else dw_ref[order]) <= tol, (name, det)


def test_uvw_fused_matches_unfused(monkeypatch):
    """'uvw' with per-edge weights runs as fused kernels; the unfused path (gathered rows, batch kernels,
    segment sums) stays selectable. Both agree, in both modes, and the fused deterministic mode gives the
    same bits on every run."""
    from openequivariance_amd._torch import ops
    problem = P.diffdock_problems()[0]
    coords, rows, cols = _graph(200, 10, seed=4)
    g = CoordGraph(coords, rows, cols)
    E = g.nnz
    gen = torch.Generator(device="cuda").manual_seed(3)
    X = torch.randn(200, problem.irreps_in1.dim, device="cuda", generator=gen)
    Y = torch.randn(E, problem.irreps_in2.dim, device="cuda", generator=gen)
    W = torch.randn(E, problem.weight_numel, device="cuda", generator=gen)
    G = torch.randn(200, problem.irreps_out.dim, device="cuda", generator=gen)
    tr, tc, tp = (torch.tensor(a, device="cuda") for a in (g.rows, g.cols, g.transpose_perm))
    out = {}
    for fuse in (1, 0):
        monkeypatch.setenv("OEQ_AMD_TUNE", f"conv_fuse_uvw={fuse}")
        for det in (True, False):
            conv = oeq.TensorProductConv(problem, deterministic=det)
            e = ops.get_entry(conv.kid)
            assert e.unfused == (fuse == 0)
            runs = []
            for _ in range(3):
                z = ops.conv_forward(X, Y, W, tr, tc, tp, conv.kid)
                runs.append((z,) + tuple(ops.conv_backward(X, Y, W, G, tr, tc, tp, conv.kid)))
            for later in runs[1:]:
                for a, b in zip(runs[0], later):
                    assert torch.equal(a, b), (fuse, det)
            out[(fuse, det)] = runs[0]
    for det in (True, False):
        for a, b in zip(out[(1, det)], out[(0, det)]):
            assert (a - b).abs().max() <= 2e-6 * b.abs().max(), det
    # the grouped mode orders a node's edges by edge id, which is the order of the sorted list here
    for a, b in zip(out[(1, True)], out[(1, False)]):
        assert torch.equal(a, b)


def test_uvw_shared_weights_fused_matches_unfused(monkeypatch):
    """Shared weights outside the matrix-core path: the fused kernels against the unfused composition, same
    bits on every run (the partial weight-gradient rows are summed in a fixed order), at a graph large enough
    for every wave of the bounded backward grid to see edges and at one where most waves see none."""
    from openequivariance_amd._torch import ops
    problem = P.FullyConnectedTPProblem("20x0e+10x1o", "40x0e+10x1o", "12x0e+6x1o", shared_weights=True,
                                        internal_weights=False, label="uvw-shared-lds")
    for n_nodes, deg in ((3000, 12), (20, 3)):
        coords, rows, cols = _graph(n_nodes, deg, seed=4)
        E = len(rows)
        gen = torch.Generator(device="cuda").manual_seed(3)
        X = torch.randn(n_nodes, problem.irreps_in1.dim, device="cuda", generator=gen)
        Y = torch.randn(E, problem.irreps_in2.dim, device="cuda", generator=gen)
        W = torch.randn(problem.weight_numel, device="cuda", generator=gen)
        G = torch.randn(n_nodes, problem.irreps_out.dim, device="cuda", generator=gen)
        order = np.random.default_rng(n_nodes).permutation(E)
        tr, tc = (torch.tensor(a[order], device="cuda") for a in (rows, cols))
        none = torch.zeros(0, dtype=torch.int64, device="cuda")
        out = {}
        for fuse in (1, 0):
            monkeypatch.setenv("OEQ_AMD_TUNE", f"conv_fuse_uvw={fuse}")
            conv = oeq.TensorProductConv(problem, deterministic=False)
            e = ops.get_entry(conv.kid)
            assert e.unfused == (fuse == 0)
            runs = []
            for _ in range(3):
                z = ops.conv_forward(X, Y, W, tr, tc, none, conv.kid)
                runs.append((z,) + tuple(ops.conv_backward(X, Y, W, G, tr, tc, none, conv.kid)))
            for later in runs[1:]:
                for a, b in zip(runs[0], later):
                    assert torch.equal(a, b), fuse
            out[fuse] = runs[0]
        for a, b in zip(out[1], out[0]):
            assert (a - b).abs().max() <= 4e-6 * b.abs().max(), n_nodes


SHARED_SINGLE_CHANNEL = ["uvw-cfg4-mfma", "uvw-shared-mfma-padded", "uvw-shared-tetris"]


@pytest.mark.parametrize("name", SHARED_SINGLE_CHANNEL)
def test_shared_weight_uvw_runs_factored(name, monkeypatch):
    """One weight tensor for all edges and single-channel second operands: the sum over a receiver's edges
    commutes with the channel mix, so the convolution runs as the fused 'uvu' convolution of the contraction
    followed by one mix per node (core/problems.py: factor_shared_uvw): no gathered [E, L1] rows, no [E, L3]
    messages. Same results as the routes that mix per edge (matrix-core batch kernels on gathered rows, fused
    general kernels), first and second order; problems with several channels in the second operand keep
    those routes."""
    from openequivariance_amd._torch import ops
    make = next(c[1] for c in CASES if c[0] == name)
    problem = make()
    coords, rows, cols = _graph(300, 8, seed=12)
    E = len(rows)
    order = np.random.default_rng(2).permutation(E)
    tr, tc = (torch.tensor(a[order], device="cuda") for a in (rows, cols))
    none = torch.zeros(0, dtype=torch.int64, device="cuda")
    gen = torch.Generator(device="cuda").manual_seed(3)
    X, A = (torch.randn(300, problem.irreps_in1.dim, device="cuda", generator=gen) for _ in range(2))
    Y, B = (torch.randn(E, problem.irreps_in2.dim, device="cuda", generator=gen) for _ in range(2))
    W, C = (torch.randn(problem.weight_numel, device="cuda", generator=gen) for _ in range(2))
    G = torch.randn(300, problem.irreps_out.dim, device="cuda", generator=gen)
    out = {}
    for knobs in ("conv_factor=1", "conv_factor=0,conv_mfma_min_weights=0", "conv_factor=0,conv_mfma_min_weights=100000000"):
        monkeypatch.setenv("OEQ_AMD_TUNE", knobs)
        conv = oeq.TensorProductConv(problem, deterministic=False)
        e = ops.get_entry(conv.kid)
        assert bool(e.factored) == (knobs == "conv_factor=1") and not (e.factored and e.unfused)
        out[knobs] = (ops.conv_forward(X, Y, W, tr, tc, none, conv.kid),) + \
            tuple(ops.conv_backward(X, Y, W, G, tr, tc, none, conv.kid)) + \
            tuple(ops.conv_double_backward(X, Y, W, G, A, B, C, tr, tc, none, conv.kid))
    ref = out["conv_factor=1"]
    for knobs, got in out.items():
        for a, b in zip(got, ref):
            assert float((a - b).abs().max() / b.abs().max()) <= 2e-5, knobs
    # several channels in the second operand: not of this shape
    monkeypatch.setenv("OEQ_AMD_TUNE", "")
    multi = next(c[1] for c in CASES if c[0] == "uvw-shared-mfma-mul2")()
    assert ops.get_entry(oeq.TensorProductConv(multi, deterministic=False).kid).factored is None


def test_reference_toy_graph():
    """The 3-node / 4-edge graph of the reference's tutorial
    (tests/example_test.py:46-82): atomic and deterministic calls agree with the
    oracle; sender_perm is the argsort by sender of the receiver-sorted edges."""
    problem = P.config1_single_uvu()
    rows = np.array([0, 1, 1, 2])
    cols = np.array([1, 0, 2, 1])
    rng = np.random.default_rng(0)
    X, Y, W = (rng.uniform(size=s).astype(np.float32) for s in ((3, 5), (4, 7), (4, 1)))
    z_ref = R.conv_forward(R.Problem.from_spec(problem), X, Y, W, rows, cols)
    tX, tY, tW = (torch.tensor(a, device="cuda") for a in (X, Y, W))
    tr, tc = torch.tensor(rows, device="cuda"), torch.tensor(cols, device="cuda")
    z = oeq.TensorProductConv(problem, deterministic=False).forward(tX, tY, tW, tr, tc)
    assert err(z, z_ref) <= 1e-5
    sender_perm = torch.argsort(tc, stable=True)
    z = oeq.TensorProductConv(problem, deterministic=True).forward(tX, tY, tW, tr, tc, sender_perm)
    assert err(z, z_ref) <= 1e-5


def test_deterministic_mode_is_bitwise_reproducible():
    problem = P.config5_mace_conv()
    coords, rows, cols = _graph(300, 16, seed=2, punch_holes=False)
    g = CoordGraph(coords, rows, cols)
    E = g.nnz
    gen = torch.Generator(device="cuda").manual_seed(0)
    X = torch.randn(300, 2048, device="cuda", generator=gen, requires_grad=True)
    Y = torch.randn(E, 16, device="cuda", generator=gen, requires_grad=True)
    W = torch.randn(E, 2944, device="cuda", generator=gen, requires_grad=True)
    G = torch.randn(300, 12672, device="cuda", generator=gen)
    tr, tc, tp = (torch.tensor(a, device="cuda") for a in (g.rows, g.cols, g.transpose_perm))
    conv = oeq.TensorProductConv(problem, deterministic=True)
    results = []
    for _ in range(5):
        for t in (X, Y, W):
            t.grad = None
        z = conv(X, Y, W, tr, tc, tp)
        z.backward(G)
        results.append((z.detach().clone(), X.grad.clone(), Y.grad.clone(), W.grad.clone()))
        torch.randn(1 << 22, device="cuda")  # unrelated work between runs
    for other in results[1:]:
        for a, b in zip(results[0], other):
            assert torch.equal(a, b)
    # deterministic=False on the same (sorted) list groups the edges in the same order: same bits; on a
    # shuffled list the output and the per-edge gradients are again the same bits from run to run (fixed
    # summation order), the sender gradient is accumulated with float atomics and agrees to tolerance
    conv_a = oeq.TensorProductConv(problem, deterministic=False)
    za = conv_a(X, Y, W, tr, tc)
    assert torch.equal(za, results[0][0])
    shuffle = torch.randperm(E, device="cuda", generator=gen)
    Ys, Ws, rs, cs = (t.detach()[shuffle].contiguous() for t in (Y, W, tr, tc))
    Xd = X.detach()
    runs = []
    for _ in range(4):
        Xr, Yr, Wr = (t.clone().requires_grad_(True) for t in (Xd, Ys, Ws))
        zs = conv_a(Xr, Yr, Wr, rs, cs)
        zs.backward(G)
        runs.append((zs.detach().clone(), Xr.grad.clone(), Yr.grad.clone(), Wr.grad.clone()))
        torch.randn(1 << 22, device="cuda")
    for other in runs[1:]:
        for n, (a, b) in enumerate(zip(runs[0], other)):
            if n == 1:
                assert (a - b).abs().max() / a.abs().max() <= 1e-5
            else:
                assert torch.equal(a, b)
    assert (runs[0][1] - results[0][1]).abs().max() / results[0][1].abs().max() <= 1e-5
    scale = results[0][0].abs().max()
    assert (runs[0][0] - results[0][0]).abs().max() / scale <= 1e-5


def test_no_edges_and_no_nodes():
    problem = P.config1_single_uvu()
    for det in (False, True):
        conv = oeq.TensorProductConv(problem, deterministic=det)
        e = torch.zeros(0, dtype=torch.int64, device="cuda")
        X = torch.rand(4, 5, device="cuda", requires_grad=True)
        Y = torch.rand(0, 7, device="cuda", requires_grad=True)
        W = torch.rand(0, 1, device="cuda", requires_grad=True)
        z = conv(X, Y, W, e, e, e if det else None)
        assert z.shape == (4, 5) and torch.count_nonzero(z) == 0
        z.backward(torch.ones_like(z))
        assert torch.count_nonzero(X.grad) == 0


def test_star_graph_closed_form():
    """All edges into node 0: Z[0] is the plain sum of the per-edge products."""
    problem = P.config2_nequip_uvu()
    n, E = 9, 8
    rows = np.zeros(E, dtype=np.int64)
    cols = np.arange(1, n, dtype=np.int64)
    X, Y, W, _ = _buffers(problem, n, E, seed=4)
    tp = oeq.TensorProduct(problem)
    msgs = tp(torch.tensor(X[cols], device="cuda"), torch.tensor(Y, device="cuda"), torch.tensor(W, device="cuda"))
    conv = oeq.TensorProductConv(problem, deterministic=True)
    tr, tc = torch.tensor(rows, device="cuda"), torch.tensor(cols, device="cuda")
    z = conv(torch.tensor(X, device="cuda"), torch.tensor(Y, device="cuda"), torch.tensor(W, device="cuda"), tr, tc,
             torch.arange(E, device="cuda"))
    assert torch.count_nonzero(z[1:]) == 0
    assert (z[0] - msgs.double().sum(0).float()).abs().max() / z[0].abs().max() <= 1e-5


def test_conv_input_validation():
    problem = P.config1_single_uvu()
    conv = oeq.TensorProductConv(problem, deterministic=True)
    X, Y, W = torch.rand(3, 5, device="cuda"), torch.rand(4, 7, device="cuda"), torch.rand(4, 1, device="cuda")
    rows = torch.tensor([0, 1, 1, 2], device="cuda")
    cols = torch.tensor([1, 0, 2, 1], device="cuda")
    perm = torch.argsort(cols, stable=True)
    conv(X, Y, W, rows, cols, perm)
    with pytest.raises(RuntimeError, match="Shape mismatch"):
        conv(X, Y[:3], W, rows, cols, perm)
    with pytest.raises(RuntimeError, match="Shape mismatch"):
        conv(X, Y, W, rows, cols, perm[:2])
    with pytest.raises(RuntimeError, match="Dtype mismatch"):
        conv(X, Y, W, rows.int(), cols, perm)
    with pytest.raises(RuntimeError, match="is not on the GPU"):
        conv(X, Y, W, rows.cpu(), cols, perm)


def test_edge_list_validation(monkeypatch):
    """With the edge-list check switched on, a corrupt list is reported before any kernel is launched; with it
    off (the default, as in the reference) the kernels force every index into range, so the same lists give
    meaningless but finite-sized work and no access outside the operands."""
    from openequivariance_amd._torch import ops
    problem = P.config1_single_uvu()
    X, Y, W = torch.rand(3, 5, device="cuda"), torch.rand(4, 7, device="cuda"), torch.rand(4, 1, device="cuda")
    rows = torch.tensor([0, 1, 1, 2], device="cuda")
    cols = torch.tensor([1, 0, 2, 1], device="cuda")
    perm = torch.argsort(cols, stable=True)
    det = oeq.TensorProductConv(problem, deterministic=True)
    grp = oeq.TensorProductConv(problem, deterministic=False)
    bad_lists = [
        ("out of range in tensor 'cols'", det, rows, torch.tensor([1, 0, 3, 1], device="cuda"), perm),
        ("out of range in tensor 'rows'", grp, torch.tensor([0, -1, 1, 2], device="cuda"), cols, None),
        ("'rows' is not sorted", det, torch.tensor([1, 0, 1, 2], device="cuda"), cols, perm),
        ("not a permutation", det, rows, cols, torch.tensor([1, 1, 3, 2], device="cuda")),
        ("not a permutation", det, rows, cols, torch.tensor([1, 0, 4, 2], device="cuda")),
        ("does not list the edges by sender", det, rows, cols, torch.tensor([0, 1, 2, 3], device="cuda")),
    ]
    monkeypatch.setattr(ops, "CHECK_INDICES", True)
    det(X, Y, W, rows, cols, perm)
    grp(X, Y, W, rows, cols)
    for msg, conv, r, c, p in bad_lists:
        with pytest.raises(RuntimeError, match=msg):
            conv(X, Y, W, r, c, p)
    monkeypatch.setattr(ops, "CHECK_INDICES", False)
    monkeypatch.setenv("OEQ_AMD_CHECK_INDICES", "1")
    with pytest.raises(RuntimeError, match="out of range"):
        grp(X, Y, W, rows, torch.tensor([1, 0, 2, 7], device="cuda"))
    monkeypatch.setenv("OEQ_AMD_CHECK_INDICES", "0")
    # unchecked: indices are forced into range on the device; the calls complete and touch only their operands
    guard = torch.full((64,), 7.0, device="cuda")
    for msg, conv, r, c, p in bad_lists:
        Xg, Yg, Wg = (t.clone().requires_grad_(True) for t in (X, Y, W))
        z = conv(Xg, Yg, Wg, r, c, p)
        z.sum().backward()
        torch.cuda.synchronize()
        assert z.shape == (3, 5) and Xg.grad.shape == (3, 5)
    assert bool((guard == 7.0).all())


def test_conv_double_backward_runs():
    problem = P.config1_single_uvu(np.float64)
    conv = oeq.TensorProductConv(problem, deterministic=True)
    rows = torch.tensor([0, 1, 1, 2], device="cuda")
    cols = torch.tensor([1, 0, 2, 1], device="cuda")
    perm = torch.argsort(cols, stable=True)
    X = torch.rand(3, 5, device="cuda", dtype=torch.float64, requires_grad=True)
    Y = torch.rand(4, 7, device="cuda", dtype=torch.float64, requires_grad=True)
    W = torch.rand(4, 1, device="cuda", dtype=torch.float64, requires_grad=True)
    assert torch.autograd.gradcheck(lambda a, b, c: conv(a, b, c, rows, cols, perm), (X, Y, W), eps=1e-6, atol=1e-6)
    assert torch.autograd.gradgradcheck(lambda a, b, c: conv(a, b, c, rows, cols, perm), (X, Y, W), eps=1e-6,
                                        atol=1e-6)


def _hub_graph(k):
    """Node 0 receives from, and sends to, each of the nodes 1..k."""
    spokes = np.arange(1, k + 1, dtype=np.int64)
    rows = np.concatenate([np.zeros(k, dtype=np.int64), spokes])
    cols = np.concatenate([spokes, np.zeros(k, dtype=np.int64)])
    return CoordGraph(np.zeros((k + 1, 3)), rows, cols)


KAHAN = [
    ("cfg1", P.config1_single_uvu),
    ("cfg2", P.config2_nequip_uvu),
    ("mace-medium", lambda: P.mace_problems()[1]),
    ("uvw", lambda: _fc(False)),
]


@pytest.mark.parametrize("name,make", KAHAN, ids=[c[0] for c in KAHAN])
def test_kahan_summation(name, make):
    """kahan=True gives the same result within tolerance, and on a node with thousands of
    same-sign terms its fp32 sums (Z of the hub in forward, dX of the hub in backward) are
    markedly closer to the float64 oracle than plain summation."""
    problem = make()
    k = 3000
    g = _hub_graph(k)
    n, E = k + 1, 2 * k
    X, Y, W, G = _buffers(problem, n, E, seed=9)
    ref = R.Problem.from_spec(problem)
    z_ref = R.conv_forward(ref, X, Y, W, g.rows, g.cols)
    dx_ref, dy_ref, dw_ref = R.conv_backward(ref, X, Y, W, G, g.rows, g.cols)
    tr, tc, tp = (torch.tensor(a, device="cuda") for a in (g.rows, g.cols, g.transpose_perm))
    hub_err = {}
    for kahan in (False, True):
        conv = oeq.TensorProductConv(problem, deterministic=True, kahan=kahan)
        tX = torch.tensor(X, device="cuda", requires_grad=True)
        tY = torch.tensor(Y, device="cuda", requires_grad=True)
        tW = torch.tensor(W, device="cuda", requires_grad=True)
        z = conv(tX, tY, tW, tr, tc, tp)
        z.backward(torch.tensor(G, device="cuda"))
        assert err(z, z_ref) <= 1e-5 and err(tX.grad, dx_ref) <= 1e-5
        assert err(tY.grad, dy_ref) <= 1e-5 and err(tW.grad, dw_ref) <= 1e-5
        hub_err[kahan] = (err(z[0], z_ref[0]), err(tX.grad[0], dx_ref[0]))
    # uncompensated fp32 sums of 3000 terms lose a few bits; the compensated ones stay at rounding level
    assert hub_err[True][0] <= 2e-7 and hub_err[True][1] <= 2e-7, hub_err
    print(name, hub_err)
    for plain, comp in zip(hub_err[False], hub_err[True]):
        # narrow problems pack many rows per wave, which already splits the sum into short partial sums,
        # and so does the chunked walk of a long segment in the uncompensated forward
        assert comp <= max(plain, 1e-7) and (plain <= 1.5e-7 or comp < 0.5 * plain), hub_err


@pytest.mark.parametrize("name,make", [("cfg2", P.config2_nequip_uvu), ("cfg5-f32", P.config5_mace_conv),
                                       ("odd-shared", lambda: _odd(True))], ids=["cfg2", "cfg5-f32", "odd-shared"])
def test_float_atomic_kernels(name, make, monkeypatch):
    """deterministic=False normally groups the edges on the device and walks them per node; the
    kernels that walk edge ranges and flush with float atomics stay selectable and must agree."""
    monkeypatch.setenv("OEQ_AMD_TUNE", "conv_sort=0")
    problem = make()
    tol = tol_of(problem)
    coords, rows, cols = _graph(40, 6, seed=2)
    E = len(rows)
    X, Y, W, G = _buffers(problem, 40, E, seed=77)
    ref = R.Problem.from_spec(problem)
    z_ref = R.conv_forward(ref, X, Y, W, rows, cols)
    dx_ref, dy_ref, dw_ref = R.conv_backward(ref, X, Y, W, G, rows, cols)
    conv = oeq.TensorProductConv(problem, deterministic=False)
    from openequivariance_amd import runtime as rt
    from openequivariance_amd._torch import ops
    assert ops.get_entry(conv.kid).kernels().dims["deterministic"] == rt.CONV_ATOMIC
    tX, tY, tW = (torch.tensor(a, device="cuda", requires_grad=True) for a in (X, Y, W))
    z = conv(tX, tY, tW, torch.tensor(rows, device="cuda"), torch.tensor(cols, device="cuda"))
    z.backward(torch.tensor(G, device="cuda"))
    for got, want in ((z, z_ref), (tX.grad, dx_ref), (tY.grad, dy_ref), (tW.grad, dw_ref)):
        assert err(got, want) <= tol


def test_float_atomic_kernels_on_a_larger_graph(monkeypatch):
    """The float-atomics kernels (edge ranges per wave, flush with atomics at every change of receiver) on
    2 400 nodes and about 19 000 shuffled edges: many ranges per receiver and many receivers per range."""
    monkeypatch.setenv("OEQ_AMD_TUNE", "conv_sort=0")
    problem = P.config2_nequip_uvu()
    n = 2400
    coords, rows, cols = _graph(n, 8, seed=8)
    order = np.random.default_rng(4).permutation(len(rows))
    rows, cols = rows[order], cols[order]
    E = len(rows)
    X, Y, W, G = _buffers(problem, n, E, seed=78)
    ref = R.Problem.from_spec(problem)
    z_ref = R.conv_forward(ref, X, Y, W, rows, cols)
    dx_ref, dy_ref, dw_ref = R.conv_backward(ref, X, Y, W, G, rows, cols)
    conv = oeq.TensorProductConv(problem, deterministic=False)
    from openequivariance_amd import runtime as rt
    from openequivariance_amd._torch import ops
    assert ops.get_entry(conv.kid).kernels().dims["deterministic"] == rt.CONV_ATOMIC
    tX, tY, tW = (torch.tensor(a, device="cuda", requires_grad=True) for a in (X, Y, W))
    z = conv(tX, tY, tW, torch.tensor(rows, device="cuda"), torch.tensor(cols, device="cuda"))
    z.backward(torch.tensor(G, device="cuda"))
    for got, want in ((z, z_ref), (tX.grad, dx_ref), (tY.grad, dy_ref), (tW.grad, dw_ref)):
        assert err(got, want) <= 1e-5


def test_shared_weight_gradient_bits_do_not_depend_on_the_index_build():
    """Shared weights: every wave group of the (bounded) backward grid sums the weight gradient over the nodes
    it visits, so the walk order has to be a function of the edge list: the same bits from three index
    builds, on a graph with more nodes than the grid has wave groups."""
    from openequivariance_amd._torch import ops
    problem = _odd(True)
    n = 9000
    coords, rows, cols = _graph(n, 6, seed=10)
    order = np.random.default_rng(6).permutation(len(rows))
    rows, cols = rows[order], cols[order]
    E = len(rows)
    X, Y, W, G = _buffers(problem, n, E, seed=79)
    conv = oeq.TensorProductConv(problem, deterministic=False)
    tX, tY, tW, tG = (torch.tensor(a, device="cuda") for a in (X, Y, W, G))
    tr, tc = torch.tensor(rows, device="cuda"), torch.tensor(cols, device="cuda")
    dummy = torch.zeros(1, dtype=torch.int64, device="cuda")
    ks = ops.get_entry(conv.kid).kernels()
    assert ks.dims["order_hops"] > 0 and ks.dims["wpartial_per_block"] > 0
    ops.clear_index_cache()
    first = ops.conv_backward(tX, tY, tW, tG, tr, tc, dummy, conv.kid)
    _, _, dw_ref = R.conv_backward(R.Problem.from_spec(problem), X, Y, W, G, rows, cols)
    assert err(first[2], dw_ref) <= 1e-5
    for _ in range(3):
        ops.clear_index_cache()
        torch.randn(1 << 22, device="cuda")
        again = ops.conv_backward(tX, tY, tW, tG, tr, tc, dummy, conv.kid)
        assert torch.equal(again[2], first[2]) and torch.equal(again[1], first[1])


def test_grouped_mode_handles_hubs_and_many_nodes():
    """The device-side grouping (histogram, one-block scan, scatter) over more nodes than one scan
    sweep covers, with isolated nodes and one hub that receives from and sends to 5000 nodes."""
    problem = P.config1_single_uvu()
    n = 20000
    rng = np.random.default_rng(3)
    hub = np.arange(1, 5001, dtype=np.int64)
    rows = np.concatenate([np.zeros(5000, dtype=np.int64), hub, rng.integers(6000, n, size=30000)])
    cols = np.concatenate([hub, np.zeros(5000, dtype=np.int64), rng.integers(6000, n, size=30000)])
    order = rng.permutation(len(rows))
    rows, cols = rows[order], cols[order]
    E = len(rows)
    X, Y, W, G = _buffers(problem, n, E, seed=5)
    ref = R.Problem.from_spec(problem)
    z_ref = R.conv_forward(ref, X, Y, W, rows, cols)
    dx_ref, dy_ref, dw_ref = R.conv_backward(ref, X, Y, W, G, rows, cols)
    conv = oeq.TensorProductConv(problem, deterministic=False)
    tX, tY, tW = (torch.tensor(a, device="cuda", requires_grad=True) for a in (X, Y, W))
    z = conv(tX, tY, tW, torch.tensor(rows, device="cuda"), torch.tensor(cols, device="cuda"))
    z.backward(torch.tensor(G, device="cuda"))
    for got, want in ((z, z_ref), (tX.grad, dx_ref), (tY.grad, dy_ref), (tW.grad, dw_ref)):
        assert err(got, want) <= 1e-5


@pytest.mark.parametrize("hubs,degree", [(3, 2100), (130, 2060)], ids=["listed", "more-than-the-list-holds"])
def test_grouping_orders_long_segments(hubs, degree):
    """Receivers with more than 2048 edges are ranked by the whole grid instead of one wave (up to 126 of them;
    beyond that the waves take them again). Either way the grouping is the ascending one: on a list that is
    already sorted, deterministic=False sums in the order of the sorted list and gives the bits of
    deterministic=True; on a shuffled list the output keeps the same bits from run to run."""
    problem = P.config1_single_uvu()
    rng = np.random.default_rng(hubs)
    n = hubs + 500
    rows = np.concatenate([np.repeat(np.arange(hubs, dtype=np.int64), degree), rng.integers(hubs, n, size=4000)])
    cols = rng.integers(0, n, size=len(rows))
    order = np.lexsort((cols, rows))
    rows, cols = rows[order], cols[order]
    E = len(rows)
    X, Y, W, G = _buffers(problem, n, E, seed=hubs)
    z_ref = R.conv_forward(R.Problem.from_spec(problem), X, Y, W, rows, cols)
    tX, tY, tW, tr, tc = (torch.tensor(a, device="cuda") for a in (X, Y, W, rows, cols))
    # the sender of the reverse edge need not exist for a forward call: any permutation serves
    z_sorted = oeq.TensorProductConv(problem, deterministic=True)(tX, tY, tW, tr, tc, torch.arange(E, device="cuda"))
    conv = oeq.TensorProductConv(problem, deterministic=False)
    z = conv(tX, tY, tW, tr, tc)
    assert err(z, z_ref) <= 1e-5
    assert torch.equal(z, z_sorted)
    shuffle = torch.tensor(rng.permutation(E), device="cuda")
    Ys, Ws, rs, cs = (t[shuffle].contiguous() for t in (tY, tW, tr, tc))
    first = conv(tX, Ys, Ws, rs, cs)
    assert err(first, z_ref) <= 1e-5
    for _ in range(3):
        torch.randn(1 << 22, device="cuda")
        assert torch.equal(conv(tX, Ys, Ws, rs, cs), first)


KNOBS = ["conv_pipe_f=0,conv_pipe_b=1", "conv_pipe_f=1,conv_pipe_b=2", "conv_pipe_f=3,conv_pipe_b=3",
         "conv_pipe_f=4,conv_pipe_b=4", "conv_pipe_f=4,conv_q=1",  # weights two edges ahead (forward)
         "conv_xcd=1,conv_gres=0", "conv_nt=0,conv_acc=48", "conv_sort=0,conv_tra=0", "conv_sort=0,conv_pipe_f=3,conv_nt=0",
         "conv_wf=0,conv_wb=0,conv_gf=1,conv_gb=1",
         # sender gradients: ordered reduction / float atomics / arrival counting; walk order off, 1 and 3 hops;
         # wave-shared product table forward only, backward only and in both directions; lanes without a
         # channel zeroed after each load
         "conv_dxm=0,conv_hops=0,conv_q=1", "conv_dxm=1,conv_hops=1", "conv_dxm=2,conv_hops=3,conv_q=3",
         "conv_q=2,conv_qaf=16,conv_qab=200,conv_qpin=0", "tp_mask=1",
         # edge segments cut into chunks of 2 / 3 edges (every node of these graphs has extra walk positions),
         # and never
         "conv_hub=2", "conv_hub=3,conv_xcd=1,conv_hops=0", "conv_hub=0",
         # sender gradients by a second walk over the senders' edges (forward kernel of the adjoint problem), whole
         # segments and chunks of 2; and never
         "conv_dxs=1", "conv_dxs=1,conv_hub=2,conv_hops=1", "conv_dxs=0",
         # ... that kernel with a third wave per SIMD where its registers allow, and held to it
         "conv_dxs=1,conv_wx=23", "conv_dxs=1,conv_wx=3",
         # a node's output gradient shared between that many waves in the backward kernel (1: a single owner)
         "conv_ngrp=1", "conv_ngrp=2,conv_hub=2", "conv_ngrp=3", "conv_ngrp=4,conv_hub=3",
         # ... whose summed sender gradient leaves as float atomics (deterministic=False; the sorted mode ignores it)
         "conv_ngrp=2,conv_dxm=1"]


@pytest.mark.parametrize("knobs", KNOBS)
def test_kernel_shape_knobs_keep_results(knobs, monkeypatch):
    """Every alternative the OEQ_AMD_TUNE switches select (edge-loop pipelining variants, LDS staging,
    XCD remap, register residency, streaming hints, output segmentation, float-atomics kernels with and
    without the LDS transpose) computes the same convolution."""
    monkeypatch.setenv("OEQ_AMD_TUNE", knobs)
    # (a problem with lanes without a channel as well: the arrival-counting variant must step aside there)
    for make in (P.config5_mace_conv, P.config2_nequip_uvu, _ragged):
        problem = make()
        coords, rows, cols = _graph(36, 6, seed=4)
        E = len(rows)
        X, Y, W, G = _buffers(problem, 36, E, seed=21)
        ref = R.Problem.from_spec(problem)
        z_ref = R.conv_forward(ref, X, Y, W, rows, cols)
        dx_ref, dy_ref, dw_ref = R.conv_backward(ref, X, Y, W, G, rows, cols)
        g = CoordGraph(coords, rows, cols)
        for det in (True, False):
            conv = oeq.TensorProductConv(problem, deterministic=det)
            tX = torch.tensor(X, device="cuda", requires_grad=True)
            tY = torch.tensor(Y[g.order], device="cuda", requires_grad=True)
            tW = torch.tensor(W[g.order], device="cuda", requires_grad=True)
            perm = torch.tensor(g.transpose_perm, device="cuda") if det else None
            z = conv(tX, tY, tW, torch.tensor(g.rows, device="cuda"), torch.tensor(g.cols, device="cuda"), perm)
            z.backward(torch.tensor(G, device="cuda"))
            assert err(z, z_ref) <= 1e-5, (knobs, det)
            assert err(tX.grad, dx_ref) <= 1e-5, (knobs, det)
            assert err(tY.grad.cpu().numpy(), dy_ref[g.order]) <= 1e-5, (knobs, det)
            assert err(tW.grad.cpu().numpy(), dw_ref[g.order]) <= 1e-5, (knobs, det)


def test_sender_gradient_modes():
    """The three ways the receiver walk hands the per-edge sender-gradient terms on (oeq_dx_mode): the
    ordered reduction by a second kernel and the in-kernel reduction by the last arrival give the same
    bits; float atomics agree to tolerance. The defaults: caller-sorted mode keeps the ordered reduction,
    deterministic=False uses the atomics. The walk order derived from the graph changes no bit."""
    import os
    from openequivariance_amd import runtime as rt
    from openequivariance_amd._torch import ops
    problem = P.config5_mace_conv()
    coords, rows, cols = _graph(400, 20, seed=6)
    g = CoordGraph(coords, rows, cols)
    E = g.nnz
    gen = torch.Generator(device="cuda").manual_seed(3)
    X = torch.randn(400, 2048, device="cuda", generator=gen)
    Y = torch.randn(E, 16, device="cuda", generator=gen)
    W = torch.randn(E, 2944, device="cuda", generator=gen)
    G = torch.randn(400, 12672, device="cuda", generator=gen)
    tr, tc, tp = (torch.tensor(a, device="cuda") for a in (g.rows, g.cols, g.transpose_perm))
    saved = os.environ.get("OEQ_AMD_TUNE")
    out = {}
    try:
        for tune in ("conv_dxm=0,conv_hops=0", "conv_dxm=0", "conv_dxm=1", "conv_dxm=2"):
            os.environ["OEQ_AMD_TUNE"] = tune
            conv = oeq.TensorProductConv(problem, deterministic=True)
            ks = ops.get_entry(conv.kid).kernels()
            assert ks.dims["dx_mode"] == int(tune.split(",")[0][-1])
            out[tune] = (ops.conv_forward(X, Y, W, tr, tc, tp, conv.kid),) + tuple(
                ops.conv_backward(X, Y, W, G, tr, tc, tp, conv.kid))
    finally:
        if saved is None:
            os.environ.pop("OEQ_AMD_TUNE", None)
        else:
            os.environ["OEQ_AMD_TUNE"] = saved
    base = out["conv_dxm=0,conv_hops=0"]
    for tune in ("conv_dxm=0", "conv_dxm=2"):
        for a, b in zip(base, out[tune]):
            assert torch.equal(a, b), tune
    z, dx, dy, dw = out["conv_dxm=1"]
    assert torch.equal(z, base[0]) and torch.equal(dy, base[2]) and torch.equal(dw, base[3])
    assert (dx - base[1]).abs().max() <= 1e-5 * base[1].abs().max()
    assert ops.get_entry(oeq.TensorProductConv(problem, deterministic=True).kid).kernels().dims["dx_mode"] == rt.DX_TERMS
    assert ops.get_entry(oeq.TensorProductConv(problem, deterministic=False).kid).kernels().dims["dx_mode"] == rt.DX_ATOMIC


def test_edge_list_index_is_reused_and_invalidated():
    """The ops keep the index of the last few edge lists: a second call over the same tensors builds nothing,
    a call after the tensors were written to (or with other tensors of the same contents) builds again, and the
    results are the same bits as with the cache switched off."""
    from openequivariance_amd._torch import ops
    problem = P.config2_nequip_uvu()
    coords, rows, cols = _graph(80, 8, seed=9)
    g = CoordGraph(coords, rows, cols)
    E = g.nnz
    gen = torch.Generator(device="cuda").manual_seed(5)
    X = torch.randn(80, problem.irreps_in1.dim, device="cuda", generator=gen)
    Y = torch.randn(E, problem.irreps_in2.dim, device="cuda", generator=gen)
    W = torch.randn(E, problem.weight_numel, device="cuda", generator=gen)
    G = torch.randn(80, problem.irreps_out.dim, device="cuda", generator=gen)
    for det in (True, False):
        conv = oeq.TensorProductConv(problem, deterministic=det)
        tr, tc, tp = (torch.tensor(a, device="cuda") for a in (g.rows, g.cols, g.transpose_perm))
        builds = []
        ks = ops.get_entry(conv.kid).kernels()
        real = ks.conv_index_build
        ks.conv_index_build = lambda *a, **k: (builds.append(1), real(*a, **k))[1]
        try:
            ops.clear_index_cache()
            z1 = ops.conv_forward(X, Y, W, tr, tc, tp, conv.kid)
            first = len(builds)
            assert first == 1
            z2 = ops.conv_forward(X, Y, W, tr, tc, tp, conv.kid)
            g1 = ops.conv_backward(X, Y, W, G, tr, tc, tp, conv.kid)
            assert len(builds) == first, "same tensors, same stream: the index is reused"
            assert torch.equal(z1, z2)
            # written to in place (same values): the version counter moves, the index is rebuilt
            tc.add_(0)
            z3 = ops.conv_forward(X, Y, W, tr, tc, tp, conv.kid)
            assert len(builds) == first + 1 and torch.equal(z3, z1)
            # a different edge list in the same storage must not be served the old index
            flipped = torch.tensor(g.cols[::-1].copy(), device="cuda")
            tc.copy_(flipped)
            tp2 = torch.tensor(np.lexsort((g.rows, g.cols[::-1])), device="cuda")
            z4 = ops.conv_forward(X, Y, W, tr, tc, tp2, conv.kid)
            monkey_off = ops.INDEX_CACHE_ENTRIES
            ops.INDEX_CACHE_ENTRIES = 0
            try:
                z5 = ops.conv_forward(X, Y, W, tr, tc, tp2, conv.kid)
                tc.copy_(torch.tensor(g.cols, device="cuda"))
                g2 = ops.conv_backward(X, Y, W, G, tr, tc, tp, conv.kid)
            finally:
                ops.INDEX_CACHE_ENTRIES = monkey_off
            assert torch.equal(z4, z5) and not torch.equal(z4, z1)
            assert torch.equal(g1[1], g2[1]) and torch.equal(g1[2], g2[2])
            assert (g1[0] - g2[0]).abs().max() <= 1e-5 * g2[0].abs().max()
        finally:
            ks.conv_index_build = real
            ops.clear_index_cache()


def test_kernel_set_compiled_side_by_side_runs(monkeypatch, tmp_path):
    """A kernel set whose kernels were compiled in shares by child processes reaches the library as a pack of
    code objects: it loads, every kernel is found (one of them sits inside a namespace), and it computes the
    bits of the set compiled whole."""
    from openequivariance_amd import runtime as rt
    problem = P.nequix_problems()[2]
    coords, rows, cols = _graph(60, 8, seed=11)
    g = CoordGraph(coords, rows, cols)
    X, Y, W, G = _buffers(problem, 60, g.nnz, seed=5)

    def run():
        conv = oeq.TensorProductConv(problem, deterministic=True)
        tX, tY, tW = (torch.tensor(a, device="cuda", requires_grad=True) for a in (X, Y[g.order], W[g.order]))
        z = conv(tX, tY, tW, torch.tensor(g.rows, device="cuda"), torch.tensor(g.cols, device="cuda"),
                 torch.tensor(g.transpose_perm, device="cuda"))
        z.backward(torch.tensor(G, device="cuda"))
        return [t.detach().cpu().numpy() for t in (z, tX.grad, tY.grad, tW.grad)]

    whole = run()
    monkeypatch.setattr(rt, "PARALLEL_MIN_BYTES", 0)
    monkeypatch.setenv("OEQ_AMD_COMPILE_JOBS", "4")
    monkeypatch.setenv("OEQ_AMD_CACHE_DIR", str(tmp_path))
    monkeypatch.setenv("OEQ_AMD_TUNE", "conv_hub=255")  # (a kernel set of its own: nothing to find in any cache)
    shares = run()
    packs = [f for f in tmp_path.iterdir() if f.read_bytes().startswith(rt.PACK_MAGIC)]
    assert len(packs) == 1 and len(rt.unpack_code(packs[0].read_bytes())) == 4
    for a, b in zip(whole, shares):
        assert np.array_equal(a, b)


@pytest.mark.parametrize("det", [True, False])
def test_autotune_keeps_results(det):
    """`TensorProductConv.autotune` times the alternative kernel shapes on the given inputs and may adopt one: the
    module computes the same convolution afterwards, and the knob string it returns rebuilds the adopted shape."""
    import json
    problem = P.ChannelwiseTPP("96x0e+96x1o", "0e+1o+2e+3o", "0e+1o+2e+3o+4e", "autotuned")
    coords, rows, cols = _graph(300, 12, seed=3)
    g = CoordGraph(coords, rows, cols)
    X, Y, W, G = _buffers(problem, 300, g.nnz, seed=8)
    ref = R.Problem.from_spec(problem)
    z_ref = R.conv_forward(ref, X, Y, W, rows, cols)
    dx_ref, dy_ref, dw_ref = R.conv_backward(ref, X, Y, W, G, rows, cols)
    conv = oeq.TensorProductConv(problem, deterministic=det)
    args = [torch.tensor(a, device="cuda") for a in (X, Y[g.order], W[g.order], g.rows, g.cols)]
    perm = torch.tensor(g.transpose_perm, device="cuda") if det else None
    allowed = set(conv.AUTOTUNE_FORWARD) | set(conv.AUTOTUNE_BACKWARD) | {"conv_dxm=0", "conv_dxm=1"}
    tune = conv.autotune(*args, perm, repeats=2)
    assert set(filter(None, tune.split(","))) <= allowed
    assert json.loads(bytes(conv.spec.tolist()).decode())["tune"] == tune
    tX, tY, tW = (a.clone().requires_grad_(True) for a in args[:3])
    z = conv(tX, tY, tW, args[3], args[4], perm)
    z.backward(torch.tensor(G, device="cuda"))
    assert err(z, z_ref) <= 1e-5 and err(tX.grad, dx_ref) <= 1e-5
    assert err(tY.grad.cpu().numpy(), dy_ref[g.order]) <= 1e-5 and err(tW.grad.cpu().numpy(), dw_ref[g.order]) <= 1e-5
    # a 'uvw' problem has no alternatives
    fc = oeq.TensorProductConv(_fc(False), deterministic=False)
    before = fc.kid
    assert fc.autotune(*[torch.zeros(1, device="cuda")] * 3, args[3][:1], args[4][:1]) == "" and fc.kid == before
