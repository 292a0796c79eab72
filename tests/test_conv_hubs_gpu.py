"""Nodes with very many edges: their edge segments are walked in chunks by different wave groups
(extra walk positions, rows of the extra chunks added in chunk order by `fixup_forward`), so the time of a
call does not grow with the largest degree. Against the oracle in both modes, first and second order, with
shared weights, and bit for bit across index builds. The reference cuts the edge list into equal ranges per
warp and fixes up the boundaries (templates/loop_unroll_conv_det.cuh:34-66, 96-179)."""

import numpy as np
import pytest
import torch

import openequivariance_amd as oeq
from openequivariance_amd import runtime as rt
from openequivariance_amd._torch import ops
from openequivariance_amd.core import problems as P
from openequivariance_amd.core.graph import CoordGraph
from oracle import e3nn_ref as R
from gpu_util import err, tol_of

pytestmark = pytest.mark.gpu


def _hub_graph(n_nodes, hub_degree, n_background, seed, second_hub=0):
    """Node 0 receives from and sends to `hub_degree` other nodes (node 7 likewise, `second_hub` of them);
    `n_background` random edges among the rest; node 3 isolated."""
    rng = np.random.default_rng(seed)
    spokes = rng.choice(np.arange(8, n_nodes), size=hub_degree, replace=False).astype(np.int64)
    rows = [np.zeros(hub_degree, dtype=np.int64), spokes]
    cols = [spokes, np.zeros(hub_degree, dtype=np.int64)]
    if second_hub:
        sp2 = rng.choice(np.arange(8, n_nodes), size=second_hub, replace=False).astype(np.int64)
        rows += [np.full(second_hub, 7, dtype=np.int64), sp2]
        cols += [sp2, np.full(second_hub, 7, dtype=np.int64)]
    rows.append(rng.integers(8, n_nodes, size=n_background))
    cols.append(rng.integers(8, n_nodes, size=n_background))
    rows, cols = np.concatenate(rows), np.concatenate(cols)
    keep = (rows != 3) & (cols != 3)
    return rows[keep], cols[keep]


def _buffers(problem, n_nodes, E, seed):
    rng = np.random.default_rng(seed)
    dt = np.dtype(problem.irrep_dtype)
    X = rng.normal(size=(n_nodes, problem.irreps_in1.dim)).astype(dt)
    Y = rng.normal(size=(E, problem.irreps_in2.dim)).astype(dt)
    W = rng.normal(size=(problem.weight_numel,) if problem.shared_weights else (E, problem.weight_numel)).astype(dt)
    G = rng.normal(size=(n_nodes, problem.irreps_out.dim)).astype(dt)
    return X, Y, W, G


def _odd_shared():
    return oeq.TPProblem("5x1e+3x2e", "2x1e+1x0e", "5x1e+3x2e+5x0e",
                         [(0, 0, 0, "uvu", True), (0, 1, 0, "uvu", True), (1, 0, 1, "uvu", True),
                          (0, 0, 2, "uvu", True)], shared_weights=True, internal_weights=False, label="odd-uvu")


def _uvw(shared):
    # 'uvw' with channels on the second operand as well, so that shared weights do not factor out of the
    # sum over edges: the fused per-edge walk runs in both cases
    return oeq.TPProblem("12x0e+7x1o", "2x0e+1x1o", "9x0e+12x1o+5x1e",
                         [(0, 0, 0, "uvw", True), (1, 1, 0, "uvw", True), (0, 1, 1, "uvw", True),
                          (1, 0, 1, "uvw", True), (1, 1, 2, "uvw", True)], shared_weights=shared,
                         internal_weights=False, label="uvw-shared" if shared else "uvw")


HUBS = [
    # (name, problem, nodes, hub degree, second hub, background edges)
    ("cfg2-hub12000", P.config2_nequip_uvu, 14000, 12000, 700, 20000),
    ("cfg1-hub30000", P.config1_single_uvu, 40000, 30000, 257, 50000),
    ("cfg5-hub1100", P.config5_mace_conv, 1500, 1100, 0, 800),          # two 64-channel chunks per row
    ("mace-large-hub600", lambda: P.mace_problems()[0], 900, 600, 0, 500),
    ("odd-shared-hub5000", _odd_shared, 6000, 5000, 300, 4000),         # bounded grid, strided walk
    ("benzene-hub700", lambda: P.nequip_problems()[3], 900, 700, 0, 300),  # node shared between waves
    ("uvw-hub4000", lambda: _uvw(False), 5000, 4000, 300, 3000),        # the channel-mixing walk
    ("uvw-shared-hub4000", lambda: _uvw(True), 5000, 4000, 300, 3000),
    ("e3tools-hub700", lambda: P.e3tools_problems()[0], 900, 700, 0, 300),
    # last layer of a network (long X rows, short output rows): the sender gradients come from the sender-side walk,
    # whose long segments are cut into chunks like the receiver side's
    ("last-layer-hub3000", lambda: P.nequix_problems()[2], 4000, 3000, 300, 3000),
]


@pytest.mark.parametrize("name,make,n_nodes,hub,hub2,background", HUBS, ids=[h[0] for h in HUBS])
def test_hub_matches_oracle_in_both_modes(name, make, n_nodes, hub, hub2, background):
    problem = make()
    tol = tol_of(problem)
    rows, cols = _hub_graph(n_nodes, hub, background, seed=1, second_hub=hub2)
    E = len(rows)
    X, Y, W, G = _buffers(problem, n_nodes, E, seed=2)
    ref = R.Problem.from_spec(problem)
    z_ref = R.conv_forward(ref, X, Y, W, rows, cols)
    dx_ref, dy_ref, dw_ref = R.conv_backward(ref, X, Y, W, G, rows, cols)
    rng = np.random.default_rng(3)
    for det in ([False] if problem.shared_weights else [False, True]):
        if det:
            g = CoordGraph(np.zeros((n_nodes, 3)), rows, cols)
            order, r_, c_, perm = g.order, g.rows, g.cols, g.transpose_perm
        else:
            order = rng.permutation(E)
            r_, c_, perm = rows[order], cols[order], None
        conv = oeq.TensorProductConv(problem, deterministic=det)
        ks = ops.get_entry(conv.kid).kernels()
        limit = ks.dims["hub_limit"]
        assert 0 < limit < hub, "the hub is meant to be cut into several chunks"
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
        # the same bits from a rebuilt index (the table of extra positions is a function of the edge list)
        ops.clear_index_cache()
        z2 = conv(tX.detach(), tY.detach(), tW.detach(), tr, tc, tp)
        assert torch.equal(z2, z.detach()), (name, det)


def test_chunked_walk_is_a_function_of_the_edge_list():
    """Forward and the per-edge gradients of a hub graph: bit-identical between runs, between index builds, and
    between the caller-sorted mode and deterministic=False on the same sorted list; the sender gradient of the
    sorted mode likewise."""
    problem = P.config2_nequip_uvu()
    n = 5000
    rows, cols = _hub_graph(n, 3000, 6000, seed=5, second_hub=500)
    g = CoordGraph(np.zeros((n, 3)), rows, cols)
    E = g.nnz
    gen = torch.Generator(device="cuda").manual_seed(0)
    X = torch.randn(n, problem.irreps_in1.dim, device="cuda", generator=gen)
    Y = torch.randn(E, problem.irreps_in2.dim, device="cuda", generator=gen)
    W = torch.randn(E, problem.weight_numel, device="cuda", generator=gen)
    G = torch.randn(n, problem.irreps_out.dim, device="cuda", generator=gen)
    tr, tc, tp = (torch.tensor(a, device="cuda") for a in (g.rows, g.cols, g.transpose_perm))
    det = oeq.TensorProductConv(problem, deterministic=True)
    at = oeq.TensorProductConv(problem, deterministic=False)
    z = ops.conv_forward(X, Y, W, tr, tc, tp, det.kid)
    dx, dy, dw = ops.conv_backward(X, Y, W, G, tr, tc, tp, det.kid)
    for _ in range(3):
        ops.clear_index_cache()
        torch.randn(1 << 22, device="cuda")
        assert torch.equal(ops.conv_forward(X, Y, W, tr, tc, tp, det.kid), z)
        again = ops.conv_backward(X, Y, W, G, tr, tc, tp, det.kid)
        assert all(torch.equal(a, b) for a, b in zip(again, (dx, dy, dw)))
    dummy = torch.zeros(1, dtype=torch.int64, device="cuda")
    assert torch.equal(ops.conv_forward(X, Y, W, tr, tc, dummy, at.kid), z)
    dxa, dya, dwa = ops.conv_backward(X, Y, W, G, tr, tc, dummy, at.kid)
    assert torch.equal(dya, dy) and torch.equal(dwa, dw)
    assert float((dxa - dx).abs().max() / dx.abs().max()) <= 1e-5


@pytest.mark.parametrize("make", [P.config2_nequip_uvu, lambda: _uvw(False)], ids=["uvu", "uvw"])
def test_hub_second_order_matches_composition(make):
    """The fused second-order pair on a hub graph (kernel A writes rows of extra chunks, kernel B walks
    them) against the composition of first-order calls, which is linear algebra on the same operands."""
    problem = make()
    n = 2500
    rows, cols = _hub_graph(n, 1500, 2500, seed=6)
    g = CoordGraph(np.zeros((n, 3)), rows, cols)
    E = g.nnz
    gen = torch.Generator(device="cuda").manual_seed(1)
    dims = (problem.irreps_in1.dim, problem.irreps_in2.dim, problem.weight_numel, problem.irreps_out.dim)
    X, A = (torch.randn(n, dims[0], device="cuda", generator=gen) for _ in range(2))
    Y, B = (torch.randn(E, dims[1], device="cuda", generator=gen) for _ in range(2))
    W, C = (torch.randn(E, dims[2], device="cuda", generator=gen) for _ in range(2))
    G = torch.randn(n, dims[3], device="cuda", generator=gen)
    tr, tc, tp = (torch.tensor(a, device="cuda") for a in (g.rows, g.cols, g.transpose_perm))
    conv = oeq.TensorProductConv(problem, deterministic=True)
    ks = ops.get_entry(conv.kid).kernels()
    assert ks.has_double_backward() and 0 < ks.dims["hub_limit"] < 1500
    fused = ops.conv_double_backward(X, Y, W, G, A, B, C, tr, tc, tp, conv.kid)
    with torch.no_grad():
        composed = ops._second_order(lambda p, q, r: ops.conv_forward(p, q, r, tr, tc, tp, conv.kid),
                                     lambda p, q, r, s: ops.conv_backward(p, q, r, s, tr, tc, tp, conv.kid),
                                     X, Y, W, G, A, B, C)
    for got, want in zip(fused, composed):
        assert float((got - want).abs().max() / want.abs().max()) <= 1e-5


def test_static_entry_point_walks_whole_segments():
    """oeq_conv_forward_static has no scratch for the rows of extra chunks: it walks a hub's segment whole
    and agrees with the chunked walk to rounding."""
    problem = P.config1_single_uvu()
    n = 3000
    rows, cols = _hub_graph(n, 2000, 3000, seed=7)
    g = CoordGraph(np.zeros((n, 3)), rows, cols)
    E = g.nnz
    gen = torch.Generator(device="cuda").manual_seed(2)
    X = torch.rand(n, 5, device="cuda", generator=gen)
    Y = torch.rand(E, 7, device="cuda", generator=gen)
    W = torch.rand(E, 1, device="cuda", generator=gen)
    tr, tc, tp = (torch.tensor(a, device="cuda") for a in (g.rows, g.cols, g.transpose_perm))
    conv = oeq.TensorProductConv(problem, deterministic=True)
    z = ops.conv_forward(X, Y, W, tr, tc, tp, conv.kid)
    ks = ops.get_entry(conv.kid).kernels()
    out = torch.empty_like(z)
    ks.conv_forward_static(n, E, X.data_ptr(), Y.data_ptr(), W.data_ptr(), out.data_ptr(), tr.data_ptr(),
                           tc.data_ptr(), torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert float((out - z).abs().max() / z.abs().max()) <= 1e-5
    assert torch.equal(out[8:], z[8:]), "nodes without extra chunks: same bits"
