"""The fused second-order kernels (`double_backward_A` / `double_backward_B`) against the composition of
first-order kernels, which tests/test_higher_derivatives_gpu.py checks against float64 autograd through the
CPU restatement. Also through autograd: the force-training pattern (gradient of a function of the first
gradients) with the fused route switched on and off."""

import numpy as np
import pytest
import torch

import openequivariance_amd as oeq
from openequivariance_amd import runtime as rt
from openequivariance_amd._torch import ops
from openequivariance_amd.codegen import uvu_double
from openequivariance_amd.core import problems as P
from openequivariance_amd.core.graph import CoordGraph, periodic_radius_graph
from oracle import e3nn_ref as R
from gpu_util import tol_of

pytestmark = pytest.mark.gpu


def _f64(problem):
    q = problem.clone()
    q.irrep_dtype, q.weight_dtype = np.float64, np.float64
    return q


def _ir_mul(problem):
    q = problem.clone()
    q.layout = "ir_mul"
    return q


def _odd():
    # packed rows (5 channels), mul2 > 1, a block no instruction reads and one no instruction writes
    return oeq.TPProblem("5x1e+3x2e+2x0e", "2x1e+1x0e", "5x1e+3x2e+5x0e+4x1o",
                         [(0, 0, 0, "uvu", True), (0, 1, 0, "uvu", True), (1, 0, 1, "uvu", True),
                          (0, 0, 2, "uvu", True)], shared_weights=False, internal_weights=False)


def _folded():
    # wide row with a different multiplicity per irrep, unread input block, unwritten output block
    return oeq.TPProblem("100x0e+70x1o+40x2e+96x1e", "1x0e+2x1o", "100x0e+70x1o+100x1o+40x1o+33x2e",
                         [(0, 0, 0, "uvu", True), (1, 0, 1, "uvu", True), (0, 1, 2, "uvu", True),
                          (2, 1, 3, "uvu", True, 0.7)], shared_weights=False, internal_weights=False)


def _wide_v():
    # more second-operand channels than the emitters unroll: the v loop stays a loop
    return oeq.TPProblem("4x1e+7x0e", "12x1e+10x0e", "4x0e+4x1e+7x1e",
                         [(0, 0, 0, "uvu", True), (0, 1, 1, "uvu", True), (1, 0, 2, "uvu", True)],
                         shared_weights=False, internal_weights=False)


CASES = [
    ("cfg1", P.config1_single_uvu, 1000),
    ("wide-v", _wide_v, 211),
    ("folded-gaps", _folded, 61),
    ("very-wide-ragged", lambda: oeq.TPProblem(
        "300x0e+70x1o+20x2e", "1x0e+1x1o", "300x0e+70x1o+300x1o+20x1o",
        [(0, 0, 0, "uvu", True), (1, 0, 1, "uvu", True), (0, 1, 2, "uvu", True), (2, 1, 3, "uvu", True)],
        shared_weights=False, internal_weights=False), 37),
    ("odd", _odd, 333),
    ("odd-f64", lambda: _f64(_odd()), 333),
    ("cfg2", P.config2_nequip_uvu, 257),
    ("cfg2-f64", lambda: _f64(P.config2_nequip_uvu()), 129),
    ("cfg2-ir_mul", lambda: _ir_mul(P.config2_nequip_uvu()), 129),
    ("cfg3", P.config3_mace_uvu, 67),
    ("cfg3-f64", lambda: _f64(P.config3_mace_uvu()), 33),
    ("lips", lambda: P.nequip_problems()[0], 129),
    ("benzene", lambda: P.nequip_problems()[3], 33),
    ("nequix-first", lambda: P.nequix_problems()[0], 65),
    ("sevennet-main", lambda: P.seven_net_problems()[1], 65),
    ("mace-large-ir_mul", lambda: _ir_mul(P.mace_problems()[0]), 33),
]


def _shared(problem):
    q = problem.clone()
    q.shared_weights = True
    return q


# shared weights (batch kernels only): one weight vector, its gradient summed over the rows
SHARED = [
    ("cfg2-shared", lambda: _shared(P.config2_nequip_uvu()), 257),
    ("cfg2-shared-f64", lambda: _shared(_f64(P.config2_nequip_uvu())), 129),
    ("cfg3-shared", lambda: _shared(P.config3_mace_uvu()), 67),
    ("odd-shared", lambda: _shared(_odd()), 333),
    ("cfg1-shared", lambda: _shared(P.config1_single_uvu()), 1000),
    ("folded-gaps-shared", lambda: _shared(_folded()), 61),
]


def _fc(shared, in2="1x0e+2x1o"):
    return P.FullyConnectedTPProblem("4x0e+3x1o", in2, "5x0e+2x1o+1x2e", shared_weights=shared,
                                     internal_weights=False, label="fc-uvw")


def _fc_general(out):
    return P.FullyConnectedTPProblem("20x0e+10x1o", "40x0e+10x1o", out, shared_weights=True, internal_weights=False,
                                     label="general-fc-uvw")


def _wide_fc(shared, in2="1x0e+1x1o"):
    # channel blocks that are no multiples of 16 and wider than a wave (shared weights: on the matrix cores with
    # padded tiles, one sub-path per channel of the second operand)
    return P.FullyConnectedTPProblem("70x0e+20x1o", in2, "70x0e+20x1o", shared_weights=shared,
                                     internal_weights=False, label="wide-fc-uvw")


# fully connected ('uvw') problems: per-row weights (weight tiles in LDS, single-channel operands, direct access)
# and shared weights outside the matrix-core path (gradients in registers, in LDS, or summed in global memory)
UVW = [
    ("uvw-fc", lambda: _fc(False), 129),
    ("uvw-fc-f64", lambda: _f64(_fc(False)), 65),
    ("uvw-fc-mul2", lambda: _fc(False, "2x0e+3x1o"), 65),
    ("uvw-diffdock", lambda: P.diffdock_problems()[0], 65),
    ("uvw-diffdock-f64", lambda: _f64(P.diffdock_problems()[0]), 33),
    ("uvw-e3tools-conv", lambda: P.e3tools_problems()[0], 65),
    ("uvw-wide", lambda: _wide_fc(False), 17),
    ("uvw-fc-shared", lambda: _fc(True), 129),
    ("uvw-fc-shared-f64", lambda: _f64(_fc(True)), 65),
    ("uvw-tetris-1-shared", lambda: P.tetris_poly_problems()[0], 129),
    ("uvw-tetris-2-shared", lambda: P.tetris_poly_problems()[1], 65),
    ("uvw-wide-shared", lambda: _wide_fc(True), 600),
    ("uvw-wide-mul2-shared", lambda: _wide_fc(True, "2x0e+1x1o"), 300),
    # off the matrix cores (second operand of more than 64 values): weight gradient in an LDS copy per wave, and in
    # partial rows in global memory
    ("uvw-lds-shared", lambda: _fc_general("12x0e+6x1o"), 200),
    ("uvw-global-shared-f64", lambda: _f64(_fc_general("40x0e+20x1o")), 100),
]
UVW_CONV = [c for c in UVW if not c[0].endswith(("shared", "shared-f64"))]
# shared weights in the fused convolution: the three ways of summing the weight gradient (registers, LDS copy per
# wave, partial rows in global memory when the weight tensor exceeds 64 KB)
UVW_CONV_SHARED = [c for c in UVW if c[0].endswith(("shared", "shared-f64")) and "wide" not in c[0]]


def _fc_shared(in1, in2, out):
    return P.FullyConnectedTPProblem(in1, in2, out, shared_weights=True, internal_weights=False, label=f"fc-shared {in1}")


# shared weights and a single-channel second operand: the matrix-core kernels (second-order pair = variants of the
# first-order kernels with the summed contraction, run on both weight tensors); multiplicities that are no
# multiples of 16 on padded tiles
MFMA = [
    ("cfg4", P.config4_uvw_shared, 83),
    ("cfg4-f64", lambda: P.config4_uvw_shared(np.float64), 37),
    ("mfma-mixed", lambda: _fc_shared("64x0e+32x1o+16x2e", "1x0e+1x1o", "48x0e+80x1o+16x2e"), 50),
    ("mfma-mixed-f64", lambda: _f64(_fc_shared("64x0e+32x1o+16x2e", "1x0e+1x1o", "48x0e+80x1o+16x2e")), 33),
    ("mfma-128", lambda: _fc_shared("128x0e+128x1o", "1x0e+1x1o", "128x0e+128x1o"), 45),
    ("mfma-pad-diffdock", lambda: _shared(P.diffdock_problems()[0]), 50),
    ("mfma-pad-mid-f64", lambda: _f64(_fc_shared("40x0e+30x1o", "1x0e+1x1o", "50x0e+20x1o+10x2e")), 35),
    ("mfma-pad-wide", lambda: _fc_shared("100x0e+70x1o", "1x0e+1x1o", "33x0e+20x1o"), 50),
    ("mfma-mul3-f64", lambda: _f64(_fc_shared("64x0e+64x1o", "3x0e+2x1o", "64x0e+64x1o")), 33),
    ("mfma-64-l3", lambda: _fc_shared("64x0e+64x1o+64x2e+64x3o", "1x0e+1x1o+1x2e+1x3o", "64x0e+64x1o+64x2e+64x3o"), 35),
    ("mfma-50-l3-f64", lambda: _f64(_fc_shared("50x0e+50x1o+50x2e+50x3o", "1x0e+1x1o+1x2e+1x3o",
                                               "50x0e+50x1o+50x2e+50x3o")), 33),
    ("mfma-mul2-pad", lambda: _fc_shared("40x0e+30x1o", "2x0e+1x1o", "25x0e+10x1o+5x2e"), 50),
    ("mfma-gaps", lambda: oeq.TPProblem(
        "32x0e+16x1o+32x2e", "1x0e+1x1o", "32x0e+16x1o+48x2e+16x1e",
        [(0, 0, 0, "uvw", True), (1, 1, 0, "uvw", True), (0, 1, 1, "uvw", True), (2, 0, 2, "uvw", True, 0.7)],
        shared_weights=True, internal_weights=False, label="mfma-gaps"), 50),
]


def _rand(rng, shape, dt):
    return torch.tensor(rng.uniform(-1, 1, size=shape).astype(dt), device="cuda")


def _check(names, fused, composed, tol):
    for name, a, b in zip(names, fused, composed):
        e = R.normalized_error(a.cpu().numpy(), b.cpu().numpy())
        assert e <= tol, (name, e)


@pytest.mark.parametrize("name,make,batch", CASES + SHARED + UVW + MFMA, ids=[c[0] for c in CASES + SHARED + UVW + MFMA])
def test_tp_fused_matches_composition(name, make, batch):
    problem = make()
    tp = oeq.TensorProduct(problem)
    e = ops.get_entry(tp.kid)
    assert e.kernels().has_double_backward()
    dt = np.dtype(problem.irrep_dtype)
    rng = np.random.default_rng(5)
    x, a = (_rand(rng, (batch, e.L1), dt) for _ in range(2))
    y, b = (_rand(rng, (batch, e.L2), dt) for _ in range(2))
    w, c = (_rand(rng, (e.WN,) if problem.shared_weights else (batch, e.WN), dt) for _ in range(2))
    g = _rand(rng, (batch, e.L3), dt)
    fused = ops.tp_double_backward(x, y, w, g, a, b, c, tp.kid)
    composed = ops._second_order(lambda p, q, r: ops.tp_forward(p, q, r, tp.kid),
                                 lambda p, q, r, s: ops.tp_backward(p, q, r, s, tp.kid), x, y, w, g, a, b, c)
    _check(("dx", "dy", "dw", "gg"), fused, composed, tol_of(problem))


def _graph(n=60):
    coords, rows, cols, _ = periodic_radius_graph(n, 8.0, 3.2, seed=3)
    return CoordGraph(coords, rows, cols)


CONV_CASES = [c for c in CASES if c[0] not in ("cfg1",)] + [("cfg1", P.config1_single_uvu, 0)] + UVW_CONV


@pytest.mark.parametrize("det", [True, False], ids=["sorted", "grouped"])
@pytest.mark.parametrize("name,make,batch", CONV_CASES, ids=[c[0] for c in CONV_CASES])
def test_conv_fused_matches_composition(name, make, batch, det, monkeypatch):
    problem = make()
    gph = _graph()
    n, E = gph.coords.shape[0], gph.nnz
    if name in ("benzene", "sevennet-main"):
        # more paths than the fused convolution kernels are built for by default
        monkeypatch.setattr(uvu_double, "CONV_MAX_PATHS", 1000)
    conv = oeq.TensorProductConv(problem, deterministic=det)
    e = ops.get_entry(conv.kid)
    assert e.kernels().has_double_backward()
    dt = np.dtype(problem.irrep_dtype)
    rng = np.random.default_rng(6)
    if det:
        rows, cols, perm = gph.rows, gph.cols, gph.transpose_perm
    else:
        order = rng.permutation(E)
        rows, cols, perm = gph.rows[order], gph.cols[order], np.zeros(0, np.int64)
    tr, tc, tp = (torch.tensor(v, device="cuda") for v in (rows, cols, perm))
    x, a = (_rand(rng, (n, e.L1), dt) for _ in range(2))
    y, b = (_rand(rng, (E, e.L2), dt) for _ in range(2))
    w, c = (_rand(rng, (E, e.WN), dt) for _ in range(2))
    g = _rand(rng, (n, e.L3), dt)
    fused = ops.conv_double_backward(x, y, w, g, a, b, c, tr, tc, tp, conv.kid)
    composed = ops._second_order(lambda p, q, r: ops.conv_forward(p, q, r, tr, tc, tp, conv.kid),
                                 lambda p, q, r, s: ops.conv_backward(p, q, r, s, tr, tc, tp, conv.kid),
                                 x, y, w, g, a, b, c)
    _check(("dx", "dy", "dw", "gg"), fused, composed, tol_of(problem))


KAHAN_CONV = [c for c in CONV_CASES if c[0] in ("cfg2", "cfg3", "odd", "folded", "lips")] + UVW_CONV[:2]


@pytest.mark.parametrize("name,make,batch", KAHAN_CONV, ids=[c[0] for c in KAHAN_CONV])
def test_conv_kahan_has_the_fused_pair(name, make, batch):
    """kahan=True: kernel A adds each edge's three terms with a compensation term (its sums run over a node's
    edges like the forward kernel's), kernel B's sender gradients go through the compensated ordered reduction.
    Against the composition of the kahan first-order kernels and against the plain fused pair."""
    problem = make()
    gph = _graph()
    n, E = gph.coords.shape[0], gph.nnz
    conv = oeq.TensorProductConv(problem, deterministic=True, kahan=True)
    plain = oeq.TensorProductConv(problem, deterministic=True)
    e = ops.get_entry(conv.kid)
    assert e.kernels().has_double_backward()
    dt = np.dtype(problem.irrep_dtype)
    rng = np.random.default_rng(8)
    tr, tc, tp = (torch.tensor(v, device="cuda") for v in (gph.rows, gph.cols, gph.transpose_perm))
    x, a = (_rand(rng, (n, e.L1), dt) for _ in range(2))
    y, b = (_rand(rng, (E, e.L2), dt) for _ in range(2))
    w, c = (_rand(rng, (E, e.WN), dt) for _ in range(2))
    g = _rand(rng, (n, e.L3), dt)
    fused = ops.conv_double_backward(x, y, w, g, a, b, c, tr, tc, tp, conv.kid)
    composed = ops._second_order(lambda p, q, r: ops.conv_forward(p, q, r, tr, tc, tp, conv.kid),
                                 lambda p, q, r, s: ops.conv_backward(p, q, r, s, tr, tc, tp, conv.kid),
                                 x, y, w, g, a, b, c)
    _check(("dx", "dy", "dw", "gg"), fused, composed, tol_of(problem))
    _check(("dx", "dy", "dw", "gg"), fused, ops.conv_double_backward(x, y, w, g, a, b, c, tr, tc, tp, plain.kid),
           tol_of(problem))


def test_conv_kahan_second_order_on_a_hub():
    """A node with 3000 same-sign terms: the compensated kernel A is closer to the float64 sum than the plain one."""
    problem = P.config1_single_uvu()
    n, hub = 3200, 3000
    rows = np.concatenate([np.zeros(hub, np.int64), np.arange(1, 200)])
    cols = np.concatenate([np.arange(1, hub + 1), np.arange(2, 201)])
    gph = CoordGraph(np.zeros((n, 3)), rows, cols)
    E = gph.nnz
    gen = torch.Generator(device="cuda").manual_seed(3)
    mk = lambda *shape: torch.rand(*shape, device="cuda", generator=gen) + 0.5
    d = ops.get_entry(oeq.TensorProductConv(problem, deterministic=True).kid)
    x, a, y, b, w, c, g = mk(n, d.L1), mk(n, d.L1), mk(E, d.L2), mk(E, d.L2), mk(E, d.WN), mk(E, d.WN), mk(n, d.L3)
    tr, tc, tp = (torch.tensor(v, device="cuda") for v in (gph.rows, gph.cols, gph.transpose_perm))
    got = {}
    for kahan in (False, True):
        conv = oeq.TensorProductConv(problem, deterministic=True, kahan=kahan)
        assert ops.get_entry(conv.kid).kernels().has_double_backward()
        got[kahan] = ops.conv_double_backward(x, y, w, g, a, b, c, tr, tc, tp, conv.kid)[3][0].double()
    c64 = oeq.TensorProductConv(_f64(problem), deterministic=True)
    ref = ops.conv_double_backward(*(t.double() for t in (x, y, w, g, a, b, c)), tr, tc, tp, c64.kid)[3][0]
    errs = {k: float((v - ref).abs().max() / ref.abs().max()) for k, v in got.items()}
    assert errs[True] <= max(errs[False], 1e-7) and errs[True] <= 2e-7, errs


def test_float_atomics_convolution_uses_the_grouped_walk_pair(monkeypatch):
    """conv_sort=0 selects the float-atomics kernels for the first-order ops; their second-order pass runs the fused
    pair of the grouped-walk kernel set of the same problem (any edge order, fixed summation order) instead of
    composing six float-atomics launches."""
    monkeypatch.setenv("OEQ_AMD_TUNE", "conv_sort=0")
    problem = P.config2_nequip_uvu()
    conv = oeq.TensorProductConv(problem, deterministic=False)
    e = ops.get_entry(conv.kid)
    assert e.kernels().dims["deterministic"] == rt.CONV_ATOMIC and not e.kernels().has_double_backward()
    assert e.second_order_kid is not None and ops.get_entry(e.second_order_kid).kernels().has_double_backward()
    gph = _graph(300)
    n, E = gph.coords.shape[0], gph.nnz
    rng = np.random.default_rng(9)
    order = rng.permutation(E)
    tr, tc = (torch.tensor(v[order], device="cuda") for v in (gph.rows, gph.cols))
    tp = torch.zeros(0, dtype=torch.int64, device="cuda")
    x, a = (_rand(rng, (n, e.L1), np.float32) for _ in range(2))
    y, b = (_rand(rng, (E, e.L2), np.float32) for _ in range(2))
    w, c = (_rand(rng, (E, e.WN), np.float32) for _ in range(2))
    g = _rand(rng, (n, e.L3), np.float32)
    with torch.no_grad():
        assert ops._use_fused(conv.kid, None, a, b, c)
        fused = ops.conv_double_backward(x, y, w, g, a, b, c, tr, tc, tp, conv.kid)
        composed = ops._second_order(lambda p, q, r: ops.conv_forward(p, q, r, tr, tc, tp, conv.kid),
                                     lambda p, q, r, s: ops.conv_backward(p, q, r, s, tr, tc, tp, conv.kid),
                                     x, y, w, g, a, b, c)
    _check(("dx", "dy", "dw", "gg"), fused, composed, tol_of(problem))
    # and through autograd: the force-training pattern
    ts = [t.clone().requires_grad_(True) for t in (x, y, w)]
    first = torch.autograd.grad(conv(*ts, tr, tc), ts, g, create_graph=True)
    second = torch.autograd.grad(sum((t ** 2).sum() for t in first), ts)
    assert all(torch.isfinite(t).all() for t in second)


@pytest.mark.parametrize("det", [True, False], ids=["sorted", "grouped"])
def test_unfused_convolution_second_order_matches_fused(det, monkeypatch):
    """The unfused convolution (gathered rows, batch kernels, ordered sums; here selected by a knob for a problem
    that also has fused kernels) runs its second-order pass as the batch kernel pair on the gathered rows of both
    orders: same results as the fused kernels, in both edge-list modes."""
    problem = P.diffdock_problems()[0]
    gph = _graph()
    n, E = gph.coords.shape[0], gph.nnz
    rng = np.random.default_rng(8)
    if det:
        rows, cols, perm = gph.rows, gph.cols, gph.transpose_perm
    else:
        order = rng.permutation(E)
        rows, cols, perm = gph.rows[order], gph.cols[order], np.zeros(0, np.int64)
    tr, tc, tp = (torch.tensor(v, device="cuda") for v in (rows, cols, perm))
    out = {}
    for fuse in (1, 0):
        monkeypatch.setenv("OEQ_AMD_TUNE", f"conv_fuse_uvw={fuse}")
        conv = oeq.TensorProductConv(problem, deterministic=det)
        e = ops.get_entry(conv.kid)
        assert e.unfused == (fuse == 0) and e.kernels().has_double_backward()
        if fuse:
            x, a = (_rand(rng, (n, e.L1), np.float32) for _ in range(2))
            y, b = (_rand(rng, (E, e.L2), np.float32) for _ in range(2))
            w, c = (_rand(rng, (E, e.WN), np.float32) for _ in range(2))
            g = _rand(rng, (n, e.L3), np.float32)
        out[fuse] = ops.conv_double_backward(x, y, w, g, a, b, c, tr, tc, tp, conv.kid)
    _check(("dx", "dy", "dw", "gg"), out[0], out[1], tol_of(problem))
    # and through autograd, where the op is chosen by the same rule as for the fused kernels
    monkeypatch.setenv("OEQ_AMD_TUNE", "conv_fuse_uvw=0")
    conv = oeq.TensorProductConv(problem, deterministic=det)
    tx, ty, tw, tg = (t.clone().requires_grad_(True) for t in (x, y, w, g))
    z = conv(tx, ty, tw, tr, tc, tp if det else None)
    first = torch.autograd.grad(z, (tx, ty, tw), tg, create_graph=True)
    second = torch.autograd.grad(sum((p * q).sum() for p, q in zip((a, b, c), first)), (tx, ty, tw, tg))
    _check(("dx", "dy", "dw", "gg"), second, out[1], tol_of(problem))


# matrix-core problems: the convolution is unfused, its second-order pass the batch kernel pair on gathered rows
MFMA_CONV = [c for c in MFMA if c[0] in ("cfg4", "mfma-mixed-f64", "mfma-pad-diffdock", "mfma-pad-wide")] + \
    [c for c in UVW if c[0] == "uvw-wide-mul2-shared"]


@pytest.mark.parametrize("name,make,batch", SHARED + UVW_CONV_SHARED + MFMA_CONV,
                         ids=[c[0] for c in SHARED + UVW_CONV_SHARED + MFMA_CONV])
def test_conv_shared_weights_fused_matches_composition_and_oracle(name, make, batch):
    """Shared weights (device-grouped edge lists only): kernel B sums the weight gradient over all edges of a
    wave (group) and the partial rows in a fixed order. Against the composition of first-order ops and against
    float64 autograd through the CPU restatement."""
    from oracle.torch_ref import TorchConv
    problem = make()
    gph = _graph(40)
    n, E = gph.coords.shape[0], gph.nnz
    conv = oeq.TensorProductConv(problem, deterministic=False)
    e = ops.get_entry(conv.kid)
    assert e.kernels().has_double_backward()
    dt = np.dtype(problem.irrep_dtype)
    rng = np.random.default_rng(26)
    order = rng.permutation(E)
    rows, cols = gph.rows[order], gph.cols[order]
    tr, tc, tp = (torch.tensor(v, device="cuda") for v in (rows, cols, np.zeros(0, np.int64)))
    x, a = (_rand(rng, (n, e.L1), dt) for _ in range(2))
    y, b = (_rand(rng, (E, e.L2), dt) for _ in range(2))
    w, c = (_rand(rng, (e.WN,), dt) for _ in range(2))
    g = _rand(rng, (n, e.L3), dt)
    fused = ops.conv_double_backward(x, y, w, g, a, b, c, tr, tc, tp, conv.kid)
    composed = ops._second_order(lambda p, q, r: ops.conv_forward(p, q, r, tr, tc, tp, conv.kid),
                                 lambda p, q, r, s: ops.conv_backward(p, q, r, s, tr, tc, tp, conv.kid),
                                 x, y, w, g, a, b, c)
    _check(("dx", "dy", "dw", "gg"), fused, composed, tol_of(problem))
    oracle = TorchConv(R.Problem.from_spec(problem), torch.float64)
    want = _oracle_second_order(lambda p, q, r: oracle(p, q, r, torch.tensor(rows), torch.tensor(cols)), x, y, w, g, a, b, c)
    for nm, got, ref in zip(("dx", "dy", "dw", "gg"), fused, want):
        err = R.normalized_error(got.cpu().numpy(), ref)
        assert err <= tol_of(problem), (nm, err)
    # no edges: the weight gradient is a sum over nothing
    none = torch.zeros(0, dtype=torch.int64, device="cuda")
    out = ops.conv_double_backward(x, y[:0], w, g, a, b[:0], c, none, none, none, conv.kid)
    assert float(out[2].abs().max()) == 0.0 and float(out[0].abs().max()) == 0.0


def test_conv_single_kernel_variant(monkeypatch):
    """The optional single-kernel form (both results from one walk; OEQ_AMD_TUNE=dd_merge=1)."""
    monkeypatch.setenv("OEQ_AMD_TUNE", "dd_merge=1")
    for name, make in (("odd", _odd), ("cfg2", P.config2_nequip_uvu), ("cfg3", P.config3_mace_uvu)):
        test_conv_fused_matches_composition(name, make, 0, True, monkeypatch)


def test_conv_fused_isolated_nodes_and_empty():
    """Nodes without edges get zero rows; an empty edge list gives zero node gradients."""
    problem = P.config2_nequip_uvu()
    conv = oeq.TensorProductConv(problem, deterministic=True)
    e = ops.get_entry(conv.kid)
    rng = np.random.default_rng(7)
    n = 9
    rows = np.array([1, 1, 4, 4, 4, 7], np.int64)
    cols = np.array([4, 7, 1, 4, 8, 1], np.int64)
    perm = np.argsort(cols, kind="stable").astype(np.int64)
    for E, (r_, c_, p_) in ((6, (rows, cols, perm)), (0, (rows[:0], cols[:0], perm[:0]))):
        tr, tc, tp = (torch.tensor(v, device="cuda") for v in (r_, c_, p_))
        x, a = (_rand(rng, (n, e.L1), np.float32) for _ in range(2))
        y, b = (_rand(rng, (E, e.L2), np.float32) for _ in range(2))
        w, c = (_rand(rng, (E, e.WN), np.float32) for _ in range(2))
        g = _rand(rng, (n, e.L3), np.float32)
        fused = ops.conv_double_backward(x, y, w, g, a, b, c, tr, tc, tp, conv.kid)
        composed = ops._second_order(lambda p, q, r: ops.conv_forward(p, q, r, tr, tc, tp, conv.kid),
                                     lambda p, q, r, s: ops.conv_backward(p, q, r, s, tr, tc, tp, conv.kid),
                                     x, y, w, g, a, b, c)
        if E:
            _check(("dx", "dy", "dw", "gg"), fused, composed, 1e-5)
            assert float(fused[3][0].abs().max()) == 0.0  # node 0 receives nothing
        else:
            assert float(fused[0].abs().max()) == 0.0 and float(fused[3].abs().max()) == 0.0


def test_edge_cases_and_refusals(monkeypatch):
    """Empty batch: nothing launched, empty results (a shared weight gradient: zeros). Kernel sets without
    second-order kernels (built with them switched off) refuse the fused entry point loudly; autograd then composes
    first-order kernels instead."""
    problem = P.config2_nequip_uvu()
    tp = oeq.TensorProduct(problem)
    e = ops.get_entry(tp.kid)
    empty = [torch.zeros((0, n), device="cuda") for n in (e.L1, e.L2, e.WN, e.L3, e.L1, e.L2, e.WN)]
    out = ops.tp_double_backward(*empty, tp.kid)
    assert [tuple(t.shape) for t in out] == [(0, e.L1), (0, e.L2), (0, e.WN), (0, e.L3)]
    tsh = oeq.TensorProduct(_shared(problem))
    empty[2] = empty[6] = torch.rand(e.WN, device="cuda")
    out = ops.tp_double_backward(*empty, tsh.kid)
    assert tuple(out[2].shape) == (e.WN,) and float(out[2].abs().max()) == 0.0
    # every batch kernel set carries the pair by default; built without it, the entry point refuses
    monkeypatch.setenv("OEQ_AMD_TUNE", "uvw_mfma_dd=0")
    tps = oeq.TensorProduct(P.config4_uvw_shared())
    es = ops.get_entry(tps.kid)
    assert not es.kernels().has_double_backward()
    rng = np.random.default_rng(1)
    x, a = (_rand(rng, (9, es.L1), np.float32) for _ in range(2))
    y, b = (_rand(rng, (9, es.L2), np.float32) for _ in range(2))
    w, c = (_rand(rng, (es.WN,), np.float32) for _ in range(2))
    g = _rand(rng, (9, es.L3), np.float32)
    with pytest.raises(RuntimeError, match="no second-order kernels"):
        ops.tp_double_backward(x, y, w, g, a, b, c, tps.kid)
    # through autograd the shared-weight problem still differentiates twice (composition)
    ts = [t.clone().requires_grad_(True) for t in (x, y, w)]
    first = torch.autograd.grad(tps(*ts), ts, g, create_graph=True)
    second = torch.autograd.grad(sum((t ** 2).sum() for t in first), ts)
    assert all(torch.isfinite(t).all() for t in second)


def test_path_limit_of_the_fused_convolution_kernels(monkeypatch):
    """Convolutions with up to 96 paths get fused second-order kernels (SevenNet main layer: 38, NequIP
    benzene: 68); beyond the limit (lowered here through its knob) the kernel set has none and autograd
    composes first-order kernels."""
    from openequivariance_amd.codegen.lower import lower
    low = lower(P.seven_net_problems()[1])
    assert uvu_double.supported(low, conv=True) and uvu_double.supported(low)
    conv = oeq.TensorProductConv(P.seven_net_problems()[1], deterministic=True)
    assert ops.get_entry(conv.kid).kernels().has_double_backward()
    monkeypatch.setenv("OEQ_AMD_TUNE", "dd_maxp=32")
    assert not uvu_double.supported(low, conv=True)
    conv = oeq.TensorProductConv(P.seven_net_problems()[1], deterministic=True)
    assert not ops.get_entry(conv.kid).kernels().has_double_backward()


@pytest.mark.parametrize("which", ["tp", "conv"])
def test_force_training_pattern(which, monkeypatch):
    """loss = f(first gradients); its gradient w.r.t. the inputs with the fused kernels equals the
    one with the composed first-order kernels."""
    problem = P.config2_nequip_uvu()
    rng = np.random.default_rng(8)
    gph = _graph(40)
    n, E = gph.coords.shape[0], gph.nnz
    if which == "tp":
        mod = oeq.TensorProduct(problem)
        rows_n, extra = E, ()
    else:
        mod = oeq.TensorProductConv(problem, deterministic=True)
        rows_n, extra = n, tuple(torch.tensor(v, device="cuda") for v in (gph.rows, gph.cols, gph.transpose_perm))
    e = ops.get_entry(mod.kid)
    base = [_rand(rng, (rows_n, e.L1), np.float32), _rand(rng, (E, e.L2), np.float32),
            _rand(rng, (E, e.WN), np.float32)]
    g = _rand(rng, (rows_n, e.L3), np.float32)
    results = []
    for fused in (True, False):
        monkeypatch.setattr(ops, "FUSED_DOUBLE_BACKWARD", fused)
        ts = [t.clone().requires_grad_(True) for t in base]
        z = mod(*ts, *extra)
        first = torch.autograd.grad(z, ts, g, create_graph=True)
        loss = sum((t ** 2).sum() for t in first)
        results.append([t.detach() for t in torch.autograd.grad(loss, ts)])
    _check(("x", "y", "w"), results[0], results[1], 1e-5)


# ---------------------------------------------------------------------------
# the fused kernels directly against float64 autograd through the CPU restatement
# ---------------------------------------------------------------------------

def _oracle_second_order(fn, x, y, w, g, a, b, c):
    """Gradients of <a, dx> + <b, dy> + <c, dw> with respect to (x, y, w, g), where (dx, dy, dw) is the
    backward of z = fn(x, y, w) for the output gradient g; float64 autograd on the host."""
    t = [torch.tensor(v.double().cpu().numpy(), requires_grad=True) for v in (x, y, w, g)]
    cot = [torch.tensor(v.double().cpu().numpy()) for v in (a, b, c)]
    z = fn(*t[:3])
    first = torch.autograd.grad(z, t[:3], t[3], create_graph=True)
    s = sum((p * q).sum() for p, q in zip(cot, first))
    return [v.numpy() for v in torch.autograd.grad(s, t)]


ORACLE_TP = [("cfg1", P.config1_single_uvu, 64), ("cfg2", P.config2_nequip_uvu, 33), ("cfg3", P.config3_mace_uvu, 9),
             ("cfg3-f64", lambda: _f64(P.config3_mace_uvu()), 5), ("folded-gaps", _folded, 17), ("odd", _odd, 40),
             ("cfg2-shared", lambda: _shared(P.config2_nequip_uvu()), 33),
             ("cfg3-shared-f64", lambda: _shared(_f64(P.config3_mace_uvu())), 5), ("odd-shared", lambda: _shared(_odd()), 40),
             ("uvw-fc", lambda: _fc(False), 33), ("uvw-fc-mul2-f64", lambda: _f64(_fc(False, "2x0e+3x1o")), 17),
             ("uvw-diffdock", lambda: P.diffdock_problems()[0], 9), ("uvw-e3tools-conv", lambda: P.e3tools_problems()[0], 9),
             ("uvw-fc-shared", lambda: _fc(True), 33), ("uvw-tetris-1-shared", lambda: P.tetris_poly_problems()[0], 17),
             ("uvw-tetris-2-shared-f64", lambda: _f64(P.tetris_poly_problems()[1]), 9),
             ("uvw-wide-shared", lambda: _wide_fc(True), 9),
             ("mfma-cfg4", P.config4_uvw_shared, 19), ("mfma-cfg4-f64", lambda: P.config4_uvw_shared(np.float64), 17),
             ("mfma-mixed", lambda: _fc_shared("64x0e+32x1o+16x2e", "1x0e+1x1o", "48x0e+80x1o+16x2e"), 21)]


@pytest.mark.parametrize("name,make,batch", ORACLE_TP, ids=[c[0] for c in ORACLE_TP])
def test_tp_fused_matches_float64_autograd(name, make, batch):
    from oracle.torch_ref import TorchTP
    problem = make()
    tp = oeq.TensorProduct(problem)
    e = ops.get_entry(tp.kid)
    assert e.kernels().has_double_backward()
    dt = np.dtype(problem.irrep_dtype)
    rng = np.random.default_rng(15)
    x, a = (_rand(rng, (batch, e.L1), dt) for _ in range(2))
    y, b = (_rand(rng, (batch, e.L2), dt) for _ in range(2))
    w, c = (_rand(rng, (e.WN,) if problem.shared_weights else (batch, e.WN), dt) for _ in range(2))
    g = _rand(rng, (batch, e.L3), dt)
    fused = ops.tp_double_backward(x, y, w, g, a, b, c, tp.kid)
    want = _oracle_second_order(TorchTP(R.Problem.from_spec(problem), torch.float64), x, y, w, g, a, b, c)
    for nm, got, ref in zip(("dx", "dy", "dw", "gg"), fused, want):
        err = R.normalized_error(got.cpu().numpy(), ref)
        assert err <= tol_of(problem), (nm, err)


ORACLE_CONV = [("cfg2", P.config2_nequip_uvu), ("cfg5", P.config5_mace_conv),
               ("cfg5-f64", lambda: _f64(P.config5_mace_conv())), ("folded-gaps", _folded), ("odd", _odd),
               # many paths per output block: kernel A walks smaller output segments (38 and 68 paths)
               ("sevennet-main", lambda: P.seven_net_problems()[1]), ("nequip-benzene", lambda: P.nequip_problems()[3]),
               ("uvw-fc", lambda: _fc(False)), ("uvw-fc-mul2-f64", lambda: _f64(_fc(False, "2x0e+3x1o"))),
               ("uvw-diffdock", lambda: P.diffdock_problems()[0]), ("uvw-e3tools-conv", lambda: P.e3tools_problems()[0])]


@pytest.mark.parametrize("det", [True, False], ids=["sorted", "grouped"])
@pytest.mark.parametrize("name,make", ORACLE_CONV, ids=[c[0] for c in ORACLE_CONV])
def test_conv_fused_matches_float64_autograd(name, make, det):
    from oracle.torch_ref import TorchConv
    problem = make()
    gph = _graph(24)
    n, E = gph.coords.shape[0], gph.nnz
    conv = oeq.TensorProductConv(problem, deterministic=det)
    e = ops.get_entry(conv.kid)
    assert e.kernels().has_double_backward()
    dt = np.dtype(problem.irrep_dtype)
    rng = np.random.default_rng(16)
    if det:
        rows, cols, perm = gph.rows, gph.cols, gph.transpose_perm
    else:
        order = rng.permutation(E)
        rows, cols, perm = gph.rows[order], gph.cols[order], np.zeros(0, np.int64)
    tr, tc, tp = (torch.tensor(v, device="cuda") for v in (rows, cols, perm))
    x, a = (_rand(rng, (n, e.L1), dt) for _ in range(2))
    y, b = (_rand(rng, (E, e.L2), dt) for _ in range(2))
    w, c = (_rand(rng, (E, e.WN), dt) for _ in range(2))
    g = _rand(rng, (n, e.L3), dt)
    fused = ops.conv_double_backward(x, y, w, g, a, b, c, tr, tc, tp, conv.kid)
    oracle = TorchConv(R.Problem.from_spec(problem), torch.float64)
    want = _oracle_second_order(lambda p, q, r: oracle(p, q, r, torch.tensor(rows), torch.tensor(cols)),
                                x, y, w, g, a, b, c)
    for nm, got, ref in zip(("dx", "dy", "dw", "gg"), fused, want):
        err = R.normalized_error(got.cpu().numpy(), ref)
        assert err <= tol_of(problem), (nm, err)
