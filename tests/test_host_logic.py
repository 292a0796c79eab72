"""Host-side logic that needs no GPU: the description a kernel set is rebuilt from in another process
(core/spec.py: problem_to_dict / problem_from_dict; _torch/ops.py: make_spec / spec_hash) and the factored form
of the shared-weight 'uvw' convolution (core/problems.py: factor_shared_uvw), the latter against the oracle."""

import json

import numpy as np
import pytest

import openequivariance_amd as oeq
from openequivariance_amd.core import problems as P
from openequivariance_amd.core.graph import CoordGraph
from openequivariance_amd.core.spec import problem_from_dict, problem_to_dict
from oracle import e3nn_ref as R


def _zoo():
    out = [P.config1_single_uvu(), P.config2_nequip_uvu(np.float64), P.config4_uvw_shared(), P.config5_mace_conv()]
    out += P.diffdock_problems()[:1] + P.seven_net_problems()[:2]
    weighted = oeq.TPProblem("5x1e+3x2e", "2x1e+1x0e", "5x1e+3x2e+5x0e",
                             [(0, 0, 0, "uvu", True, 0.37), (0, 1, 0, "uvu", True), (1, 0, 1, "uvu", True, 2.5),
                              (0, 0, 2, "uvu", True)], shared_weights=True, internal_weights=False,
                             irrep_normalization="norm", path_normalization="path", label="weighted paths")
    ir_mul = P.config2_nequip_uvu().clone()
    ir_mul.layout = "ir_mul"
    return out + [weighted, ir_mul]


@pytest.mark.parametrize("problem", _zoo(), ids=lambda p: p.label)
def test_problem_description_round_trip(problem):
    d = problem_to_dict(problem)
    text = json.dumps(d, sort_keys=True)
    back = problem_from_dict(json.loads(text))
    assert str(back.irreps_in1) == str(problem.irreps_in1) and str(back.irreps_out) == str(problem.irreps_out)
    assert str(back.irreps_in2) == str(problem.irreps_in2)
    assert back.shared_weights == problem.shared_weights and back.internal_weights == problem.internal_weights
    assert np.dtype(back.irrep_dtype) == np.dtype(problem.irrep_dtype) and back.layout == problem.layout
    assert back.weight_numel == problem.weight_numel and back.label == problem.label
    assert len(back.instructions) == len(problem.instructions)
    for a, b in zip(back.instructions, problem.instructions):
        assert (a.i_in1, a.i_in2, a.i_out, a.connection_mode, a.has_weight) == \
               (b.i_in1, b.i_in2, b.i_out, b.connection_mode, b.has_weight)
        assert a.path_weight == b.path_weight, "path weights travel as hexadecimal floats: no rounding"
        assert tuple(a.path_shape) == tuple(b.path_shape)
    # the description of the copy is the same text: a fixed point
    assert json.dumps(problem_to_dict(back), sort_keys=True) == text


def test_kernel_set_id_is_a_function_of_the_description(monkeypatch):
    from openequivariance_amd._torch import ops
    monkeypatch.setenv("OEQ_AMD_TUNE", "")
    p = P.config2_nequip_uvu()
    s1, s2 = ops.make_spec("conv", p, True, False), ops.make_spec("conv", P.config2_nequip_uvu(), True, False)
    assert s1 == s2 and ops.spec_hash(s1) == ops.spec_hash(s2) and 0 <= ops.spec_hash(s1) < 2 ** 63
    others = [ops.make_spec("conv", p, False, False), ops.make_spec("conv", p, True, True), ops.make_spec("tp", p),
              ops.make_spec("conv", P.config2_nequip_uvu(np.float64), True, False)]
    monkeypatch.setenv("OEQ_AMD_TUNE", "conv_hub=64")
    others.append(ops.make_spec("conv", p, True, False))  # the knobs in force are part of the description
    ids = {ops.spec_hash(s) for s in others}
    assert len(ids) == len(others) and ops.spec_hash(s1) not in ids
    # an entry made from the bytes alone knows the problem's shape (kernels are not built here)
    entry = ops._entry_from_spec(s1)
    assert (entry.L1, entry.L2, entry.L3, entry.WN) == (p.irreps_in1.dim, p.irreps_in2.dim, p.irreps_out.dim,
                                                        p.weight_numel)
    assert entry.deterministic and bytes(entry.spec.numpy()) == s1
    with pytest.raises(RuntimeError):
        ops._entry_from_spec(b'{"v": 7}')


def _fc(in1, in2, out, shared=True):
    return P.FullyConnectedTPProblem(in1, in2, out, shared_weights=shared, internal_weights=False, label=f"fc {in1}")


def test_which_problems_factor():
    assert P.factor_shared_uvw(P.config4_uvw_shared()) is not None
    assert P.factor_shared_uvw(_fc("4x0e+3x1o", "1x0e+1x1o", "5x0e+2x1o", shared=False)) is None, "per-edge weights"
    assert P.factor_shared_uvw(_fc("4x0e+3x1o", "2x0e+1x1o", "5x0e+2x1o")) is None, "second operand with channels"
    assert P.factor_shared_uvw(P.config2_nequip_uvu()) is None, "'uvu' has no channel mix to factor out"


@pytest.mark.parametrize("make", [lambda: _fc("4x0e+3x1o+2x2e", "1x0e+1x1o+1x2e", "5x0e+2x1o+3x2e"),
                                  lambda: _fc("6x1o", "1x1o", "2x0e+3x1e+1x2e"),
                                  lambda: P.config4_uvw_shared(np.float64)], ids=["mixed", "one-input", "cfg4"])
def test_factored_convolution_equals_the_per_edge_one(make):
    """sum_e W (x_e (x) y_e) = W sum_e (x_e (x) y_e): the oracle's convolution of the original problem against the
    oracle's convolution of the contraction problem followed by its channel mix on one row per node."""
    problem = make()
    a, b = P.factor_shared_uvw(problem)
    rng = np.random.default_rng(0)
    n, E = 7, 40
    rows, cols = rng.integers(0, n, size=E), rng.integers(0, n, size=E)
    g = CoordGraph(np.zeros((n, 3)), rows, cols)
    X = rng.normal(size=(n, problem.irreps_in1.dim))
    Y = rng.normal(size=(g.nnz, problem.irreps_in2.dim))
    W = rng.normal(size=(problem.weight_numel,))
    want = R.conv_forward(R.Problem.from_spec(problem), X, Y, W, g.rows, g.cols)
    mid = R.conv_forward(R.Problem.from_spec(a), X, Y, np.ones(a.weight_numel), g.rows, g.cols)
    got = R.tp_forward(R.Problem.from_spec(b), mid, np.ones((n, 1)), W)
    assert np.abs(got - want).max() <= 1e-12 * max(1.0, np.abs(want).max())
    # and the weight gradient comes from the mix alone, the operand gradients through both
    G = rng.normal(size=want.shape)
    dx_ref, dy_ref, dw_ref = R.conv_backward(R.Problem.from_spec(problem), X, Y, W, G, g.rows, g.cols)
    dmid, _, dw = R.tp_backward(R.Problem.from_spec(b), mid, np.ones((n, 1)), W, G)
    dx, dy, _ = R.conv_backward(R.Problem.from_spec(a), X, Y, np.ones(a.weight_numel), dmid, g.rows, g.cols)
    scale = lambda v: max(1.0, np.abs(v).max())
    assert np.abs(dw - dw_ref).max() <= 1e-12 * scale(dw_ref)
    assert np.abs(dx - dx_ref).max() <= 1e-12 * scale(dx_ref)
    assert np.abs(dy - dy_ref).max() <= 1e-12 * scale(dy_ref)
