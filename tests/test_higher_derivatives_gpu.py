"""Second and third derivatives of the tensor product and of the convolution
(torch autograd through the custom ops) against autograd through the CPU einsum
restatement in float64. The reference checks the same quantities in
tests/batch_test.py:88-102 and tests/conv_test.py:129-171."""

import numpy as np
import pytest
import torch

import openequivariance_amd as oeq
from openequivariance_amd.core import problems as P
from openequivariance_amd.core.graph import CoordGraph, periodic_radius_graph
from oracle import e3nn_ref as R
from oracle.torch_ref import TorchConv, TorchTP

pytestmark = pytest.mark.gpu

TOL = 1e-10


def _uvu():
    return oeq.TPProblem("5x1e+3x2e", "2x1e+1x0e", "5x1e+3x2e+5x0e",
                         [(0, 0, 0, "uvu", True), (0, 1, 0, "uvu", True), (1, 0, 1, "uvu", True),
                          (0, 0, 2, "uvu", True)], shared_weights=False, internal_weights=False,
                         irrep_dtype=np.float64, weight_dtype=np.float64)


def _uvw(shared):
    return P.FullyConnectedTPProblem("4x0e+3x1o", "1x0e+2x1o", "5x0e+2x1o+1x2e", shared_weights=shared,
                                     internal_weights=False, irrep_dtype=np.float64, weight_dtype=np.float64)


def _nequip64():
    return P.config2_nequip_uvu(np.float64)


PROBLEMS = [("uvu", _uvu), ("uvw", lambda: _uvw(False)), ("uvw-shared", lambda: _uvw(True)), ("cfg2-f64", _nequip64)]


def _derivative_tower(fn, tensors, g):
    """First, second and third order quantities of z = fn(*tensors) contracted with g."""
    z = fn(*tensors)
    first = torch.autograd.grad(z, tensors, g, create_graph=True)
    s1 = sum((t ** 2).sum() for t in first)
    second = torch.autograd.grad(s1, tensors + (g,), create_graph=True)
    s2 = sum((t ** 2).sum() for t in second)
    third = torch.autograd.grad(s2, tensors + (g,))
    return [z] + list(first) + list(second) + list(third)


def _compare(gpu_fn, cpu_fn, arrays, g):
    outs = []
    for fn, dev in ((cpu_fn, "cpu"), (gpu_fn, "cuda")):
        ts = tuple(torch.tensor(a, device=dev, requires_grad=True) for a in arrays)
        tg = torch.tensor(g, device=dev, requires_grad=True)
        outs.append([t.detach().cpu().numpy() for t in _derivative_tower(fn, ts, tg)])
    names = (["z"] + [f"d{n}" for n in "xyw"] + [f"dd{n}" for n in "xywg"] + [f"ddd{n}" for n in "xywg"])
    for name, a, b in zip(names, outs[1], outs[0]):
        assert R.normalized_error(a, b) <= TOL, name


@pytest.mark.parametrize("name,make", PROBLEMS, ids=[c[0] for c in PROBLEMS])
def test_tp_second_and_third_derivatives(name, make):
    problem = make()
    B = 11
    rng = np.random.default_rng(7)
    x = rng.normal(size=(B, problem.irreps_in1.dim))
    y = rng.normal(size=(B, problem.irreps_in2.dim))
    w = rng.normal(size=(problem.weight_numel,) if problem.shared_weights else (B, problem.weight_numel))
    g = rng.normal(size=(B, problem.irreps_out.dim))
    ref = TorchTP(R.Problem.from_spec(problem), torch.float64)
    _compare(oeq.TensorProduct(problem), ref, (x, y, w), g)


@pytest.mark.parametrize("det", [True, False], ids=["deterministic", "atomic"])
@pytest.mark.parametrize("name,make", PROBLEMS, ids=[c[0] for c in PROBLEMS])
def test_conv_second_and_third_derivatives(name, make, det):
    problem = make()
    if det and problem.shared_weights:
        pytest.skip("deterministic convolution needs per-edge weights")
    n = 14
    coords, rows, cols, _ = periodic_radius_graph(n, 4, 5.0, 2)
    keep = rows != 2  # one node receives nothing; the pattern is no longer symmetric
    graph = CoordGraph(coords, rows[keep], cols[keep])
    E = graph.nnz
    rng = np.random.default_rng(8)
    X = rng.normal(size=(n, problem.irreps_in1.dim))
    Y = rng.normal(size=(E, problem.irreps_in2.dim))
    W = rng.normal(size=(problem.weight_numel,) if problem.shared_weights else (E, problem.weight_numel))
    G = rng.normal(size=(n, problem.irreps_out.dim))
    ref = TorchConv(R.Problem.from_spec(problem), torch.float64)
    r_cpu, c_cpu = torch.tensor(graph.rows), torch.tensor(graph.cols)
    r_gpu, c_gpu = r_cpu.cuda(), c_cpu.cuda()
    perm = torch.tensor(graph.transpose_perm, device="cuda") if det else None
    conv = oeq.TensorProductConv(problem, deterministic=det)
    _compare(lambda a, b, c: conv(a, b, c, r_gpu, c_gpu, perm), lambda a, b, c: ref(a, b, c, r_cpu, c_cpu),
             (X, Y, W), G)
