"""The ops (first- and second-order) can be recorded into a HIP graph (torch.cuda.graph): every launch goes to the
capturing stream, buffers are cleared by a fill kernel rather than a memset node, and scratch
comes from torch's capture-aware allocator. Each graph is replayed several times with new
input values and eager work in between, and every replay is compared with the eager result."""

import pytest
import torch

import openequivariance_amd as oeq
from openequivariance_amd._torch import ops
from openequivariance_amd.core import problems as P
from openequivariance_amd.core.graph import CoordGraph, periodic_radius_graph

pytestmark = pytest.mark.gpu


def _replay_and_compare(eager_fn, static_inputs, make_new_values, tol=0.0):
    """``tol`` > 0: outputs that depend on float atomics are compared by max normalised error."""
    # warm-up on a side stream (compiles and loads the kernels, primes the allocator)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            eager_fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = eager_fn()
    for seed in range(4):
        for t, v in zip(static_inputs, make_new_values(seed)):
            t.copy_(v)
        expected = [o.clone() for o in eager_fn()]
        torch.cuda.synchronize()
        for o in captured:
            o.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(captured, expected):
            if tol:
                assert torch.isfinite(got).all() and (got - want).abs().max() <= tol * want.abs().max(), seed
            else:
                assert torch.equal(got, want), seed
        (static_inputs[0] * 2).sum().item()  # unrelated eager work between replays


@pytest.mark.parametrize("make", [P.config2_nequip_uvu, P.config4_uvw_shared], ids=["uvu", "uvw-mfma"])
def test_tensor_product_in_a_graph(make):
    problem = make()
    tp = oeq.TensorProduct(problem)
    B = 200
    gen = torch.Generator(device="cuda").manual_seed(1)
    x = torch.randn(B, problem.irreps_in1.dim, device="cuda", generator=gen)
    y = torch.randn(B, problem.irreps_in2.dim, device="cuda", generator=gen)
    w = torch.randn((problem.weight_numel,) if problem.shared_weights else (B, problem.weight_numel), device="cuda",
                    generator=gen)
    g = torch.randn(B, problem.irreps_out.dim, device="cuda", generator=gen)

    def step():
        z = ops.tp_forward(x, y, w, tp.kid)
        dx, dy, dw = ops.tp_backward(x, y, w, g, tp.kid)
        out = [z, dx, dy, dw]
        if ops.get_entry(tp.kid).kernels().has_double_backward():  # fused second-order kernels
            out += list(ops.tp_double_backward(x, y, w, g, dx, dy, dw, tp.kid))
        return out

    def new_values(seed):
        gen2 = torch.Generator(device="cuda").manual_seed(100 + seed)
        return [torch.randn(t.shape, device="cuda", generator=gen2) for t in (x, y, w, g)]

    _replay_and_compare(step, [x, y, w, g], new_values)


@pytest.mark.parametrize("deterministic", [True, False], ids=["sorted", "grouped"])
def test_convolution_in_a_graph(deterministic):
    problem = P.config5_mace_conv()
    coords, rows, cols, _ = periodic_radius_graph(60, 8, 5.0, 3)
    gr = CoordGraph(coords, rows, cols)
    n, E = 60, gr.nnz
    tr, tc, tp = (torch.tensor(a, device="cuda") for a in (gr.rows, gr.cols, gr.transpose_perm))
    conv = oeq.TensorProductConv(problem, deterministic=deterministic)
    gen = torch.Generator(device="cuda").manual_seed(2)
    X = torch.randn(n, problem.irreps_in1.dim, device="cuda", generator=gen)
    Y = torch.randn(E, problem.irreps_in2.dim, device="cuda", generator=gen)
    W = torch.randn(E, problem.weight_numel, device="cuda", generator=gen)
    G = torch.randn(n, problem.irreps_out.dim, device="cuda", generator=gen)

    def step():
        z = ops.conv_forward(X, Y, W, tr, tc, tp, conv.kid)
        dx, dy, dw = ops.conv_backward(X, Y, W, G, tr, tc, tp, conv.kid)
        second = ops.conv_double_backward(X, Y, W, G, dx, dy, dw, tr, tc, tp, conv.kid)
        return [z, dx, dy, dw] + list(second)

    def new_values(seed):
        gen2 = torch.Generator(device="cuda").manual_seed(200 + seed)
        return [torch.randn(t.shape, device="cuda", generator=gen2) for t in (X, Y, W, G)]

    # deterministic=False accumulates the sender gradient with float atomics (and what is derived from it here)
    _replay_and_compare(step, [X, Y, W, G], new_values, tol=0.0 if deterministic else 2e-5)


@pytest.mark.parametrize("deterministic", [True, False], ids=["sorted", "grouped"])
def test_uvw_convolution_in_a_graph(deterministic):
    """The fused 'uvw' convolution (per-edge weights): index build, receiver walk, per-edge backward and the ordered
    sender-side sum are all recorded; both modes are bitwise reproducible, so every replay equals the eager result."""
    problem = P.diffdock_problems()[0]
    coords, rows, cols, _ = periodic_radius_graph(60, 8, 5.0, 3)
    gr = CoordGraph(coords, rows, cols)
    n, E = 60, gr.nnz
    tr, tc, tp = (torch.tensor(a, device="cuda") for a in (gr.rows, gr.cols, gr.transpose_perm))
    conv = oeq.TensorProductConv(problem, deterministic=deterministic)
    assert not ops.get_entry(conv.kid).unfused
    gen = torch.Generator(device="cuda").manual_seed(2)
    X = torch.randn(n, problem.irreps_in1.dim, device="cuda", generator=gen)
    Y = torch.randn(E, problem.irreps_in2.dim, device="cuda", generator=gen)
    W = torch.randn(E, problem.weight_numel, device="cuda", generator=gen)
    G = torch.randn(n, problem.irreps_out.dim, device="cuda", generator=gen)

    def step():
        z = ops.conv_forward(X, Y, W, tr, tc, tp, conv.kid)
        return [z] + list(ops.conv_backward(X, Y, W, G, tr, tc, tp, conv.kid))

    def new_values(seed):
        gen2 = torch.Generator(device="cuda").manual_seed(300 + seed)
        return [torch.randn(t.shape, device="cuda", generator=gen2) for t in (X, Y, W, G)]

    _replay_and_compare(step, [X, Y, W, G], new_values)
