"""The allocation-free convolution forward (oeq_conv_forward_static), called through the C ABI: same bits
as oeq_conv_forward on two calls in a row (the second on a smaller graph, so that stale contents of the
library's scratch array would show), in caller-sorted and in device-grouped mode; sizes beyond the static
scratch and kernel sets not yet loaded on the device are refused with a message."""

import numpy as np
import pytest
import torch

from openequivariance_amd import runtime as rt
from openequivariance_amd._torch.tensor_product_conv import build_conv_module
from openequivariance_amd.core import problems as P
from openequivariance_amd.core.graph import CoordGraph, periodic_radius_graph

pytestmark = pytest.mark.gpu


def _case(n_nodes, deg, seed, sort, problem):
    coords, rows, cols, _ = periodic_radius_graph(n_nodes, deg, 5.0, seed)
    if sort:
        g = CoordGraph(coords, rows, cols)
        rows, cols = g.rows, g.cols
    else:
        perm = np.random.default_rng(seed).permutation(len(rows))
        rows, cols = rows[perm], cols[perm]
    gen = torch.Generator(device="cuda").manual_seed(seed)
    E = len(rows)
    X = torch.randn(n_nodes, problem.irreps_in1.dim, device="cuda", generator=gen)
    Y = torch.randn(E, problem.irreps_in2.dim, device="cuda", generator=gen)
    W = torch.randn(E, problem.weight_numel, device="cuda", generator=gen)
    return X, Y, W, torch.tensor(rows, device="cuda"), torch.tensor(cols, device="cuda")


@pytest.mark.parametrize("deterministic", [True, False], ids=["sorted", "grouped"])
def test_static_forward_matches_workspace_forward(deterministic):
    problem = P.config2_nequip_uvu()
    src, dims, descs = build_conv_module(problem, deterministic)
    ks = rt.get_kernel_set(src, dims, descs)
    L3 = problem.irreps_out.dim
    stream = torch.cuda.current_stream().cuda_stream
    for n_nodes, deg, seed in ((300, 12, 1), (120, 6, 2)):  # the second call is the smaller one
        X, Y, W, r, c = _case(n_nodes, deg, seed, deterministic, problem)
        E = r.shape[0]
        want = torch.full((n_nodes, L3), float("nan"), device="cuda")
        nb = ks.conv_forward_workspace_bytes(n_nodes, E)
        assert 0 < nb <= rt.load_library().oeq_static_scratch_bytes()
        ws = torch.empty(nb, dtype=torch.uint8, device="cuda")
        ks.conv_forward(n_nodes, E, X.data_ptr(), Y.data_ptr(), W.data_ptr(), want.data_ptr(), r.data_ptr(),
                        c.data_ptr(), ws.data_ptr(), nb, stream)
        got = torch.full((n_nodes, L3), float("nan"), device="cuda")
        torch.cuda.synchronize()
        # free device memory as the driver reports it (hipMemGetInfo): an allocation inside the library would
        # show here, which torch's own allocator statistics could not see
        before = torch.cuda.mem_get_info()[0]
        ks.conv_forward_static(n_nodes, E, X.data_ptr(), Y.data_ptr(), W.data_ptr(), got.data_ptr(), r.data_ptr(),
                               c.data_ptr(), stream)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == before
        assert torch.isfinite(want).all()
        assert torch.equal(got, want), (n_nodes, deterministic)


def test_static_forward_under_graph_capture():
    """The call records nothing but kernel launches, so a HIP graph can hold it: every replay (with eager
    work and synchronisations in between) reproduces the eager result."""
    problem = P.config2_nequip_uvu()
    src, dims, descs = build_conv_module(problem, False)
    ks = rt.get_kernel_set(src, dims, descs)
    X, Y, W, r, c = _case(200, 8, 4, False, problem)
    n_nodes, E = X.shape[0], r.shape[0]
    want = torch.empty(n_nodes, problem.irreps_out.dim, device="cuda")
    nb = ks.conv_forward_workspace_bytes(n_nodes, E)
    ws = torch.empty(nb, dtype=torch.uint8, device="cuda")
    ks.conv_forward(n_nodes, E, X.data_ptr(), Y.data_ptr(), W.data_ptr(), want.data_ptr(), r.data_ptr(), c.data_ptr(),
                    ws.data_ptr(), nb, torch.cuda.current_stream().cuda_stream)  # also loads the kernels
    got = torch.zeros_like(want)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up on the capture stream
        ks.conv_forward_static(n_nodes, E, X.data_ptr(), Y.data_ptr(), W.data_ptr(), got.data_ptr(), r.data_ptr(),
                               c.data_ptr(), side.cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ks.conv_forward_static(n_nodes, E, X.data_ptr(), Y.data_ptr(), W.data_ptr(), got.data_ptr(), r.data_ptr(),
                               c.data_ptr(), torch.cuda.current_stream().cuda_stream)
    for rep in range(3):
        got.fill_(float("nan"))
        torch.randn(1 << 20, device="cuda").sum().item()  # eager work and a synchronisation between replays
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got, want), rep


def test_static_forward_refuses_what_it_cannot_do():
    problem = P.config1_single_uvu()
    src, dims, descs = build_conv_module(problem, True)
    # a kernel set of its own (not the cached one other tests may have loaded on the device already)
    ks = rt.KernelSet(rt.compile_source(src), dims, descs)
    lib = rt.load_library()
    assert lib.oeq_static_scratch_bytes() == 32 << 20
    with pytest.raises(rt.OeqError, match="static buffer holds"):
        ks.conv_forward_static(5_000_000, 10, 0, 0, 0, 0, 0, 0, 0)  # refused on size alone: nothing is touched
    X, Y, W, r, c = _case(40, 6, 3, True, problem)
    out = torch.empty(40, problem.irreps_out.dim, device="cuda")
    with pytest.raises(rt.OeqError, match="not loaded on this device"):
        ks.conv_forward_static(40, r.shape[0], X.data_ptr(), Y.data_ptr(), W.data_ptr(), out.data_ptr(), r.data_ptr(),
                               c.data_ptr(), torch.cuda.current_stream().cuda_stream)
