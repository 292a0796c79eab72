"""Row layouts (`mul_ir` / `ir_mul`): the conversion helpers and the rule that
`ir_mul` is only defined for per-channel ('uvu') problems. Mirrors the reference's
checks in tests/input_validation_test.py:143-155 and tests/batch_test.py:309-380."""

import numpy as np
import pytest

import openequivariance_amd as oeq
from openequivariance_amd.core.layout import layout_permutation, transpose_irrep_layout


def test_permutation_by_definition():
    irreps = oeq.Irreps("3x1e+2x0e+4x2o")
    x = np.arange(2 * irreps.dim, dtype=np.float64).reshape(2, irreps.dim)
    y = transpose_irrep_layout(x, irreps, "mul_ir", "ir_mul")
    off = 0
    for mul, ir in irreps:
        for u in range(mul):
            for i in range(ir.dim):
                assert y[1, off + i * mul + u] == x[1, off + u * ir.dim + i]
        off += mul * ir.dim
    back = transpose_irrep_layout(y, irreps, "ir_mul", "mul_ir")
    assert np.array_equal(back, x)
    same = transpose_irrep_layout(x, irreps, "mul_ir", "mul_ir")
    assert np.array_equal(same, x) and same is not x
    # the two directions are inverse permutations of each other
    a = layout_permutation(irreps, "mul_ir", "ir_mul")
    b = layout_permutation(irreps, "ir_mul", "mul_ir")
    assert np.array_equal(a[b], np.arange(irreps.dim))


def test_scalars_and_single_channels_do_not_move():
    irreps = oeq.Irreps("7x0e+1x3o")
    assert np.array_equal(layout_permutation(irreps, "mul_ir", "ir_mul"), np.arange(irreps.dim))


def test_torch_transpose_irreps():
    import torch

    irreps = oeq.Irreps("5x5e+2x1o")
    x = torch.randn(3, 4, irreps.dim, dtype=torch.float64, requires_grad=True)
    y = oeq.transpose_irreps(x, irreps, "mul_ir", "ir_mul")
    assert y.shape == x.shape and y.dtype == x.dtype
    ref = transpose_irrep_layout(x.detach().numpy(), irreps, "mul_ir", "ir_mul")
    assert np.array_equal(y.detach().numpy(), ref)
    assert torch.equal(oeq.transpose_irreps(y, irreps, "ir_mul", "mul_ir"), x)
    # differentiable: the gradient of sum(c * y) is c carried back through the permutation
    c = torch.randn_like(y)
    (y * c).sum().backward()
    assert torch.equal(x.grad, oeq.transpose_irreps(c, irreps, "ir_mul", "mul_ir"))
    same = oeq.transpose_irreps(x, irreps, "ir_mul", "ir_mul")
    assert torch.equal(same, x) and same.data_ptr() != x.data_ptr()
    with pytest.raises(ValueError, match="Unsupported src_layout"):
        oeq.transpose_irreps(x, irreps, "mulir", "ir_mul")
    with pytest.raises(ValueError, match="Unsupported dst_layout"):
        oeq.transpose_irreps(x, irreps, "mul_ir", "irmul")
    with pytest.raises(TypeError):
        oeq.transpose_irreps(x.detach().numpy(), irreps, "mul_ir", "ir_mul")


def test_ir_mul_rejects_uvw_problem():
    problem = oeq.TPProblem("2x0e", "1x0e", "2x0e", [(0, 0, 0, "uvw", True)], shared_weights=False,
                            internal_weights=False, layout="ir_mul")
    with pytest.raises(AssertionError, match="layout='ir_mul'"):
        oeq.TensorProduct(problem)
    with pytest.raises(AssertionError):
        oeq.TPProblem("2x0e", "1x0e", "2x0e", [(0, 0, 0, "uvu", True)], layout="mul_mul")


def test_ir_mul_kernels_compile_for_gfx950():
    from openequivariance_amd import runtime as rt
    from openequivariance_amd.codegen import uvu
    from openequivariance_amd.codegen.lower import lower
    from openequivariance_amd.core import problems as P

    problem = P.config5_mace_conv()
    problem.layout = "ir_mul"
    low = lower(problem)
    assert low.ir_mul
    for src in (uvu.tp_module(low)[0], uvu.conv_module(low, True)[0], uvu.conv_module(low, False)[0]):
        assert len(rt.compile_source(src)) > 0
