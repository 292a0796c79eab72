"""Single-instruction problems over the reference's grid of multiplicities and
irrep triples (tests/batch_test.py:145-264: powers of two, odd multiplicities 5..123,
wide rows up to 512, mul2 > 1, l up to 7), per-row weights, forward and backward
against the CPU oracle: every multiplicity with every one of the nine irrep triples, in
both precisions, as the reference's grid does."""

import numpy as np
import pytest
import torch

import openequivariance_amd as oeq
from oracle import e3nn_ref as R
from gpu_util import err, tol_of, tp_inputs

pytestmark = pytest.mark.gpu

MULS = [(1, 1, 1), (2, 1, 2), (4, 1, 4), (8, 1, 8), (16, 1, 16), (32, 1, 32), (5, 1, 5), (13, 1, 13), (19, 1, 19),
        (33, 1, 33), (49, 1, 49), (50, 1, 50), (64, 1, 64), (123, 1, 123), (128, 1, 128), (256, 1, 256),
        (512, 1, 512), (1, 2, 1), (1, 4, 1), (1, 16, 1), (1, 32, 1), (16, 3, 16), (16, 9, 16), (24, 24, 24),
        (32, 32, 32)]
IRS = [(0, 0, 0), (1, 1, 1), (1, 0, 1), (1, 2, 1), (2, 0, 2), (2, 2, 4), (2, 2, 2), (5, 3, 5), (7, 2, 5)]
UVW_MAX_MUL = 64  # the reference's uvw grid stops at 64 channels


def _grid(mode):
    out = []
    for n, m in enumerate(MULS):
        if mode == "uvw" and m[0] > UVW_MAX_MUL:
            continue
        for irs in IRS:
            for dtype in (np.float32, np.float64):
                out.append((mode, m, irs, dtype))
    return out


GRID = _grid("uvu") + _grid("uvw")


def _id(case):
    mode, m, i, dtype = case
    return f"{mode}-{m[0]}x{i[0]}e__x__{m[1]}x{i[1]}e---{m[2]}x{i[2]}e-{np.dtype(dtype).name}"


@pytest.mark.parametrize("case", GRID, ids=[_id(c) for c in GRID])
def test_single_instruction(case):
    mode, m, i, dtype = case
    problem = oeq.TPProblem(f"{m[0]}x{i[0]}e", f"{m[1]}x{i[1]}e", f"{m[2]}x{i[2]}e", [(0, 0, 0, mode, True)],
                            shared_weights=False, internal_weights=False, irrep_dtype=dtype, weight_dtype=dtype)
    tol = tol_of(problem)
    B = 19
    x, y, w, g = tp_inputs(problem, B, seed=GRID.index(case))
    ref = R.Problem.from_spec(problem)
    z_ref = R.tp_forward(ref, x, y, w)
    dx_ref, dy_ref, dw_ref = R.tp_backward(ref, x, y, w, g)
    tx, ty, tw = (torch.tensor(a, device="cuda", requires_grad=True) for a in (x, y, w))
    z = oeq.TensorProduct(problem)(tx, ty, tw)
    z.backward(torch.tensor(g, device="cuda"))
    assert err(z, z_ref) <= tol
    assert err(tx.grad, dx_ref) <= tol
    assert err(ty.grad, dy_ref) <= tol
    assert err(tw.grad, dw_ref) <= tol
