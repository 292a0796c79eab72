"""Shared helpers for the GPU parity tests."""

import numpy as np
import torch

from oracle import e3nn_ref as R

TOL = {np.dtype(np.float32): 1e-5, np.dtype(np.float64): 1e-12}


def tol_of(problem):
    """Max normalised error max|a-b|/max|b| allowed against the float64 oracle."""
    return TOL[np.dtype(problem.irrep_dtype)]


def tp_inputs(problem, B, seed=0, dist="uniform"):
    """Seeded buffers in the reference's order in1, in2, weights, out_grad
    (openequivariance/openequivariance/benchmark/test_buffers.py:14-62)."""
    rng = np.random.default_rng(seed)
    dt = np.dtype(problem.irrep_dtype)
    draw = (lambda s: rng.uniform(size=s)) if dist == "uniform" else (lambda s: rng.normal(size=s))
    x = draw((B, problem.irreps_in1.dim)).astype(dt)
    y = draw((B, problem.irreps_in2.dim)).astype(dt)
    w = draw((problem.weight_numel,) if problem.shared_weights else (B, problem.weight_numel)).astype(dt)
    g = draw((B, problem.irreps_out.dim)).astype(dt)
    return x, y, w, g


def to_gpu(*arrays, requires_grad=False):
    return tuple(torch.tensor(a, device="cuda", requires_grad=requires_grad) for a in arrays)


def err(a, b):
    if isinstance(a, torch.Tensor):
        a = a.detach().cpu().numpy()
    return R.normalized_error(a, b)
