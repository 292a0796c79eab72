"""``TensorProduct``: batched CG tensor product as a torch module.

Drop-in for the reference class
(openequivariance/openequivariance/_torch/TensorProduct.py:19-178): same
constructor, ``forward(x, y, W)``, ``.to(dtype)`` re-specialisation, pickling
by constructor arguments, and weight-reordering helpers (identities here: the
kernels read weights in e3nn order directly).
"""

from __future__ import annotations

import torch

from ..codegen.lower import lower
from ..core.spec import TPProblem
from . import ops
from .benchmarking import TensorProductTiming
from .utils import oeq_to_torch_dtype, torch_to_oeq_dtype, compute_units


def build_tp_module(problem: TPProblem):
    low = lower(problem)
    if low.mode == "uvu":
        from ..codegen import uvu
        return uvu.tp_module(low, compute_units())
    from ..codegen import uvw
    return uvw.tp_module(low, compute_units())


class TensorProduct(TensorProductTiming, torch.nn.Module):
    r"""Drop-in replacement for ``o3.TensorProduct`` from e3nn with per-problem
    HIP kernels. Supports 'uvu' and 'uvw' instructions with weights.

    :param problem: specification of the tensor product.
    :param use_opaque: deprecated, ignored.
    """

    def __init__(self, problem: TPProblem, torch_op: bool = True, use_opaque: bool = False):
        torch.nn.Module.__init__(self)
        self.input_args = {"problem": problem, "torch_op": torch_op, "use_opaque": use_opaque}
        self._init_class()

    def _init_class(self):
        problem: TPProblem = self.input_args["problem"].clone()
        self.config = problem
        low = lower(problem)  # validates (asserts) before anything else happens
        self.L1, self.L2, self.L3 = problem.irreps_in1, problem.irreps_in2, problem.irreps_out
        self.L3_dim = low.L3
        self.weight_numel = problem.weight_numel
        self.is_uvw = low.mode == "uvw"
        self._low = low
        # The ops are handed the kernel set's description (a hash and the bytes it is the hash of), so that a
        # traced or exported graph can rebuild the kernels in a process that never constructed this module.
        # A plain attribute, not a buffer: it stays in host memory whatever the module is moved to.
        self.kid = ops.register_spec(ops.make_spec("tp", problem))
        self.spec = ops.get_entry(self.kid).spec

    # -- dtype handling (TensorProduct.py:55-92) ---------------------------------
    def to(self, *args, **kwargs):
        _device, dtype, _nb, _fmt = torch._C._nn._parse_to(*args, **kwargs)
        if dtype is not None and dtype.is_floating_point:
            updated = self.input_args["problem"].clone()
            updated.irrep_dtype = torch_to_oeq_dtype(dtype)
            updated.weight_dtype = torch_to_oeq_dtype(dtype)
            self.input_args["problem"] = updated
            self._init_class()
        torch.nn.Module.to(self, *args, **kwargs)
        return self

    def _apply(self, fn, recurse=True):
        if getattr(self, "_applying", False):
            return super()._apply(fn, recurse)
        current = oeq_to_torch_dtype(self.input_args["problem"].irrep_dtype)
        probe = fn(torch.tensor(0.0, dtype=current))
        if probe.dtype != current and probe.dtype.is_floating_point:
            self._applying = True
            try:
                self.to(probe.dtype)
            finally:
                self._applying = False
        return super()._apply(fn, recurse)

    def __getstate__(self):
        return self.input_args

    def __setstate__(self, state):
        torch.nn.Module.__init__(self)
        self.input_args = state
        self._init_class()

    # -- weights ---------------------------------------------------------------
    def reorder_weights_from_e3nn(self, weights, has_batch_dim: bool = True):
        """e3nn order is the native order of these kernels."""
        return weights

    def reorder_weights_to_e3nn(self, weights, has_batch_dim: bool = True):
        return weights

    @staticmethod
    def name():
        return "LoopUnrollTP"

    def forward(self, x: torch.Tensor, y: torch.Tensor, W: torch.Tensor) -> torch.Tensor:
        r"""
        :param x: ``[batch, problem.irreps_in1.dim]``
        :param y: ``[batch, problem.irreps_in2.dim]``
        :param W: ``[batch, weight_numel]``, or ``[weight_numel]`` when ``shared_weights``
        :return: ``[batch, problem.irreps_out.dim]``
        """
        return ops.tp_forward(x, y, W, self.kid, self.spec)
