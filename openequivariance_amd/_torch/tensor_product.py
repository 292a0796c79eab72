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

    # Kernel shapes that `autotune` tries beside the default (knobs of codegen/uvu.py: tp_module): how many waves a
    # SIMD may hold, rows per block, and whether the backward kernel keeps a row's output gradient in registers. Over
    # the reference's zoo the defaults are within a few percent of the best of these, except for kernels with few
    # words per lane, where another occupancy was up to 18 % faster for some problems and 8 % slower for others.
    AUTOTUNE_FORWARD = ("tp_wf=-2", "tp_wf=23", "tp_gf=2")
    AUTOTUNE_BACKWARD = ("tp_wb=-2", "tp_wb=23", "tp_gb=2", "tp_gres=1", "tp_gres=0")

    def autotune(self, x: torch.Tensor, y: torch.Tensor, W: torch.Tensor, *, repeats: int = 5, margin: float = 0.03,
                 verbose: bool = False) -> str:
        """Times alternative kernel shapes for this problem on the given inputs (forward, then backward with a
        random output gradient) and adopts the fastest where it beats the current one by more than ``margin``.
        Every alternative computes the same product; each costs a kernel compile the first time. Returns the knob
        string in force afterwards (exporting it as ``OEQ_AMD_TUNE`` makes the choice permanent for modules built
        later). 'uvw' problems have no alternatives and are left as they are. No counterpart in the reference."""
        import json
        import numpy as np
        base = json.loads(bytes(self.spec.tolist()).decode())["tune"]
        if self.is_uvw:
            return base
        problem = self.config
        g = torch.randn(x.shape[0], self.L3_dim, device=x.device, dtype=x.dtype)

        def build(tune: str):
            with ops._tune_env(tune):
                kid = ops.register_spec(ops.make_spec("tp", problem))
            ops.get_entry(kid).kernels()
            return kid

        def clock(fn) -> float:
            fn()
            times = []
            for _ in range(repeats):
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                fn()
                b.record()
                torch.cuda.synchronize()
                times.append(a.elapsed_time(b))
            return float(np.median(times))

        def best_of(current: str, candidates, run) -> str:
            best, best_ms = current, clock(lambda: run(build(current)))
            for cand in candidates:
                tune = ",".join(t for t in (current, cand) if t)
                try:
                    ms = clock(lambda: run(build(tune)))
                except (AssertionError, RuntimeError) as err:  # a shape this problem does not have
                    if verbose:
                        print(f"[autotune] {cand}: skipped ({type(err).__name__})")
                    continue
                if verbose:
                    print(f"[autotune] {cand}: {ms:.3f} ms")
                if ms < best_ms * (1.0 - margin):
                    best, best_ms = tune, ms
            return best

        with torch.no_grad():
            tune = best_of(base, self.AUTOTUNE_FORWARD, lambda kid: ops.tp_forward(x, y, W, kid))
            tune = best_of(tune, self.AUTOTUNE_BACKWARD, lambda kid: ops.tp_backward(x, y, W, g, kid))
        if tune != base:
            self.kid = build(tune)
            self.spec = ops.get_entry(self.kid).spec
        return tune

    def forward(self, x: torch.Tensor, y: torch.Tensor, W: torch.Tensor) -> torch.Tensor:
        r"""
        :param x: ``[batch, problem.irreps_in1.dim]``
        :param y: ``[batch, problem.irreps_in2.dim]``
        :param W: ``[batch, weight_numel]``, or ``[weight_numel]`` when ``shared_weights``
        :return: ``[batch, problem.irreps_out.dim]``
        """
        return ops.tp_forward(x, y, W, self.kid, self.spec)
