"""``TensorProductConv``: fused CG tensor product + scatter-sum over a graph.

Drop-in for the reference class
(openequivariance/openequivariance/_torch/TensorProductConv.py:32-278):
``forward(X, Y, W, rows, cols, sender_perm=None)`` with ``rows`` = receivers and
``cols`` = senders; ``deterministic=True`` needs row-sorted edges and the
permutation that lists them in sender-major order.

Unlike the reference, the deterministic backward does not assume a symmetric
sparsity pattern, and the module holds no workspace of its own (scratch memory
is allocated per call from torch's stream-ordered allocator), so two streams
may use one module concurrently.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..codegen.lower import lower
from ..core.spec import TPProblem
from .. import runtime as rt
from . import ops
from .benchmarking import ConvolutionTiming
from .utils import compute_units, oeq_to_torch_dtype, torch_to_oeq_dtype


def fused(low) -> bool:
    """Whether the convolution of this problem runs as fused kernels: every 'uvu' problem, and the 'uvw'
    problems except shared-weight ones that are faster through the matrix-core batch kernels
    (``codegen/uvw.py: conv_supported``; ``OEQ_AMD_TUNE=conv_fuse_uvw=0`` sends every 'uvw' problem through the
    unfused path)."""
    if low.mode == "uvu":
        return True
    from ..codegen import uvw
    from ..codegen.uvu import tuning
    return uvw.conv_supported(low) and bool(tuning(dict(conv_fuse_uvw=1))["conv_fuse_uvw"])


def build_conv_module(problem: TPProblem, deterministic: bool, kahan: bool = False):
    low = lower(problem)
    if low.mode == "uvu":
        from ..codegen import uvu
        return uvu.conv_module(low, deterministic, compute_units(), kahan)
    from ..codegen import uvw
    if fused(low):
        return uvw.conv_module(low, deterministic, compute_units(), kahan)
    # 'uvw' with shared weights on the matrix cores: no fused kernel; the batch kernels run on gathered rows and an ordered
    # segment sum scatters the result, like the reference's unfused convolution
    # (core/ConvolutionBase.py:292-301, _torch/TensorProductConv.py:595-640).
    cu = compute_units()
    src, dims, descs = uvw.tp_module(low, cu, kahan)
    descs = list(descs) + [(rt.ROLE_SEGMENT_PTR, "oeq_segment_ptr", 256, 256, cu * 16),
                           (rt.ROLE_SEGMENT_SUM, "oeq_segment_sum", 256, 1, cu * 32),
                           (rt.ROLE_GROUP_COUNT, "oeq_group_count", 256, 256 * 4, cu * 16),
                           (rt.ROLE_GROUP_SCAN, "oeq_group_scan", 1024, 1, 1),
                           (rt.ROLE_GROUP_SCATTER, "oeq_group_scatter", 256, 256 * 4, cu * 16),
                           (rt.ROLE_GROUP_ORDER, "oeq_group_order", 256, 4, cu * 32)]
    return src, dims, descs


class TensorProductConv(ConvolutionTiming, torch.nn.Module):
    r"""Computes :math:`z_i = \sum_{(i,j,e)} W_e (x_j \otimes_{CG} y_e)` over the
    edges of a directed graph.

    :param problem: specification of the tensor product.
    :param deterministic: ``False``: any edge order; the edge indices are grouped by receiver (and by
           sender for backward) on the device at every call, ascending within a node, and the sums follow
           that grouping (so this mode, too, gives the same bits from run to run for a given edge list).
           ``True``: receiver-sorted edges and ``sender_perm`` from the caller, no grouping pass.
           *Default*: ``False``.
    :param kahan: with ``deterministic=True``: Kahan-compensated summation over the edges of a node
           (receiver's output in forward, sender's gradient in backward). *Default*: ``False``.
    :param use_opaque: deprecated, ignored.
    """

    def __init__(self, problem: TPProblem, *, deterministic: bool = False, kahan: bool = False,
                 torch_op: bool = True, use_opaque: bool = False):
        torch.nn.Module.__init__(self)
        self.input_args = {"problem": problem, "deterministic": deterministic, "kahan": kahan,
                           "torch_op": torch_op, "use_opaque": use_opaque}
        self._init_class()

    def _init_class(self):
        problem: TPProblem = self.input_args["problem"].clone()
        deterministic = bool(self.input_args["deterministic"])
        kahan = bool(self.input_args["kahan"])
        if kahan:
            assert deterministic, "kahan=True requires deterministic=True"
        if deterministic:
            assert not problem.shared_weights, "Deterministic convolution does not support shared weights"
        self.config = problem
        self.deterministic = deterministic
        low = lower(problem)
        self._low = low
        self.L1, self.L2, self.L3 = problem.irreps_in1, problem.irreps_in2, problem.irreps_out
        self.L3_dim = low.L3
        self.weight_numel = problem.weight_numel
        # the kernel set's description travels with every op call (see TensorProduct._init_class)
        self.kid = ops.register_spec(ops.make_spec("conv", problem, deterministic, kahan))
        self.spec = ops.get_entry(self.kid).spec

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

    def reorder_weights_from_e3nn(self, weights, has_batch_dim: bool = True):
        return weights

    def reorder_weights_to_e3nn(self, weights, has_batch_dim: bool = True):
        return weights

    @staticmethod
    def name():
        return "LoopUnrollConv"

    # Kernel shapes that `autotune` tries beside the default (knobs of codegen/uvu.py: conv_module). The defaults
    # are rules fitted to sweeps over some 130 problems; on a tenth of those one of these was 10 - 30 % faster in the
    # forward kernel (another split of the outputs into register-resident segments, one operand set in flight
    # instead of two, a third wave per SIMD), and the number of waves that share a node in the backward kernel and
    # the route of the sender gradients have break-even points that a given graph may move.
    AUTOTUNE_FORWARD = ("conv_acc=96", "conv_acc=64", "conv_pipe_f=0", "conv_wf=3")
    AUTOTUNE_BACKWARD = ("conv_gb=4", "conv_ngrp=1", "conv_ngrp=2", "conv_ngrp=4", "conv_dxs=1", "conv_dxs=0")

    def autotune(self, X: torch.Tensor, Y: torch.Tensor, W: torch.Tensor, rows: torch.Tensor, cols: torch.Tensor,
                 sender_perm: Optional[torch.Tensor] = None, *, repeats: int = 5, margin: float = 0.03,
                 verbose: bool = False) -> str:
        """Times alternative kernel shapes for this problem on the given inputs (forward, then backward with a
        random output gradient) and adopts the fastest where it beats the current one by more than ``margin``.
        Every alternative computes the same convolution (they are the variants the knob tests cover); each costs a
        kernel compile the first time. Returns the knob string in force afterwards: exporting it as
        ``OEQ_AMD_TUNE`` makes the choice permanent for modules built later. 'uvw' problems have no alternatives
        and are left as they are. No counterpart in the reference."""
        import json
        import numpy as np
        if self._low.mode != "uvu":
            return json.loads(bytes(self.spec.tolist()).decode())["tune"]
        if sender_perm is None:
            if self.deterministic:
                raise RuntimeError("deterministic=True needs sender_perm")
            sender_perm = rows
        problem, det, kahan = self.config, self.deterministic, bool(self.input_args["kahan"])
        base = json.loads(bytes(self.spec.tolist()).decode())["tune"]
        G = torch.randn(X.shape[0], self.L3_dim, device=X.device, dtype=X.dtype)

        def build(tune: str):
            with ops._tune_env(tune):
                kid = ops.register_spec(ops.make_spec("conv", problem, det, kahan))
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
            tune = best_of(base, self.AUTOTUNE_FORWARD,
                           lambda kid: ops.conv_forward(X, Y, W, rows, cols, sender_perm, kid))
            # (how the sender gradients travel is a choice only where the bits need not repeat from run to run)
            travel = () if det else ("conv_dxm=0", "conv_dxm=1")
            tune = best_of(tune, self.AUTOTUNE_BACKWARD + travel,
                           lambda kid: ops.conv_backward(X, Y, W, G, rows, cols, sender_perm, kid))
            if ops.get_entry(build(tune)).kernels().dims.get("dx_mode", 0) == rt.DX_SENDER_WALK:
                # the sender-walk kernel with a third wave per SIMD where its registers allow
                tune = best_of(tune, ("conv_wx=23",),
                               lambda kid: ops.conv_backward(X, Y, W, G, rows, cols, sender_perm, kid))
        if tune != base:
            self.kid = build(tune)
            self.spec = ops.get_entry(self.kid).spec
        return tune

    def forward(self, X: torch.Tensor, Y: torch.Tensor, W: torch.Tensor, rows: torch.Tensor, cols: torch.Tensor,
                sender_perm: Optional[torch.Tensor] = None) -> torch.Tensor:
        r"""
        :param X: ``[|V|, irreps_in1.dim]`` node features
        :param Y: ``[|E|, irreps_in2.dim]`` edge features
        :param W: ``[|E|, weight_numel]`` (or ``[weight_numel]`` with shared weights)
        :param rows: ``[|E|]`` int64 receiver of each edge (sorted when ``deterministic``)
        :param cols: ``[|E|]`` int64 sender of each edge
        :param sender_perm: ``[|E|]`` int64 permutation listing the edges in
               sender-major order; required when ``deterministic``
        :return: ``[|V|, irreps_out.dim]``
        """
        if sender_perm is None:
            if self.deterministic:
                raise RuntimeError("Shape mismatch for tensor 'transpose perm'. deterministic=True needs sender_perm")
            # any int64 tensor fills the op's slot (it is not read in this mode); the receivers are at hand, and
            # handing them over creates no tensor and sets no attribute while a program is being traced
            sender_perm = rows
        return ops.conv_forward(X, Y, W, rows, cols, sender_perm, self.kid, self.spec)
