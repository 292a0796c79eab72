"""Timing helpers on the two modules, with the call signatures of the reference's
``benchmark_forward`` / ``benchmark_backward`` / ``benchmark_double_backward``
(openequivariance/openequivariance/core/TensorProductBase.py:69-175,
core/ConvolutionBase.py:134-290, core/utils.py:152-205), and the numpy-in / numpy-out
helpers its correctness harness drives (``forward_cpu``, ``backward_cpu``,
``double_backward_cpu``: _torch/TensorProduct.py:138-178, _torch/TensorProductConv.py:209-275,
_torch/NPDoubleBackwardMixin.py). Despite their names the latter run on the GPU: "cpu" says where
the caller's arrays live.

``with_torch_overhead=True`` times the whole op call with events on torch's current
stream; ``False`` returns the device time of the kernels alone, taken with HIP events
around the launches inside the C ABI (the reference reads it from a profiler trace).
A large scratch tensor is overwritten before every sample so that no operand starts in
cache, as the reference's ``clear_L2_cache`` does.
"""

from __future__ import annotations

import numpy as np
import torch

from .. import runtime as rt
from . import ops

_FLUSH_BYTES = 512 << 20  # larger than the 256 MiB Infinity Cache


def _flush(device):
    buf = getattr(_flush, "buf", None)
    if buf is None or buf.device != torch.device(device):
        buf = torch.empty(_FLUSH_BYTES, dtype=torch.uint8, device=device)
        _flush.buf = buf
    buf.zero_()


def time_call(fn, num_warmup: int, num_iter: int, device="cuda", kernel_entry=None, roles=()) -> np.ndarray:
    """Milliseconds per call of ``fn`` (``num_iter`` samples). With ``kernel_entry`` and ``roles``:
    summed device time of those kernel roles instead of the elapsed time of the call."""
    out = np.zeros(num_iter, dtype=np.float32)
    for _ in range(num_warmup):
        fn()
    torch.cuda.synchronize()
    ks = kernel_entry.kernels() if kernel_entry is not None else None
    for i in range(num_iter):
        _flush(device)
        if ks is None:
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            fn()
            stop.record()
            torch.cuda.synchronize()
            out[i] = start.elapsed_time(stop)
        else:
            ks.timing_enable(True)
            try:
                fn()
                torch.cuda.synchronize()
                out[i] = sum(ks.timing_collect(role)[0] for role in roles)
            finally:
                ks.timing_enable(False)
    return out


class TensorProductTiming:
    """Mixin for ``TensorProduct``."""

    def benchmark_forward(self, num_warmup, num_iter, L1_in, L2_in, L3_buffer, weights, with_torch_overhead=True,
                          kernel_names=("forward",)) -> np.ndarray:
        x, y, w = (torch.as_tensor(a).to("cuda").detach() for a in (L1_in, L2_in, weights))
        entry = None if with_torch_overhead else ops.get_entry(self.kid)
        return time_call(lambda: self.forward(x, y, w), num_warmup, num_iter, x.device, entry, (rt.ROLE_TP_FORWARD,))

    def benchmark_backward(self, num_warmup, num_iter, L1_in, L2_in, L3_buffer, weights, with_torch_overhead=True,
                           kernel_names=("backward",)) -> np.ndarray:
        x, y, w = (torch.as_tensor(a).to("cuda").detach().requires_grad_(True) for a in (L1_in, L2_in, weights))
        g = torch.as_tensor(L3_buffer).to("cuda")
        z = self.forward(x, y, w)
        entry = None if with_torch_overhead else ops.get_entry(self.kid)
        return time_call(lambda: z.backward(gradient=g, retain_graph=True, inputs=[x, y, w]), num_warmup, num_iter,
                         x.device, entry, (rt.ROLE_TP_BACKWARD, rt.ROLE_TP_BACKWARD_WREDUCE))

    def benchmark_double_backward(self, num_warmup, num_iter, L1_in, L2_in, weights, weights_grad,
                                  with_torch_overhead=True,
                                  kernel_names=("double_backward_A", "double_backward_B")) -> np.ndarray:
        """Time of the gradient of a scalar function of the three first-order gradients with respect to
        X, Y, W and the output gradient (the reference's protocol, TensorProductBase.py:126-175; as
        there, the output gradient is the forward result and ``weights_grad`` is accepted for
        signature compatibility only)."""
        x, y, w = (torch.as_tensor(a).to("cuda").detach().requires_grad_(True) for a in (L1_in, L2_in, weights))
        z = self.forward(x, y, w)
        g = z.clone().detach().requires_grad_(True)
        first = torch.autograd.grad(z, [x, y, w], g, create_graph=True, retain_graph=True)
        dummy = sum(torch.norm(t) for t in first)
        dummy_grad = torch.ones_like(dummy)
        entry = None if with_torch_overhead else ops.get_entry(self.kid)
        roles = (rt.ROLE_DOUBLE_BACKWARD_A, rt.ROLE_DOUBLE_BACKWARD_B, rt.ROLE_TP_FORWARD, rt.ROLE_TP_BACKWARD,
                 rt.ROLE_TP_BACKWARD_WREDUCE)
        return time_call(lambda: torch.autograd.grad(dummy, [x, y, w, g], dummy_grad, retain_graph=True),
                         num_warmup, num_iter, x.device, entry, roles)

    def forward_cpu(self, L1_in, L2_in, L3_out, weights) -> None:
        x, y, w = (torch.tensor(np.asarray(a), device="cuda") for a in (L1_in, L2_in, weights))
        L3_out[:] = self.forward(x, y, w).cpu().numpy()

    def backward_cpu(self, L1_in, L1_grad, L2_in, L2_grad, L3_grad, weights, weights_grad) -> None:
        x, y, w = (torch.tensor(np.asarray(a), device="cuda", requires_grad=True) for a in (L1_in, L2_in, weights))
        self.forward(x, y, w).backward(gradient=torch.tensor(np.asarray(L3_grad), device="cuda"))
        L1_grad[:], L2_grad[:], weights_grad[:] = (t.grad.cpu().numpy() for t in (x, y, w))

    def double_backward_cpu(self, in1, in2, out_grad, weights, weights_dgrad, in1_dgrad, in2_dgrad):
        """(in1_grad, in2_grad, weights_grad, out_dgrad) as numpy arrays: the second-order map evaluated
        through autograd (_torch/NPDoubleBackwardMixin.py:17-59 of the reference)."""
        dev = "cuda"
        x, y, w, g = (torch.tensor(np.asarray(a), device=dev, requires_grad=True)
                      for a in (in1, in2, weights, out_grad))
        cot = [torch.tensor(np.asarray(a), device=dev) for a in (in1_dgrad, in2_dgrad, weights_dgrad)]
        first = torch.autograd.grad(self.forward(x, y, w), [x, y, w], g, create_graph=True, retain_graph=True)
        second = torch.autograd.grad(first, [x, y, w, g], cot)
        return tuple(t.detach().cpu().numpy() for t in second)

    double_backward = double_backward_cpu


class ConvolutionTiming:
    """Mixin for ``TensorProductConv``; ``graph`` is a ``CoordGraph``."""

    def _random_buffers(self, graph, prng_seed):
        rng = np.random.default_rng(prng_seed)
        p = self.config
        dt = np.dtype(p.irrep_dtype)
        wshape = (p.weight_numel,) if p.shared_weights else (graph.nnz, p.weight_numel)
        host = (rng.uniform(size=(graph.node_count, p.irreps_in1.dim)), rng.uniform(size=(graph.nnz, p.irreps_in2.dim)),
                rng.uniform(size=wshape), rng.uniform(size=(graph.node_count, p.irreps_out.dim)))
        return tuple(torch.tensor(a.astype(dt), device="cuda") for a in host)

    def _graph_tensors(self, graph):
        rows, cols = torch.tensor(graph.rows, device="cuda"), torch.tensor(graph.cols, device="cuda")
        perm = torch.tensor(graph.transpose_perm, device="cuda") if self.deterministic else None
        return rows, cols, perm

    def _stats(self, direction, time_millis, graph, num_warmup, num_iter, prng_seed):
        low = self._low
        flops = low.flops(direction) + (low.L3 if direction == "forward" else 0)
        es = low.elem_size
        wn = 0 if low.shared_weights else low.WN
        if direction == "forward":
            data = (graph.nnz * (low.L2 + wn) + graph.node_count * (low.L1 + low.L3)) * es
        else:
            data = (2 * graph.nnz * (low.L2 + wn) + graph.node_count * (2 * low.L1 + low.L3)) * es
        t = np.asarray(time_millis, dtype=np.float64)
        return {
            "time_millis": [float(v) for v in t], "direction": direction, "graph_node_count": graph.node_count,
            "graph_adj_nnz": graph.nnz, "num_warmup": num_warmup, "num_iter": num_iter, "prng_seed": prng_seed,
            "flops_per_tp": flops, "data_per_tp": data / max(1, graph.nnz),
            "throughputs_gflops": [float(v) for v in flops * graph.nnz / (t * 1e6)],
            "bandwidth_gbps": [float(v) for v in data / (t * 1e6)],
        }

    def forward_cpu(self, L1_in, L2_in, weights, L3_out, graph) -> None:
        x, y, w = (torch.tensor(np.asarray(a), device="cuda") for a in (L1_in, L2_in, weights))
        L3_out[:] = self.forward(x, y, w, *self._graph_tensors(graph)).cpu().numpy()

    def backward_cpu(self, L1_in, L1_grad, L2_in, L2_grad, weights, weights_grad, L3_grad, graph) -> None:
        x, y, w = (torch.tensor(np.asarray(a), device="cuda", requires_grad=True) for a in (L1_in, L2_in, weights))
        z = self.forward(x, y, w, *self._graph_tensors(graph))
        z.backward(gradient=torch.tensor(np.asarray(L3_grad), device="cuda"))
        L1_grad[:], L2_grad[:], weights_grad[:] = (t.grad.cpu().numpy() for t in (x, y, w))

    def double_backward_cpu(self, in1, in2, out_grad, weights, weights_dgrad, in1_dgrad, in2_dgrad, graph):
        """(in1_grad, in2_grad, weights_grad, out_dgrad) as numpy arrays
        (_torch/NPDoubleBackwardMixin.py:145-193 of the reference)."""
        x, y, w, g = (torch.tensor(np.asarray(a), device="cuda", requires_grad=True)
                      for a in (in1, in2, weights, out_grad))
        cot = [torch.tensor(np.asarray(a), device="cuda") for a in (in1_dgrad, in2_dgrad, weights_dgrad)]
        z = self.forward(x, y, w, *self._graph_tensors(graph))
        first = torch.autograd.grad(z, [x, y, w], g, create_graph=True, retain_graph=True)
        second = torch.autograd.grad(first, [x, y, w, g], cot)
        return tuple(t.detach().cpu().numpy() for t in second)

    def benchmark_forward(self, num_warmup, num_iter, graph, prng_seed=12345, kernel_names=("forward",)):
        X, Y, W, _ = self._random_buffers(graph, prng_seed)
        rows, cols, perm = self._graph_tensors(graph)
        t = time_call(lambda: self.forward(X, Y, W, rows, cols, perm), num_warmup, num_iter, X.device)
        return self._stats("forward", t, graph, num_warmup, num_iter, prng_seed)

    def benchmark_backward(self, num_warmup, num_iter, graph, prng_seed=12345, kernel_names=("backward",)):
        X, Y, W, G = self._random_buffers(graph, prng_seed)
        X, Y, W = (t.requires_grad_(True) for t in (X, Y, W))
        rows, cols, perm = self._graph_tensors(graph)
        z = self.forward(X, Y, W, rows, cols, perm)
        t = time_call(lambda: z.backward(gradient=G, retain_graph=True, inputs=[X, Y, W]), num_warmup, num_iter,
                      X.device)
        return self._stats("backward", t, graph, num_warmup, num_iter, prng_seed)

    def benchmark_double_backward(self, num_warmup, num_iter, graph, prng_seed=12345,
                                  kernel_names=("double_backward_A", "double_backward_B")):
        """Same protocol as the batch module's: gradient of the sum of the norms of (dX, dY, dW) with
        respect to X, Y, W and the output gradient."""
        X, Y, W, G = self._random_buffers(graph, prng_seed)
        X, Y, W, G = (t.requires_grad_(True) for t in (X, Y, W, G))
        rows, cols, perm = self._graph_tensors(graph)
        z = self.forward(X, Y, W, rows, cols, perm)
        first = torch.autograd.grad(z, [X, Y, W], G, create_graph=True, retain_graph=True)
        dummy = sum(torch.norm(t) for t in first)
        t = time_call(lambda: torch.autograd.grad(dummy, [X, Y, W, G], retain_graph=True), num_warmup, num_iter,
                      X.device)
        low = self._low
        wn = 0 if low.shared_weights else low.WN
        stats = self._stats("backward", t, graph, num_warmup, num_iter, prng_seed)
        data = (3 * graph.nnz * (low.L2 + wn) + graph.node_count * (3 * low.L1 + 2 * low.L3)) * low.elem_size
        tt = np.asarray(t, dtype=np.float64)
        stats.update(direction="double_backward", data_per_tp=data / max(1, graph.nnz),
                     bandwidth_gbps=[float(v) for v in data / (tt * 1e6)])
        stats.pop("throughputs_gflops", None)
        stats.pop("flops_per_tp", None)
        return stats
