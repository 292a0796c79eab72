"""PyTorch custom ops over the C ABI.

Stand in for the reference's native op library
(openequivariance/openequivariance/extension/torch_core.hpp:274-644:
``jit_tp_forward``, ``jit_tp_backward``, ``jit_conv_forward``,
``jit_conv_backward`` and their double-backward companions) and its Python
registrations of fake kernels, autograd and autocast
(openequivariance/openequivariance/_torch/TensorProduct.py:182-374,
_torch/TensorProductConv.py:280-568).

Like the reference's ops (``Tensor json_bytes, int hash``, torch_core.hpp:637-643)
every op takes the description of its kernel set: ``kid``, a 63-bit hash of the
serialised problem and flags, and ``spec``, a uint8 tensor holding those bytes.
The hash finds the compiled kernel set in a process-wide registry; a process
that has never seen it (an exported program loaded elsewhere) rebuilds the set
from the bytes, so a traced graph means the same thing in every process.
Callers inside one process may leave ``spec`` out. Argument checks raise
``RuntimeError`` with the reference's wording (torch_core.hpp:109-134).

Second and higher derivatives need no extra kernels: with
S(x, y, w, g) = <g, TP(x, y, w)> multilinear, the backward op returns
(dS/dx, dS/dy, dS/dw) and its own vector-Jacobian product is a sum of three
forward and three backward calls with one argument replaced by a cotangent.
"""

from __future__ import annotations

import contextlib
import hashlib
import json
import os
import threading
from typing import Dict, List, Optional, Tuple

import torch

from .. import runtime as rt

_registry: Dict[int, "KernelEntry"] = {}
_registry_lock = threading.RLock()


class KernelEntry:
    """Lazily compiled kernel set + the shape facts the ops validate against."""

    def __init__(self, build_fn, L1, L2, L3, WN, shared, torch_dtype, deterministic=False, unfused=False):
        self.build_fn = build_fn  # () -> (source, dims, descs)
        self.unfused = unfused  # convolution = gather + batch kernels + scatter (no fused kernel for this problem)
        self.L1, self.L2, self.L3, self.WN = L1, L2, L3, WN
        self.shared = shared
        self.dtype = torch_dtype
        self.deterministic = deterministic
        self.spec: Optional[torch.Tensor] = None  # the bytes this entry was built from (uint8, host)
        # Shared-weight 'uvw' convolution as contraction + channel mix per node (core/problems.py:
        # factor_shared_uvw): ids of the two kernel sets that then do the work, else None.
        self.factored: Optional[Tuple[int, int]] = None
        # Float-atomics convolution kernels (conv_sort=0) have no second-order pair of their own: id of the
        # grouped-walk kernel set of the same problem, whose fused pair takes the edges in any order as well.
        self.second_order_kid: Optional[int] = None
        self._ks: Optional[rt.KernelSet] = None
        self._lock = threading.Lock()

    def kernels(self) -> rt.KernelSet:
        if self._ks is None:
            with self._lock:
                if self._ks is None:
                    src, dims, descs = self.build_fn()
                    self._ks = rt.get_kernel_set(src, dims, descs)
        return self._ks


# ---------------------------------------------------------------------------
# kernel sets by description
# ---------------------------------------------------------------------------

_tune_lock = threading.RLock()


@contextlib.contextmanager
def _tune_env(tune: str):
    """The kernel-shape knobs (``OEQ_AMD_TUNE``) that were in force when a description was written are part
    of it: they are put back while its kernels are generated, whenever and wherever that happens."""
    with _tune_lock:
        saved = os.environ.get("OEQ_AMD_TUNE")
        os.environ["OEQ_AMD_TUNE"] = tune
        try:
            yield
        finally:
            if saved is None:
                os.environ.pop("OEQ_AMD_TUNE", None)
            else:
                os.environ["OEQ_AMD_TUNE"] = saved


def make_spec(kind: str, problem, deterministic: bool = False, kahan: bool = False) -> bytes:
    """Serialised description of a kernel set: ``kind`` 'tp' or 'conv', the problem, the module's flags and
    the tuning knobs in force (cf. the reference's kernel JSON, torch_core.hpp:144-178)."""
    from ..core.spec import problem_to_dict
    assert kind in ("tp", "conv")
    desc = {"v": 1, "kind": kind, "problem": problem_to_dict(problem), "deterministic": bool(deterministic),
            "kahan": bool(kahan), "tune": os.environ.get("OEQ_AMD_TUNE", "")}
    return json.dumps(desc, sort_keys=True, separators=(",", ":")).encode()


def spec_hash(spec: bytes) -> int:
    return int.from_bytes(hashlib.sha256(spec).digest()[:8], "little") & ((1 << 63) - 1)


def _entry_from_spec(spec: bytes) -> KernelEntry:
    from ..codegen.lower import lower
    from ..core.spec import problem_from_dict
    from .tensor_product import build_tp_module
    from .tensor_product_conv import build_conv_module, fused
    from .utils import oeq_to_torch_dtype
    desc = json.loads(spec.decode())
    if desc.get("v") != 1 or desc.get("kind") not in ("tp", "conv"):
        raise RuntimeError("unreadable kernel-set description")
    problem = problem_from_dict(desc["problem"])
    tune, det, kahan = desc["tune"], desc["deterministic"], desc["kahan"]
    low = lower(problem)
    dtype = oeq_to_torch_dtype(problem.irrep_dtype)
    if desc["kind"] == "tp":
        def build():
            with _tune_env(tune):
                return build_tp_module(problem)
        entry = KernelEntry(build, low.L1, low.L2, low.L3, low.WN, low.shared_weights, dtype)
    else:
        def build():
            with _tune_env(tune):
                return build_conv_module(problem, det, kahan)
        factored = None
        with _tune_env(tune):
            from ..codegen.uvu import tuning
            from ..core.problems import factor_shared_uvw
            knobs = tuning(dict(conv_fuse_uvw=1, conv_factor=1))
            parts = factor_shared_uvw(problem) if (knobs["conv_fuse_uvw"] and knobs["conv_factor"]) else None
            if parts is not None and not det:
                factored = (register_spec(make_spec("conv", parts[0], False, False)),
                            register_spec(make_spec("tp", parts[1])))
            unfused = factored is None and not fused(low)
            sibling = None
            if low.mode == "uvu" and not det and not tuning(dict(conv_sort=1))["conv_sort"]:
                walk = dict(desc, tune=(tune + "," if tune else "") + "conv_sort=1")
                sibling = register_spec(json.dumps(walk, sort_keys=True, separators=(",", ":")).encode())
        entry = KernelEntry(build, low.L1, low.L2, low.L3, low.WN, low.shared_weights, dtype, deterministic=det,
                            unfused=unfused)
        entry.factored = factored
        entry.second_order_kid = sibling
    entry.spec = torch.frombuffer(bytearray(spec), dtype=torch.uint8)
    return entry


def register_spec(spec: bytes) -> int:
    """The id of the kernel set a description stands for (its hash); the set is entered into the registry
    unless it is there already. Kernels are generated and compiled at first use."""
    kid = spec_hash(spec)
    with _registry_lock:
        if kid not in _registry:
            _registry[kid] = _entry_from_spec(spec)
    return kid


def get_entry(kid: int, spec: Optional[torch.Tensor] = None) -> KernelEntry:
    entry = _registry.get(kid)
    if entry is not None:
        return entry
    if spec is None:
        raise RuntimeError(f"unknown kernel id {kid}: no kernel set with this hash in this process, and the "
                           "call carries no description to build it from")
    try:
        data = bytes(spec.detach().cpu().contiguous().numpy().tobytes())
    except Exception as exc:  # a tensor without data: tracing in a process that never built this kernel set
        raise RuntimeError(f"kernel id {kid} is unknown in this process and its description cannot be read "
                           "while tracing; call the module once outside tracing first") from exc
    if spec_hash(data) != kid:
        raise RuntimeError(f"kernel id {kid} does not match the description that came with it")
    register_spec(data)
    return _registry[kid]


_DTYPE_CODE = {torch.float32: 1, torch.float64: 2, torch.int32: 3, torch.int64: 4, torch.uint8: 5}


def check_tensor(t: torch.Tensor, shape: List[int], dtype: torch.dtype, name: str):
    """torch_core.hpp:109-134."""
    if t.dim() != len(shape) or any(int(a) != int(b) for a, b in zip(t.shape, shape)):
        raise RuntimeError(
            f"Shape mismatch for tensor '{name}'. Expected: {list(shape)}. Got: {list(t.shape)}"
        )
    if not t.is_cuda:
        raise RuntimeError(f"Tensor '{name}' is not on the GPU.")
    if t.dtype != dtype:
        raise RuntimeError(
            f"Dtype mismatch for tensor '{name}'. Expected: {_DTYPE_CODE.get(dtype, dtype)}. "
            f"Got: {_DTYPE_CODE.get(t.dtype, t.dtype)}"
        )


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _wshape(e: KernelEntry, n: int) -> List[int]:
    return [e.WN] if e.shared else [n, e.WN]


# ---------------------------------------------------------------------------
# batch tensor product
# ---------------------------------------------------------------------------


@torch.library.custom_op("oeq_amd::tp_forward", mutates_args=(), device_types="cuda")
def tp_forward(L1_in: torch.Tensor, L2_in: torch.Tensor, W: torch.Tensor, kid: int,
               spec: Optional[torch.Tensor] = None) -> torch.Tensor:
    e = get_entry(kid, spec)
    n = L1_in.shape[0] if L1_in.dim() > 0 else -1
    check_tensor(L1_in, [n, e.L1], e.dtype, "L1_in")
    check_tensor(L2_in, [n, e.L2], e.dtype, "L2_in")
    check_tensor(W, _wshape(e, n), e.dtype, "W")
    x, y, w = L1_in.contiguous(), L2_in.contiguous(), W.contiguous()
    out = x.new_empty((n, e.L3))
    with torch.cuda.device(x.device):
        e.kernels().tp_forward(n, x.data_ptr(), y.data_ptr(), w.data_ptr(), out.data_ptr(), _stream())
    return out


@tp_forward.register_fake
def _(L1_in, L2_in, W, kid, spec=None):
    e = get_entry(kid, spec)
    return L1_in.new_empty((L1_in.shape[0], e.L3))


@torch.library.custom_op("oeq_amd::tp_backward", mutates_args=(), device_types="cuda")
def tp_backward(L1_in: torch.Tensor, L2_in: torch.Tensor, W: torch.Tensor, L3_grad: torch.Tensor,
                kid: int, spec: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    e = get_entry(kid, spec)
    n = L1_in.shape[0] if L1_in.dim() > 0 else -1
    check_tensor(L1_in, [n, e.L1], e.dtype, "L1_in")
    check_tensor(L2_in, [n, e.L2], e.dtype, "L2_in")
    check_tensor(W, _wshape(e, n), e.dtype, "W")
    check_tensor(L3_grad, [n, e.L3], e.dtype, "L3_grad")
    x, y, w, g = L1_in.contiguous(), L2_in.contiguous(), W.contiguous(), L3_grad.contiguous()
    dx, dy, dw = torch.empty_like(x), torch.empty_like(y), torch.empty_like(w)
    with torch.cuda.device(x.device):
        ks = e.kernels()
        nb = ks.tp_backward_workspace_bytes(n)
        ws = torch.empty(max(nb, 1), dtype=torch.uint8, device=x.device)
        ks.tp_backward(n, x.data_ptr(), dx.data_ptr(), y.data_ptr(), dy.data_ptr(), w.data_ptr(), dw.data_ptr(),
                       g.data_ptr(), ws.data_ptr() if nb else 0, nb, _stream())
    return dx, dy, dw


@tp_backward.register_fake
def _(L1_in, L2_in, W, L3_grad, kid, spec=None):
    return torch.empty_like(L1_in), torch.empty_like(L2_in), torch.empty_like(W)


def _tp_fwd_setup(ctx, inputs, output):
    ctx.kid, ctx.spec = inputs[3], inputs[4]
    ctx.save_for_backward(inputs[0], inputs[1], inputs[2])


def _tp_fwd_backward(ctx, grad):
    x, y, w = ctx.saved_tensors
    dx, dy, dw = tp_backward(x, y, w, grad, ctx.kid, ctx.spec)
    return dx, dy, dw, None, None


tp_forward.register_autograd(_tp_fwd_backward, setup_context=_tp_fwd_setup)


def _tp_bwd_setup(ctx, inputs, output):
    ctx.kid, ctx.spec = inputs[4], inputs[5]
    ctx.save_for_backward(inputs[0], inputs[1], inputs[2], inputs[3])


def _sum2(a, b):
    """a + b where either may be missing; in place on ``a`` (a fresh kernel output nothing else holds)
    when no graph is being recorded, which saves a pass over a weight-sized tensor."""
    if a is None or b is None:
        return b if a is None else a
    return a + b if torch.is_grad_enabled() else a.add_(b)


def _second_order(forward, backward, x, y, w, g, ddx, ddy, ddw):
    """Gradients of ``backward(x, y, w, g) -> (dx, dy, dw)`` contracted with (ddx, ddy, ddw). The
    tensor product is linear in each of x, y, w and g, so every term is the forward or backward
    kernel applied with one operand replaced by its cotangent (the reference has two dedicated
    kernels for this, double_backward_A/B in templates/loop_unroll_batch.cuh:148-317). Terms of
    cotangents autograd did not ask for (None) are skipped."""
    dx = dy = dw = gg = None
    if ddy is not None:
        dx1, _, dw1 = backward(x, ddy, w, g)
        dx, dw = dx1, dw1
        gg = forward(x, ddy, w)
    if ddw is not None:
        dx2, dy2, _ = backward(x, y, ddw, g)
        dx, dy = _sum2(dx, dx2), dy2
        gg = _sum2(gg, forward(x, y, ddw))
    if ddx is not None:
        _, dy3, dw3 = backward(ddx, y, w, g)
        dy, dw = _sum2(dy, dy3), _sum2(dw, dw3)
        gg = _sum2(gg, forward(ddx, y, w))
    return dx, dy, dw, gg


# The fused second-order kernels are used when no graph is being recorded for a third derivative (then
# the composition of differentiable first-order ops is needed) and at least two of the three cotangents
# are present (a missing one is passed as zeros; with a single cotangent the two first-order calls of
# the composition read less). Tests switch this off to compare the two routes.
FUSED_DOUBLE_BACKWARD = True


def _use_fused(kid, spec, ddx, ddy, ddw) -> bool:
    if not FUSED_DOUBLE_BACKWARD or torch.is_grad_enabled():
        return False
    if sum(t is not None for t in (ddx, ddy, ddw)) < 2:
        return False
    entry = get_entry(kid, spec)
    if entry.second_order_kid is not None:
        entry = get_entry(entry.second_order_kid)
    return bool(entry.factored) or entry.kernels().has_double_backward()


def _zeros_if_none(t, like):
    return torch.zeros_like(like) if t is None else t


@torch.library.custom_op("oeq_amd::tp_double_backward", mutates_args=(), device_types="cuda")
def tp_double_backward(L1_in: torch.Tensor, L2_in: torch.Tensor, W: torch.Tensor, L3_grad: torch.Tensor,
                       L1_dgrad: torch.Tensor, L2_dgrad: torch.Tensor, W_dgrad: torch.Tensor,
                       kid: int, spec: Optional[torch.Tensor] = None
                       ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """(L1_grad, L2_grad, W_grad, L3_dgrad): the op of the reference's jit_tp_double_backward
    (extension/torch_core.hpp:357-420)."""
    e = get_entry(kid, spec)
    n = L1_in.shape[0] if L1_in.dim() > 0 else -1
    for t, name in ((L1_in, "L1_in"), (L1_dgrad, "L1_dgrad")):
        check_tensor(t, [n, e.L1], e.dtype, name)
    for t, name in ((L2_in, "L2_in"), (L2_dgrad, "L2_dgrad")):
        check_tensor(t, [n, e.L2], e.dtype, name)
    for t, name in ((W, "W"), (W_dgrad, "W_dgrad")):
        check_tensor(t, _wshape(e, n), e.dtype, name)
    check_tensor(L3_grad, [n, e.L3], e.dtype, "L3_grad")
    x, y, w, g = L1_in.contiguous(), L2_in.contiguous(), W.contiguous(), L3_grad.contiguous()
    a, b, c = L1_dgrad.contiguous(), L2_dgrad.contiguous(), W_dgrad.contiguous()
    dx, dy, dw, gg = torch.empty_like(x), torch.empty_like(y), torch.empty_like(w), torch.empty_like(g)
    with torch.cuda.device(x.device):
        ks = e.kernels()
        nb = ks.tp_double_backward_workspace_bytes(n)
        ws = torch.empty(max(nb, 1), dtype=torch.uint8, device=x.device)
        ks.tp_double_backward(n, x.data_ptr(), y.data_ptr(), w.data_ptr(), g.data_ptr(), a.data_ptr(),
                              b.data_ptr(), c.data_ptr(), dx.data_ptr(), dy.data_ptr(), dw.data_ptr(),
                              gg.data_ptr(), ws.data_ptr(), nb, _stream())
    return dx, dy, dw, gg


@tp_double_backward.register_fake
def _(L1_in, L2_in, W, L3_grad, L1_dgrad, L2_dgrad, W_dgrad, kid, spec=None):
    return torch.empty_like(L1_in), torch.empty_like(L2_in), torch.empty_like(W), torch.empty_like(L3_grad)


def _tp_bwd_backward(ctx, ddx, ddy, ddw):
    x, y, w, g = ctx.saved_tensors
    kid, spec = ctx.kid, ctx.spec
    if _use_fused(kid, spec, ddx, ddy, ddw):
        dx, dy, dw, gg = tp_double_backward(x, y, w, g, _zeros_if_none(ddx, x), _zeros_if_none(ddy, y),
                                            _zeros_if_none(ddw, w), kid, spec)
        return dx, dy, dw, gg, None, None
    dx, dy, dw, gg = _second_order(lambda a, b, c: tp_forward(a, b, c, kid, spec),
                                   lambda a, b, c, d: tp_backward(a, b, c, d, kid, spec), x, y, w, g, ddx, ddy, ddw)
    return dx, dy, dw, gg, None, None


tp_backward.register_autograd(_tp_bwd_backward, setup_context=_tp_bwd_setup)


# ---------------------------------------------------------------------------
# fused convolution
# ---------------------------------------------------------------------------


# Edge-list validation before any kernel is launched: ``CHECK_INDICES = True`` here, or
# OEQ_AMD_CHECK_INDICES=1 in the environment. Off by default, like in the reference (which checks
# shapes, dtypes and devices only, torch_core.hpp:109-134): the check synchronises with the device.
# Without it a corrupt edge list cannot make the kernels read or write outside their operands (every
# index is forced into range on the device), but the sums it gives are then meaningless.
CHECK_INDICES = False


def check_edge_list(nodes: int, rows: torch.Tensor, cols: torch.Tensor, perm: Optional[torch.Tensor],
                    deterministic: bool):
    """RuntimeError unless 0 <= rows, cols < nodes and, for the caller-sorted mode, rows is non-decreasing
    and perm is a permutation of the edges that lists them by non-decreasing sender."""
    nnz = rows.shape[0]
    if nnz == 0:
        return
    for name, t in (("rows", rows), ("cols", cols)):
        lo, hi = int(t.min()), int(t.max())
        if lo < 0 or hi >= nodes:
            raise RuntimeError(f"Index out of range in tensor '{name}': values span [{lo}, {hi}], "
                               f"the graph has {nodes} nodes")
    if deterministic:
        if nnz > 1 and bool((rows[1:] < rows[:-1]).any()):
            raise RuntimeError("Tensor 'rows' is not sorted: deterministic=True needs the edges sorted by receiver")
        lo, hi = int(perm.min()), int(perm.max())
        if lo < 0 or hi >= nnz or int(torch.bincount(perm, minlength=nnz).max()) != 1:
            raise RuntimeError("Tensor 'transpose perm' is not a permutation of the edges")
        by_sender = cols[perm]
        if nnz > 1 and bool((by_sender[1:] < by_sender[:-1]).any()):
            raise RuntimeError("Tensor 'transpose perm' does not list the edges by sender")


def _check_indices_enabled() -> bool:
    import os
    return CHECK_INDICES or os.environ.get("OEQ_AMD_CHECK_INDICES", "0") not in ("", "0")


def _walk_dims(e: KernelEntry) -> dict:
    """Dims of the kernel set that walks the graph for this entry (the contraction part of a factored one)."""
    return (get_entry(e.factored[0]) if e.factored else e).kernels().dims


def _conv_checks(e: KernelEntry, L1_in, L2_in, W, rows, cols, perm, L3_grad=None):
    nodes = L1_in.shape[0] if L1_in.dim() > 0 else -1
    nnz = rows.shape[0] if rows.dim() > 0 else -1
    check_tensor(L1_in, [nodes, e.L1], e.dtype, "L1_in")
    check_tensor(L2_in, [nnz, e.L2], e.dtype, "L2_in")
    check_tensor(W, _wshape(e, nnz), e.dtype, "W")
    if L3_grad is not None:
        check_tensor(L3_grad, [nodes, e.L3], e.dtype, "L3_grad")
    check_tensor(rows, [nnz], torch.int64, "rows")
    check_tensor(cols, [nnz], torch.int64, "cols")
    if e.deterministic:
        check_tensor(perm, [nnz], torch.int64, "transpose perm")
    if _check_indices_enabled():
        check_edge_list(nodes, rows, cols, perm if e.deterministic else None, bool(e.deterministic))
    if e.deterministic:
        pass
    elif (torch.are_deterministic_algorithms_enabled() and not e.unfused
          and (_walk_dims(e)["deterministic"] == rt.CONV_ATOMIC
               or (L3_grad is not None and _walk_dims(e).get("dx_mode", 0) == rt.DX_ATOMIC))):
        # counterpart of at::globalContext().alertNotDeterministic (torch_core.hpp:448) for the calls that
        # use float atomics: the backward of deterministic=False (sender gradients), and both directions
        # of the float-atomics kernels. The grouped forward sums in a fixed order and needs no alert.
        msg = ("OpenEquivariance_conv_atomic does not have a deterministic implementation, but you set "
               "'torch.use_deterministic_algorithms(True)'. Use TensorProductConv(..., deterministic=True).")
        if torch.is_deterministic_algorithms_warn_only_enabled():
            import warnings
            warnings.warn(msg)
        else:
            raise RuntimeError(msg)
    return nodes, nnz


# ---------------------------------------------------------------------------
# index of an edge list, kept between calls
# ---------------------------------------------------------------------------

# A walk-mode convolution first derives an index from the edge list (CSR pointers, edge grouping, walk
# order; include/oeq_amd.h, oeq_conv_index_build). The layers of a model, and the forward and backward of
# each, usually run over the same edge tensors, so the ops keep the last few indices and reuse one when a
# call brings the same tensors (same storage, same version counters, i.e. not written to since), on the same
# stream, for a kernel set that indexes the same way. The cache holds references to the edge tensors, so
# their memory cannot be handed to different data while an entry exists. 0 switches the cache off.
INDEX_CACHE_ENTRIES = 4
_index_cache: List[dict] = []
_index_cache_lock = threading.Lock()


def clear_index_cache():
    with _index_cache_lock:
        _index_cache.clear()


def _version_of(t: torch.Tensor) -> Optional[int]:
    """Version counter of a tensor, None where there is none (tensors made under
    ``torch.inference_mode()`` do not track one: reading it raises)."""
    if t.is_inference():
        return None
    try:
        return t._version
    except RuntimeError:
        return None


def _conv_index(ks, nodes: int, nnz: int, r: torch.Tensor, c: torch.Tensor, p: Optional[torch.Tensor],
                need_sender_side: bool):
    """(index tensor, sender_side flag) for the edge list; built now unless a valid one is cached."""
    dims = ks.dims
    stream = _stream()
    grouped = dims["deterministic"] == rt.CONV_GROUPED
    # the sender side is cheap to add when the caller brings the sender-major permutation, costly when the
    # library has to group the edges by sender itself: then only the calls that need it build it
    sender_side = need_sender_side or (not grouped and p is not None and p.numel() == nnz)
    key = (dims["deterministic"], dims.get("order_hops", 0), dims.get("hub_limit", 0), nodes, nnz, r.data_ptr(),
           c.data_ptr(),
           p.data_ptr() if (p is not None and not grouped) else 0, stream, r.device.index)
    versions = (_version_of(r), _version_of(c), _version_of(p) if (p is not None and not grouped) else 0)
    # an edge tensor without a version counter could be rewritten unnoticed: such a call builds its index
    # and keeps nothing
    caching = (INDEX_CACHE_ENTRIES > 0 and not torch.cuda.is_current_stream_capturing()
               and None not in versions)
    if caching:
        with _index_cache_lock:
            for i, ent in enumerate(_index_cache):
                if ent["key"] == key and ent["versions"] == versions and (ent["sender_side"] or not sender_side):
                    _index_cache.append(_index_cache.pop(i))
                    return ent["index"], ent["sender_side"]
    nb = ks.conv_index_bytes(nodes, nnz, sender_side)
    index = torch.empty(max(nb, 1), dtype=torch.uint8, device=r.device)
    ks.conv_index_build(nodes, nnz, r.data_ptr(), c.data_ptr(), p.data_ptr() if (p is not None and not grouped) else 0,
                        sender_side, index.data_ptr(), nb, stream)
    if caching:
        with _index_cache_lock:
            _index_cache[:] = [ent for ent in _index_cache if ent["key"] != key]
            _index_cache.append({"key": key, "versions": versions, "sender_side": sender_side, "index": index,
                                 "refs": (r, c, p)})
            del _index_cache[:-INDEX_CACHE_ENTRIES]
    return index, sender_side


def _segment_sum(ks, src: torch.Tensor, n_segments: int, keys: torch.Tensor, perm: Optional[torch.Tensor]):
    """Ordered sum of the rows of ``src`` over runs of equal ``keys`` (read through ``perm`` if given)."""
    dst = src.new_empty((n_segments, src.shape[1]))
    nb = ks.segment_sum_workspace_bytes(n_segments)
    ws = torch.empty(max(nb, 1), dtype=torch.uint8, device=src.device)
    ks.segment_sum(n_segments, src.shape[0], src.shape[1], src.data_ptr(), dst.data_ptr(), keys.data_ptr(),
                   perm.data_ptr() if perm is not None else 0, ws.data_ptr(), nb, _stream())
    return dst


def _scatter_rows(e: KernelEntry, ks, src, n_segments, keys, perm):
    """Sum edge rows into node rows in a fixed order: along the caller's sorted list when deterministic,
    else after grouping the edge indices by key on the device (the reference's unfused path,
    core/ConvolutionBase.py:292-301, uses a float-atomics scatter_add)."""
    if e.deterministic:
        return _segment_sum(ks, src, n_segments, keys, perm)
    dst = src.new_empty((n_segments, src.shape[1]))
    nb = ks.grouped_sum_workspace_bytes(n_segments, src.shape[0])
    ws = torch.empty(max(nb, 1), dtype=torch.uint8, device=src.device)
    ks.grouped_sum(n_segments, src.shape[0], src.shape[1], src.data_ptr(), dst.data_ptr(), keys.data_ptr(),
                   ws.data_ptr(), nb, _stream())
    return dst


def _unfused_forward(e, ks, x, y, w, r, c, nodes, nnz):
    xe = x.index_select(0, c)
    msg = x.new_empty((nnz, e.L3))
    ks.tp_forward(nnz, xe.data_ptr(), y.data_ptr(), w.data_ptr(), msg.data_ptr(), _stream())
    return _scatter_rows(e, ks, msg, nodes, r, None)


def _unfused_backward(e, ks, x, y, w, g, r, c, p, nodes, nnz):
    xe, ge = x.index_select(0, c), g.index_select(0, r)
    dxe, dy, dw = torch.empty_like(xe), torch.empty_like(y), torch.empty_like(w)
    nb = ks.tp_backward_workspace_bytes(nnz)
    ws = torch.empty(max(nb, 1), dtype=torch.uint8, device=x.device)
    ks.tp_backward(nnz, xe.data_ptr(), dxe.data_ptr(), y.data_ptr(), dy.data_ptr(), w.data_ptr(), dw.data_ptr(),
                   ge.data_ptr(), ws.data_ptr() if nb else 0, nb, _stream())
    return _scatter_rows(e, ks, dxe, nodes, c, p if e.deterministic else None), dy, dw


def _unfused_double_backward(e, ks, x, y, w, g, a, b, c, r, cc, p, nodes, nnz):
    """Second-order pass of the unfused convolution: the batch kernel pair on gathered rows, the per-edge
    sender gradients and second cotangents summed into node rows in the order of the first-order passes."""
    xe, ae, ge = x.index_select(0, cc), a.index_select(0, cc), g.index_select(0, r)
    dxe, dy, dw, gge = torch.empty_like(xe), torch.empty_like(y), torch.empty_like(w), torch.empty_like(ge)
    nb = ks.tp_double_backward_workspace_bytes(nnz)
    ws = torch.empty(max(nb, 1), dtype=torch.uint8, device=x.device)
    ks.tp_double_backward(nnz, xe.data_ptr(), y.data_ptr(), w.data_ptr(), ge.data_ptr(), ae.data_ptr(), b.data_ptr(),
                          c.data_ptr(), dxe.data_ptr(), dy.data_ptr(), dw.data_ptr(), gge.data_ptr(), ws.data_ptr(), nb,
                          _stream())
    return (_scatter_rows(e, ks, dxe, nodes, cc, p if e.deterministic else None), dy, dw,
            _scatter_rows(e, ks, gge, nodes, r, None))


_ones_cache: Dict[tuple, torch.Tensor] = {}


def _ones(n: int, like: torch.Tensor, cols: Optional[int] = None) -> torch.Tensor:
    """A tensor of ones ([n] or [n, cols]) in the dtype and on the device of ``like``; the few shapes a model
    uses are kept (they are read-only operands of the factored convolution)."""
    key = (n, cols, like.dtype, like.device)
    t = _ones_cache.get(key)
    if t is None:
        if len(_ones_cache) > 64:
            _ones_cache.clear()
        t = torch.ones((n,) if cols is None else (n, cols), dtype=like.dtype, device=like.device)
        _ones_cache[key] = t
    return t


def _factored_forward(e: KernelEntry, x, y, w, r, c, p):
    """Shared weights, single-channel second operands: contraction summed per receiver by the fused 'uvu'
    convolution of the first part, then ONE channel mix per node (core/problems.py: factor_shared_uvw)."""
    kid_a, kid_b = e.factored
    mid = conv_forward(x, y, _ones(get_entry(kid_a).WN, x), r, c, p, kid_a)
    return tp_forward(mid, _ones(x.shape[0], x, 1), w, kid_b)


def _factored_backward(e: KernelEntry, x, y, w, g, r, c, p):
    kid_a, kid_b = e.factored
    ones_a, ones_b = _ones(get_entry(kid_a).WN, x), _ones(x.shape[0], x, 1)
    mid = conv_forward(x, y, ones_a, r, c, p, kid_a)            # recomputed: one node-sized tensor
    dmid, _, dw = tp_backward(mid, ones_b, w, g, kid_b)         # mix: gradients of the node sums and of W
    dx, dy, _ = conv_backward(x, y, ones_a, dmid, r, c, p, kid_a)
    return dx, dy, dw


@torch.library.custom_op("oeq_amd::conv_forward", mutates_args=(), device_types="cuda")
def conv_forward(L1_in: torch.Tensor, L2_in: torch.Tensor, W: torch.Tensor, rows: torch.Tensor,
                 cols: torch.Tensor, transpose_perm: torch.Tensor, kid: int,
                 spec: Optional[torch.Tensor] = None) -> torch.Tensor:
    e = get_entry(kid, spec)
    nodes, nnz = _conv_checks(e, L1_in, L2_in, W, rows, cols, transpose_perm)
    x, y, w = L1_in.contiguous(), L2_in.contiguous(), W.contiguous()
    r, c = rows.contiguous(), cols.contiguous()
    if e.factored:
        return _factored_forward(e, x, y, w, r, c, transpose_perm)
    if e.unfused:
        with torch.cuda.device(x.device):
            return _unfused_forward(e, e.kernels(), x, y, w, r, c, nodes, nnz)
    out = x.new_empty((nodes, e.L3))
    with torch.cuda.device(x.device):
        ks = e.kernels()
        if ks.dims["deterministic"] == rt.CONV_ATOMIC or nodes == 0 or nnz == 0:
            ks.conv_forward(nodes, nnz, x.data_ptr(), y.data_ptr(), w.data_ptr(), out.data_ptr(), r.data_ptr(),
                            c.data_ptr(), 0, 0, _stream())
        else:
            perm = transpose_perm.contiguous() if e.deterministic else None
            # the forward walk needs the receiver side only; where the backward pass will want the edges grouped
            # by sender as well, both are built now, so that one index serves the whole step
            both = ks.dims["deterministic"] == rt.CONV_GROUPED and ks.dims.get("dx_mode", 0) != rt.DX_ATOMIC
            index, side = _conv_index(ks, nodes, nnz, r, c, perm, both)
            nb = ks.conv_forward_scratch_bytes(nodes, nnz)
            ws = torch.empty(max(nb, 1), dtype=torch.uint8, device=x.device)
            ks.conv_forward_indexed(nodes, nnz, x.data_ptr(), y.data_ptr(), w.data_ptr(), out.data_ptr(), r.data_ptr(),
                                    c.data_ptr(), index.data_ptr(), index.numel(), side, ws.data_ptr() if nb else 0, nb,
                                    _stream())
    return out


@conv_forward.register_fake
def _(L1_in, L2_in, W, rows, cols, transpose_perm, kid, spec=None):
    e = get_entry(kid, spec)
    return L1_in.new_empty((L1_in.shape[0], e.L3))


@torch.library.custom_op("oeq_amd::conv_backward", mutates_args=(), device_types="cuda")
def conv_backward(L1_in: torch.Tensor, L2_in: torch.Tensor, W: torch.Tensor, L3_grad: torch.Tensor,
                  rows: torch.Tensor, cols: torch.Tensor, transpose_perm: torch.Tensor,
                  kid: int, spec: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    e = get_entry(kid, spec)
    nodes, nnz = _conv_checks(e, L1_in, L2_in, W, rows, cols, transpose_perm, L3_grad)
    x, y, w, g = L1_in.contiguous(), L2_in.contiguous(), W.contiguous(), L3_grad.contiguous()
    r, c, p = rows.contiguous(), cols.contiguous(), transpose_perm.contiguous()
    if e.factored:
        return _factored_backward(e, x, y, w, g, r, c, p)
    if e.unfused:
        with torch.cuda.device(x.device):
            return _unfused_backward(e, e.kernels(), x, y, w, g, r, c, p, nodes, nnz)
    dx, dy, dw = torch.empty_like(x), torch.empty_like(y), torch.empty_like(w)
    with torch.cuda.device(x.device):
        ks = e.kernels()
        pp = p.data_ptr() if e.deterministic else 0
        if ks.dims["deterministic"] == rt.CONV_ATOMIC or nodes == 0 or nnz == 0:
            ks.conv_backward(nodes, nnz, x.data_ptr(), dx.data_ptr(), y.data_ptr(), dy.data_ptr(), w.data_ptr(),
                             dw.data_ptr(), g.data_ptr(), r.data_ptr(), c.data_ptr(), pp, 0, 0, _stream())
        else:
            terms = ks.dims.get("dx_mode", 0) != rt.DX_ATOMIC
            index, side = _conv_index(ks, nodes, nnz, r, c, p if e.deterministic else None, terms)
            nb = ks.conv_backward_scratch_bytes(nodes, nnz)
            ws = torch.empty(max(nb, 1), dtype=torch.uint8, device=x.device)
            ks.conv_backward_indexed(nodes, nnz, x.data_ptr(), dx.data_ptr(), y.data_ptr(), dy.data_ptr(), w.data_ptr(),
                                     dw.data_ptr(), g.data_ptr(), r.data_ptr(), c.data_ptr(), pp, index.data_ptr(),
                                     index.numel(), side, ws.data_ptr() if nb else 0, nb, _stream())
    return dx, dy, dw


@conv_backward.register_fake
def _(L1_in, L2_in, W, L3_grad, rows, cols, transpose_perm, kid, spec=None):
    return torch.empty_like(L1_in), torch.empty_like(L2_in), torch.empty_like(W)


def _conv_fwd_setup(ctx, inputs, output):
    ctx.kid, ctx.spec = inputs[6], inputs[7]
    ctx.save_for_backward(*inputs[:6])


def _conv_fwd_backward(ctx, grad):
    x, y, w, rows, cols, perm = ctx.saved_tensors
    dx, dy, dw = conv_backward(x, y, w, grad, rows, cols, perm, ctx.kid, ctx.spec)
    return dx, dy, dw, None, None, None, None, None


conv_forward.register_autograd(_conv_fwd_backward, setup_context=_conv_fwd_setup)


def _conv_bwd_setup(ctx, inputs, output):
    ctx.kid, ctx.spec = inputs[7], inputs[8]
    ctx.save_for_backward(*inputs[:7])


@torch.library.custom_op("oeq_amd::conv_double_backward", mutates_args=(), device_types="cuda")
def conv_double_backward(L1_in: torch.Tensor, L2_in: torch.Tensor, W: torch.Tensor, L3_grad: torch.Tensor,
                         L1_dgrad: torch.Tensor, L2_dgrad: torch.Tensor, W_dgrad: torch.Tensor,
                         rows: torch.Tensor, cols: torch.Tensor, transpose_perm: torch.Tensor,
                         kid: int, spec: Optional[torch.Tensor] = None
                         ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """(L1_grad, L2_grad, W_grad, L3_dgrad): the op of the reference's jit_conv_double_backward
    (extension/torch_core.hpp:544-625)."""
    e = get_entry(kid, spec)
    if e.second_order_kid is not None:
        e = get_entry(e.second_order_kid)
    nodes, nnz = _conv_checks(e, L1_in, L2_in, W, rows, cols, transpose_perm, L3_grad)
    _conv_checks(e, L1_dgrad, L2_dgrad, W_dgrad, rows, cols, transpose_perm)
    x, y, w, g = L1_in.contiguous(), L2_in.contiguous(), W.contiguous(), L3_grad.contiguous()
    a, b, c = L1_dgrad.contiguous(), L2_dgrad.contiguous(), W_dgrad.contiguous()
    r, cc, p = rows.contiguous(), cols.contiguous(), transpose_perm.contiguous()
    if e.factored:
        # the map is linear in each of X, Y, W: its second-order pass is a sum of first-order calls, each of
        # them the cheap factored form (one channel mix per node)
        with torch.no_grad():
            return _second_order(lambda p1, q1, r1: _factored_forward(e, p1, q1, r1, r, cc, p),
                                 lambda p1, q1, r1, s1: _factored_backward(e, p1, q1, r1, s1, r, cc, p),
                                 x, y, w, g, a, b, c)
    if e.unfused:
        with torch.cuda.device(x.device):
            return _unfused_double_backward(e, e.kernels(), x, y, w, g, a, b, c, r, cc, p, nodes, nnz)
    dx, dy, dw, gg = torch.empty_like(x), torch.empty_like(y), torch.empty_like(w), torch.empty_like(g)
    with torch.cuda.device(x.device):
        ks = e.kernels()
        pp = p.data_ptr() if e.deterministic else 0
        if nodes == 0 or nnz == 0:
            ks.conv_double_backward(nodes, nnz, x.data_ptr(), y.data_ptr(), w.data_ptr(), g.data_ptr(), a.data_ptr(),
                                    b.data_ptr(), c.data_ptr(), dx.data_ptr(), dy.data_ptr(), dw.data_ptr(),
                                    gg.data_ptr(), r.data_ptr(), cc.data_ptr(), pp, 0, 0, _stream())
        else:
            index, _side = _conv_index(ks, nodes, nnz, r, cc, p if e.deterministic else None, True)
            nb = ks.conv_double_backward_scratch_bytes(nodes, nnz)
            ws = torch.empty(max(nb, 1), dtype=torch.uint8, device=x.device)
            ks.conv_double_backward_indexed(nodes, nnz, x.data_ptr(), y.data_ptr(), w.data_ptr(), g.data_ptr(),
                                            a.data_ptr(), b.data_ptr(), c.data_ptr(), dx.data_ptr(), dy.data_ptr(),
                                            dw.data_ptr(), gg.data_ptr(), r.data_ptr(), cc.data_ptr(), pp,
                                            index.data_ptr(), index.numel(), ws.data_ptr() if nb else 0, nb, _stream())
    return dx, dy, dw, gg


@conv_double_backward.register_fake
def _(L1_in, L2_in, W, L3_grad, L1_dgrad, L2_dgrad, W_dgrad, rows, cols, transpose_perm, kid, spec=None):
    return torch.empty_like(L1_in), torch.empty_like(L2_in), torch.empty_like(W), torch.empty_like(L3_grad)


def _conv_bwd_backward(ctx, ddx, ddy, ddw):
    x, y, w, g, rows, cols, perm = ctx.saved_tensors
    kid, spec = ctx.kid, ctx.spec
    if _use_fused(kid, spec, ddx, ddy, ddw):
        dx, dy, dw, gg = conv_double_backward(x, y, w, g, _zeros_if_none(ddx, x), _zeros_if_none(ddy, y),
                                              _zeros_if_none(ddw, w), rows, cols, perm, kid, spec)
        return dx, dy, dw, gg, None, None, None, None, None
    dx, dy, dw, gg = _second_order(lambda a, b, c: conv_forward(a, b, c, rows, cols, perm, kid, spec),
                                   lambda a, b, c, d: conv_backward(a, b, c, d, rows, cols, perm, kid, spec),
                                   x, y, w, g, ddx, ddy, ddw)
    return dx, dy, dw, gg, None, None, None, None, None


conv_backward.register_autograd(_conv_bwd_backward, setup_context=_conv_bwd_setup)


# Mixed precision: the kernels are compiled for one dtype; under autocast the
# ops run in that dtype (cf. the reference's register_autocast to float32,
# _torch/TensorProduct.py:362-374).
def _register_autocast():
    for op in (tp_forward, tp_backward, conv_forward, conv_backward):
        try:
            op.register_autocast("cuda", torch.float32)
        except Exception:  # older/newer torch without this hook: ops still validate dtypes
            pass


_register_autocast()
