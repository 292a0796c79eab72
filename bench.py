#!/usr/bin/env python3
"""Benchmark of the fused equivariant graph convolution at MACE shape.

One step = forward + backward of ``TensorProductConv`` (deterministic mode) on a
synthetic periodic radius graph: N = 50000 nodes, mean degree ~32 (E ~ 1.6 M),
X = 128x{0e,1o,2e,3o}, Y = spherical harmonics lmax 3, 23 'uvu' paths, fp32.
All inputs are resident in HBM before the timed region starts. The default
``deterministic=False`` mode on shuffled edges (device-side grouping, sender
gradients by float atomics; and the reference-style float-atomics kernels for
comparison) is timed beside it and reported in ``modes``. Next to the HBM
roofline the record carries the vector-ALU bound of the step (the kernels are
compiled without packed FP32 instructions) and the stream ceilings measured on
the same GPU by ./hbm_stream.

Prints ONE JSON line (rank 0). ``value`` = edges per second of the whole step.
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
FP32_VECTOR_PEAK_TFLOPS = 157.3  # published; reached with packed FP32 instructions, which this build does not use


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--nodes", type=int, default=50000)
    ap.add_argument("--degree", type=float, default=32.0)
    ap.add_argument("--atomic-steps", type=int, default=3)
    ap.add_argument("--cpu-receivers", type=int, default=48, help="receivers in the CPU-baseline sub-graph (0 = skip)")
    ap.add_argument("--no-atomic", action="store_true")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the side measurements (spatially ordered nodes, batch tensor-product configs)")
    ap.add_argument("--with-double", action="store_true",
                    help="with --no-extras: still run the second-order (double backward) side measurement")
    ap.add_argument("--only-tp", default=None, metavar="N",
                    help="run only the batched tensor-product side measurement for config N (1, 2, 3, 3d, 4, 4d, dd) "
                         "and print its row; used for per-kernel profiles")
    return ap.parse_args()


def time_steps(fn, steps, warmup):
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def cpu_baseline(problem, graph, Ysh, n_receivers, seed=0):
    """e3nn-equivalent torch-CPU einsum + index_add (oracle/torch_ref.py), forward
    and backward, on the sub-graph made of the first receivers and all their
    edges; same problem, fp32, all host threads."""
    import numpy as np
    import torch
    from oracle import e3nn_ref as R
    from oracle.torch_ref import TorchConv

    cores = os.cpu_count() or 1
    threads = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(threads)
    e_end = int(np.searchsorted(graph.rows, n_receivers, side="left"))
    rows = torch.tensor(graph.rows[:e_end])
    cols_np = graph.cols[:e_end]
    # compact the senders that occur so the sample does not carry all 50000 rows of X
    uniq, inv = np.unique(np.concatenate([cols_np, np.arange(n_receivers)]), return_inverse=True)
    cols = torch.tensor(inv[:e_end])
    n_local = len(uniq)
    gen = torch.Generator().manual_seed(seed)
    X = torch.randn(n_local, problem.irreps_in1.dim, generator=gen, requires_grad=True)
    Y = torch.tensor(Ysh[:e_end], requires_grad=True)
    W = torch.randn(e_end, problem.weight_numel, generator=gen, requires_grad=True)
    conv = TorchConv(R.Problem.from_spec(problem), torch.float32)
    # receivers keep their ids 0..n_receivers-1 only if those ids are the first n_receivers of uniq
    recv_local = torch.tensor(np.searchsorted(uniq, graph.rows[:e_end]))

    def step():
        for t in (X, Y, W):
            t.grad = None
        Z = conv(X, Y, W, recv_local, cols)
        Z.backward(torch.ones_like(Z))

    step()
    reps, t0 = 0, time.perf_counter()
    while reps < 3 or (time.perf_counter() - t0 < 10.0 and reps < 50):
        step()
        reps += 1
    dt = (time.perf_counter() - t0) / reps
    return {
        "value": e_end / dt, "unit": "edges/s", "cores": threads, "kind": "port",
        "sample": f"fwd+bwd on the sub-graph of the first {n_receivers} receivers ({e_end} edges, {n_local} nodes), "
                  f"torch-CPU einsum + index_add restatement of e3nn (e3nn not installed), fp32, {reps} reps",
        "seconds_per_step": dt, "host_cpus": cores,
    }


def tp_config_table(dev, only=None):
    """Side measurements: the batched tensor product at configs 1-4 (forward and backward timed
    separately, median of 10). Bytes = every operand once per row (shared weights once per call);
    FLOPs by the reference's convention, and dense 2*u*w*(2l+1) per path for the MFMA config."""
    import numpy as np
    import torch

    import openequivariance_amd as oeq
    from openequivariance_amd._torch import ops
    from openequivariance_amd.codegen.lower import lower
    from openequivariance_amd.core import problems as P

    # 512 MiB written before every timed call: twice the 256 MB Infinity Cache, so no operand of the call is
    # still cached from the previous iteration (the reference flushes 100 MB, backend_hip.hpp:88-95)
    flush = torch.empty(512 << 20, dtype=torch.uint8, device=dev)

    def med(fn, warm=3, it=10):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        ts = []
        for _ in range(it):
            flush.zero_()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            fn()
            b.record()
            torch.cuda.synchronize()
            ts.append(a.elapsed_time(b))
        return float(np.median(ts))

    cases = [("cfg1 single uvu f32", P.config1_single_uvu(), 100000), ("cfg2 nequip uvu f32", P.config2_nequip_uvu(), 200000),
             ("cfg3 mace uvu f32", P.config3_mace_uvu(), 500000), ("cfg3 mace uvu f64", P.config3_mace_uvu(np.float64), 500000),
             ("cfg4 uvw shared f32 (MFMA)", P.config4_uvw_shared(), 262144),
             ("cfg4 uvw shared f64 (MFMA)", P.config4_uvw_shared(np.float64), 131072),
             ("DiffDock L=1 uvw per-row weights f32", P.diffdock_problems()[0], 100000)]
    # multiplicities that are no multiples of 16 (48 and 10 channels) with shared weights: matrix cores, padded tiles
    padded = P.diffdock_problems()[0].clone()
    padded.shared_weights = True
    cases.append(("DiffDock L=1 uvw shared f32 (MFMA, padded tiles)", padded, 262144))
    if only is not None:
        cases = [cases[["1", "2", "3", "3d", "4", "4d", "dd", "pad"].index(only)]]
    table = []
    for name, prob, B in cases:
        low = lower(prob)
        es = low.elem_size
        dt = torch.float32 if es == 4 else torch.float64
        x = torch.randn(B, low.L1, device=dev, dtype=dt)
        y = torch.randn(B, low.L2, device=dev, dtype=dt)
        w = torch.randn((low.WN,) if prob.shared_weights else (B, low.WN), device=dev, dtype=dt)
        g = torch.randn(B, low.L3, device=dev, dtype=dt)
        tp = oeq.TensorProduct(prob)
        tf = med(lambda: ops.tp_forward(x, y, w, tp.kid))
        tb = med(lambda: ops.tp_backward(x, y, w, g, tp.kid))
        wrow = 0 if prob.shared_weights else low.WN
        wcall = low.WN * es if prob.shared_weights else 0
        fb = B * (low.L1 + low.L2 + low.L3 + wrow) * es + wcall
        bb = B * (2 * low.L1 + 2 * low.L2 + low.L3 + 2 * wrow) * es + 2 * wcall
        row = {"config": name, "rows": B, "fwd_ms": tf, "bwd_ms": tb,
               "fwd_rows_per_s": B / tf * 1e3, "bwd_rows_per_s": B / tb * 1e3,
               "fwd_gflops": B * low.flops("forward") / tf / 1e6, "bwd_gflops": B * low.flops("backward") / tb / 1e6,
               "fwd_hbm_frac": fb / tf / 1e6 / HBM_PEAK_GBS, "bwd_hbm_frac": bb / tb / 1e6 / HBM_PEAK_GBS}
        if low.mode == "uvw" and prob.shared_weights:
            dense = sum(2 * low.in1[p.i1].mul * low.in2[p.i2].mul * low.out[p.io].mul * low.out[p.io].d for p in low.paths)
            row["fwd_dense_tflops"] = B * dense / tf / 1e9
            row["bwd_dense_tflops"] = 2 * B * dense / tb / 1e9
            peak = 157.3 if es == 4 else 78.6  # dense MFMA TFLOP/s, fp32 / fp64
            row["fwd_mfma_frac"] = row["fwd_dense_tflops"] / peak
            row["bwd_mfma_frac"] = row["bwd_dense_tflops"] / peak
        if name.startswith(("cfg2", "cfg4 uvw shared f32", "DiffDock")) and ops.get_entry(tp.kid).kernels().has_double_backward():
            # second-order pass (the backward of the backward): the fused kernel pair beside the composition of
            # three forward and three backward calls; bytes = every operand once per kernel
            a, b, c = torch.randn_like(x), torch.randn_like(y), torch.randn_like(w)
            t2 = med(lambda: ops.tp_double_backward(x, y, w, g, a, b, c, tp.kid), it=7)
            tc = med(lambda: ops._second_order(lambda p, q, r: ops.tp_forward(p, q, r, tp.kid),
                                               lambda p, q, r, s_: ops.tp_backward(p, q, r, s_, tp.kid),
                                               x, y, w, g, a, b, c), warm=1, it=3)
            db = B * (5 * low.L1 + 5 * low.L2 + 5 * wrow + 2 * low.L3) * es + 5 * wcall
            row["second_order"] = {"fused_ms": t2, "composed_first_order_ms": tc,
                                   "hbm_frac": db / t2 / 1e6 / HBM_PEAK_GBS}
            del a, b, c
        table.append(row)
        del x, y, w, g
        torch.cuda.empty_cache()
    del flush
    return table


def uvw_conv_table(dev, nodes=12000):
    """Side measurement: the fused 'uvw' convolution with per-edge weights (DiffDock, e3tools) on a graph of
    the headline's density, forward and backward, beside the unfused path (gathered rows, batch kernels,
    segment sums) that it replaces, and the second-order kernel pair beside the composition of first-order
    calls. Bytes = every operand once per kernel (W and dW dominate: 27-30 KB per edge)."""
    import numpy as np
    import torch

    import openequivariance_amd as oeq
    from openequivariance_amd._torch import ops
    from openequivariance_amd.codegen.lower import lower
    from openequivariance_amd.core import problems as P
    from openequivariance_amd.core.graph import CoordGraph, periodic_radius_graph

    coords, rows, cols, _vec = periodic_radius_graph(nodes, 32.0 * (nodes / 50000) ** (1 / 3), 5.0, 0)
    g = CoordGraph(coords, rows, cols)
    E = g.nnz
    tr, tc, tp = (torch.tensor(a, device=dev) for a in (g.rows, g.cols, g.transpose_perm))

    def med(fn, warm=2, it=7):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        ts = []
        for _ in range(it):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            fn()
            b.record()
            torch.cuda.synchronize()
            ts.append(a.elapsed_time(b))
        return float(np.median(ts))

    table = []
    saved = os.environ.get("OEQ_AMD_TUNE")
    try:
        for prob in (P.diffdock_problems()[0], P.e3tools_problems()[0]):
            low = lower(prob)
            X, Y = torch.randn(nodes, low.L1, device=dev), torch.randn(E, low.L2, device=dev)
            W, G = torch.randn(E, low.WN, device=dev), torch.randn(nodes, low.L3, device=dev)
            fb = 4 * (E * (low.WN + low.L2 + low.L1) + nodes * low.L3)
            bb = 4 * (E * (2 * low.WN + 2 * low.L2 + low.L1) + nodes * (low.L3 + low.L1))
            row = {"config": prob.label, "nodes": nodes, "edges": E, "mode": "deterministic"}
            for key, fuse in (("fused", 1), ("unfused", 0)):
                os.environ["OEQ_AMD_TUNE"] = ((saved + ",") if saved else "") + f"conv_fuse_uvw={fuse}"
                kid = oeq.TensorProductConv(prob, deterministic=True).kid
                tf = med(lambda: ops.conv_forward(X, Y, W, tr, tc, tp, kid))
                tb = med(lambda: ops.conv_backward(X, Y, W, G, tr, tc, tp, kid))
                row[key] = {"fwd_ms": tf, "bwd_ms": tb, "fwd_hbm_frac": fb / tf / 1e6 / HBM_PEAK_GBS,
                            "bwd_hbm_frac": bb / tb / 1e6 / HBM_PEAK_GBS}
                if fuse and ops.get_entry(kid).kernels().has_double_backward():
                    # second-order pass: the fused kernel pair beside three forward and three backward calls
                    A_, B_, C_ = torch.randn_like(X), torch.randn_like(Y), torch.randn_like(W)
                    t2 = med(lambda: ops.conv_double_backward(X, Y, W, G, A_, B_, C_, tr, tc, tp, kid), it=5)
                    tc2 = med(lambda: ops._second_order(
                        lambda p, q, r: ops.conv_forward(p, q, r, tr, tc, tp, kid),
                        lambda p, q, r, s_: ops.conv_backward(p, q, r, s_, tr, tc, tp, kid), X, Y, W, G, A_, B_, C_),
                        warm=1, it=3)
                    # per-edge tensors: Y, B, W, C read by both kernels, dY and dW written; node tensors once per
                    # kernel (the per-edge dX terms and the re-gathered sender rows are not algorithmic)
                    db = 4 * (E * 5 * (low.WN + low.L2) + nodes * (5 * low.L1 + 2 * low.L3))
                    row["second_order"] = {"fused_ms": t2, "composed_first_order_ms": tc2,
                                           "hbm_frac": db / t2 / 1e6 / HBM_PEAK_GBS}
                    del A_, B_, C_
            table.append(row)
            del X, Y, W, G
            torch.cuda.empty_cache()
        # Shared weights (one weight tensor for all edges), shuffled edge list: the factored form (contraction
        # summed per receiver by the fused 'uvu' convolution, then one channel mix per NODE on the matrix
        # cores) beside the two routes that mix per edge: the matrix-core batch kernels on gathered rows with
        # ordered segment sums ("per_edge_mfma"), and the fused general kernels ("per_edge_general").
        shared_dd = P.diffdock_problems()[0].clone()
        shared_dd.shared_weights = True
        shared_dd.label = "DiffDock-L=1 shared weights"
        perm = torch.randperm(E, device=dev)
        rs, cs = tr[perm].contiguous(), tc[perm].contiguous()
        none = torch.zeros(0, dtype=torch.int64, device=dev)
        for prob in (shared_dd, P.config4_uvw_shared()):
            low = lower(prob)
            X, Y = torch.randn(nodes, low.L1, device=dev), torch.randn(E, low.L2, device=dev)
            W, G = torch.randn(low.WN, device=dev), torch.randn(nodes, low.L3, device=dev)
            A_, B_, C_ = torch.randn_like(X), torch.randn_like(Y), torch.randn_like(W)
            row = {"config": prob.label, "nodes": nodes, "edges": E, "mode": "deterministic=False, shuffled edges"}
            for key, knobs in (("factored", "conv_factor=1"), ("per_edge_mfma", "conv_factor=0,conv_mfma_min_weights=0"),
                               ("per_edge_general", "conv_factor=0,conv_mfma_min_weights=100000000")):
                os.environ["OEQ_AMD_TUNE"] = ((saved + ",") if saved else "") + knobs
                kid = oeq.TensorProductConv(prob, deterministic=False).kid
                row[key] = {"fwd_ms": med(lambda: ops.conv_forward(X, Y, W, rs, cs, none, kid)),
                            "bwd_ms": med(lambda: ops.conv_backward(X, Y, W, G, rs, cs, none, kid)),
                            "second_order_ms": med(lambda: ops.conv_double_backward(X, Y, W, G, A_, B_, C_, rs, cs, none,
                                                                                    kid), warm=1, it=3)}
            table.append(row)
            del X, Y, W, G, A_, B_, C_
            torch.cuda.empty_cache()
    finally:
        if saved is None:
            os.environ.pop("OEQ_AMD_TUNE", None)
        else:
            os.environ["OEQ_AMD_TUNE"] = saved
    return table


def hbm_ceilings():
    """Read-only / write-only / copy stream rates of this GPU (./hbm_stream, built by __graft_entry__.build())."""
    import subprocess
    exe = os.path.join(ROOT, "hbm_stream")
    if not os.path.exists(exe):
        return None
    try:
        res = subprocess.run([exe], capture_output=True, text=True, timeout=120)
        return json.loads(res.stdout.strip().splitlines()[-1]) if res.returncode == 0 else None
    except Exception:
        return None


def main():
    args = parse()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU only (no collectives, no sharding); "
              "use --gpus 1. (Sharding would split the receivers into contiguous blocks with a halo "
              "exchange of sender rows; it is not built.)", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    if args.only_tp is not None:
        assert torch.cuda.is_available(), "bench.py needs a GPU"
        print(json.dumps(tp_config_table("cuda:0", args.only_tp)[0]))
        return

    import openequivariance_amd as oeq
    from openequivariance_amd import runtime as rt
    from openequivariance_amd._torch import ops
    from openequivariance_amd.codegen.lower import lower
    from openequivariance_amd.core import problems as P
    from openequivariance_amd.core.graph import CoordGraph, periodic_radius_graph
    from openequivariance_amd.core.sh import spherical_harmonics

    assert torch.cuda.is_available(), "bench.py needs a GPU (there is no CPU fallback for the product path)"
    dev = "cuda:0"
    torch.cuda.set_device(0)
    problem = P.config5_mace_conv()
    low = lower(problem)
    L1, L2, L3, WN = low.L1, low.L2, low.L3, low.WN

    coords, rows, cols, vec = periodic_radius_graph(args.nodes, args.degree, 5.0, seed=0)
    graph = CoordGraph(coords, rows, cols, "periodic-radius")
    N, E = graph.node_count, graph.nnz
    Ysh = spherical_harmonics(3, vec).astype(np.float32)[graph.order]

    gen = torch.Generator(device=dev).manual_seed(0)
    X = torch.randn(N, L1, device=dev, generator=gen)
    W = torch.randn(E, WN, device=dev, generator=gen)
    G = torch.randn(N, L3, device=dev, generator=gen)
    Y = torch.tensor(Ysh, device=dev)
    tr, tc, tp = (torch.tensor(a, device=dev) for a in (graph.rows, graph.cols, graph.transpose_perm))

    es = 4
    fwd_bytes = (E * (L2 + WN) + N * (L1 + L3)) * es
    bwd_bytes = (2 * E * (L2 + WN) + N * (L1 + L3) + N * L1) * es
    fwd_flops, bwd_flops = low.flops("forward") + L3, low.flops("backward")  # per edge (conv adds the scatter)

    # ---- deterministic mode: the timed K steps --------------------------------
    conv = oeq.TensorProductConv(problem, deterministic=True)
    kid = conv.kid

    def step_det():
        ops.conv_forward(X, Y, W, tr, tc, tp, kid)
        ops.conv_backward(X, Y, W, G, tr, tc, tp, kid)

    ms_det = time_steps(step_det, args.steps, args.warmup)

    # per-kernel durations with HIP events on the launch stream, over K more steps
    ks = ops.get_entry(kid).kernels()
    ks_source = ops.get_entry(kid).build_fn()[0]  # the generated HIP source of this kernel set
    ks.timing_enable(True)
    for _ in range(args.steps):
        step_det()
    torch.cuda.synchronize()
    kt = {name: ks.timing_collect(role) for name, role in
          (("forward", rt.ROLE_CONV_FORWARD), ("backward", rt.ROLE_CONV_BACKWARD),
           ("fixup_backward", rt.ROLE_CONV_FIXUP_BACKWARD), ("oeq_segment_ptr", rt.ROLE_SEGMENT_PTR))}
    ks.timing_enable(False)
    avg = {k: (v[0] / v[1] if v[1] else 0.0) for k, v in kt.items()}

    # dominant kernel: conv `backward` (reads X[cols], Y, W, dZ; writes dY, dW and the per-edge dX terms)
    bwd_kernel_bytes = (2 * E * (L2 + WN) + N * (L1 + L3)) * es
    achieved = bwd_kernel_bytes / (avg["backward"] * 1e-3) / 1e9
    roofline = {
        "bound": "hbm", "kernel": "backward (TensorProductConv, deterministic)",
        "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
        "traffic": None,
        "algorithmic_bytes_per_launch": bwd_kernel_bytes, "avg_kernel_ms": avg["backward"],
        "launches_timed": kt["backward"][1],
    }
    # The same fraction per op, with the kernels an op cannot do without counted in: the backward op is
    # `backward` + `fixup_backward` (+ the index kernels) and moves bwd_bytes; forward moves fwd_bytes.
    index_ms = avg["oeq_segment_ptr"] * (kt["oeq_segment_ptr"][1] / max(1, kt["backward"][1]))
    bwd_op_ms = avg["backward"] + avg["fixup_backward"]
    roofline["ops"] = {
        "forward": {"algorithmic_bytes": fwd_bytes, "kernel_ms": avg["forward"],
                    "frac": fwd_bytes / (avg["forward"] * 1e-3) / 1e9 / HBM_PEAK_GBS},
        "backward_op": {"algorithmic_bytes": bwd_bytes, "kernel_ms": bwd_op_ms, "kernels": ["backward", "fixup_backward"],
                        "frac": bwd_bytes / (bwd_op_ms * 1e-3) / 1e9 / HBM_PEAK_GBS},
        "index_kernels_ms_per_step": index_ms,
    }
    # Bounds of the step (time at 100 % of a rate). The arithmetic is ordinary v_fma_f32 (every HIP file of this
    # build is compiled without packed FP32 instructions); the rate the vector units reach with those, and the
    # rate a stream of reads reaches once writes are mixed in, are measured on this box by ./hbm_stream.
    ceilings = None if args.no_extras else hbm_ceilings()
    step_flops = (fwd_flops + bwd_flops) * E
    roofline["bounds_ms"] = {
        "hbm_at_8_TBps": (fwd_bytes + bwd_bytes) / HBM_PEAK_GBS / 1e6,
        "fp32_vector_at_published_peak": step_flops / (FP32_VECTOR_PEAK_TFLOPS * 1e9),
    }
    if ceilings:
        roofline["bounds_ms"]["fp32_vector_unpacked_as_measured"] = step_flops / (ceilings["valu_fp32_tflops_unpacked"] * 1e9)
        # this step writes 40 % of its algorithmic bytes: the measured rate of a read stream with writes mixed in
        roofline["bounds_ms"]["hbm_at_measured_read_write_mix"] = (fwd_bytes + bwd_bytes) / ceilings["read_with_writes_1_2"] / 1e6
        # the step against that measured rate (frac above is against the published 8 TB/s)
        roofline["step_frac_of_measured_read_write_mix"] = roofline["bounds_ms"]["hbm_at_measured_read_write_mix"] / ms_det

    modes = {
        "deterministic": {
            "ms_per_step": ms_det, "edges_per_s": E / (ms_det * 1e-3),
            "gflops": (fwd_flops + bwd_flops) * E / (ms_det * 1e-3) / 1e9,
            "hbm_roofline_frac": (fwd_bytes + bwd_bytes) / (ms_det * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "kernel_ms": avg,
        }
    }

    # The ops keep the index derived from an edge list (CSR pointers, walk order) between calls on the same
    # tensors, as the layers of a model and their backward passes are; the same step with that cache off,
    # i.e. the index rebuilt by every forward and every backward:
    cache_entries, ops.INDEX_CACHE_ENTRIES = ops.INDEX_CACHE_ENTRIES, 0
    try:
        ms_cold = time_steps(step_det, max(3, args.steps // 2), 1)
    finally:
        ops.INDEX_CACHE_ENTRIES = cache_entries
    modes["deterministic_index_rebuilt_every_call"] = {
        "ms_per_step": ms_cold, "edges_per_s": E / (ms_cold * 1e-3),
        "hbm_roofline_frac": (fwd_bytes + bwd_bytes) / (ms_cold * 1e-3) / 1e9 / HBM_PEAK_GBS}

    # ---- deterministic=False (the API default): any edge order --------------------
    if not args.no_atomic:
        perm = torch.randperm(E, device=dev, generator=gen)
        Ya, Wa, ra, ca = Y[perm].contiguous(), W[perm].contiguous(), tr[perm].contiguous(), tc[perm].contiguous()
        dummy = torch.zeros(1, dtype=torch.int64, device=dev)

        def mode_entry(ms, steps):
            return {"ms_per_step": ms, "edges_per_s": E / (ms * 1e-3),
                    "gflops": (fwd_flops + bwd_flops) * E / (ms * 1e-3) / 1e9,
                    "hbm_roofline_frac": (fwd_bytes + bwd_bytes) / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "steps": steps}

        # default: the library groups the shuffled edges by receiver / sender on the device, then walks them
        conv_a = oeq.TensorProductConv(problem, deterministic=False)

        def step_unsorted():
            ops.conv_forward(X, Ya, Wa, ra, ca, dummy, conv_a.kid)
            ops.conv_backward(X, Ya, Wa, G, ra, ca, dummy, conv_a.kid)

        modes["nondeterministic_shuffled_edges"] = mode_entry(time_steps(step_unsorted, args.steps, 1), args.steps)
        cache_entries, ops.INDEX_CACHE_ENTRIES = ops.INDEX_CACHE_ENTRIES, 0
        try:
            modes["nondeterministic_shuffled_edges_index_rebuilt_every_call"] = mode_entry(
                time_steps(step_unsorted, max(3, args.steps // 2), 1), max(3, args.steps // 2))
        finally:
            ops.INDEX_CACHE_ENTRIES = cache_entries

        # the float-atomics kernels (edge ranges, flush at every change of receiver), same shuffled edges
        saved = os.environ.get("OEQ_AMD_TUNE")
        os.environ["OEQ_AMD_TUNE"] = ((saved + ",") if saved else "") + "conv_sort=0"
        try:
            conv_f = oeq.TensorProductConv(problem, deterministic=False)
            ops.get_entry(conv_f.kid).kernels()
        finally:
            if saved is None:
                del os.environ["OEQ_AMD_TUNE"]
            else:
                os.environ["OEQ_AMD_TUNE"] = saved

        def step_atomic():
            ops.conv_forward(X, Ya, Wa, ra, ca, dummy, conv_f.kid)
            ops.conv_backward(X, Ya, Wa, G, ra, ca, dummy, conv_f.kid)

        modes["float_atomics_shuffled_edges"] = mode_entry(time_steps(step_atomic, args.atomic_steps, 1),
                                                           args.atomic_steps)
        del Ya, Wa

    extras = {}
    if not args.no_extras:
        # Same graph with nodes numbered along a Z-order curve (core/graph.py: spatial_order): a
        # relabelling the caller can apply once per structure; it lets gathered sender rows hit in L2.
        from openequivariance_amd.core.graph import relabel_nodes, spatial_order
        order_n = spatial_order(coords)
        rows_s, cols_s = relabel_nodes(order_n, rows, cols)
        gs = CoordGraph(coords[order_n], rows_s, cols_s, "periodic-radius-zorder")
        Ys = torch.tensor(spherical_harmonics(3, vec).astype(np.float32)[gs.order], device=dev)
        trs, tcs, tps = (torch.tensor(a, device=dev) for a in (gs.rows, gs.cols, gs.transpose_perm))

        def step_sp():
            ops.conv_forward(X, Ys, W, trs, tcs, tps, kid)
            ops.conv_backward(X, Ys, W, G, trs, tcs, tps, kid)

        ms_sp = time_steps(step_sp, args.steps, args.warmup)
        modes["deterministic_zorder_nodes"] = {
            "ms_per_step": ms_sp, "edges_per_s": E / (ms_sp * 1e-3),
            "gflops": (fwd_flops + bwd_flops) * E / (ms_sp * 1e-3) / 1e9,
            "hbm_roofline_frac": (fwd_bytes + bwd_bytes) / (ms_sp * 1e-3) / 1e9 / HBM_PEAK_GBS,
        }
        del Ys, trs, tcs, tps

        # The same graph plus one hub: node 0 receives from and sends to 20 000 further nodes. Edge segments
        # longer than dims["hub_limit"] edges are walked in chunks by different wave groups, so the step should
        # cost what its 2.5 % more edges cost, not the hub's degree times one edge's latency.
        rng = np.random.default_rng(1)
        spokes = rng.choice(np.arange(1, N), size=20000, replace=False).astype(np.int64)
        spokes = spokes[~np.isin(spokes, cols[rows == 0])]  # keep the edge list free of duplicates
        rows_h = np.concatenate([rows, np.zeros(len(spokes), dtype=np.int64), spokes])
        cols_h = np.concatenate([cols, spokes, np.zeros(len(spokes), dtype=np.int64)])
        dirs = rng.normal(size=(len(spokes), 3))
        vec_h = np.concatenate([vec, dirs, -dirs])
        gh = CoordGraph(coords, rows_h, cols_h, "periodic-radius-plus-hub")
        Eh = gh.nnz
        Yh = torch.tensor(spherical_harmonics(3, vec_h).astype(np.float32)[gh.order], device=dev)
        Wh = torch.randn(Eh, WN, device=dev, generator=gen)
        trh, tch, tph = (torch.tensor(a, device=dev) for a in (gh.rows, gh.cols, gh.transpose_perm))

        def step_hub():
            ops.conv_forward(X, Yh, Wh, trh, tch, tph, kid)
            ops.conv_backward(X, Yh, Wh, G, trh, tch, tph, kid)

        ms_hub = time_steps(step_hub, max(3, args.steps // 2), 2)
        ks.timing_enable(True)
        step_hub()
        torch.cuda.synchronize()
        hub_split = {name: ks.timing_collect(role)[0] for name, role in
                     (("forward", rt.ROLE_CONV_FORWARD), ("fixup_forward", rt.ROLE_CONV_FIXUP_FORWARD),
                      ("backward", rt.ROLE_CONV_BACKWARD), ("fixup_backward", rt.ROLE_CONV_FIXUP_BACKWARD))}
        ks.timing_enable(False)
        modes["deterministic_plus_hub_of_20000_edges"] = {
            "ms_per_step": ms_hub, "edges": Eh, "edges_per_s": Eh / (ms_hub * 1e-3),
            "ms_per_step_relative_to_config5": ms_hub / ms_det, "hub_limit": ks.dims.get("hub_limit", 0),
            "kernel_ms": hub_split,
        }
        del Yh, Wh, trh, tch, tph

    # Second-order kernels at the same shape (the backward of the backward, as in force training):
    # the fused pair against the composition of three forward and three backward calls.
    if (not args.no_extras or args.with_double) and ks.has_double_backward():
        from openequivariance_amd import runtime as rt
        A_, B_, C_ = torch.randn_like(X), torch.randn_like(Y), torch.randn_like(W)

        def step_dd():
            ops.conv_double_backward(X, Y, W, G, A_, B_, C_, tr, tc, tp, kid)

        def step_composed():
            with torch.no_grad():
                ops._second_order(lambda p, q, r: ops.conv_forward(p, q, r, tr, tc, tp, kid),
                                  lambda p, q, r, s: ops.conv_backward(p, q, r, s, tr, tc, tp, kid),
                                  X, Y, W, G, A_, B_, C_)

        ms_dd = time_steps(step_dd, max(3, args.steps // 4), 2)
        ks.timing_enable(True)
        step_dd()
        torch.cuda.synchronize()
        split = {name: ks.timing_collect(role)[0] for name, role in
                 (("double_backward_A", rt.ROLE_DOUBLE_BACKWARD_A), ("double_backward_B", rt.ROLE_DOUBLE_BACKWARD_B),
                  ("fixup_backward", rt.ROLE_CONV_FIXUP_BACKWARD))}
        ks.timing_enable(False)
        ms_cmp = time_steps(step_composed, 2, 1)
        dd_bytes = 4 * (E * 3 * (L2 + WN) + N * (3 * L1 + 2 * L3))
        extras["double_backward"] = {
            "fused_ms": ms_dd, "composed_first_order_ms": ms_cmp, "kernel_ms": split,
            "hbm_roofline_frac": dd_bytes / (ms_dd * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "algorithmic_bytes_per_edge": dd_bytes / E,
        }
        del A_, B_, C_

    cpu = None
    if args.cpu_receivers > 0:
        cpu = cpu_baseline(problem, graph, Ysh, args.cpu_receivers)

    if not args.no_extras:
        del X, W, G, Y
        torch.cuda.empty_cache()
        extras["tp_configs"] = tp_config_table(dev)
        extras["uvw_conv"] = uvw_conv_table(dev)

    traffic_path = os.path.join(ROOT, "profiles", "conv_cfg5_traffic.json")
    if os.path.exists(traffic_path):
        # HBM bytes per launch of the dominant kernel, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of
        # this same command (scaled by a copy-kernel calibration); see profiles/conv_cfg5_deterministic.md
        with open(traffic_path) as f:
            tr = json.load(f)
        # the counters belong to the kernels they were measured on: the file names the hash of that kernel
        # source, and a different source here means the figures are stale (traffic stays null until the
        # profile is taken again)
        if tr.get("edges") == E and tr.get("source_hash") == rt.cache_key(ks_source):
            roofline["traffic"] = tr["backward_bytes_per_launch"]
            roofline["traffic_per_kernel"] = tr.get("per_kernel")
        else:
            roofline["traffic_note"] = ("profiles/conv_cfg5_traffic.json was measured on another kernel source "
                                        f"or by another compiler ({tr.get('source_hash')} != {rt.cache_key(ks_source)})")

    out = {
        "metric": "fused conv fwd+bwd edges/s at MACE shape (deterministic mode)",
        "value": E / (ms_det * 1e-3), "unit": "edges/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_det,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "cfg5: TensorProductConv fwd+bwd, MACE shape 128x{0e,1o,2e,3o} x SH(lmax3), 23 uvu paths",
                   "nodes": N, "edges": E, "L1": L1, "L2": L2, "L3": L3, "weight_numel": WN,
                   "graph": "uniform points in a periodic cube, cutoff 5.0, directed both ways, seed 0"},
        "gflops": modes["deterministic"]["gflops"],
        "hbm_roofline_frac_step": modes["deterministic"]["hbm_roofline_frac"],
        "algorithmic_bytes_per_edge": {"forward": fwd_bytes / E, "backward": bwd_bytes / E},
        "flops_per_edge": {"forward": fwd_flops, "backward": bwd_flops},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "modes": modes,
        "hbm_stream_ceilings": ceilings,
        # what tells a slow box from a fast one: the device, its nominal clock, and the time of a fixed amount of
        # vector arithmetic (./hbm_stream: 2 x 524 288 wave64 multiply-adds per SIMD)
        "device": {"name": torch.cuda.get_device_name(0), "compute_units": rt.device_props(0).compute_units,
                   "clock_khz_nominal": rt.device_props(0).clock_khz,
                   "valu_fixed_work_ms": ceilings["valu_fixed_work_ms"] if ceilings else None},
    }
    out.update(extras)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
