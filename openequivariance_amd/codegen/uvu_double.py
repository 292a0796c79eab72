"""HIP source generator for the second-order ('double backward') kernels of 'uvu' problems.

The first backward pass maps (X, Y, W, dZ) to (dX, dY, dW). Differentiating it once more, with
cotangents (A, B, C) for (dX, dY, dW), gives, because the tensor product ``F`` is linear in each
operand,

    d/d(dZ) = F(A, Y, W) + F(X, B, W) + F(X, Y, C)                         (kernel ``double_backward_A``)
    d/dX    = dX-part of backward(., B, W; dZ) + backward(., Y, C; dZ)
    d/dY    = dY-part of backward(A, ., W; dZ) + backward(X, ., C; dZ)     (kernel ``double_backward_B``)
    d/dW    = dW-part of backward(A, Y, .; dZ) + backward(X, B, .; dZ)

The reference computes the same two groups with its kernels ``double_backward_A`` /
``double_backward_B`` (openequivariance/openequivariance/templates/loop_unroll_batch.cuh:148-317,
templates/loop_unroll_conv_det.cuh, wired in extension/torch_core.hpp:357-420 and 544-625). Here each
kernel reads every operand once: per path the CG products of Y and of B are formed side by side, and
the weights W and C are streamed together, where composing the first-order kernels would make three
passes over the weight-sized tensors for each group.

Work decomposition is that of the first-order kernels (lane = channel, a wave or a group of chunk
waves per row / per receiver node, register-resident accumulators over a node's edges, per-edge dX
terms reduced by the sender-ordered second pass). Shared weights: the weight gradient is summed per wave
group in registers (over the rows, or the edges of the nodes, the group handles) and across groups by the
first-order pass's ordered reduction.
"""

from __future__ import annotations

import os

from typing import Dict, List, Optional, Tuple

from .common import Src
from .lower import Lowered, Path
from .uvu import UNROLL_V_LIMIT, UvuEmitter


# Convolution: above this many paths (after folding of wide rows) the kernels' register needs (two
# operand sets per path in flight beside X, A, dX, dY and the gradient slice) make them spill so much that
# they no longer beat the composition of first-order kernels (measured: SevenNet main layer, 38 paths,
# 63 - 80 ms against 66 ms; NequIP benzene, 68 paths, 155 - 175 ms against 118 ms; NequiX main layer, 27
# paths, 28 against 35 ms). The batch kernels are 3 - 4 times faster than the composition for all of them.
CONV_MAX_PATHS = 96


def supported(low: Lowered, conv: bool = False) -> bool:
    """Batch kernels: every 'uvu' problem. Convolution: up to CONV_MAX_PATHS paths."""
    if low.mode != "uvu":
        return False
    from .uvu import tuning
    return not conv or len(low.paths) <= tuning(dict(dd_maxp=CONV_MAX_PATHS))["dd_maxp"]


def dwv_live(value: str, guard: Optional[str]) -> str:
    return value if guard in (None, "true") else f"({guard} ? {value} : T(0))"


class DoubleEmitter(UvuEmitter):
    """Adds ``double_backward_A`` / ``double_backward_B`` (batch and convolution flavours) to a module
    whose structs (X_t, G_t) the base emitter has already written."""

    # ------------------------------------------------------------ operands
    def _y_of(self, row: str):
        def y(p: Path, v: str, j: int) -> str:
            return f"{row}[{self._y_index(self.low.in2[p.i2], v, j)}]"
        return y

    def _w_of(self, row: str):
        low = self.low

        def w(p: Path, v: str) -> str:
            mul = low.in1[p.i1].mul
            wp = self._ptr(row, (f"{p.woff} + ({v})", low.in2[p.i2].mul), mul)
            ld = f"__builtin_nontemporal_load({wp})" if (self.nt & 1) and not low.shared_weights else f"*{wp}"
            return self._operand(mul, ld)
        return w

    def _two_products(self, s: Src, p: Path, v: str) -> Dict[int, Tuple[str, str, bool]]:
        """|c| * y_j and |c| * b_j for the distinct (|c|, j) of a path: nnz index -> (qy, qb, negative)."""
        yacc, bacc = self._y_of("yrow"), self._y_of("brow")
        for j in sorted({j for _, j, _, _ in p.nnz}):
            s(f"const T y{j} = {yacc(p, v, j)};")
            s(f"const T b{j} = {bacc(p, v, j)};")
        names: Dict[Tuple[str, int], int] = {}
        out = {}
        for n, (i, j, k, c) in enumerate(p.nnz):
            key = (self.lit(abs(c)), j)
            if key not in names:
                names[key] = len(names)
                s(f"const T q{names[key]} = T({key[0]}) * y{j};")
                s(f"const T r{names[key]} = T({key[0]}) * b{j};")
            out[n] = (f"q{names[key]}", f"r{names[key]}", c < 0)
        return out

    # ------------------------------------------------------------ kernel A cores
    def emit_double_cores(self, s: Src):
        """dda_seg<i>: adds one row's / one edge's three forward terms to the accumulators of segment i."""
        low = self.low

        def emit():
            for si, seg in enumerate(self.segments):
                s.open(
                    f"OEQ_DEV void dda_seg{si}{self._sfx()}(const X_t& x, const X_t& xa, const T* __restrict__ yrow, "
                    "const T* __restrict__ brow, const T* __restrict__ wrow, const T* __restrict__ crow, "
                    f"const int u, D{si}_t& a)"
                )
                wacc, cacc = self._w_of("wrow"), self._w_of("crow")
                seg_paths = [p for p in self._paths() if p.io in seg]
                preload_w = (self.forms and sum(low.in2[q.i2].mul for q in seg_paths) <= 48
                             and all(low.in2[q.i2].mul <= UNROLL_V_LIMIT for q in seg_paths))
                if preload_w:
                    # the weights are folded into the X operands at the top of every path: all requested here
                    for q in seg_paths:
                        for v in range(low.in2[q.i2].mul):
                            s(f"const T wv{q.index}_{v} = {wacc(q, str(v))};")
                            s(f"const T cv{q.index}_{v} = {cacc(q, str(v))};")
                for p in seg_paths:
                    s(f"// path {p.index}")

                    def body(v, p=p, preload_w=preload_w):
                        # z''_k = sum c [ y_j (w a_i + c_w x_i) + b_j (w x_i) ]: with the weights folded into two
                        # per-lane vectors first, a term costs two multiply-adds instead of three plus the
                        # weighting of two partial results; the coefficient then rides on (|c|, j) products
                        # or, summing the terms of equal |c| first, on the result - whichever is fewer.
                        if not self.forms:
                            return body_plain(v, p)
                        yacc, bacc = self._y_of("yrow"), self._y_of("brow")
                        for j in sorted({j for _, j, _, _ in p.nnz}):
                            s(f"const T y{j} = {yacc(p, v, j)};")
                            s(f"const T b{j} = {bacc(p, v, j)};")
                        s(f"const T wv = {f'wv{p.index}_{v}' if preload_w else wacc(p, v)};")
                        s(f"const T cv = {f'cv{p.index}_{v}' if preload_w else cacc(p, v)};")
                        for i in sorted({i for i, _, _, _ in p.nnz}):
                            s(f"const T r{i} = wv * x.b{p.i1}[{i}];")
                            s(f"const T p{i} = wv * xa.b{p.i1}[{i}] + cv * x.b{p.i1}[{i}];")
                        cj, ci, ck, nc = self._form_counts(p)
                        ks = sorted({k for _, _, k, _ in p.nnz})
                        if ck <= 2 * cj + len(ks):
                            sums = {}
                            for i, j, k, c in p.nnz:
                                key = (self.lit(abs(c)), k)
                                neg = c < 0
                                if key not in sums:
                                    sums[key] = f"s{len(sums)}"
                                    s(f"T {sums[key]} = {'-' if neg else ''}y{j} * p{i};")
                                else:
                                    s(f"{sums[key]} {'-=' if neg else '+='} y{j} * p{i};")
                                s(f"{sums[key]} {'-=' if neg else '+='} b{j} * r{i};")
                            for (m, k), name in sums.items():
                                s(f"a.o{p.io}[{k}] += T({m}) * {name};")
                        else:
                            qs = {}
                            started = set()
                            for i, j, k, c in p.nnz:
                                key = (self.lit(abs(c)), j)
                                if key not in qs:
                                    qs[key] = len(qs)
                                    s(f"const T q{qs[key]} = T({key[0]}) * y{j};")
                                    s(f"const T qb{qs[key]} = T({key[0]}) * b{j};")
                                n_ = qs[key]
                                neg = c < 0
                                if k not in started:
                                    s(f"T t{k} = {'-' if neg else ''}q{n_} * p{i};")
                                    started.add(k)
                                else:
                                    s(f"t{k} {'-=' if neg else '+='} q{n_} * p{i};")
                                s(f"t{k} {'-=' if neg else '+='} qb{n_} * r{i};")
                            for k in sorted(started):
                                s(f"a.o{p.io}[{k}] += t{k};")

                    def body_plain(v, p):
                        prods = self._two_products(s, p, v)
                        started = set()
                        for n, (i, j, k, c) in enumerate(p.nnz):
                            qy, qb, neg = prods[n]
                            xi, ai = f"x.b{p.i1}[{i}]", f"xa.b{p.i1}[{i}]"
                            sign = "-" if neg else ""
                            if k not in started:
                                s(f"T t{k} = {sign}{qy} * {ai}; T s{k} = {sign}{qy} * {xi};")
                                started.add(k)
                            else:
                                op = "-=" if neg else "+="
                                s(f"t{k} {op} {qy} * {ai}; s{k} {op} {qy} * {xi};")
                            s(f"t{k} {'-=' if neg else '+='} {qb} * {xi};")
                        s(f"const T wv = {wacc(p, v)};")
                        s(f"const T cv = {cacc(p, v)};")
                        for k in sorted(started):
                            s(f"a.o{p.io}[{k}] += wv * t{k} + cv * s{k};")

                    self._for_v(s, p, body)
                s.close()

        self._per_chunk(s, emit, in_kernel=False)

    # ------------------------------------------------------------ kernel B paths
    def _ddb_paths(self, s: Src, g_on_demand_row: Optional[str], fence: bool, deferred: bool,
                   dw_guard: Optional[str], paths: Optional[List[Path]] = None, fwd_acc: bool = False):
        """Straight-line second-order backward of all paths. In scope: x, xa (X_t), dx (X_t), dy[],
        yrow, brow, wrow, crow, dwrow, u, and gr (G_t) or the row pointer named ``g_on_demand_row``.
        ``fwd_acc``: the three forward terms of kernel A are added to ``a`` (G_t) as well, from the same
        operand registers."""
        low = self.low
        wacc, cacc = self._w_of("wrow"), self._w_of("crow")
        ordered = sorted(self._paths(paths), key=lambda q: (q.io, q.index))
        since_fence = 0
        preload_w = (self.forms and not fwd_acc and sum(low.in2[q.i2].mul for q in ordered) <= 48
                     and all(low.in2[q.i2].mul <= UNROLL_V_LIMIT for q in ordered))
        if preload_w:
            # every path's W and C value is wanted at the top of its code (the weights are folded into the Y
            # operands first): requested here, all together, or each path would wait for its own pair
            for q in ordered:
                for v in range(low.in2[q.i2].mul):
                    s(f"const T wv{q.index}_{v} = {wacc(q, str(v))};")
                    s(f"const T cv{q.index}_{v} = {cacc(q, str(v))};")
        for n_path, p in enumerate(ordered):
            b1, b2, bo = low.in1[p.i1], low.in2[p.i2], low.out[p.io]
            V = b2.mul
            s(f"// path {p.index}")
            s.open("")
            if g_on_demand_row is not None:
                s(f"T gk[{bo.d}];")
                s.open("")
                base, st = self._lane_ptr(bo)
                s(f"const T* gp = {self._gptr(g_on_demand_row, base, bo.mul)};")
                for k in range(bo.d):
                    s(f"gk[{k}] = gp[{k * st}];")
                s.close()
                gname = lambda k: f"gk[{k}]"
            else:
                gname = lambda k, io=p.io: f"gr.o{io}[{k}]"
            base_slot = self.wslot[p.index]

            def body(v, p=p, b1=b1, b2=b2, V=V, gname=gname, base_slot=base_slot):
                ks = sorted({k for _, _, k, _ in p.nnz})
                js = sorted({j for _, j, _, _ in p.nnz})
                fold = self.forms and not fwd_acc
                if fold:
                    # d/dX_i = sum c g_k (w b_j + c_w y_j): the weights are folded into one vector over j first, so
                    # a term costs one multiply-add (two before, plus the weighting of g_k twice)
                    yacc, bacc = self._y_of("yrow"), self._y_of("brow")
                    for j in js:
                        s(f"const T y{j} = {yacc(p, v, j)};")
                        s(f"const T b{j} = {bacc(p, v, j)};")
                    s(f"const T wv = {f'wv{p.index}_{v}' if preload_w else wacc(p, v)};")
                    s(f"const T cv = {f'cv{p.index}_{v}' if preload_w else cacc(p, v)};")
                    for j in js:
                        s(f"const T m{j} = wv * b{j} + cv * y{j};")
                    prods = self._scaled(s, p, 1, lambda j: f"m{j}", "qm")
                else:
                    prods = self._two_products(s, p, v)
                    s(f"const T wv = {wacc(p, v)};")
                    s(f"const T cv = {cacc(p, v)};")
                # One output component k at a time, so that what is derived from g_k (its products with the
                # weights and with the X / A components) is dead before the next k: in any other order
                # these temporaries, two sets of them here, cost more registers than the operands.
                #   d/dX_i += (|c| b_j)(g_k w) + (|c| y_j)(g_k c)
                #   h_j = sum_ik c x_i g_k,  ha_j = sum_ik c a_i g_k
                for j in js:
                    s(f"T h{j} = T(0), ha{j} = T(0);")
                for k in ks:
                    s.open("")
                    of_k = [(n, t) for n, t in enumerate(p.nnz) if t[2] == k]
                    if fold:
                        for n, (i, j, _, c) in of_k:
                            qm, neg = prods[n]
                            s(f"dx.b{p.i1}[{i}] {'-=' if neg else '+='} {qm} * {gname(k)};")
                    else:
                        s(f"const T gw = {gname(k)} * wv; const T gc = {gname(k)} * cv;")
                        for n, (i, j, _, c) in of_k:
                            qy, qb, neg = prods[n]
                            op = "-=" if neg else "+="
                            s(f"dx.b{p.i1}[{i}] {op} {qb} * gw; dx.b{p.i1}[{i}] {op} {qy} * gc;")
                    for i in sorted({t[0] for _, t in of_k}):
                        s(f"{{ const T xg = x.b{p.i1}[{i}] * {gname(k)}; const T ag = xa.b{p.i1}[{i}] * {gname(k)};")
                        for n, (i2, j, _, c) in of_k:
                            if i2 == i:
                                s(f"  h{j} += T({self.lit(c)}) * xg; ha{j} += T({self.lit(c)}) * ag;")
                        s("}")
                    s.close()
                # d/dW = sum_j b_j h_j + y_j ha_j ; d/dY_j = c h_j + w ha_j
                s(f"T dwv = b{js[0]} * h{js[0]};")
                s(f"dwv += y{js[0]} * ha{js[0]};")
                for j in js[1:]:
                    s(f"dwv += b{j} * h{j}; dwv += y{j} * ha{j};")
                if low.shared_weights:
                    # summed over the wave's rows in registers; rows past the end of the batch are duplicates
                    s(f"dwacc[{base_slot} + {v}] += {dwv_live('dwv', dw_guard)};")
                elif deferred:
                    s(f"dwkeep[{base_slot} + {v}] = dwv;")
                else:
                    dwp = self._dump_unless(self._store_cond(b1.mul, dw_guard),
                                            self._ptr("dwrow", (f"{p.woff} + ({v})", V)))
                    s(f"__builtin_nontemporal_store(dwv, {dwp});" if self.nt & 2 else f"*{dwp} = dwv;")
                for j in js:
                    s(f"dy[{self._y_index(b2, v, j)}] += cv * h{j}; dy[{self._y_index(b2, v, j)}] += wv * ha{j};")
                if fwd_acc:
                    for k in ks:
                        s.open("")
                        s("T ft = T(0), fs = T(0);")
                        for n, (i, j, k2, c) in enumerate(p.nnz):
                            if k2 != k:
                                continue
                            qy, qb, neg = prods[n]
                            op = "-=" if neg else "+="
                            xi, ai = f"x.b{p.i1}[{i}]", f"xa.b{p.i1}[{i}]"
                            s(f"ft {op} {qy} * {ai}; ft {op} {qb} * {xi}; fs {op} {qy} * {xi};")
                        s(f"a.o{p.io}[{k}] += wv * ft + cv * fs;")
                        s.close()

            self._for_v(s, p, body)
            s.close()
            if fence and g_on_demand_row is not None:
                since_fence += bo.d * self.words
                nxt = ordered[n_path + 1] if n_path + 1 < len(ordered) else None
                if nxt is None or since_fence + low.out[nxt.io].d * self.words > self.fence_words:
                    s("__builtin_amdgcn_sched_barrier(0);")
                    since_fence = 0
            elif self.fence_paths and (n_path + 1) % self.fence_paths == 0 and n_path + 1 < len(ordered):
                # resident gradients: the scheduler would still request every path's W and C values up
                # front, two registers per path on top of X, A, dX, dY and the gradient slice
                s("__builtin_amdgcn_sched_barrier(0);")

    fence_paths = 0   # resident gradients: a scheduling fence after every so many paths (0: none)
    force_resident: Optional[bool] = None

    def double_b_resident(self) -> bool:
        """The row's / node's output-gradient slice stays in registers beside X, A, dX and dY."""
        low = self.low
        if self.force_resident is not None:
            return self.force_resident
        x = sum(low.in1[b].d for b in self.used_in1)
        g = sum(low.out[io].d for io in self.used_out)
        # X, A, dX, dY, the gradient slice, and the W and C values of every path (requested up front)
        return self.words * (g + 3 * x + self.l2_pad + 2 * self.n_wslots) + 40 <= 232

    # ------------------------------------------------------------ batch kernels
    def emit_tp_double_a(self, s: Src, G: int, waves_per_eu: int = 0):
        low = self.low
        block = 64 * self.NCH * G
        s.open(
            f'extern "C" __global__ {self._attrs(block, waves_per_eu)} void double_backward_A(i64 num_batch, '
            "const T* __restrict__ L1_in, const T* __restrict__ L1_dgrad, const T* __restrict__ L2_in, "
            "const T* __restrict__ L2_dgrad, const T* __restrict__ W, const T* __restrict__ W_dgrad, "
            "T* __restrict__ L3_dgrad)"
        )
        self._lane_prologue(s)
        if self.tr_stores & 1 and self.R == 1:
            s(f"__shared__ T s_tr[{self.NCH * G}][{64 * max(b.d for b in low.out)}];")
        s(f"const i64 ngroups = (num_batch + {self.R - 1}) / {self.R};")
        s.open(f"for (i64 grp = (i64)blockIdx.x * {G} + g; grp < ngroups; grp += (i64)gridDim.x * {G})")
        s(f"const i64 row = grp * {self.R} + r;")
        s("const bool live = row < num_batch;")
        s("const i64 rowc = live ? row : num_batch - 1;")
        s(f"const T* xrow = L1_in + rowc * {low.L1};")
        s(f"const T* arow = L1_dgrad + rowc * {low.L1};")
        s(f"const T* yrow = L2_in + rowc * {low.L2};")
        s(f"const T* brow = L2_dgrad + rowc * {low.L2};")
        s(f"const T* wrow = W{'' if low.shared_weights else f' + rowc * {low.WN}'};")
        s(f"const T* crow = W_dgrad{'' if low.shared_weights else f' + rowc * {low.WN}'};")
        s(f"T* zrow = L3_dgrad + rowc * {low.L3};")
        live = "live"
        if self.R == 1:
            s.open("if (live)")
            live = "true"

        def row_body():
            s("X_t x, xa;")
            self._load_x(s, "xrow", self.used_in1)
            self._load_x(s, "arow", self.used_in1, "xa")
            for si in range(len(self.segments)):
                if self.cur_chunk is not None and not self._out_of(self.segments[si]):
                    continue
                s.open("")
                s(f"D{si}_t a; zero_dseg{si}(a);")
                s(f"dda_seg{si}{self._sfx()}(x, xa, yrow, brow, wrow, crow, u, a);")
                self._store_seg(s, si, "zrow", live)
                s.close()

        self._per_chunk(s, row_body)
        self._zero_untouched_out(s, "zrow", live)
        if self.R == 1:
            s.close()
        s.close()
        s.close()
        return block

    def emit_tp_double_b(self, s: Src, G: int, waves_per_eu: int = 0):
        low = self.low
        if self.NCH > 1:
            G = 1  # the dY reduction across chunk waves uses block barriers
        block = 64 * self.NCH * G
        s.open(
            f'extern "C" __global__ {self._attrs(block, waves_per_eu)} void double_backward_B(i64 num_batch, '
            "const T* __restrict__ L1_in, const T* __restrict__ L1_dgrad, const T* __restrict__ L2_in, "
            "const T* __restrict__ L2_dgrad, const T* __restrict__ W, const T* __restrict__ W_dgrad, "
            "const T* __restrict__ L3_grad, T* __restrict__ L1_grad, T* __restrict__ L2_grad, T* __restrict__ W_grad, "
            "T* __restrict__ wpartial)"
        )
        self._lane_prologue(s)
        shared = low.shared_weights
        if self.NCH > 1:
            s(f"__shared__ T s_dy[{G}][{self.NCH}][{self.l2_pad}];")
        if self.tr_stores & 2 and self.R == 1:
            s(f"__shared__ T s_tr[{self.NCH * G}][{64 * max(b.d for b in low.in1)}];")
        if shared:
            s(f"T dwacc[{self.n_wslots}];")
            s(f"for (int t = 0; t < {self.n_wslots}; ++t) dwacc[t] = T(0);")
        s(f"const i64 ngroups = (num_batch + {self.R - 1}) / {self.R};")
        s.open(f"for (i64 base = (i64)blockIdx.x * {G}; base < ngroups; base += (i64)gridDim.x * {G})")
        s("const i64 grp = base + g;")
        s(f"const i64 row = grp * {self.R} + r;")
        s("const bool live = row < num_batch;")
        s("const i64 rowc = live ? row : num_batch - 1;")
        s(f"const T* xrow = L1_in + rowc * {low.L1};")
        s(f"const T* arow = L1_dgrad + rowc * {low.L1};")
        s(f"const T* yrow = L2_in + rowc * {low.L2};")
        s(f"const T* brow = L2_dgrad + rowc * {low.L2};")
        s(f"const T* wrow = W{'' if shared else f' + rowc * {low.WN}'};")
        s(f"const T* crow = W_dgrad{'' if shared else f' + rowc * {low.WN}'};")
        s(f"const T* grow = L3_grad + rowc * {low.L3};")
        if not shared:
            s(f"T* dwrow = W_grad + rowc * {low.WN};")
        live = "live"
        if self.R == 1:
            s.open("if (live)")
            live = "true"
        resident = self.double_b_resident()

        def row_body():
            s("X_t x, xa, dx;")
            self._load_x(s, "xrow", self.used_in1)
            self._load_x(s, "arow", self.used_in1, "xa")
            self._zero_x(s, "dx")
            s(f"T dy[{self.l2_pad}];")
            s(f"for (int t = 0; t < {self.l2_pad}; ++t) dy[t] = T(0);")
            deferred = not shared and self._dw_deferred(live)
            if deferred:
                s(f"T dwkeep[{self.n_wslots}];")
            if resident:
                s("G_t gr;")
                self._load_g(s, "grow", self.used_out)
                self._ddb_paths(s, None, False, deferred, live)
            else:
                self._ddb_paths(s, "grow", True, deferred, live)
            self._pin_gradients(s, self.used_in1, deferred)
            if deferred:
                self._flush_dwkeep(s, live)
            s(f"T* dxrow = L1_grad + rowc * {low.L1};")
            self._store_dx(s, "dxrow", live, nt=bool(self.nt & 2))
            self._zero_untouched_in1(s, "dxrow", live)
            self._dy_finish(s, f"L2_grad + rowc * {low.L2}", live)

        self._per_chunk(s, row_body)
        if self.R == 1:
            s.close()
        s.close()
        if shared:
            # as in the first-order backward: fold the row groups of the wave, then every wave group writes one
            # partial row, which a second kernel sums in block order
            if self.R > 1:
                s.open(f"for (int t = 0; t < {self.n_wslots}; ++t)")
                m = self.LPR
                while m < 64:
                    s(f"dwacc[t] += __shfl_xor(dwacc[t], {m});")
                    m *= 2
                s.close()
            s(f"T* prow = wpartial + ((i64)blockIdx.x * {G} + g) * {low.WN};")
            for p, slot in self._dw_slots():
                b1, V = low.in1[p.i1], low.in2[p.i2].mul
                s.open(f"if (r == 0 && u < {b1.mul})")
                s(f"for (int v = 0; v < {V}; ++v) prow[{p.woff} + u * {V} + v] = dwacc[{slot} + v];")
                s.close()
        s.close()
        return block

    # ------------------------------------------------------------ convolution kernels
    _CONV_OPERANDS = (
        "const T* __restrict__ L1_in, const T* __restrict__ L1_dgrad, const T* __restrict__ L2_in, "
        "const T* __restrict__ L2_dgrad, const T* __restrict__ W, const T* __restrict__ W_dgrad, "
    )

    def _edge_rows(self, s: Src, e: str):
        low = self.low
        s(f"const i64 eid = OEQ_EDGE({e});")
        s("const i64 sender = oeq_idx(cols[eid], node_count);")
        s(f"const T* xrow = L1_in + sender * {low.L1};")
        s(f"const T* arow = L1_dgrad + sender * {low.L1};")
        s(f"const T* yrow = L2_in + eid * {low.L2};")
        s(f"const T* brow = L2_dgrad + eid * {low.L2};")
        s(f"const T* wrow = W{'' if low.shared_weights else f' + eid * {low.WN}'};")
        s(f"const T* crow = W_dgrad{'' if low.shared_weights else f' + eid * {low.WN}'};")

    def emit_conv_double_a(self, s: Src, G: int, waves_per_eu: int = 0, xcd: int = 1, segw: int = 1):
        """Receiver-major walk: the node's accumulators stay in registers over its edges. With ``segw``
        > 1 the output segments of a node are shared between that many waves, which walk its edges side
        by side (fewer registers per wave, more waves in flight)."""
        low = self.low
        segw = max(1, min(segw, len(self.segments))) if self.R == 1 else 1
        block = 64 * self.NCH * G * segw
        s.open(
            f'extern "C" __global__ {self._attrs(block, waves_per_eu)} void double_backward_A(i64 node_count, '
            f"i64 nnz, {self._CONV_OPERANDS}T* __restrict__ L3_dgrad, const i64* __restrict__ rows, "
            "const i64* __restrict__ cols, const i64* __restrict__ rowptr, const i64* __restrict__ eperm, "
            f"const i64* __restrict__ order{self.HUB_PARAMS}{self.HUB_ROWS_PARAM})"
        )
        self._lane_prologue(s, segw)
        if self.tr_stores & 1 and self.R == 1:
            s(f"__shared__ T s_tr[{self.NCH * G * segw}][{64 * max(low.out[io].d for io in self.used_out)}];")
        self._node_loop_open(s, G, xcd)
        s(f"T* zrow = hubpos >= 0 ? hub_rows + hubpos * {low.L3} : L3_dgrad + node * {low.L3};")
        for si in range(len(self.segments)):
            s.open(f"if (sg == {si % segw})" if segw > 1 else "")

            def node_body(si=si):
                if self.cur_chunk is not None and not self._out_of(self.segments[si]):
                    return
                s(f"D{si}_t a; zero_dseg{si}(a);")
                if self.kahan:
                    s(f"D{si}_t c; zero_dseg{si}(c);")
                s.open(f"for (i64 e = e0 + r; e < e1; e += {self.R})")
                self._edge_rows(s, "e")
                s("X_t x, xa;")
                self._load_x(s, "xrow", self.seg_in1[si])
                self._load_x(s, "arow", self.seg_in1[si], "xa")
                s(f"dda_seg{si}{self._sfx()}(x, xa, yrow, brow, wrow, crow, u, {'c' if self.kahan else 'a'});")
                if self.kahan:
                    s(f"kahan_dseg{si}(c, a);")
                s.close()
                if self.R > 1:
                    for io in self.segments[si]:
                        for k in range(low.out[io].d):
                            m = self.LPR
                            while m < 64:
                                s(f"a.o{io}[{k}] += __shfl_xor(a.o{io}[{k}], {m});")
                                m *= 2
                self._store_seg(s, si, "zrow", "r == 0" if self.R > 1 else "true")

            self._per_chunk(s, node_body)
            s.close()
        self._zero_untouched_out(s, "zrow", "r == 0 && sg == 0" if segw > 1 else "r == 0")
        s.close()
        s.close()
        return block

    def emit_conv_double_b(self, s: Src, G: int, waves_per_eu: int = 0, xcd: int = 1):
        """Receiver-major walk with the node's output-gradient slice in registers (when it fits); the
        per-edge d/dX terms go to ``dx_tmp`` for the sender-ordered reduction, as in the first-order
        backward kernel."""
        low = self.low
        if self.NCH > 1:
            G = 1
        block = 64 * self.NCH * G
        s.open(
            f'extern "C" __global__ {self._attrs(block, waves_per_eu)} void double_backward_B(i64 node_count, '
            f"i64 nnz, {self._CONV_OPERANDS}const T* __restrict__ L3_grad, T* __restrict__ L2_grad, "
            "T* __restrict__ W_grad, const i64* __restrict__ rows, const i64* __restrict__ cols, "
            "const i64* __restrict__ rowptr, T* __restrict__ dx_tmp, const i64* __restrict__ eperm, "
            f"T* __restrict__ L3_dgrad, const i64* __restrict__ order, T* __restrict__ wpartial{self.HUB_PARAMS})"
        )
        self._lane_prologue(s)
        shared = low.shared_weights
        assert not (shared and self.merged)
        if self.NCH > 1:
            s(f"__shared__ T s_dy[{G}][{self.NCH}][{self.l2_pad}];")
        if (self.tr_stores & 2 or (self.merged and self.tr_stores & 1)) and self.R == 1:
            dmax = max([low.in1[b].d for b in self.used_in1] + [low.out[io].d for io in self.used_out])
            s(f"__shared__ T s_tr[{self.NCH * G}][{64 * dmax}];")
        if shared:
            # summed over all edges of all nodes of the wave group; one partial row per group at the end
            s(f"T dwacc[{self.n_wslots}];")
            s(f"for (int t = 0; t < {self.n_wslots}; ++t) dwacc[t] = T(0);")
        resident = self.double_b_resident() or self.merged
        self._node_loop_open(s, G, xcd)

        def node_body():
            if resident:
                s("G_t gr;")
                self._load_g(s, f"L3_grad + node * {low.L3}", self.used_out)
            if self.merged:
                s("G_t a;")
                for io in self._out_of(self.used_out):
                    for k in range(low.out[io].d):
                        s(f"a.o{io}[{k}] = T(0);")
            # with more than one chunk every wave of the block walks the same edges: the block barriers
            # of the dY reduction are reached uniformly
            s.open(f"for (i64 e = e0 + r; e < e1; e += {self.R})")
            self._edge_rows(s, "e")
            if not shared:
                s(f"T* dwrow = W_grad + eid * {low.WN};")
            s("X_t x, xa, dx;")
            self._load_x(s, "xrow", self.used_in1)
            self._load_x(s, "arow", self.used_in1, "xa")
            self._zero_x(s, "dx")
            s(f"T dy[{self.l2_pad}];")
            s(f"for (int t = 0; t < {self.l2_pad}; ++t) dy[t] = T(0);")
            deferred = not shared and self._dw_deferred(None)
            if deferred:
                s(f"T dwkeep[{self.n_wslots}];")
            if resident:
                self._ddb_paths(s, None, False, deferred, None, fwd_acc=self.merged)
            else:
                s(f"const T* grow = L3_grad + node * {low.L3};")
                # without this the compiler hoists the loads of the node's gradient row out of the edge
                # loop, i.e. makes it register resident after all
                s(f'asm volatile("" : "+{"s" if self.R == 1 else "v"}"(grow));')
                self._ddb_paths(s, "grow", True, deferred, None)
            self._pin_gradients(s, self.used_in1, deferred)
            if deferred:
                self._flush_dwkeep(s, None)
            s(f"T* dxrow = dx_tmp + eid * {low.L1};")
            self._store_dx(s, "dxrow", "true", nt=bool(self.nt & 2))
            self._zero_untouched_in1(s, "dxrow", "true")
            self._dy_finish(s, f"L2_grad + eid * {low.L2}", "true")
            s.close()
            if self.merged:
                if self.R > 1:  # fold the lane groups of packed rows (fixed order) into group 0
                    for io in self._out_of(self.used_out):
                        for k in range(low.out[io].d):
                            m = self.LPR
                            while m < 64:
                                s(f"a.o{io}[{k}] += __shfl_xor(a.o{io}[{k}], {m});")
                                m *= 2
                segments, self.segments = self.segments, [self.used_out]
                try:
                    self._store_seg(s, 0, f"(L3_dgrad + node * {low.L3})", "r == 0" if self.R > 1 else "true")
                finally:
                    self.segments = segments

        self._per_chunk(s, node_body)
        if self.merged:
            self._zero_untouched_out(s, f"(L3_dgrad + node * {low.L3})", "r == 0")
        s.close()
        if shared:
            if self.R > 1:
                s.open(f"for (int t = 0; t < {self.n_wslots}; ++t)")
                m = self.LPR
                while m < 64:
                    s(f"dwacc[t] += __shfl_xor(dwacc[t], {m});")
                    m *= 2
                s.close()
            s(f"T* prow = wpartial + ((i64)blockIdx.x * {G} + g) * {low.WN};")
            for p, slot in self._dw_slots():
                b1, V = low.in1[p.i1], low.in2[p.i2].mul
                s.open(f"if (r == 0 && u < {b1.mul})")
                s(f"for (int v = 0; v < {V}; ++v) prow[{p.woff} + u * {V} + v] = dwacc[{slot} + v];")
                s.close()
        s.close()
        return block


    # ---- kernel B with a node's output blocks shared between several waves ------------------------
    merged = False     # kernel B also accumulates and writes kernel A's result (no separate kernel A)
    need_limit = 200   # register estimate above which a node's output blocks are shared between waves

    def merged_fits_one_wave(self) -> bool:
        low = self.low
        x = sum(low.in1[b].d for b in self.used_in1)
        g = sum(low.out[io].d for io in self.used_out)
        return self.words * (2 * g + 3 * x + self.l2_pad + 2 * self.n_wslots) + 40 <= 232

    def plan_double_groups(self, max_waves: int) -> Optional[List[List[int]]]:
        """Output blocks per wave when one wave cannot keep X, A, dX, dY, the node's gradient slice and
        the in-flight W / C values of all paths in registers: None when one wave can (or when the
        kernel shape does not allow the split)."""
        low = self.low
        if self.R != 1 or not self.can_preload:
            return None
        x = sum(low.in1[b].d for b in self.used_in1)
        fixed = self.words * (3 * x + self.l2_pad) + 40
        sizes = [low.out[io].d for io in self.used_out]
        per_path = {io: sum(2 * low.in2[p.i2].mul for p in low.paths if p.io == io) for io in self.used_out}

        def need(grp):
            return fixed + self.words * sum(low.out[io].d * (2 if self.merged else 1) + per_path[io] for io in grp)

        forced = getattr(self, "group_count", 0)
        if need(self.used_out) <= self.need_limit and not forced:
            return None
        # the waves exchange their dX terms through LDS: [waves][chunks][X components][64 lanes]
        lds_per_wave = self.NCH * x * 64 * low.elem_size
        max_waves = min(max_waves, 60000 // lds_per_wave, len(sizes))

        def balanced(n: int) -> List[List[int]]:
            target = -(-sum(sizes) // n)
            groups, cur, tot = [], [], 0
            for io, d in zip(self.used_out, sizes):
                if cur and tot + d > target and len(groups) < n - 1:
                    groups.append(cur)
                    cur, tot = [], 0
                cur.append(io)
                tot += d
            groups.append(cur)
            return groups

        if forced:
            return None if forced == 1 or max_waves < 2 else balanced(min(forced, max_waves))
        # Two waves while half of what varies with the share (gradient slice, W and C values) fits beside what
        # every wave holds, else four: with the count forced to 1 .. 4 on 15 problems (config-5 graph) two waves
        # were best up to an estimate of 231 words for such a share (SevenNet main layer: -16 % against the three
        # that a fixed limit per wave gave) and four from 343 on (NequIP benzene -14 % against seven); three never
        # won.
        if self.need_limit == 200 and max_waves >= 2:
            share2 = fixed + -(-(need(self.used_out) - fixed) // 2)
            if share2 <= 250 or max_waves < 4:
                return balanced(2)
            return balanced(4)
        n = 2
        while n <= max_waves:
            groups = balanced(n)
            if all(need(grp) <= self.need_limit for grp in groups) or n == max_waves:
                return groups
            n += 1
        return None

    def emit_conv_double_b_split(self, s: Src, groups: List[List[int]], waves_per_eu: int = 0, xcd: int = 1) -> int:
        """All waves of a block walk the edges of one node; wave ``sg`` keeps the gradient of its output
        blocks resident and handles the paths into them (their d/dW is final); an edge's partial d/dX and
        d/dY are summed over the waves through LDS in a fixed order."""
        low = self.low
        SW = len(groups)
        block = 64 * self.NCH * SW
        xoff, XW = {}, 0
        for b in self.used_in1:
            xoff[b] = XW
            XW += low.in1[b].d
        gpaths = [[p for p in low.paths if p.io in grp] for grp in groups]
        gin1 = [sorted({p.i1 for p in ps}) for ps in gpaths]
        s.open(
            f'extern "C" __global__ {self._attrs(block, waves_per_eu)} void double_backward_B(i64 node_count, '
            f"i64 nnz, {self._CONV_OPERANDS}const T* __restrict__ L3_grad, T* __restrict__ L2_grad, "
            "T* __restrict__ W_grad, const i64* __restrict__ rows, const i64* __restrict__ cols, "
            "const i64* __restrict__ rowptr, T* __restrict__ dx_tmp, const i64* __restrict__ eperm, "
            f"T* __restrict__ L3_dgrad, const i64* __restrict__ order, T* __restrict__ wpartial{self.HUB_PARAMS})"
        )
        self._lane_prologue(s, SW)
        s(f"__shared__ T s_dy[{SW * self.NCH}][{self.l2_pad}];")
        s(f"__shared__ T s_dx[{SW}][{self.NCH}][{XW}][64];")
        if self.merged and self.tr_stores & 1:
            s(f"__shared__ T s_tr[{self.NCH * SW}][{64 * max(low.out[io].d for io in self.used_out)}];")
        self._node_loop_open(s, 1, xcd)
        for si in range(SW):
            s.open(f"if (sg == {si})")

            def sg_body(si=si):
                s("G_t gr;")
                self._load_g(s, f"L3_grad + node * {low.L3}", groups[si])
                if self.merged:
                    s("G_t a;")
                    for io in self._out_of(groups[si]):
                        for k in range(low.out[io].d):
                            s(f"a.o{io}[{k}] = T(0);")
                # every wave of the block runs the same number of edges, so the block barriers match up
                s.open("for (i64 e = e0; e < e1; ++e)")
                self._edge_rows(s, "e")
                s(f"T* dwrow = W_grad + eid * {low.WN};")
                s("X_t x, xa, dx;")
                self._load_x(s, "xrow", gin1[si])
                self._load_x(s, "arow", gin1[si], "xa")
                self._zero_x(s, "dx")
                s(f"T dy[{self.l2_pad}];")
                s(f"for (int t = 0; t < {self.l2_pad}; ++t) dy[t] = T(0);")
                deferred = self._dw_deferred(None)
                if deferred:
                    s(f"T dwkeep[{self.n_wslots}];")
                self._ddb_paths(s, None, False, deferred, None, gpaths[si], fwd_acc=self.merged)
                self._pin_gradients(s, gin1[si], deferred, gpaths[si])
                if deferred:
                    low_paths, low.paths = low.paths, gpaths[si]
                    try:
                        self._flush_dwkeep(s, None)
                    finally:
                        low.paths = low_paths
                for b in self._in1_of(gin1[si]):
                    for i in range(low.in1[b].d):
                        s(f"s_dx[{si}][chunk][{xoff[b] + i}][ul] = dx.b{b}[{i}];")
                s.open("")
                cur, dup = self._dy_reduce(s)
                s.open(f"if ((ul & {dup}) == 0)")
                for j in range(cur):
                    s(f"s_dy[{si} * {self.NCH} + chunk][dyidx + {j}] = rv[{j}];")
                s.close()
                s.close()
                s("__syncthreads();")
                # the used input blocks are shared out between the waves for the final sum and store
                s(f"T* dxrow = dx_tmp + eid * {low.L1};")
                for n, b in enumerate(self.used_in1):
                    if n % SW != si or not self._has(low.in1[b].mul):
                        continue
                    blk = low.in1[b]
                    contributors = [c for c in range(SW) if b in gin1[c]]
                    self._open_if(s, self._store_cond(blk.mul))
                    base, st = self._lane_ptr(blk)
                    s(f"T* dp = {self._ptr('dxrow', base)};")
                    for i in range(blk.d):
                        terms = " + ".join(f"s_dx[{c}][chunk][{xoff[b] + i}][ul]" for c in contributors)
                        val = f"({terms})" if contributors else "T(0)"
                        if self.nt & 2:
                            s(f"__builtin_nontemporal_store({val}, dp + {i * st});")
                        else:
                            s(f"dp[{i * st}] = {val};")
                    s.close()
                if si == 0:
                    self._zero_untouched_in1(s, "dxrow", "true")
                    s.open("if (chunk == 0)")
                    s.open(f"for (int j = lane; j < {low.L2}; j += 64)")
                    s("T tot = s_dy[0][j];")
                    s(f"for (int cc = 1; cc < {SW * self.NCH}; ++cc) tot += s_dy[cc][j];")
                    s(f"L2_grad[eid * {low.L2} + j] = tot;")
                    s.close()
                    s.close()
                s("__syncthreads();")
                s.close()
                if self.merged:
                    segments, self.segments = self.segments, groups
                    try:
                        self._store_seg(s, si, f"(L3_dgrad + node * {low.L3})", "true")
                    finally:
                        self.segments = segments

            self._per_chunk(s, sg_body)
            s.close()
        if self.merged:
            self._zero_untouched_out(s, f"(L3_dgrad + node * {low.L3})", "sg == 0")
        s.close()
        s.close()
        return block


def add_tp_kernels(s: Src, low: Lowered, base: UvuEmitter, tune: dict, groups_b: int = 4,
                   compute_units: int = 256) -> List[tuple]:
    """Append the batch double-backward kernels to a module; returns their launch descriptors. ``groups_b``:
    wave groups per block of the first-order backward kernel."""
    from .. import runtime as rt

    em = DoubleEmitter(low, acc_budget_words=64)
    em.nt = base.nt
    em.mask_loads = base.mask_loads
    em.forms = base.forms
    em.tr_stores = base.tr_stores
    em.fence_words = 48
    # the accumulator structs of this emitter's (smaller) segments
    _emit_segment_structs(s, em, "D")
    em.emit_double_cores(s)
    wide = low.n_chunks > 1
    G = 1 if wide else 4
    # shared weights: kernel B writes one partial weight-gradient row per wave group, as the first-order
    # backward does, and the runtime sizes both from the same figure (groups per block); bounded grid
    G_b = 1 if em.NCH > 1 else (groups_b if low.shared_weights else G)
    blk_a = em.emit_tp_double_a(s, G, tune.get("dd_wa", 2))
    blk_b = em.emit_tp_double_b(s, G_b, tune.get("dd_wb", 2))
    return [(rt.ROLE_DOUBLE_BACKWARD_A, "double_backward_A", blk_a, G * em.R, 0),
            (rt.ROLE_DOUBLE_BACKWARD_B, "double_backward_B", blk_b, G_b * em.R,
             compute_units * 8 if low.shared_weights else 0)]


def add_conv_kernels(s: Src, low: Lowered, base: UvuEmitter, tune: dict, xcd: int, groups_b: int = 0,
                     compute_units: int = 256, kahan: bool = False) -> List[tuple]:
    """Append the convolution double-backward kernels (receiver-major walk) to a module. Shared weights: kernel B
    runs with the first-order backward kernel's wave groups per block (``groups_b``) on a bounded grid, one
    partial weight-gradient row per group, and is never split between waves or merged with kernel A."""
    from .. import runtime as rt

    def kernel_a_need(e: DoubleEmitter) -> int:
        """Registers kernel A needs for its widest output segment: the accumulators, X and A of the input
        blocks the segment's paths read, one W and one C value per path."""
        worst = 0
        for si, seg in enumerate(e.segments):
            acc = (2 if kahan else 1) * sum(low.out[io].d for io in seg)  # (and their compensation terms)
            xin = sum(low.in1[b].d for b in e.seg_in1[si])
            wc = sum(2 * low.in2[p.i2].mul for p in low.paths if p.io in seg)
            worst = max(worst, e.words * (acc + 2 * xin + wc))
        return worst

    # Output segment size of kernel A: 112 accumulator words where the widest segment then fits (the MACE
    # shape: one segment, 177 words); problems with many paths per output block (SevenNet, NequIP benzene)
    # spill there, up to 149 registers, and take the largest budget that leaves the widest segment under
    # 160 words - with the spills the fused pair was slower than composing first-order kernels.
    if tune.get("dd_acc", 0) > 0:
        em = DoubleEmitter(low, acc_budget_words=tune["dd_acc"], kahan=kahan)
    else:
        em = DoubleEmitter(low, acc_budget_words=56 if kahan else 112, kahan=kahan)
        if kernel_a_need(em) > 200:
            for budget in (80, 64, 48, 32, 24, 16):
                if kahan and budget > 48:
                    continue
                em = DoubleEmitter(low, acc_budget_words=budget, kahan=kahan)
                if kernel_a_need(em) <= 160:
                    break
    em.nt = base.nt
    em.mask_loads = base.mask_loads
    em.forms = base.forms
    em.tr_stores = base.tr_stores
    em.fence_words = tune.get("dd_fw", 32)
    em.fence_paths = tune.get("dd_fp", 0)
    if tune.get("dd_gres", -1) >= 0:
        em.force_resident = bool(tune["dd_gres"])
    _emit_segment_structs(s, em, "D")
    em.emit_double_cores(s)
    G = max(1, tune.get("dd_g", 2) // em.NCH) if em.R == 1 else 4
    em.need_limit = tune.get("dd_need", 200)
    em.group_count = tune.get("dd_ngrp", 0)
    # dd_merge=1: one kernel for both results (W, C and the gathered X, A rows are then read once instead of
    # twice). Measured slower on MI355X for every shape tried (MACE shape 37 - 85 ms against 33 ms for the
    # pair): its accumulators on top of kernel B's state spill whatever the split, so it is off by default.
    shared = low.shared_weights
    em.merged = bool(tune.get("dd_merge", 0)) and not shared and not kahan
    groups = em.plan_double_groups(max(1, 8 // em.NCH)) if tune.get("dd_split", 1) and not shared else None
    if em.merged and not groups and not em.merged_fits_one_wave():
        em.merged = False
        groups = em.plan_double_groups(max(1, 8 // em.NCH)) if tune.get("dd_split", 1) else None
    descs = []
    if not em.merged:
        segw = min(len(em.segments), max(1, tune.get("dd_segw", 4)), max(1, 8 // em.NCH)) if em.R == 1 else 1
        G_a = max(1, min(G, 8 // (em.NCH * segw)))
        if len(em.segments) > 1 and "dd_g" not in os.environ.get("OEQ_AMD_TUNE", ""):
            # several output segments: one node per block, as in the first-order forward kernel (second-order op:
            # SevenNet main layer -4 %, three more mixed-multiplicity shapes -2 % .. -3 %, nothing slower)
            G_a = 1
        blk_a = em.emit_conv_double_a(s, G_a, tune.get("dd_wa", 2), xcd, segw)
        descs.append((rt.ROLE_DOUBLE_BACKWARD_A, "double_backward_A", blk_a, G_a, 0, xcd))
    if groups:
        blk_b = em.emit_conv_double_b_split(s, groups, tune.get("dd_wb", 2), xcd)
        G_b = 1
    elif shared:
        G_b = 1 if em.NCH > 1 else groups_b
        blk_b = em.emit_conv_double_b(s, G_b, tune.get("dd_wb", 2), 1)
        return descs + [(rt.ROLE_DOUBLE_BACKWARD_B, "double_backward_B", blk_b, G_b, compute_units * 8, 1)]
    else:
        blk_b = em.emit_conv_double_b(s, G, tune.get("dd_wb", 2), xcd)
        G_b = 1 if em.NCH > 1 else G
    return descs + [(rt.ROLE_DOUBLE_BACKWARD_B, "double_backward_B", blk_b, G_b, 0, xcd)]


def _emit_segment_structs(s: Src, em: DoubleEmitter, prefix: str):
    """This emitter's output segments can differ from the first-order kernels': its accumulator
    structs get their own names (D<i>_t, zero_dseg<i>)."""
    low = em.low
    for si, seg in enumerate(em.segments):
        s(f"struct {prefix}{si}_t {{")
        for io in seg:
            s(f"    T o{io}[{low.out[io].d}];")
        s("};")
        s.open(f"OEQ_DEV void zero_{prefix.lower()}seg{si}({prefix}{si}_t& a)")
        for io in seg:
            for k in range(low.out[io].d):
                s(f"a.o{io}[{k}] = T(0);")
        s.close()
        if em.kahan:
            # c: one edge's terms plus the rounding error carried over; afterwards what did not fit into a
            s.open(f"OEQ_DEV void kahan_{prefix.lower()}seg{si}({prefix}{si}_t& c, {prefix}{si}_t& a)")
            for io in seg:
                for k in range(low.out[io].d):
                    e = f"o{io}[{k}]"
                    s(f"{{ const T y = c.{e}; const T t = a.{e} + y; c.{e} = y - (t - a.{e}); a.{e} = t; }}")
            s.close()
