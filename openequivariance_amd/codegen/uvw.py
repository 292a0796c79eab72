"""HIP source generator for fully-connected ('uvw') tensor products.

Replaces the reference's 'uvw' branch of the unrolled templates and its
register-tiled warp matmul (openequivariance/openequivariance/templates/
loop_unroll_tp.cuh:55-84, 217-272 and templates/wmm.cuh:1-87).

Two kernel families are generated:

* a general one (any multiplicities, per-row or shared weights): lanes are
  input channels ``u`` for the CG contraction and for everything in the backward
  pass; the forward channel mix runs with lanes = output channels ``w`` and reads
  the per-``u`` intermediates back from LDS as broadcasts;
* for shared weights, MFMA kernels (see ``uvw_mfma.py``) that batch rows so that the
  channel mix is a dense GEMM; they take every problem except those whose padded
  16-channel tiles would be mostly zeros or whose tiles exceed the LDS.

The general family also carries the second-order pair ``double_backward_A`` / ``double_backward_B`` (the
reference's kernels of that name, templates/loop_unroll_batch.cuh:148-317 and
templates/loop_unroll_conv_det.cuh:296-548): the forward- and backward-shaped kernels written with
``second=True``, which read the operands of both orders in one pass.
"""

from __future__ import annotations

from typing import Dict, Tuple

from .common import Src, prelude, utility_kernels
from .lower import Lowered, Path, float_literal

WAVES_PER_BLOCK = 4
# the chunk table of long edge segments and the rows of the extra chunks, as the last kernel arguments of the
# receiver walks
HUB_PARAMS = (", const i64* __restrict__ hubptr, const i64* __restrict__ hubnode, i64 hub_limit, i64 hub_units, "
              "T* __restrict__ hub_rows")


def _pow2ceil(n: int) -> int:
    return 1 << max(0, (n - 1).bit_length())


class UvwEmitter:
    def __init__(self, low: Lowered):
        assert low.mode == "uvw"
        from .uvu import tuning
        self.tune = tuning(dict(uvw_unroll=16, uvw_tile=24576, uvw_regdw=1, conv_hops=2, conv_fuse_uvw=1, uvw_dd=1,
                                uvw_dda_split=0, uvw_dda_unroll=4, conv_hub=256))
        self.TILE_BYTES = self.tune["uvw_tile"]
        self.low = low
        self.T = low.ctype
        self.l2_pad = _pow2ceil(low.L2)
        self.max_d3 = max(low.out[p.io].d for p in low.paths)
        self.second = False         # set while the second-order kernel B is being written
        self.wvec_declared = False

    def lit(self, v: float) -> str:
        return float_literal(v, self.T)

    def _products(self, s: Src, p: Path, second: bool = False) -> Dict[int, Tuple[str, bool]]:
        """|c| * y_j for the distinct (|c|, j) of a path: nnz index -> (name, negative). ``second``: the same
        products of the second row ``brow`` as well, under the name with a ``b`` appended."""
        b2 = self.low.in2[p.i2]
        for j in sorted({j for _, j, _, _ in p.nnz}):
            s(f"const T y{j} = yrow[{b2.off} + v * {b2.d} + {j}];")
            if second:
                s(f"const T b{j} = brow[{b2.off} + v * {b2.d} + {j}];")
        names, out = {}, {}
        for n, (i, j, k, c) in enumerate(p.nnz):
            key = (self.lit(abs(c)), j)
            if key not in names:
                names[key] = f"q{len(names)}"
                s(f"const T {names[key]} = T({key[0]}) * y{j};")
                if second:
                    s(f"const T {names[key]}b = T({key[0]}) * b{j};")
            out[n] = (names[key], c < 0)
        return out

    def _row_loop_open(self, s: Src, waves: int = WAVES_PER_BLOCK):
        s("const int lane = oeq_lane();")
        s("const int wave = oeq_wave();")
        s(f"for (i64 base = (i64)blockIdx.x * {waves}; base < num_batch; "
          f"base += (i64)gridDim.x * {waves}) {{")
        s.level += 1
        s("const i64 row = base + wave;")
        s("const bool live = row < num_batch;")
        s("const i64 rowc = live ? row : num_batch - 1;")

    # ------------------------------------------------------------- forward
    def _forward_block(self, s: Src, io: int, acc: str = "acc", second: bool = False):
        """Adds the contribution of one row (xrow, yrow, wrow) to the channels w = wc + lane of output block
        ``io``: the CG contraction with lanes = u goes to the wave's LDS tile, the channel mix reads it
        back as broadcasts with lanes = w. ``second``: the three forward terms of the second-order pass,
        F(a, y, w) + F(x, b, w) + F(x, y, c), as two channel mixes: the contraction of (a, y) and (x, b) mixed
        with w, that of (x, y) with c."""
        low = self.low
        bo = low.out[io]
        if second:
            return self._forward_block_second(s, io, acc)
        for p in [q for q in low.paths if q.io == io]:
            b1, b2 = low.in1[p.i1], low.in2[p.i2]
            s(f"// path {p.index}: l=({b1.l},{b2.l},{bo.l}) {b1.mul}x{b2.mul}->{bo.mul}")
            s.open(f"for (int v = 0; v < {b2.mul}; ++v)")
            s.open(f"for (int uc = 0; uc < {b1.mul}; uc += 64)")
            s.open("")
            s("const int u = uc + lane;")
            s(f"T x[{b1.d}];")
            s.open(f"if (u < {b1.mul})")
            for i in range(b1.d):
                s(f"x[{i}] = xrow[{b1.off} + u * {b1.d} + {i}];")
            s.close(" else {")
            s.level += 1
            for i in range(b1.d):
                s(f"x[{i}] = T(0);")
            s.close()
            prods = self._products(s, p)
            started = set()
            for n, (i, j, k, c) in enumerate(p.nnz):
                q, neg = prods[n]
                if k not in started:
                    s(f"T t{k} = {'-' if neg else ''}{q} * x[{i}];")
                    started.add(k)
                else:
                    s(f"t{k} {'-=' if neg else '+='} {q} * x[{i}];")
            # the tile is private to the wave (one row per wave): wave-level ordering is enough
            s("oeq_wave_sync();")
            for k in range(bo.d):
                s(f"s_t[wave][{k}][lane] = {'t%d' % k if k in started else 'T(0)'};")
            s("oeq_wave_sync();")
            s.close()
            s(f"const int nu = ({b1.mul} - uc < 64) ? {b1.mul} - uc : 64;")
            s(f"const T* wp = wrow + {p.woff} + ((i64)uc * {b2.mul} + v) * {bo.mul} + w;")
            s.open(f"if (w < {bo.mul})")
            s.open("for (int uu = 0; uu < nu; ++uu)")
            s(f"const T wv = wp[(i64)uu * {b2.mul * bo.mul}];")
            for k in range(bo.d):
                s(f"{acc}[{k}] += wv * s_t[wave][{k}][uu];")
            s.close()
            s.close()
            s.close()
            s.close()

    def _forward_block_second(self, s: Src, io: int, acc: str):
        low = self.low
        bo = low.out[io]
        D = self.max_d3
        for p in [q for q in low.paths if q.io == io]:
            b1, b2 = low.in1[p.i1], low.in2[p.i2]
            s(f"// path {p.index}: l=({b1.l},{b2.l},{bo.l}) {b1.mul}x{b2.mul}->{bo.mul}")
            s.open(f"for (int v = 0; v < {b2.mul}; ++v)")
            s.open(f"for (int uc = 0; uc < {b1.mul}; uc += 64)")
            s.open("")
            s("const int u = uc + lane;")
            s(f"T x[{b1.d}], a[{b1.d}];")
            s.open(f"if (u < {b1.mul})")
            for i in range(b1.d):
                s(f"x[{i}] = xrow[{b1.off} + u * {b1.d} + {i}]; a[{i}] = arow[{b1.off} + u * {b1.d} + {i}];")
            s.close(" else {")
            s.level += 1
            for i in range(b1.d):
                s(f"x[{i}] = T(0); a[{i}] = T(0);")
            s.close()
            prods = self._products(s, p, second=True)
            started = set()
            for n, (i, j, k, c) in enumerate(p.nnz):
                q, neg = prods[n]
                sg, op = ("-" if neg else ""), ("-=" if neg else "+=")
                if k not in started:
                    s(f"T t{k} = {sg}{q} * a[{i}]; T r{k} = {sg}{q} * x[{i}];")
                    started.add(k)
                else:
                    s(f"t{k} {op} {q} * a[{i}]; r{k} {op} {q} * x[{i}];")
                s(f"t{k} {op} {q}b * x[{i}];")
            s("oeq_wave_sync();")
            for k in range(bo.d):
                s(f"s_t[wave][{k}][lane] = {'t%d' % k if k in started else 'T(0)'};")
                s(f"s_t[wave][{D + k}][lane] = {'r%d' % k if k in started else 'T(0)'};")
            s("oeq_wave_sync();")
            s.close()
            s(f"const int nu = ({b1.mul} - uc < 64) ? {b1.mul} - uc : 64;")
            s(f"const i64 woff = {p.woff} + ((i64)uc * {b2.mul} + v) * {bo.mul} + w;")
            s.open(f"if (w < {bo.mul})")
            mode, unroll = self.tune["uvw_dda_split"], self.tune["uvw_dda_unroll"]
            if mode:
                # one weight stream per loop, as in the first-order kernel
                for row, base in (("wrow", 0), ("crow", D)):
                    s(f"const T* {row[0]}p = {row} + woff;")
                    if unroll:
                        s(f"#pragma unroll {unroll}")
                    s.open("for (int uu = 0; uu < nu; ++uu)")
                    s(f"const T wv = {row[0]}p[(i64)uu * {b2.mul * bo.mul}];")
                    for k in range(bo.d):
                        s(f"{acc}[{k}] += wv * s_t[wave][{base + k}][uu];")
                    s.close()
            else:
                if unroll:
                    s(f"#pragma unroll {unroll}")
                s.open("for (int uu = 0; uu < nu; ++uu)")
                s(f"const T wv = wrow[woff + (i64)uu * {b2.mul * bo.mul}];")
                s(f"const T cv = crow[woff + (i64)uu * {b2.mul * bo.mul}];")
                for k in range(bo.d):
                    s(f"{acc}[{k}] += wv * s_t[wave][{k}][uu]; {acc}[{k}] += cv * s_t[wave][{D + k}][uu];")
                s.close()
            s.close()
            s.close()
            s.close()

    def emit_forward(self, s: Src, second: bool = False):
        """``second``: the kernel double_backward_A (three forward terms into L3_dgrad)."""
        low = self.low
        block = 64 * WAVES_PER_BLOCK
        if second:
            s.open(
                f'extern "C" __global__ __launch_bounds__({block}) void double_backward_A(i64 num_batch, '
                "const T* __restrict__ L1_in, const T* __restrict__ L1_dgrad, const T* __restrict__ L2_in, "
                "const T* __restrict__ L2_dgrad, const T* __restrict__ W, const T* __restrict__ W_dgrad, "
                "T* __restrict__ L3_out)"
            )
        else:
            s.open(
                f'extern "C" __global__ __launch_bounds__({block}) void forward(i64 num_batch, '
                "const T* __restrict__ L1_in, const T* __restrict__ L2_in, const T* __restrict__ W, "
                "T* __restrict__ L3_out)"
            )
        s(f"__shared__ T s_t[{WAVES_PER_BLOCK}][{self.max_d3 * (2 if second else 1)}][64];")
        self._row_loop_open(s)
        s(f"const T* xrow = L1_in + rowc * {low.L1};")
        s(f"const T* yrow = L2_in + rowc * {low.L2};")
        s(f"const T* wrow = W{'' if low.shared_weights else f' + rowc * {low.WN}'};")
        if second:
            s(f"const T* arow = L1_dgrad + rowc * {low.L1};")
            s(f"const T* brow = L2_dgrad + rowc * {low.L2};")
            s(f"const T* crow = W_dgrad{'' if low.shared_weights else f' + rowc * {low.WN}'};")
        s(f"T* zrow = L3_out + rowc * {low.L3};")
        for io, bo in enumerate(low.out):
            s(f"// ---- out[{io}]: {bo.mul} x l={bo.l}")
            s.open(f"for (int wc = 0; wc < {bo.mul}; wc += 64)")
            s("const int w = wc + lane;")
            s(f"T acc[{bo.d}];")
            for k in range(bo.d):
                s(f"acc[{k}] = T(0);")
            self._forward_block(s, io, second=second)
            s.open(f"if (live && w < {bo.mul})")
            for k in range(bo.d):
                s(f"zrow[{bo.off} + w * {bo.d} + {k}] = acc[{k}];")
            s.close()
            s.close()
        s.close()
        s.close()
        return block

    def emit_conv_forward(self, s: Src, kahan: bool = False, second: bool = False):
        """Fused convolution, forward: the waves of a block share a receiver node's output segments (64
        channels of one output block each, lanes = w) and each keeps its segments in registers over the
        node's edges, whose senders' rows, Y rows and weight rows it reads in place: no gathered copy of X
        and no per-edge message tensor. The nodes are taken in the walk order of the index, the edges of a
        node in list order (so the sums do not depend on scheduling); with ``kahan`` each edge's message is
        added with a compensation term. ``second``: the kernel double_backward_A of the convolution (the three
        forward terms of the second-order pass, same walk). Returns (block size, nodes per block)."""
        low = self.low
        segs = [(io, wc) for io, bo in enumerate(low.out) for wc in range(0, bo.mul, 64)
                if any(p.io == io for p in low.paths)]
        empty = [io for io in range(len(low.out)) if not any(p.io == io for p in low.paths)]
        wpn = max(1, min(WAVES_PER_BLOCK, len(segs)))  # waves per node
        G = WAVES_PER_BLOCK // wpn
        block = 64 * wpn * G
        if second:
            s.open(
                f'extern "C" __global__ __launch_bounds__({block}) void double_backward_A(i64 node_count, i64 nnz, '
                "const T* __restrict__ L1_in, const T* __restrict__ L1_dgrad, const T* __restrict__ L2_in, "
                "const T* __restrict__ L2_dgrad, const T* __restrict__ W, const T* __restrict__ W_dgrad, "
                "T* __restrict__ L3_out, const i64* __restrict__ rows, const i64* __restrict__ cols, "
                "const i64* __restrict__ rowptr, const i64* __restrict__ eperm, const i64* __restrict__ order"
                f"{HUB_PARAMS})"
            )
        else:
            s.open(
                f'extern "C" __global__ __launch_bounds__({block}) void forward(i64 node_count, i64 nnz, '
                "const T* __restrict__ L1_in, const T* __restrict__ L2_in, const T* __restrict__ W, "
                "T* __restrict__ L3_out, const i64* __restrict__ rows, const i64* __restrict__ cols, "
                "const i64* __restrict__ rowptr, const i64* __restrict__ eperm, const i64* __restrict__ order"
                f"{HUB_PARAMS})"
            )
        s(f"__shared__ T s_t[{wpn * G}][{self.max_d3 * (2 if second else 1)}][64];")
        s("const int lane = oeq_lane();")
        s("const int wave = oeq_wave();")
        s(f"const int g = wave / {wpn}, sg = wave % {wpn};")
        # Walk positions: the first hub_units of them are the extra chunks of nodes with more than hub_limit
        # edges (their partial rows go to hub_rows and are added in chunk order afterwards), then one position
        # per node, which takes the node's first chunk.
        s("const i64 walk_end = hub_units + node_count;")
        s.open(f"for (i64 base = (i64)blockIdx.x * {G}; base < walk_end; base += (i64)gridDim.x * {G})")
        s("const i64 wpos = base + g;")
        s("const bool extra = wpos < hub_units;")
        s("const bool live = extra ? wpos < hubptr[node_count] : wpos < walk_end;")
        s("i64 node = 0, e0 = 0, e1 = 0;")
        s(f"T* zrow = L3_out;")
        s.open("if (live && extra)")
        s("node = oeq_idx(hubnode[wpos], node_count);")
        s("e0 = oeq_pos(rowptr[node] + (wpos - hubptr[node] + 1) * hub_limit, nnz);")
        s("e1 = oeq_pos(rowptr[node + 1], nnz);")
        s("if (e1 - e0 > hub_limit) e1 = e0 + hub_limit;")
        s(f"zrow = hub_rows + wpos * {low.L3};")
        s.close()
        s.open("else if (live)")
        s("const i64 vnode = wpos - hub_units;")
        s("node = order ? oeq_idx(order[vnode], node_count) : vnode;")
        s("e0 = oeq_pos(rowptr[node], nnz);")
        s("e1 = oeq_pos(rowptr[node + 1], nnz);")
        s("if (hub_limit > 0 && e1 - e0 > hub_limit) e1 = e0 + hub_limit;")
        s(f"zrow = L3_out + node * {low.L3};")
        s.close()
        for io in empty:
            # an output block no path writes: zeros
            bo = low.out[io]
            s.open("if (live && sg == 0)")
            s(f"for (int t = lane; t < {bo.mul * bo.d}; t += 64) zrow[{bo.off} + t] = T(0);")
            s.close()
        for si, (io, wc) in enumerate(segs):
            bo = low.out[io]
            s(f"// ---- out[{io}]: {bo.mul} x l={bo.l}, channels {wc}..")
            s.open(f"if (sg == {si % wpn})")
            s(f"const int wc = {wc};")
            s("const int w = wc + lane;")
            s(f"T acc[{bo.d}];")
            for k in range(bo.d):
                s(f"acc[{k}] = T(0);")
            if kahan:
                s(f"T comp[{bo.d}];")
                for k in range(bo.d):
                    s(f"comp[{k}] = T(0);")
            s.open("for (i64 pos = e0; pos < e1; ++pos)")
            s("const i64 e = oeq_idx(OEQ_EDGE(pos), nnz);")
            s("const i64 sender = oeq_idx(cols[e], node_count);")
            s(f"const T* xrow = L1_in + sender * {low.L1};")
            s(f"const T* yrow = L2_in + e * {low.L2};")
            s(f"const T* wrow = W{'' if low.shared_weights else f' + e * {low.WN}'};")
            if second:
                s(f"const T* arow = L1_dgrad + sender * {low.L1};")
                s(f"const T* brow = L2_dgrad + e * {low.L2};")
                s(f"const T* crow = W_dgrad{'' if low.shared_weights else f' + e * {low.WN}'};")
            if kahan:
                s(f"T msg[{bo.d}];")
                for k in range(bo.d):
                    s(f"msg[{k}] = T(0);")
                self._forward_block(s, io, "msg", second=second)
                for k in range(bo.d):
                    s(f"{{ const T y = msg[{k}] - comp[{k}]; const T t = acc[{k}] + y; "
                      f"comp[{k}] = (t - acc[{k}]) - y; acc[{k}] = t; }}")
            else:
                self._forward_block(s, io, second=second)
            s.close()
            s.open(f"if (live && w < {bo.mul})")
            for k in range(bo.d):
                s(f"zrow[{bo.off} + w * {bo.d} + {k}] = acc[{k}];")
            s.close()
            s.close()
        s.close()
        s.close()
        return block, G

    # ------------------------------------------------------------ backward
    # TILE_BYTES (set from the uvw_tile knob): per-wave LDS budget for one path's weight tile; larger
    # blocks are accessed directly. 24 KB takes in [64 x 80] blocks (e3tools convolution: 44 % -> 59 % of
    # HBM peak); with the loads of the next tile in flight during a step, fewer waves per CU no longer hurt.

    def _tile_plan(self, p: Path):
        """Per-row weights of a path and one 64-channel chunk of u form a contiguous [rows, V, W] block.
        Returns (max elements of such a block, vector width in elements for 16-byte copies) when it fits
        the per-wave LDS tile, else None."""
        low = self.low
        if low.shared_weights:
            return None
        b1, b2, bo = low.in1[p.i1], low.in2[p.i2], low.out[p.io]
        if b1.mul == 1:
            return None  # one input channel: handled with lanes = output channels instead
        per_u = b2.mul * bo.mul
        rows = min(64, b1.mul)
        elems = rows * per_u
        if elems * low.elem_size > self.TILE_BYTES:
            return None
        vw = 16 // low.elem_size
        chunk_starts = range(0, b1.mul, 64)
        aligned = low.WN % vw == 0 and all((p.woff + uc * per_u) % vw == 0 and
                                           (min(64, b1.mul - uc) * per_u) % vw == 0 for uc in chunk_starts)
        return elems, (vw if aligned else 1)

    def emit_backward(self, s: Src, conv: bool = False, second: bool = False, force_waves: int = 0):
        """``conv``: the fused convolution's backward. An edge is a row: X comes from the sender's row,
        the output gradient from the receiver's, the X gradient goes to the edge's row of ``dx_tmp``
        (summed per sender, in the order of the sender-major list, by ``fixup_backward``). The edges need no
        order here, so the kernel strides over the edge list as it is.

        ``second``: the kernel double_backward_B. With cotangents (a, b, c) of the first-order (dX, dY, dW) and
        G = W g, H = C g (two channel mixes where the composition of first-order kernels runs three):
        d/dX_i = sum c (b_j G_k + y_j H_k), d/dY_j = sum c (a_i G_k + x_i H_k),
        d/dW[u,v,w] = sum_k f_k g[w,k] with f_k = sum c (y_j a_i + b_j x_i). Same work decomposition and weight
        staging as the first-order kernel, with a second tile for C. ``force_waves``: waves per block (shared
        weights: the partial weight-gradient rows are counted per block of the first-order kernel)."""
        low = self.low
        shared = low.shared_weights
        self.second = second
        plans = {p.index: self._tile_plan(p) for p in low.paths}
        tiled = [p for p in low.paths if plans[p.index]]
        waves = WAVES_PER_BLOCK
        if tiled:
            # rows of the tile start an odd number of elements apart: lanes reading the same column of
            # their rows hit different banks
            tile_elems = (max(min(64, low.in1[p.i1].mul) * self._row_stride(p) for p in tiled) + 3) // 4 * 4
            vw = 16 // low.elem_size
            if not getattr(self, "wvec_declared", False):
                s(f"struct __attribute__((aligned(16))) wvec_t {{ T v[{vw}]; }};")
                self.wvec_declared = True
            # keep a block's LDS near 40 KB, so that four blocks (and at least four waves) share a CU; the
            # second-order kernel holds two tiles per wave and is given twice that
            per_wave = tile_elems * low.elem_size * (2 if second else 1)
            waves = max(1, min(WAVES_PER_BLOCK, (81920 if second else 40960) // per_wave))
        # shared weights: each wave sums its rows' weight gradients in an LDS copy of the weight tensor
        # (when that fits) and writes it out once, instead of a read-modify-write of global memory per row
        self.shared_lds = False
        self.reg_dw = False
        if shared:
            # Small shared weight tensors with at most 64 input channels per path: lane u keeps its rows
            # dW[u, :, :] of every path in registers over all the rows the wave handles (no read-modify-write
            # of LDS per row), and reads W from one padded LDS copy per block with constant offsets.
            dw_regs = sum(low.in2[p.i2].mul * low.out[p.io].mul for p in low.paths) * (low.elem_size // 4)
            self.wsh_base, off = {}, 0
            for p in low.paths:
                self.wsh_base[p.index] = off
                off += low.in1[p.i1].mul * self._row_stride(p)
            self.wsh_elems = off
            if (self.tune["uvw_regdw"] and dw_regs <= 176 and all(1 < low.in1[p.i1].mul <= 64 for p in low.paths)
                    and off * low.elem_size * (2 if second else 1) <= 49152
                    and (not force_waves or force_waves == WAVES_PER_BLOCK)):
                self.reg_dw = True
                waves = WAVES_PER_BLOCK
        if shared and not self.reg_dw:
            fit = 65536 // (low.WN * low.elem_size)
            if force_waves:
                waves = force_waves
                self.shared_lds = fit >= force_waves
            elif fit >= 1:
                self.shared_lds = True
                waves = min(WAVES_PER_BLOCK, fit)
        if not second:
            self.backward_waves = waves
        block = 64 * waves
        name = "double_backward_B" if second else "backward"
        operands = ("const T* __restrict__ L1_in, const T* __restrict__ L1_dgrad, const T* __restrict__ L2_in, "
                    "const T* __restrict__ L2_dgrad, const T* __restrict__ W, const T* __restrict__ W_dgrad, "
                    "const T* __restrict__ L3_grad, ")
        # register-resident weight gradients: left to one wave per SIMD with up to 512 registers (e3tools
        # transformer block: 0.29 ms against 0.57 ms with spills at 256; uvw_regdw=2 selects the latter)
        attr = " __attribute__((amdgpu_waves_per_eu(2, 2)))" if (self.reg_dw and self.tune["uvw_regdw"] == 2) else ""
        if second and conv:
            s.open(
                f'extern "C" __global__ __launch_bounds__({block}){attr} void {name}(i64 node_count, i64 nnz, '
                + operands + "T* __restrict__ L2_grad, T* __restrict__ W_grad, const i64* __restrict__ rows, "
                "const i64* __restrict__ cols, const i64* __restrict__ rowptr, T* __restrict__ dx_tmp, "
                "const i64* __restrict__ eperm, T* __restrict__ L3_dgrad, const i64* __restrict__ order, "
                "T* __restrict__ wpartial)"
            )
            s("const i64 num_batch = nnz;")
        elif second:
            s.open(
                f'extern "C" __global__ __launch_bounds__({block}){attr} void {name}(i64 num_batch, '
                + operands + "T* __restrict__ L1_grad, T* __restrict__ L2_grad, T* __restrict__ W_grad, "
                "T* __restrict__ wpartial)"
            )
        elif conv:
            s.open(
                f'extern "C" __global__ __launch_bounds__({block}){attr} void backward(i64 node_count, i64 nnz, '
                "const T* __restrict__ L1_in, T* __restrict__ L1_grad, const T* __restrict__ L2_in, "
                "T* __restrict__ L2_grad, const T* __restrict__ W, T* __restrict__ W_grad, "
                "const T* __restrict__ L3_grad, const i64* __restrict__ rows, const i64* __restrict__ cols, "
                "const i64* __restrict__ rowptr, T* __restrict__ dx_tmp, const i64* __restrict__ eperm, "
                "T* __restrict__ wpartial, const i64* __restrict__ colptr, const i64* __restrict__ sperm, "
                "int* __restrict__ arrivals, const i64* __restrict__ order)"
            )
            s("const i64 num_batch = nnz;")
        else:
            s.open(
                f'extern "C" __global__ __launch_bounds__({block}){attr} void backward(i64 num_batch, '
                "const T* __restrict__ L1_in, T* __restrict__ L1_grad, const T* __restrict__ L2_in, "
                "T* __restrict__ L2_grad, const T* __restrict__ W, T* __restrict__ W_grad, "
                "const T* __restrict__ L3_grad, T* __restrict__ wpartial)"
            )
        if tiled:
            # one path's weights of the row, then (in place) its weight gradients
            s(f"__shared__ __attribute__((aligned(16))) T s_w[{waves}][{tile_elems}];")
            if second:
                s(f"__shared__ __attribute__((aligned(16))) T s_c[{waves}][{tile_elems}];")
        if shared:
            s(f"T* prow = wpartial + ((i64)blockIdx.x * {waves} + oeq_wave()) * {low.WN};")
            if self.reg_dw:
                s(f"__shared__ T s_wsh[{self.wsh_elems}];")
                if second:
                    s(f"__shared__ T s_csh[{self.wsh_elems}];")
                for p in low.paths:
                    per_u, S = low.in2[p.i2].mul * low.out[p.io].mul, self._row_stride(p)
                    s(f"for (int t = threadIdx.x; t < {low.in1[p.i1].mul * per_u}; t += {block}) "
                      f"s_wsh[{self.wsh_base[p.index]} + t / {per_u} * {S - per_u} + t] = W[{p.woff} + t];")
                    if second:
                        s(f"for (int t = threadIdx.x; t < {low.in1[p.i1].mul * per_u}; t += {block}) "
                          f"s_csh[{self.wsh_base[p.index]} + t / {per_u} * {S - per_u} + t] = W_dgrad[{p.woff} + t];")
                    s(f"T dwr{p.index}[{per_u}];")
                    s(f"for (int t = 0; t < {per_u}; ++t) dwr{p.index}[t] = T(0);")
                s("__syncthreads();")
            elif self.shared_lds:
                s(f"__shared__ T s_dw[{waves}][{low.WN}];")
                s(f"for (int t = oeq_lane(); t < {low.WN}; t += 64) s_dw[oeq_wave()][t] = T(0);")
                s("oeq_wave_sync();")
            else:
                s("bool first = true;")
        if tiled:
            steps0 = [(i1, c, p) for i1, b1 in enumerate(low.in1) for c in range((b1.mul + 63) // 64)
                      for p in low.paths if p.i1 == i1 and plans[p.index]]
            nv_max = max(self._pad_vectors(st[2], st[1] * 64, plans[st[2].index][1]) for st in steps0)
            s(f"wvec_t pf[{nv_max}];  // the next weight tile on its way from global memory to LDS")
            if second:
                s(f"wvec_t pfc[{nv_max}];")
        self._row_loop_open(s, waves)
        if conv:
            s("const i64 sender = oeq_idx(cols[rowc], node_count);")
            s(f"const T* xrow = L1_in + sender * {low.L1};")
            s(f"const T* grow = L3_grad + oeq_idx(rows[rowc], node_count) * {low.L3};")
            s(f"T* dxrow = dx_tmp + rowc * {low.L1};")
            if second:
                s(f"const T* arow = L1_dgrad + sender * {low.L1};")
        else:
            s(f"const T* xrow = L1_in + rowc * {low.L1};")
            s(f"const T* grow = L3_grad + rowc * {low.L3};")
            s(f"T* dxrow = L1_grad + rowc * {low.L1};")
            if second:
                s(f"const T* arow = L1_dgrad + rowc * {low.L1};")
        if second:
            s(f"const T* brow = L2_dgrad + rowc * {low.L2};")
            s(f"const T* crow = W_dgrad{'' if shared else f' + rowc * {low.WN}'};")
        s(f"const T* yrow = L2_in + rowc * {low.L2};")
        s(f"const T* wrow = W{'' if shared else f' + rowc * {low.WN}'};")
        if not shared:
            s(f"T* dwrow = W_grad + rowc * {low.WN};")
        s(f"T dy[{self.l2_pad}];")
        s(f"for (int t = 0; t < {self.l2_pad}; ++t) dy[t] = T(0);")
        pipelined = bool(tiled)
        if pipelined:
            # Every (input block, 64-channel chunk, path) is a step known at generation time. The weight
            # tile of the next tiled step is requested from global memory into registers (pf) before the
            # current step computes, and written to LDS when that step is done: one exposed memory latency
            # per row instead of one per path.
            steps = [(i1, c, p) for i1, b1 in enumerate(low.in1) for c in range((b1.mul + 63) // 64)
                     for p in low.paths if p.i1 == i1]
            tsteps = [st for st in steps if plans[st[2].index]]
            self._pad_issue(s, tsteps[0][2], tsteps[0][1] * 64, plans[tsteps[0][2].index][1])
        for i1, b1 in enumerate(low.in1):
            paths = [p for p in low.paths if p.i1 == i1]
            s(f"// ---- in1[{i1}]: {b1.mul} x l={b1.l}")
            chunks = range((b1.mul + 63) // 64) if pipelined else [None]
            for c in chunks:
                if c is None:
                    s.open(f"for (int uc = 0; uc < {b1.mul}; uc += 64)")
                else:
                    s.open("")
                    s(f"const int uc = {c * 64};")
                s("const int u = uc + lane;")
                s(f"const bool uok = u < {b1.mul};")
                s(f"T x[{b1.d}], dx[{b1.d}];")
                for i in range(b1.d):
                    s(f"x[{i}] = uok ? xrow[{b1.off} + u * {b1.d} + {i}] : T(0); dx[{i}] = T(0);")
                if second:
                    s(f"T a[{b1.d}];")
                    for i in range(b1.d):
                        s(f"a[{i}] = uok ? arow[{b1.off} + u * {b1.d} + {i}] : T(0);")
                for p in paths:
                    b2, bo = low.in2[p.i2], low.out[p.io]
                    s(f"// path {p.index}: l=({b1.l},{b2.l},{bo.l})")
                    if plans[p.index] and pipelined:
                        k = tsteps.index((i1, c, p))
                        nxt = tsteps[k + 1] if k + 1 < len(tsteps) else None
                        self._bwd_path_padded(s, p, plans[p.index][1], c * 64,
                                              (nxt[2], nxt[1] * 64, plans[nxt[2].index][1]) if nxt else None)
                    elif self.reg_dw:
                        self._bwd_path_regdw(s, p)
                    elif b1.mul == 1:
                        self._bwd_path_single_u(s, p)
                    else:
                        self._bwd_path_direct(s, p)
                s.open("if (live && uok)")
                for i in range(b1.d):
                    s(f"dxrow[{b1.off} + u * {b1.d} + {i}] = dx[{i}];")
                s.close()
                s.close()
        if shared and not self.shared_lds and not self.reg_dw:
            s("first = false;")
        # dY: butterfly over the 64 lanes
        n = self.l2_pad
        s(f"T rv[{n}];")
        for j in range(n):
            s(f"rv[{j}] = dy[{j}];")
        s("int dyidx = 0;")
        cur, dup, m = n, 0, 32
        while m >= 1:
            if cur > 1:
                half = cur // 2
                s.open("")
                s(f"const bool hi = (lane & {m}) != 0;")
                for j in range(half):
                    s(f"{{ const T keep = hi ? rv[{j + half}] : rv[{j}]; const T send = hi ? rv[{j}] : rv[{j + half}]; "
                      f"rv[{j}] = keep + __shfl_xor(send, {m}); }}")
                s(f"dyidx += hi ? {half} : 0;")
                s.close()
                cur = half
            else:
                s(f"rv[0] += __shfl_xor(rv[0], {m});")
                dup |= m
            m //= 2
        s.open(f"if (live && (lane & {dup}) == 0)")
        for j in range(cur):
            s(f"if (dyidx + {j} < {low.L2}) L2_grad[rowc * {low.L2} + dyidx + {j}] = rv[{j}];")
        s.close()
        s.close()
        if shared and self.reg_dw:
            # lane u owns rows [u, :, :] of every path's weight gradient
            for p in low.paths:
                per_u = low.in2[p.i2].mul * low.out[p.io].mul
                s.open(f"if (oeq_lane() < {low.in1[p.i1].mul})")
                for t in range(per_u):
                    s(f"prow[{p.woff} + oeq_lane() * {per_u} + {t}] = dwr{p.index}[{t}];")
                s.close()
        elif shared and self.shared_lds:
            s("oeq_wave_sync();")
            s(f"for (int t = oeq_lane(); t < {low.WN}; t += 64) prow[t] = s_dw[oeq_wave()][t];")
        elif shared:
            # a wave that saw no row still owns a partial row: clear it
            s.open("if (first)")
            s(f"for (int t = oeq_lane(); t < {low.WN}; t += 64) prow[t] = T(0);")
            s.close()
        s.close()
        return block

    def _cg_backward(self, s: Src, p: Path, prods, gname: str = "G"):
        """dx, dy contributions of one (path, v) from G_k, and f_k = sum c x_i y_j (returns the k set)."""
        b2 = self.low.in2[p.i2]
        fstart = set()
        if getattr(self, "second", False):
            # second order: G_k = (W g)_k, H_k = (C g)_k; the products of the second row are named q<n>b
            for n, (i, j, k, c) in enumerate(p.nnz):
                q, neg = prods[n]
                op = "-=" if neg else "+="
                s(f"dx[{i}] {op} {q}b * {gname}{k}; dx[{i}] {op} {q} * H{k};")
                if k not in fstart:
                    s(f"T f{k} = {'-' if neg else ''}{q} * a[{i}];")
                    fstart.add(k)
                else:
                    s(f"f{k} {op} {q} * a[{i}];")
                s(f"f{k} {op} {q}b * x[{i}];")
            pair = {}
            for n, (i, j, k, c) in enumerate(p.nnz):
                if (i, k) not in pair:
                    pair[(i, k)] = f"xg{len(pair)}"
                    s(f"const T {pair[(i, k)]} = a[{i}] * {gname}{k} + x[{i}] * H{k};")
                s(f"dy[{b2.off} + v * {b2.d} + {j}] += T({self.lit(c)}) * {pair[(i, k)]};")
            return sorted(fstart)
        for n, (i, j, k, c) in enumerate(p.nnz):
            q, neg = prods[n]
            s(f"dx[{i}] {'-=' if neg else '+='} {q} * {gname}{k};")
            if k not in fstart:
                s(f"T f{k} = {'-' if neg else ''}{q} * x[{i}];")
                fstart.add(k)
            else:
                s(f"f{k} {'-=' if neg else '+='} {q} * x[{i}];")
        pair = {}
        for n, (i, j, k, c) in enumerate(p.nnz):
            if (i, k) not in pair:
                pair[(i, k)] = f"xg{len(pair)}"
                s(f"const T {pair[(i, k)]} = x[{i}] * {gname}{k};")
            s(f"dy[{b2.off} + v * {b2.d} + {j}] += T({self.lit(c)}) * {pair[(i, k)]};")
        return sorted(fstart)

    def _bwd_path_regdw(self, s: Src, p: Path):
        """Shared weights, lane = u, weight gradients in registers (``dwr<path>``) over all rows of the
        wave; W from the block's padded LDS copy (rows an odd number of elements apart: no bank
        conflicts, constant offsets), dZ of the output irrep through the scalar cache."""
        low = self.low
        b1, b2, bo = low.in1[p.i1], low.in2[p.i2], low.out[p.io]
        V, Wn, d3 = b2.mul, bo.mul, bo.d
        S = self._row_stride(p)
        s.open("")
        s(f"const T* gq = grow + {bo.off};  // wave-uniform")
        s(f"const T* wl = s_wsh + {self.wsh_base[p.index]} + (uok ? u : 0) * {S};")
        second = self.second
        if second:
            s(f"const T* cl = s_csh + {self.wsh_base[p.index]} + (uok ? u : 0) * {S};")
        for vv in range(V):
            s.open("")
            s(f"const int v = {vv};")
            prods = self._products(s, p, second)
            for k in range(d3):
                s(f"T G{k} = T(0);" + (f" T H{k} = T(0);" if second else ""))
            for w in range(Wn):
                s(f"{{ const T wv = wl[{vv * Wn + w}]; " +
                  " ".join(f"G{k} += wv * gq[{w * d3 + k}];" for k in range(d3)) + " }")
                if second:
                    s(f"{{ const T cv = cl[{vv * Wn + w}]; " +
                      " ".join(f"H{k} += cv * gq[{w * d3 + k}];" for k in range(d3)) + " }")
            ks = self._cg_backward(s, p, prods)
            s.open("if (uok && live)")
            for w in range(Wn):
                terms = " + ".join(f"f{k} * gq[{w * d3 + k}]" for k in ks)
                s(f"dwr{p.index}[{vv * Wn + w}] += {terms};")
            s.close()
            s.close()
        s.close()

    def _bwd_path_single_u(self, s: Src, p: Path):
        """A path whose first operand has one channel (spherical harmonics of an edge, say): lanes are the
        output channels w instead of u, of which there is only one. G_k = sum_w W[w] g[w,k] is a wave
        reduction, the weight gradient dW[w] = sum_k f_k g[w,k] is one value per lane (coalesced), and
        the dX / dY terms are wave-uniform: lane 0 (the lane that owns u = 0 in the surrounding code)
        adds them to its accumulators."""
        low = self.low
        shared = low.shared_weights
        b1, b2, bo = low.in1[p.i1], low.in2[p.i2], low.out[p.io]
        Wn, d3 = bo.mul, bo.d
        nchunk = (Wn + 63) // 64
        second = self.second
        s.open("")
        s(f"T xu[{b1.d}];")
        for i in range(b1.d):
            s(f"xu[{i}] = xrow[{b1.off} + {i}];")
        if second:
            s(f"T au[{b1.d}];")
            for i in range(b1.d):
                s(f"au[{i}] = arow[{b1.off} + {i}];")
        s.open(f"for (int v = 0; v < {b2.mul}; ++v)")
        prods = self._products(s, p, second)
        s(f"const int wbase = {p.woff} + v * {Wn};")
        for k in range(d3):
            s(f"T G{k} = T(0);" + (f" T H{k} = T(0);" if second else ""))
        if nchunk == 1:
            s(f"T gv[{d3}];")
        for c in range(nchunk):
            s.open("")
            s(f"const int w = {c * 64} + lane;")
            s(f"const bool wok = w < {Wn};")
            s(f"const int wc = wok ? w : {Wn - 1};")
            s("const T wv = wok ? wrow[wbase + wc] : T(0);")
            if second:
                s("const T cv = wok ? crow[wbase + wc] : T(0);")
            for k in range(d3):
                ld = f"grow[{bo.off} + wc * {d3} + {k}]"
                if nchunk == 1:
                    s(f"gv[{k}] = wok ? {ld} : T(0);")
                    s(f"G{k} += wv * gv[{k}];")
                    if second:
                        s(f"H{k} += cv * gv[{k}];")
                elif second:
                    s(f"{{ const T gl = {ld}; G{k} += wv * gl; H{k} += cv * gl; }}")
                else:
                    s(f"G{k} += wv * {ld};")
            s.close()
        for k in range(d3):
            for m in (32, 16, 8, 4, 2, 1):
                s(f"G{k} += __shfl_xor(G{k}, {m});")
                if second:
                    s(f"H{k} += __shfl_xor(H{k}, {m});")
        # wave-uniform from here on; only lane 0 (uok) keeps the dX / dY terms
        fstart = set()
        for n, (i, j, k, c) in enumerate(p.nnz):
            q, neg = prods[n]
            first_op = "xu" if not second else "au"
            if k not in fstart:
                s(f"T f{k} = {'-' if neg else ''}{q} * {first_op}[{i}];")
                fstart.add(k)
            else:
                s(f"f{k} {'-=' if neg else '+='} {q} * {first_op}[{i}];")
            if second:
                s(f"f{k} {'-=' if neg else '+='} {q}b * xu[{i}];")
        s.open("if (uok)")
        for n, (i, j, k, c) in enumerate(p.nnz):
            q, neg = prods[n]
            if second:
                op = "-=" if neg else "+="
                s(f"dx[{i}] {op} {q}b * G{k}; dx[{i}] {op} {q} * H{k};")
                s(f"dy[{b2.off} + v * {b2.d} + {j}] += T({self.lit(c)}) * (au[{i}] * G{k} + xu[{i}] * H{k});")
            else:
                s(f"dx[{i}] {'-=' if neg else '+='} {q} * G{k};")
                s(f"dy[{b2.off} + v * {b2.d} + {j}] += T({self.lit(c)}) * (xu[{i}] * G{k});")
        s.close()
        ks = sorted(fstart)
        for c in range(nchunk):
            s.open("")
            s(f"const int w = {c * 64} + lane;")
            s(f"const bool wok = w < {Wn};")
            s(f"const int wc = wok ? w : {Wn - 1};")
            gk = (lambda k: f"gv[{k}]") if nchunk == 1 else (lambda k: f"grow[{bo.off} + wc * {d3} + {k}]")
            s(f"T dwv = f{ks[0]} * {gk(ks[0])};")
            for k in ks[1:]:
                s(f"dwv += f{k} * {gk(k)};")
            if shared and self.shared_lds:
                s("if (wok && live) s_dw[wave][wbase + w] += dwv;")
            elif shared:
                s("if (!live) dwv = T(0);")
                s("if (wok) prow[wbase + w] = first ? dwv : prow[wbase + w] + dwv;")
            else:
                s("if (wok && live) dwrow[wbase + w] = dwv;")
            s.close()
        s.close()
        s.close()

    def _bwd_path_direct(self, s: Src, p: Path):
        """Weights read and weight gradients written straight from / to global memory, lane = u."""
        low = self.low
        shared = low.shared_weights
        b2, bo = low.in2[p.i2], low.out[p.io]
        second = self.second
        s.open(f"for (int v = 0; v < {b2.mul}; ++v)")
        prods = self._products(s, p, second)
        s(f"const i64 wbase = {p.woff} + ((i64)u * {b2.mul} + v) * {bo.mul};")
        # G_k = sum_w W[u,v,w] * g[w,k]
        for k in range(bo.d):
            s(f"T G{k} = T(0);" + (f" T H{k} = T(0);" if second else ""))
        s.open("if (uok)")
        s.open(f"for (int w = 0; w < {bo.mul}; ++w)")
        s("const T wv = wrow[wbase + w];")
        if second:
            s("const T cv = crow[wbase + w];")
        for k in range(bo.d):
            if second:
                s(f"{{ const T gl = grow[{bo.off} + w * {bo.d} + {k}]; G{k} += wv * gl; H{k} += cv * gl; }}")
            else:
                s(f"G{k} += wv * grow[{bo.off} + w * {bo.d} + {k}];")
        s.close()
        s.close()
        ks = self._cg_backward(s, p, prods)
        # dW[u,v,w] = sum_k f_k * g[w,k]
        if shared and self.shared_lds:
            # lane u visits w in the rotated order (u + t) mod W: the lanes' LDS addresses then fall into
            # different banks although their rows are a multiple of W apart
            s.open("if (uok && live)")
            s(f"int w = lane % {bo.mul};")
            s(f"T* drow = s_dw[wave] + wbase;")
            s.open(f"for (int t = 0; t < {bo.mul}; ++t)")
            terms = [f"f{k} * grow[{bo.off} + w * {bo.d} + {k}]" for k in ks]
            s(f"T dwv = {terms[0]};")
            for t in terms[1:]:
                s(f"dwv += {t};")
            s("drow[w] += dwv;")
            s(f"w = (w + 1 == {bo.mul}) ? 0 : w + 1;")
            s.close()
            s.close()
            s.close()
            return
        s.open(f"if (uok{' && live' if not shared else ''})")
        s.open(f"for (int w = 0; w < {bo.mul}; ++w)")
        terms = [f"f{k} * grow[{bo.off} + w * {bo.d} + {k}]" for k in ks]
        s(f"T dwv = {terms[0]};")
        for t in terms[1:]:
            s(f"dwv += {t};")
        if shared:
            s("if (!live) dwv = T(0);")
            s("prow[wbase + w] = first ? dwv : prow[wbase + w] + dwv;")
        else:
            s("dwrow[wbase + w] = dwv;")
        s.close()
        s.close()
        s.close()

    def _row_stride(self, p: Path) -> int:
        per_u = self.low.in2[p.i2].mul * self.low.out[p.io].mul
        return per_u | 1

    def _pad_geometry(self, p: Path, uc: int, vw: int):
        low = self.low
        b1, b2, bo = low.in1[p.i1], low.in2[p.i2], low.out[p.io]
        per_u = b2.mul * bo.mul
        nrows = min(64, b1.mul - uc)
        return per_u, nrows * per_u, p.woff + uc * per_u, self._row_stride(p)

    def _pad_vectors(self, p: Path, uc: int, vw: int) -> int:
        _, nel, _, _ = self._pad_geometry(p, uc, vw)
        return -(-nel // (64 * vw))

    def _pad_issue(self, s: Src, p: Path, uc: int, vw: int):
        """Request this lane's share of a step's contiguous weight block (coalesced 16-byte reads); in the
        second-order kernel the same block of the second weight tensor as well."""
        per_u, nel, tbase, _ = self._pad_geometry(p, uc, vw)
        for pf, row in (("pf", "wrow"), ("pfc", "crow"))[:2 if getattr(self, "second", False) else 1]:
            for q in range(self._pad_vectors(p, uc, vw)):
                t = f"(lane + {64 * q}) * {vw}"
                guard = "" if (64 * q + 64) * vw <= nel else f"if ({t} < {nel}) "
                if vw > 1:
                    s(f"{guard}{pf}[{q}] = *(const wvec_t*)({row} + {tbase} + {t});")
                else:
                    s(f"{guard}{pf}[{q}].v[0] = {row}[{tbase} + {t}];")

    def _pad_commit(self, s: Src, p: Path, uc: int, vw: int):
        """Registers -> padded LDS tile (row r of the block starts at r * S)."""
        per_u, nel, _, S = self._pad_geometry(p, uc, vw)
        for pf, tw in (("pf", "tw"), ("pfc", "tc"))[:2 if getattr(self, "second", False) else 1]:
            for q in range(self._pad_vectors(p, uc, vw)):
                t = f"(lane + {64 * q}) * {vw}"
                s.open("" if (64 * q + 64) * vw <= nel else f"if ({t} < {nel})")
                s(f"const int t = {t};")
                if per_u % vw == 0:
                    s(f"const int tr = t / {per_u};")
                    s(f"T* dst = {tw} + tr * {S - per_u} + t;")
                    for i in range(vw):
                        s(f"dst[{i}] = {pf}[{q}].v[{i}];")
                else:  # a vector can straddle two rows
                    for i in range(vw):
                        s(f"{tw}[(t + {i}) / {per_u} * {S - per_u} + t + {i}] = {pf}[{q}].v[{i}];")
                s.close()

    def _bwd_path_padded(self, s: Src, p: Path, vw: int, uc: int, nxt):
        """One step of the pipelined per-row-weight backward. The step's weights are in ``pf``; they go
        to the wave's LDS tile, whose rows start an odd number of elements apart: lane u can then walk
        its row front to back (all lanes at the same column) without bank conflicts and with addresses
        that are constants within the unrolled loops. dZ of the path's output irrep is the same for every
        lane: it is read through the scalar cache and enters the multiply-adds as scalar operands. Weight
        gradients replace the weights in the tile, which is copied out coalesced. ``nxt``: the next tiled
        step, whose weights are requested as soon as ``pf`` is free."""
        low = self.low
        b1, b2, bo = low.in1[p.i1], low.in2[p.i2], low.out[p.io]
        V, Wn = b2.mul, bo.mul
        per_u, nel, tbase, S = self._pad_geometry(p, uc, vw)
        unroll = max(1, self.tune["uvw_unroll"])
        s.open("")
        second = self.second
        s("T* tw = s_w[wave];")
        if second:
            s("T* tc = s_c[wave];")
        s(f"const T* gq = grow + {bo.off};  // wave-uniform")
        s("oeq_wave_sync();  // the previous step's tile is no longer read")
        self._pad_commit(s, p, uc, vw)
        if nxt is not None:
            self._pad_issue(s, *nxt)
        s("oeq_wave_sync();")
        s("const int urow = uok ? lane : 0;  // lanes without a channel read row 0 and store nothing")
        s.open(f"for (int v = 0; v < {V}; ++v)")
        prods = self._products(s, p, second)
        s(f"T* trow = tw + urow * {S} + v * {Wn};")
        if second:
            s(f"const T* crw = tc + urow * {S} + v * {Wn};")
        for k in range(bo.d):
            s(f"T G{k} = T(0);" + (f" T H{k} = T(0);" if second else ""))
        s(f"#pragma unroll {unroll}")
        s.open(f"for (int w = 0; w < {Wn}; ++w)")
        s("const T wv = trow[w];")
        if second:
            s("const T cv = crw[w];")
        for k in range(bo.d):
            s(f"G{k} += wv * gq[w * {bo.d} + {k}];")
            if second:
                s(f"H{k} += cv * gq[w * {bo.d} + {k}];")
        s.close()
        ks = self._cg_backward(s, p, prods)
        s.open("if (uok)")
        s(f"#pragma unroll {unroll}")
        s.open(f"for (int w = 0; w < {Wn}; ++w)")
        terms = [f"f{k} * gq[w * {bo.d} + {k}]" for k in ks]
        s(f"T dwv = {terms[0]};")
        for t in terms[1:]:
            s(f"dwv += {t};")
        s("trow[w] = dwv;")
        s.close()
        s.close()
        s.close()
        s("oeq_wave_sync();")
        s.open("if (live)")
        for q in range(self._pad_vectors(p, uc, vw)):
            t = f"(lane + {64 * q}) * {vw}"
            s.open("" if (64 * q + 64) * vw <= nel else f"if ({t} < {nel})")
            s(f"const int t = {t};")
            if vw > 1:
                s("wvec_t val;")
                for i in range(vw):
                    if per_u % vw == 0:
                        s(f"val.v[{i}] = tw[t / {per_u} * {S - per_u} + t + {i}];")
                    else:
                        s(f"val.v[{i}] = tw[(t + {i}) / {per_u} * {S - per_u} + t + {i}];")
                s(f"*(wvec_t*)(dwrow + {tbase} + t) = val;")
            else:
                s(f"dwrow[{tbase} + t] = tw[t / {per_u} * {S - per_u} + t];")
            s.close()
        s.close()
        s.close()


def conv_supported(low: Lowered) -> bool:
    """Problems the fused 'uvw' convolution kernels cover: per-edge weights, and shared weights unless the unfused
    path (gathered rows through the MFMA kernels, ordered sums) is the faster one: problems the matrix-core path
    takes with at least ``conv_mfma_min_weights`` weights. Below that the gathers and sums of the unfused path cost
    more than the matrix cores save (12 000 nodes / 532 k edges, forward / backward, unfused MFMA against fused
    general kernels: 256 weights 0.45 / 0.72 against 0.20 / 0.56 ms, 664 weights 0.72 / 1.49 against 0.70 / 0.82 ms,
    2 190 weights 0.96 / 3.3 against 0.89 / 7.9 ms, 6 928 weights 0.87 / 1.6 against 1.16 / 11.7 ms)."""
    if low.mode != "uvw":
        return False
    if not low.shared_weights:
        return True
    from . import uvw_mfma
    from .uvu import tuning
    return not uvw_mfma.supported(low) or low.WN < tuning(dict(conv_mfma_min_weights=2048))["conv_mfma_min_weights"]


def conv_module(low: Lowered, deterministic: bool, compute_units: int = 256, kahan: bool = False):
    """Source + launch descriptors of the fused 'uvw' convolution (per-edge weights; replaces the
    reference's 'uvw' branch inside its convolution templates, templates/loop_unroll_conv_atomic.cuh:52-180
    and loop_unroll_conv_det.cuh:187-293). Same kernel roles, argument lists and index as the 'uvu'
    convolution: a receiver walk for the forward pass, per-edge gradients plus the ordered sender-side
    sum for the backward pass. ``deterministic``: the caller brings receiver-sorted edges and the
    sender-major permutation; otherwise the library groups the edge ids on the device first."""
    from .. import runtime as rt
    from .common import fixup_backward_kernel

    assert conv_supported(low)
    shared = low.shared_weights
    em = UvwEmitter(low)
    s = Src()
    s(prelude(low.ctype))
    s(utility_kernels(kahan))
    s("#define OEQ_EDGE(j) (eperm ? eperm[(j)] : (j))")
    blk_f, G_f = em.emit_conv_forward(s, kahan)
    blk_b = em.emit_backward(s, conv=True)
    s(fixup_backward_kernel(low.L1, kahan, True))
    cu = compute_units
    # shared weights: every wave of the backward grid writes one partial weight-gradient row (summed in order
    # by oeq_wreduce), so that grid is bounded
    max_b = cu * (3 if em.shared_lds else 2) if shared else cu * 16
    second = []
    if em.tune["uvw_dd"]:
        # second-order pair: the same receiver walk / per-edge pass with the operands of both orders (with
        # ``kahan`` kernel A adds each edge's three terms with a compensation term, like the forward kernel)
        blk_da, G_da = em.emit_conv_forward(s, kahan, second=True)
        blk_db = em.emit_backward(s, conv=True, second=True, force_waves=em.backward_waves if shared else 0)
        second = [(rt.ROLE_DOUBLE_BACKWARD_A, "double_backward_A", blk_da, G_da, cu * 32),
                  (rt.ROLE_DOUBLE_BACKWARD_B, "double_backward_B", blk_db, 1, max_b)]
    descs = second + [
        (rt.ROLE_FILL_ZERO, "oeq_fill_zero", 256, 256 * 16, cu * 16),
        (rt.ROLE_SEGMENT_PTR, "oeq_segment_ptr", 256, 256, cu * 16),
        (rt.ROLE_CONV_FORWARD, "forward", blk_f, G_f, cu * 32),
        # strides over the edges: the grid need not follow the node count it is derived from
        (rt.ROLE_CONV_BACKWARD, "backward", blk_b, 1, max_b),
        (rt.ROLE_TP_BACKWARD_WREDUCE, "oeq_wreduce", 256, 64, 0),
        (rt.ROLE_CONV_FIXUP_BACKWARD, "fixup_backward", 256, 1, 0),
        (rt.ROLE_GROUP_COUNT, "oeq_group_count", 256, 256 * 4, cu * 16),
        (rt.ROLE_GROUP_SCAN, "oeq_group_scan", 1024, 1, 1),
        (rt.ROLE_GROUP_SCATTER, "oeq_group_scatter", 256, 256 * 4, cu * 16),
        (rt.ROLE_GROUP_ORDER, "oeq_group_order", 256, 4, cu * 32),
        (rt.ROLE_ORDER_HOP, "oeq_order_hop", 256, 256, cu * 16),
        (rt.ROLE_HUB_COUNT, "oeq_hub_count", 256, 256, cu * 16),
        (rt.ROLE_HUB_FILL, "oeq_hub_fill", 256, 256, cu * 16),
        (rt.ROLE_CONV_FIXUP_FORWARD, "fixup_forward", 256, 1, cu * 32),
    ]
    t = em.tune
    # Compensated sums run over whole segments (a compensation term does not carry across chunks).
    hub_limit = 0 if kahan else max(0, t["conv_hub"])
    dims = dict(L1_dim=low.L1, L2_dim=low.L2, L3_dim=low.L3, weight_numel=low.WN, elem_size=low.elem_size,
                shared_weights=int(shared), deterministic=rt.CONV_SORTED if deterministic else rt.CONV_GROUPED,
                wpartial_per_block=em.backward_waves if shared else 0, dx_mode=rt.DX_TERMS, n_chunks=1,
                order_hops=max(0, t["conv_hops"]), hub_limit=hub_limit)
    return s.text(), dims, descs


def tp_module(low: Lowered, compute_units: int = 256, kahan: bool = False):
    """``kahan`` only affects the ordered segment sum used by the unfused convolution."""
    from .. import runtime as rt

    if low.shared_weights and not kahan:
        from . import uvw_mfma
        from .uvu import tuning
        if uvw_mfma.supported(low) and tuning(dict(uvw_mfma=1))["uvw_mfma"]:
            return uvw_mfma.tp_module(low, compute_units)
    em = UvwEmitter(low)
    s = Src()
    s(prelude(low.ctype))
    s(utility_kernels(kahan))
    blk_f = em.emit_forward(s)
    blk_b = em.emit_backward(s)
    max_blocks_b = compute_units * (3 if em.shared_lds else 2)
    second = []
    if em.tune["uvw_dd"]:
        blk_da = em.emit_forward(s, second=True)
        blk_db = em.emit_backward(s, second=True, force_waves=em.backward_waves if low.shared_weights else 0)
        waves_db = blk_db // 64
        second = [(rt.ROLE_DOUBLE_BACKWARD_A, "double_backward_A", blk_da, WAVES_PER_BLOCK, compute_units * 16),
                  (rt.ROLE_DOUBLE_BACKWARD_B, "double_backward_B", blk_db, waves_db,
                   max_blocks_b if low.shared_weights else compute_units * 16)]
    descs = second + [
        (rt.ROLE_TP_FORWARD, "forward", blk_f, WAVES_PER_BLOCK, compute_units * 16),
        (rt.ROLE_TP_BACKWARD, "backward", blk_b, em.backward_waves,
         max_blocks_b if low.shared_weights else compute_units * 16),
        (rt.ROLE_FILL_ZERO, "oeq_fill_zero", 256, 256 * 16, compute_units * 16),
        (rt.ROLE_TP_BACKWARD_WREDUCE, "oeq_wreduce", 256, 64, 0),
    ]
    dims = dict(L1_dim=low.L1, L2_dim=low.L2, L3_dim=low.L3, weight_numel=low.WN, elem_size=low.elem_size,
                shared_weights=int(low.shared_weights), deterministic=0,
                wpartial_per_block=em.backward_waves if low.shared_weights else 0)
    return s.text(), dims, descs
