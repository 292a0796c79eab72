"""MFMA kernels for shared-weight 'uvw' tensor products (fp32).

With one weight tensor for the whole batch the channel mix of a path,
``Z[b][w,k] += sum_u W[u,w] * T[b][u,k]`` with ``T[b][u,k] = sum_ij c_ijk X[b][u,i] Y[b][j]``,
is a dense GEMM once rows are batched: ``[(b,k)] x [u] x [w]``. These kernels
run it on the matrix cores with ``v_mfma_f32_16x16x4_f32`` (true fp32, needed for
the 1e-5 parity bound) and keep the sparse CG part on the vector ALU. The
reference does this mix with a scalar-FMA warp matmul on 32-wide chunks
(openequivariance/openequivariance/templates/wmm.cuh:1-87,
loop_unroll_tp.cuh:55-84, 217-272).

Work decomposition: a block of 4 waves owns a tile of 16 batch rows at a time.

* forward: the block computes T of one path for the tile into LDS (lanes = u,
  4 rows per wave), then each wave multiplies the 16 x d3 row block with its own
  16-wide slices of the output channels; accumulators of an output irrep live in
  registers across all paths that feed it.
* backward: the dZ tile is staged in LDS once. Per path, G = dZ W^T comes out of
  MFMA in a layout (lane = 4 rows x one channel) on which the vector-ALU part
  (dX, dY and T) runs directly; T goes to LDS and the weight gradient
  dW += T^T dZ is accumulated by MFMA in registers over all tiles of the block
  (wave = 16-channel slice of u). Blocks write partial weight gradients that a
  second kernel sums in block order: no atomics, deterministic.

Operand layouts of v_mfma_f32_16x16x4_f32 used below (lane l of 64):
A[m][k]: m = l % 16, k = l / 16;  B[k][n]: k = l / 16, n = l % 16;
D[m][n]: n = l % 16, m = 4 * (l / 16) + i for the i-th of 4 result registers.
"""

from __future__ import annotations

from typing import Dict, List, Tuple

from .common import Src, prelude, utility_kernels
from .lower import Lowered, Path, float_literal

RT = 16          # rows per tile
WAVES = 4        # waves per block
TPAD = RT + 1    # padded row stride of the T tile in LDS (bank spread)


def supported(low: Lowered) -> bool:
    if low.mode != "uvw" or not low.shared_weights or low.ctype != "float":
        return False
    if low.L3 > 2048 or low.L2 > 32:
        return False
    for p in low.paths:
        a, b, o = low.in1[p.i1], low.in2[p.i2], low.out[p.io]
        if b.mul != 1 or a.mul != 64 or o.mul % 64 != 0 or o.mul > 256:
            return False
    n_dw = sum((low.in1[p.i1].mul // 64) * (low.out[p.io].mul // 16) * 4 for p in low.paths)
    return n_dw <= 256


def _pow2ceil(n: int) -> int:
    return 1 << max(0, (n - 1).bit_length())


class MfmaEmitter:
    def __init__(self, low: Lowered):
        self.low = low
        self.max_d3 = max(low.out[p.io].d for p in low.paths)
        self.gstride = low.L3 + (1 if low.L3 % 32 != 1 else 0)  # odd-ish row stride of the dZ tile in LDS
        if self.gstride % 2 == 0:
            self.gstride += 1

    def lit(self, v):
        return float_literal(v, "float")

    # ---- CG part of one path for one (row, channel): t_k, and in the backward dx, dy
    def _emit_path_fns(self, s: Src):
        low = self.low
        for p in low.paths:
            b1, b2, bo = low.in1[p.i1], low.in2[p.i2], low.out[p.io]
            js = sorted({j for _, j, _, _ in p.nnz})

            def products():
                names, out = {}, {}
                for n, (i, j, k, c) in enumerate(p.nnz):
                    key = (self.lit(abs(c)), j)
                    if key not in names:
                        names[key] = f"q{len(names)}"
                        s(f"const T {names[key]} = T({key[0]}) * y[{b2.off + j}];")
                    out[n] = (names[key], c < 0)
                return out

            # forward: t[k] = sum c x_i y_j
            s.open(f"OEQ_DEV void cg_fwd{p.index}(const T* __restrict__ xp, const T* __restrict__ y, T (&t)[{bo.d}])")
            for i in range(b1.d):
                s(f"const T x{i} = xp[{i}];")
            prods = products()
            started = set()
            for n, (i, j, k, c) in enumerate(p.nnz):
                q, neg = prods[n]
                if k not in started:
                    s(f"t[{k}] = {'-' if neg else ''}{q} * x{i};")
                    started.add(k)
                else:
                    s(f"t[{k}] {'-=' if neg else '+='} {q} * x{i};")
            for k in range(bo.d):
                if k not in started:
                    s(f"t[{k}] = T(0);")
            s.close()
            # backward: given G[k] = sum_w W[u,w] dZ[w,k]
            s.open(
                f"OEQ_DEV void cg_bwd{p.index}(const T* __restrict__ xp, const T* y, const T (&G)[{bo.d}], "
                f"T (&dx)[{b1.d}], T (&dy)[{low.L2}], T (&t)[{bo.d}])"
            )
            for i in range(b1.d):
                s(f"const T x{i} = xp[{i}];")
            prods = products()
            started = set()
            for n, (i, j, k, c) in enumerate(p.nnz):
                q, neg = prods[n]
                s(f"dx[{i}] {'-=' if neg else '+='} {q} * G[{k}];")
                if k not in started:
                    s(f"t[{k}] = {'-' if neg else ''}{q} * x{i};")
                    started.add(k)
                else:
                    s(f"t[{k}] {'-=' if neg else '+='} {q} * x{i};")
            for k in range(bo.d):
                if k not in started:
                    s(f"t[{k}] = T(0);")
            pair = {}
            for n, (i, j, k, c) in enumerate(p.nnz):
                if (i, k) not in pair:
                    pair[(i, k)] = f"xg{len(pair)}"
                    s(f"const T {pair[(i, k)]} = x{i} * G[{k}];")
                s(f"dy[{b2.off + j}] += T({self.lit(c)}) * {pair[(i, k)]};")
            s.close()

    # ------------------------------------------------------------- forward
    def emit_forward(self, s: Src):
        low = self.low
        s.open(
            f'extern "C" __global__ __launch_bounds__({64 * WAVES}) void forward(i64 num_batch, '
            "const T* __restrict__ L1_in, const T* __restrict__ L2_in, const T* __restrict__ W, T* __restrict__ L3_out)"
        )
        s(f"__shared__ T s_T[{self.max_d3}][64][{TPAD}];")
        s("const int lane = oeq_lane();")
        s("const int wave = oeq_wave();")
        s("const int l16 = lane & 15, lq = lane >> 4;")
        s(f"const i64 ntiles = (num_batch + {RT - 1}) / {RT};")
        s.open("for (i64 tile = blockIdx.x; tile < ntiles; tile += gridDim.x)")
        s(f"const i64 row0 = tile * {RT};")
        for io, bo in enumerate(low.out):
            paths = [p for p in low.paths if p.io == io]
            ntw = bo.mul // 64  # 16-wide output slices per wave
            s(f"// ---- out[{io}]: {bo.mul} x l={bo.l}")
            s.open("")
            s(f"v4f acc[{bo.d}][{ntw}];")
            for k in range(bo.d):
                for j in range(ntw):
                    s(f"acc[{k}][{j}] = v4f{{0.f, 0.f, 0.f, 0.f}};")
            for p in paths:
                b1 = low.in1[p.i1]
                s(f"// path {p.index}: l=({b1.l},{low.in2[p.i2].l},{bo.l})")
                s.open(f"for (int uc = 0; uc < {b1.mul}; uc += 64)")
                s("__syncthreads();")
                s.open(f"for (int rr = 0; rr < {RT // WAVES}; ++rr)")
                s(f"const int r = wave * {RT // WAVES} + rr;")
                s("i64 row = row0 + r; if (row >= num_batch) row = num_batch - 1;")
                s(f"T t[{bo.d}];")
                s(f"cg_fwd{p.index}(L1_in + row * {low.L1} + {b1.off} + (uc + lane) * {b1.d}, L2_in + row * {low.L2}, t);")
                for k in range(bo.d):
                    s(f"s_T[{k}][lane][r] = t[{k}];")
                s.close()
                s("__syncthreads();")
                s("#pragma unroll 4")
                s.open("for (int st = 0; st < 16; ++st)")
                for k in range(bo.d):
                    s(f"const T a{k} = s_T[{k}][4 * st + lq][l16];")
                for j in range(ntw):
                    s(f"const T b{j} = W[{p.woff} + (i64)(uc + 4 * st + lq) * {bo.mul} + {16 * WAVES * j} + wave * 16 + l16];")
                for j in range(ntw):
                    for k in range(bo.d):
                        s(f"acc[{k}][{j}] = __builtin_amdgcn_mfma_f32_16x16x4f32(a{k}, b{j}, acc[{k}][{j}], 0, 0, 0);")
                s.close()
                s.close()
            # D layout: rows 4*lq + i, column (channel) l16 of the wave's slice
            for j in range(ntw):
                s.open("for (int i = 0; i < 4; ++i)")
                s("const i64 row = row0 + 4 * lq + i;")
                s.open("if (row < num_batch)")
                s(f"T* zp = L3_out + row * {low.L3} + {bo.off} + ({16 * WAVES * j} + wave * 16 + l16) * {bo.d};")
                for k in range(bo.d):
                    s(f"zp[{k}] = acc[{k}][{j}][i];")
                s.close()
                s.close()
            s.close()
        s.close()
        s.close()

    # ------------------------------------------------------------ backward
    def dw_layout(self) -> Dict[int, Tuple[int, int]]:
        """path -> (first accumulator index, number of 16-wide w slices)."""
        out, n = {}, 0
        for p in self.low.paths:
            nw = self.low.out[p.io].mul // 16
            out[p.index] = (n, nw)
            n += nw
        self.n_dw = n
        return out

    def _stage_tile(self, s: Src, with_y: bool):
        low = self.low
        s("__syncthreads();")
        s.open(f"for (int t = tid; t < {RT * low.L3}; t += {64 * WAVES})")
        s(f"const int r = t / {low.L3}, c = t % {low.L3};")
        s(f"s_g[r][c] = (row0 + r < num_batch) ? L3_grad[(row0 + r) * {low.L3} + c] : T(0);")
        s.close()
        if with_y:
            s.open(f"for (int t = tid; t < {RT * low.L2}; t += {64 * WAVES})")
            s(f"const int r = t / {low.L2}, c = t % {low.L2};")
            s(f"s_y[r][c] = (row0 + r < num_batch) ? L2_in[(row0 + r) * {low.L2} + c] : T(0);")
            s.close()
        s("__syncthreads();")

    def emit_backward(self, s: Src):
        """Two sweeps over the block's tiles inside one kernel, so that the
        register sets of the two halves (dX/dY state vs. the weight-gradient
        accumulators) are never live together."""
        low = self.low
        dwl = self.dw_layout()
        L2p = low.L2
        s.open(
            f'extern "C" __global__ __launch_bounds__({64 * WAVES}) void backward(i64 num_batch, '
            "const T* __restrict__ L1_in, T* __restrict__ L1_grad, const T* __restrict__ L2_in, "
            "T* __restrict__ L2_grad, const T* __restrict__ W, T* __restrict__ W_grad, "
            "const T* __restrict__ L3_grad, T* __restrict__ wpartial)"
        )
        s(f"__shared__ T s_g[{RT}][{self.gstride}];")
        s(f"__shared__ T s_T[{self.max_d3}][64][{TPAD}];")
        s(f"__shared__ T s_y[{RT}][{L2p}];")
        s(f"__shared__ T s_dy[{WAVES}][{RT}][{L2p}];")
        s("const int lane = oeq_lane();")
        s("const int wave = oeq_wave();")
        s("const int l16 = lane & 15, lq = lane >> 4;")
        s("const int tid = (int)threadIdx.x;")
        s(f"const i64 ntiles = (num_batch + {RT - 1}) / {RT};")

        # ---------------- sweep 1: dX, dY --------------------------------------
        s.open("for (i64 tile = blockIdx.x; tile < ntiles; tile += gridDim.x)")
        s(f"const i64 row0 = tile * {RT};")
        self._stage_tile(s, with_y=True)
        s(f"T dy[4][{L2p}];")
        s(f"for (int i = 0; i < 4; ++i) for (int j = 0; j < {L2p}; ++j) dy[i][j] = T(0);")
        for i1, b1 in enumerate(low.in1):
            paths = [p for p in low.paths if p.i1 == i1]
            s(f"// ---- in1[{i1}]: {b1.mul} x l={b1.l}")
            if not paths:
                s.open(f"for (int t = tid; t < {RT * b1.mul * b1.d}; t += {64 * WAVES})")
                s(f"const int r = t / {b1.mul * b1.d}, c = t % {b1.mul * b1.d};")
                s(f"if (row0 + r < num_batch) L1_grad[(row0 + r) * {low.L1} + {b1.off} + c] = T(0);")
                s.close()
                continue
            s.open("")
            s(f"T dx[4][{b1.d}];")
            s(f"for (int i = 0; i < 4; ++i) for (int c = 0; c < {b1.d}; ++c) dx[i][c] = T(0);")
            s("const int u = wave * 16 + l16;")
            for p in paths:
                b2, bo = low.in2[p.i2], low.out[p.io]
                s(f"// path {p.index}: l=({b1.l},{b2.l},{bo.l})")
                s.open("")
                # G[k] = sum_w dZ[(r,k), w] * W[u, w]   (A = dZ tile, B = W^T)
                s(f"v4f G[{bo.d}];")
                for k in range(bo.d):
                    s(f"G[{k}] = v4f{{0.f, 0.f, 0.f, 0.f}};")
                s("#pragma unroll 2")
                s.open(f"for (int st = 0; st < {bo.mul // 4}; ++st)")
                for k in range(bo.d):
                    s(f"const T a{k} = s_g[l16][{bo.off} + (4 * st + lq) * {bo.d} + {k}];")
                s(f"const T b = W[{p.woff} + (i64)u * {bo.mul} + 4 * st + lq];")
                for k in range(bo.d):
                    s(f"G[{k}] = __builtin_amdgcn_mfma_f32_16x16x4f32(a{k}, b, G[{k}], 0, 0, 0);")
                s.close()
                # vector-ALU part on the D layout: lane = rows 4*lq+i, channel u
                s("#pragma unroll")
                s.open("for (int i = 0; i < 4; ++i)")
                s("i64 row = row0 + 4 * lq + i; if (row >= num_batch) row = num_batch - 1;")
                s(f"T Gk[{bo.d}], t[{bo.d}];")
                for k in range(bo.d):
                    s(f"Gk[{k}] = G[{k}][i];")
                s(f"cg_bwd{p.index}(L1_in + row * {low.L1} + {b1.off} + u * {b1.d}, s_y[4 * lq + i], Gk, dx[i], dy[i], t);")
                s.close()
                s.close()
            s.open("for (int i = 0; i < 4; ++i)")
            s("const i64 row = row0 + 4 * lq + i;")
            s.open("if (row < num_batch)")
            s(f"T* dp = L1_grad + row * {low.L1} + {b1.off} + u * {b1.d};")
            for c in range(b1.d):
                s(f"dp[{c}] = dx[i][{c}];")
            s.close()
            s.close()
            s.close()
        # dY: sum over the 16 channels of the lane group, then over the 4 waves through LDS
        s.open("for (int i = 0; i < 4; ++i)")
        s.open(f"for (int j = 0; j < {L2p}; ++j)")
        s("T v = dy[i][j];")
        for m in (1, 2, 4, 8):
            s(f"v += __shfl_xor(v, {m});")
        s("if (l16 == 0) s_dy[wave][4 * lq + i][j] = v;")
        s.close()
        s.close()
        s("__syncthreads();")
        s.open(f"for (int t = tid; t < {RT * low.L2}; t += {64 * WAVES})")
        s(f"const int r = t / {low.L2}, c = t % {low.L2};")
        s("const T tot = ((s_dy[0][r][c] + s_dy[1][r][c]) + s_dy[2][r][c]) + s_dy[3][r][c];")
        s(f"if (row0 + r < num_batch) L2_grad[(row0 + r) * {low.L2} + c] = tot;")
        s.close()
        s.close()

        # ---------------- sweep 2: dW ------------------------------------------
        s(f"v4f dw[{self.n_dw}];")
        for n in range(self.n_dw):
            s(f"dw[{n}] = v4f{{0.f, 0.f, 0.f, 0.f}};")
        s.open("for (i64 tile = blockIdx.x; tile < ntiles; tile += gridDim.x)")
        s(f"const i64 row0 = tile * {RT};")
        self._stage_tile(s, with_y=False)
        for p in low.paths:
            b1, b2, bo = low.in1[p.i1], low.in2[p.i2], low.out[p.io]
            base, nw = dwl[p.index]
            s(f"// path {p.index}: l=({b1.l},{b2.l},{bo.l})")
            s("__syncthreads();  // readers of the previous s_T are done")
            s.open(f"for (int rr = 0; rr < {RT // WAVES}; ++rr)")
            s(f"const int r = wave * {RT // WAVES} + rr;")
            s("i64 row = row0 + r; if (row >= num_batch) row = num_batch - 1;")
            s(f"T t[{bo.d}];")
            s(f"cg_fwd{p.index}(L1_in + row * {low.L1} + {b1.off} + lane * {b1.d}, L2_in + row * {low.L2}, t);")
            for k in range(bo.d):
                s(f"s_T[{k}][lane][r] = t[{k}];")
            s.close()
            s("__syncthreads();")
            # dW[u, w] += sum_(k,r) T[(k,r), u] * dZ[(k,r), w]   (A = T^T, B = dZ tile; zero dZ rows past the batch)
            s("#pragma unroll 2")
            s.open(f"for (int st = 0; st < {4 * bo.d}; ++st)")
            s("const int kq = 4 * st + lq;")
            s("const int kk = kq >> 4, rr = kq & 15;")
            s("const T a = s_T[kk][wave * 16 + l16][rr];")
            for n in range(nw):
                s(f"const T b{n} = s_g[rr][{bo.off} + ({16 * n} + l16) * {bo.d} + kk];")
            for n in range(nw):
                s(f"dw[{base + n}] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b{n}, dw[{base + n}], 0, 0, 0);")
            s.close()
        s.close()
        # partial weight gradient of this block (D layout: rows = channels u, columns = w)
        s(f"T* prow = wpartial + (i64)blockIdx.x * {low.WN};")
        for p in low.paths:
            base, nw = dwl[p.index]
            bo = low.out[p.io]
            for n in range(nw):
                s.open("for (int i = 0; i < 4; ++i)")
                s(f"prow[{p.woff} + (i64)(wave * 16 + 4 * lq + i) * {bo.mul} + {16 * n} + l16] = dw[{base + n}][i];")
                s.close()
        s.close()


def tp_module(low: Lowered, compute_units: int = 256):
    from .. import runtime as rt

    em = MfmaEmitter(low)
    s = Src()
    s(prelude(low.ctype))
    s("typedef float v4f __attribute__((ext_vector_type(4)));")
    s(utility_kernels())
    em._emit_path_fns(s)
    em.emit_forward(s)
    em.emit_backward(s)
    max_blocks_b = compute_units * 2
    descs = [
        (rt.ROLE_TP_FORWARD, "forward", 64 * WAVES, RT, compute_units * 8),
        (rt.ROLE_TP_BACKWARD, "backward", 64 * WAVES, RT, max_blocks_b),
        (rt.ROLE_FILL_ZERO, "oeq_fill_zero", 256, 256 * 16, compute_units * 16),
        (rt.ROLE_TP_BACKWARD_WREDUCE, "oeq_wreduce", 256, 256, 0),
    ]
    dims = dict(L1_dim=low.L1, L2_dim=low.L2, L3_dim=low.L3, weight_numel=low.WN, elem_size=low.elem_size,
                shared_weights=1, deterministic=0, wpartial_per_block=1)
    return s.text(), dims, descs
