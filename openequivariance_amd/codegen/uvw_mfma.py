"""MFMA kernels for shared-weight 'uvw' tensor products (fp32 and fp64).

With one weight tensor for the whole batch the channel mix of a path,
``Z[b][w,k] += sum_u W[u,w] * T[b][u,k]`` with ``T[b][u,k] = sum_ij c_ijk X[b][u,i] Y[b][j]``,
is a dense GEMM once rows are batched: ``[(b,k)] x [u] x [w]``. These kernels
run it on the matrix cores with ``v_mfma_f32_16x16x4_f32`` (true fp32, needed for
the 1e-5 parity bound) or ``v_mfma_f64_16x16x4_f64`` and keep the sparse CG part on the vector ALU. The
reference does this mix with a scalar-FMA warp matmul on 32-wide chunks
(openequivariance/openequivariance/templates/wmm.cuh:1-87,
loop_unroll_tp.cuh:55-84, 217-272).

A path whose second operand has V channels is V such mixes, one per channel v with
the weight matrix ``W[:, v, :]``.

Work decomposition: irrep blocks are cut into pieces of at most 64 channels
(a piece whose channel count is no multiple of 16 is padded to one with zero
weights: its missing channels are never loaded or stored), a path into one sub-path per channel of the second
operand and pair of
pieces with its own 64 x 64 (or smaller) corner of the path's weight matrix. A
block of 4 waves owns a tile of 16 batch rows at a time; wave ``w`` owns output
channels (forward) or input channels (backward) ``16w .. 16w+15`` of a piece
(waves beyond a narrow piece's channels sit out the multiplies). Forward and
backward are each a short sequence of kernels launched back to back with the
same arguments; with pieces on both sides a kernel takes one piece and the
sub-paths that meet it from the k-th piece of the other side, and all but the
first kernel of a piece add to what is already there (a tile is always handled
by the same thread of the same block, so the order of these additions is fixed):

* forward, one kernel per output irrep: the wave's slices of the weight
  matrices of the paths feeding that irrep stay in registers in MFMA B-operand
  layout (16 registers per path) for the whole kernel. Per path the block
  computes T for the tile into LDS (lanes = u, 4 rows per wave; the X values of
  the next path are fetched into registers while the current path's MFMAs run),
  then each wave multiplies the 16 x d3 row block by its weight slice. The T
  tile is double buffered: one block barrier per path.
* backward, one kernel per input irrep (dX and the dY terms of its paths): the
  dZ tile is staged in LDS; per path G = dZ W^T comes out of MFMA in a layout
  (lane = 4 rows x one channel) on which the vector-ALU part runs directly, with
  W^T slices register-resident. A tile is always handled by the same thread of
  the same block, so later kernels add their dY terms with plain
  read-modify-writes in a fixed order.
* backward, one kernel per output irrep (dW of the paths feeding it): T is
  recomputed into LDS and dW += T^T dZ is accumulated by MFMA in registers over
  all tiles of the block. Blocks write partial weight gradients that a last
  kernel sums in block order: no atomics, deterministic.

Splitting by irrep keeps each kernel under 256 registers (two waves per SIMD),
so one wave's LDS/global latencies hide behind the other's MFMAs.

Operand layouts of the two 16x16x4 instructions used below (lane l of 64):
A[m][k]: m = l % 16, k = l / 16;  B[k][n]: k = l / 16, n = l % 16;
D[m][n]: n = l % 16, and for the i-th of 4 result registers m = 4 * (l / 16) + i in fp32,
m = l / 16 + 4 * i in fp64.

The second-order pair (``second_order_kernels``) reuses these kernels under other operand bindings: the
forward and dW kernels with the contraction ``T(a, y) + T(x, b)`` of both operand pairs, the forward and dX
kernels once per weight tensor (W, then the cotangent of dW, adding to the first result).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import List

from .common import Src, prelude, utility_kernels
from .lower import Lowered, Path, float_literal

RT = 16          # rows per tile
WAVES = 4        # waves per block
TPAD = RT + 1    # padded row stride of the T tile in LDS (bank spread)
LDS_BUDGET = 160 * 1024 - 2048   # bytes of LDS a kernel may declare (the CU has 160 KB)
MFMA = "oeq_mfma"  # v_mfma_f32_16x16x4_f32 or v_mfma_f64_16x16x4_f64, see tp_module
# fp32 problems, split-operand form: every fp32 operand is written as the sum of three bf16 numbers (8 mantissa bits
# each: 24 in all, the fp32 mantissa), a product as the six cross products of weight 2^-16 and above, each of them exact
# in fp32, summed in fp32 by v_mfma_f32_16x16x32_bf16. That instruction does 8 times the multiplies of the fp32 one in
# half its time (16 against 32 cycles), runs on a pipe of its own (the fp32 matrix instruction shares the vector
# datapath), and the three dropped products are of the size of an fp32 rounding error.
BF3_ROW = 72     # elements per row of a bf16 operand plane in LDS: 64 + 8, rows start 36 words apart
BF3_TERMS = ((2, 0), (0, 2), (1, 1), (1, 0), (0, 1), (0, 0))  # (part of A, part of B), smallest products first


def c4(n: int) -> int:
    """k-steps of 4 that cover n channels."""
    return (n + 3) // 4


def c16(n: int) -> int:
    """16-channel tiles that cover n channels."""
    return (n + 15) // 16


def piece_of(low: Lowered) -> int:
    """Channels per piece of an irrep block (``uvw_piece`` overrides: 16, 32, 48 or 64)."""
    from .uvu import tuning
    forced = tuning(dict(uvw_piece=0))["uvw_piece"]
    return forced if forced in (16, 32, 48, 64) else 64


@dataclass
class VBlock:
    """A piece (at most 64 channels) of an irrep block."""
    off: int
    mul: int
    l: int
    orig: int     # index of the block it was cut from
    chunk: int    # which piece of that block

    @property
    def d(self) -> int:
        return 2 * self.l + 1


@dataclass
class VPath:
    """The part of a path between one piece of its input block and one piece of its output block: a
    U x Wn corner of the path's weight matrix, whose rows are ``ld`` words apart."""
    index: int
    p: Path
    vi: int
    vo: int
    U: int
    Wn: int
    woff: int
    ld: int
    ub: int
    wb: int
    v: int = 0    # channel of the second operand (its own sub-path: W[u, v, w] is a U x Wn matrix for every v)
    part: int = 0  # which part of its group, where the group's weight slices exceed a kernel's registers (_groups)

    def tag(self, side: str) -> str:
        """Names the group of sub-paths a kernel takes from the other side of a piece on ``side``."""
        k = self.ub if side == "vo" else self.wb
        return f"{k}" + (f"p{self.part}" if self.part else "")


def _pieces(blocks, piece: int) -> List[VBlock]:
    out = []
    for i, b in enumerate(blocks):
        for c in range((b.mul + piece - 1) // piece):
            out.append(VBlock(b.off + c * piece * b.d, min(piece, b.mul - c * piece), b.l, i, c))
    return out


def _split(low: Lowered):
    PIECE = piece_of(low)
    vin, vout = _pieces(low.in1, PIECE), _pieces(low.out, PIECE)
    vpaths = []
    for p in low.paths:
        wtot, V = low.out[p.io].mul, low.in2[p.i2].mul
        for v in range(V):
            for vi, a in enumerate(vin):
                if a.orig != p.i1:
                    continue
                for vo, o in enumerate(vout):
                    if o.orig != p.io:
                        continue
                    # W[u, v, w] of the path: rows (u) are V * wtot words apart
                    vpaths.append(VPath(len(vpaths), p, vi, vo, a.mul, o.mul,
                                        p.woff + (a.chunk * PIECE * V + v) * wtot + o.chunk * PIECE, V * wtot,
                                        a.chunk, o.chunk, v))
    return vin, vout, vpaths


# Most registers (in elements) that the resident weight slices of one kernel take, per pass: a group of sub-paths
# beyond that (or beyond what the kernel's other registers leave, see the ``limit`` functions of the emitters) is
# cut into parts with a kernel each (an irrep fed by more than five 64-channel paths, say).
SLICE_REGS = {"forward": 80, "dx": 80, "dw": 80}


def _slice_regs(vp: VPath, which: str, bf3: bool = False) -> int:
    if bf3 and which == "forward":
        return 12 * ((vp.U + 31) // 32)  # three parts of 8 bf16 (4 registers) per 32 input channels
    return c4(vp.U) if which == "forward" else 4 * c16(vp.Wn)


def _groups(vpaths: List[VPath], side: str, n_blocks: int, which: str, limit=None, bf3: bool = False):
    """Kernels of one pass (``which``: 'forward', 'dx' or 'dw'): for every piece on ``side`` ('vo' or 'vi') its
    sub-paths grouped by the piece index on the other side (all channels of the second operand), a group cut into
    parts whose weight slices fit ``limit(piece, sub-paths)`` registers. Returns [(piece, [sub-paths], first
    kernel of that piece?)]; a piece without paths gets one entry with an empty list."""
    other = "ub" if side == "vo" else "wb"
    out = []
    for b in range(n_blocks):
        mine = [vp for vp in vpaths if getattr(vp, side) == b]
        keys = sorted({getattr(vp, other) for vp in mine})
        if not keys:
            out.append((b, [], True))
        for n, key in enumerate(keys):
            parts, room = [], 0
            sel = sorted((q for q in mine if getattr(q, other) == key), key=lambda q: (q.v, q.index))
            budget = min(SLICE_REGS[which], limit(b, sel)) if limit else SLICE_REGS[which]
            total = sum(_slice_regs(vp, which, bf3) for vp in sel)
            if total > budget:  # parts of about equal size
                budget = max(-(-total // -(-total // budget)), max(_slice_regs(vp, which, bf3) for vp in sel))
            for vp in sel:
                need = _slice_regs(vp, which, bf3)
                if not parts or need > room:
                    parts.append([])
                    room = budget
                parts[-1].append(vp)
                room -= need
                vp.part = len(parts) - 1
            out += [(b, part, n == 0 and c == 0) for c, part in enumerate(parts)]
    return out


def supported(low: Lowered) -> bool:
    if low.mode != "uvw" or not low.shared_weights or low.ctype not in ("float", "double") or low.ir_mul:
        return False
    if low.L2 > 64:  # (per-lane dY accumulators of the dX kernels: 4 rows x L2)
        return False
    # the dX kernels keep a whole 16-row dZ tile in LDS beside the Y rows and the partial dY of the four waves
    # (fp64: rows of up to about 1 000 elements)
    if (RT * (low.L3 + 36) + (1 + WAVES) * RT * low.L2) * low.elem_size > LDS_BUDGET:
        return False
    # ... the forward kernels two copies of the T tile of an output piece (fp64: l <= 4), the dW kernels one copy
    # beside the piece's dZ columns
    tl = piece_of(low)
    for p in low.paths:
        o = low.out[p.io]
        cols = min(o.mul, tl) * o.d
        if max(2 * o.d * tl * TPAD + 2 * RT * low.L2,
               RT * (cols + 36) + o.d * tl * TPAD + 2 * RT * low.L2) * low.elem_size > LDS_BUDGET:
            return False
    vin, vout, vpaths = _split(low)
    # Multiplicities that are no multiples of 16 run on tiles padded with zero weights. Where nearly all of a
    # tile would be padding the general kernels are the better choice: ``uvw_mfma_fill`` = least share (percent)
    # of the multiplies that must be real ones. Measured at 262 144 rows, backward, padded tiles against general
    # kernels: share 0.80 (48 and 10 channels) 0.54 / 6.8 ms, 0.39 (10 -> 17, 9, 33 channels) 1.4 / 5.3 ms, 0.25
    # (8 channels) 0.17 / 0.23 ms, 0.06 (tetris polynomial, 1 - 6 channels) 2.5 / 2.0 ms.
    from .uvu import tuning
    real = sum(vp.U * vp.Wn for vp in vpaths)
    padded = sum(16 * c16(vp.U) * 16 * c16(vp.Wn) for vp in vpaths)
    if 100 * real < tuning(dict(uvw_mfma_fill=25))["uvw_mfma_fill"] * padded:
        return False
    return True


class MfmaEmitter:
    def __init__(self, low: Lowered):
        self.low = low
        self.vin, self.vout, self.vpaths = _split(low)
        self.max_d3 = max(low.out[p.io].d for p in low.paths)
        self.max_d1 = max(low.in1[p.i1].d for p in low.paths)
        self.words = low.elem_size // 4
        self.vw = 16 // low.elem_size  # elements per 16-byte vector
        # Row stride of the dZ tile in LDS: 4 mod 32 words. Rows then start on 16-byte boundaries (the tile is
        # filled with 16-byte stores), and the 32 lanes of a half-wave that read one column of 16 rows, at two
        # k-steps d words apart (d odd), fall into 32 different banks.
        self.gstride = self._tile_stride(low.L3)
        # batch row (within the tile) of the i-th of a lane's four results: fp32 4 * (lane / 16) + i, fp64
        # lane / 16 + 4 * i (the two instructions lay their 16 x 16 result out differently)
        self.row = (lambda i: f"(4 * lq + {i})") if low.elem_size == 4 else (lambda i: f"(lq + 4 * {i})")
        self.tlanes = piece_of(low)  # lanes that hold a channel in the CG part (rows of the T tile)
        from .uvu import tuning
        # waves per SIMD: fp64 runs one (512 registers; the register budgets below are in elements, of two
        # registers there). With 32-channel pieces and two waves fp64 was 2.3x slower: half the waves of a
        # block sit out the multiplies and there are four times as many kernels.
        wpe = 2 if self.words == 1 else 1
        self.tune = tuning(dict(uvw_wf=wpe, uvw_wx=wpe, uvw_ww=wpe, uvw_blocks=2, uvw_pipe=1, uvw_regs=220,
                                uvw_merge=1, uvw_fregs=232, uvw_wregs=232, uvw_xregs=215, uvw_mfma_dd=1, uvw_gdma=1,
                                uvw_bf3=0))
        # Forward kernels in the split-operand form (see BF3_TERMS). Off by default: correct to the fp32 bound, but
        # its weight slices take 24 registers per path where the fp32 form takes 16, so config 4's forward becomes
        # four kernels instead of two, and what those cost is their passes over X and Z, not their multiplies
        # (1.09 against 0.90 ms). One kernel over all paths of a tile, with the split weight slices streamed from a
        # buffer instead of living in registers, was tried as well: 1.10 ms, with the matrix pipe busy 18 % and
        # the vector unit 20 % of the time - eleven block barriers per 16-row tile with about 600 cycles of matrix
        # work between them. A third form without LDS or barriers (a wave owns 16 rows and all output channels,
        # lane = (row, 8 input channels): the contraction lands in the A-operand layout in registers; weight
        # slices streamed from L2) took 1.22 ms: 256 registers leave no room to request the next step's operands
        # while the current step is multiplied, so every step waits for its loads.
        self.bf3 = (self.words == 1 and bool(self.tune["uvw_bf3"])
                    and 2 * self.max_d3 * 3 * RT * BF3_ROW * 2 + 2 * RT * low.L2 * 4 <= LDS_BUDGET)

    # Variant of the kernels being written (see second_order_kernels): a name prefix, the kernel signature, the
    # lines that bind the names the bodies use (L1_in, L2_in, W, ...) to its parameters, whether every result is
    # added to what the output holds, and whether the contraction T is that of the second-order pass,
    # T(a, y) + T(x, b), with the second pair of operands bound to L1_alt / L2_alt.
    prefix = ""
    sy, sdy = "s_y", "s_dy[wave]"   # where the dX kernels find the tile's Y rows and leave their partial dY
    alias: List[str] = []
    accumulate = False
    t1 = False

    def lit(self, v):
        return float_literal(v, self.low.ctype)

    # ---- CG part of one path for one (row, channel)
    def _emit_path_fns(self, s: Src):
        low = self.low
        # second operands with several channels: the functions take the offset of the channel's values in the row
        self.multi_v = any(low.in2[p.i2].mul > 1 for p in low.paths)
        yo, yo_par = (" + yo", ", const int yo") if self.multi_v else ("", "")
        for p in low.paths:
            b1, b2, bo = low.in1[p.i1], low.in2[p.i2], low.out[p.io]

            def products(p=p, b2=b2):
                names, out = {}, {}
                for n, (i, j, k, c) in enumerate(p.nnz):
                    key = (self.lit(abs(c)), j)
                    if key not in names:
                        names[key] = f"q{len(names)}"
                        s(f"const T {names[key]} = T({key[0]}) * y[{b2.off + j}{yo}];")
                    out[n] = (names[key], c < 0)
                return out

            # t[k] = sum c x_i y_j
            s.open(f"OEQ_DEV void cg_fwd{p.index}(const T (&x)[{self.max_d1}], const T* y, T (&t)[{bo.d}]{yo_par})")
            prods = products()
            started = set()
            for n, (i, j, k, c) in enumerate(p.nnz):
                q, neg = prods[n]
                if k not in started:
                    s(f"t[{k}] = {'-' if neg else ''}{q} * x[{i}];")
                    started.add(k)
                else:
                    s(f"t[{k}] {'-=' if neg else '+='} {q} * x[{i}];")
            for k in range(bo.d):
                if k not in started:
                    s(f"t[{k}] = T(0);")
            s.close()
            # given G[k] = sum_w W[u,w] dZ[w,k]:  dx_i += c y_j G_k,  dy_j += c x_i G_k
            s.open(
                f"OEQ_DEV void cg_bwd{p.index}(const T (&x)[{self.max_d1}], const T* y, const T (&G)[{bo.d}], "
                f"T (&dx)[{b1.d}], T (&dy)[{low.L2}]{yo_par})"
            )
            prods = products()
            for n, (i, j, k, c) in enumerate(p.nnz):
                q, neg = prods[n]
                s(f"dx[{i}] {'-=' if neg else '+='} {q} * G[{k}];")
            pair = {}
            for n, (i, j, k, c) in enumerate(p.nnz):
                if (i, k) not in pair:
                    pair[(i, k)] = f"xg{len(pair)}"
                    s(f"const T {pair[(i, k)]} = x[{i}] * G[{k}];")
                s(f"dy[{b2.off + j}{yo}] += T({self.lit(c)}) * {pair[(i, k)]};")
            s.close()

    def _prologue(self, s: Src):
        s("const int lane = oeq_lane();")
        s("const int wave = oeq_wave();")
        s("const int l16 = lane & 15, lq = lane >> 4;")
        s("const int tid = (int)threadIdx.x;")
        s(f"const i64 ntiles = (num_batch + {RT - 1}) / {RT};")
        s("(void)tid; (void)lane;")

    def _stage_y(self, s: Src):
        low = self.low
        s.open(f"for (int t = tid; t < {RT * low.L2}; t += {64 * WAVES})")
        s(f"const int r = t / {low.L2}, c = t % {low.L2};")
        s(f"s_y[r][c] = (row0 + r < num_batch) ? L2_in[(row0 + r) * {low.L2} + c] : T(0);")
        if self.t1:
            s(f"s_y2[r][c] = (row0 + r < num_batch) ? L2_alt[(row0 + r) * {low.L2} + c] : T(0);")
        s.close()

    def _tile_stride(self, ncols: int) -> int:
        """Row stride (elements) of an LDS tile with ncols columns: 16 bytes mod 128 when rows can start on
        16-byte boundaries (see ``gstride``), else one element mod 32."""
        want = self.vw if ncols % self.vw == 0 else 1
        stride = ncols + want
        while stride % 32 != want:
            stride += 1
        return stride

    def _stage_g(self, s: Src, col0: int = 0, ncols: int = None, local: bool = False):
        """dZ tile (columns col0 .. col0+ncols) -> LDS, rows past the batch zeroed. All loads of a
        thread are issued before the first LDS store, so their latencies overlap. ``local``: s_g holds
        only those columns (column c of the row at index c - col0)."""
        low = self.low
        ncols = low.L3 if ncols is None else ncols
        dst0 = 0 if local else col0
        nthreads = 64 * WAVES
        VW = self.vw
        if low.L3 % VW == 0 and col0 % VW == 0 and ncols % VW == 0:
            # each wave moves its 4 rows, 64 lanes x 16 bytes at a time: every address is affine in the lane id
            rpw, nc4 = RT // WAVES, ncols // VW
            J = (nc4 + 63) // 64
            # (at most five vectors per row in flight: 80 registers; longer rows in several rounds)
            for j0 in range(0, J, 5):
                js = range(j0, min(J, j0 + 5))
                s.open("")
                s(f"oeq_vec16 gv[{rpw * len(js)}];")
                for phase in ("load", "store"):
                    for rr in range(rpw):
                        for j in js:
                            part = (j + 1) * 64 > nc4
                            cv = f"(lane + {64 * j})"
                            r = f"(wave * {rpw} + {rr})"
                            slot = rr * len(js) + j - j0
                            if phase == "load":
                                cond = f"row0 + {r} < num_batch" + (f" && {cv} < {nc4}" if part else "")
                                s(f"gv[{slot}] = ({cond}) ? *(const oeq_vec16*)(L3_grad + (row0 + {r}) * {low.L3} + "
                                  f"{col0} + {VW} * {cv}) : oeq_vec16(T(0));")
                            else:
                                guard = f"if ({cv} < {nc4}) " if part else ""
                                s(f"{guard}*(oeq_vec16*)&s_g[{r}][{dst0} + {VW} * {cv}] = gv[{slot}];")
                s.close()
        else:
            s.open(f"for (int t = tid; t < {RT * ncols}; t += {nthreads})")
            s(f"const int r = t / {ncols}, c = t % {ncols};")
            s(f"s_g[r][{dst0} + c] = (row0 + r < num_batch) ? L3_grad[(row0 + r) * {low.L3} + {col0} + c] : T(0);")
            s.close()

    def _dma_g(self, s: Src, tile: str, buf: str):
        """The dZ tile of ``tile`` -> s_g[buf] by direct global-to-LDS loads (no registers, nothing to wait for
        here): every wave moves its 4 rows, 64 lanes x 16 bytes per instruction to consecutive LDS addresses.
        Rows past the batch read the last row (the dX kernels sum nothing over rows, and store nothing for them).
        Only whole instructions go that way. The rest of a row (fewer than 64 vectors) is loaded into ``gtail``
        here and stored by ``_put_g_tail``: a direct load under a lane condition sits in divergent control flow, and
        there one compiler version (the hiprtc of ROCm 7.2) has been seen to merge it with the next row's direct load
        into one instruction whose LDS base is taken from the first active lane - a float64 problem with 65 vectors
        per row then got wrong sender gradients."""
        low = self.low
        VW, rpw = self.vw, RT // WAVES
        nc4 = low.L3 // VW
        s.open("")
        s(f"const i64 nrow0 = ({tile}) * {RT};")
        for rr in range(rpw):
            s.open("")
            s(f"i64 row = nrow0 + wave * {rpw} + {rr}; if (row >= num_batch) row = num_batch - 1;")
            s(f"const T* src = L3_grad + row * {low.L3};")
            for j in range(nc4 // 64):
                s(f"__builtin_amdgcn_global_load_lds((const OEQ_GPTR)(src + {VW} * (lane + {64 * j})), "
                  f"(OEQ_LPTR)&s_g[{buf}][wave * {rpw} + {rr}][{VW * 64 * j}], 16, 0, 0);")
            if nc4 % 64:
                jt = nc4 // 64
                s(f"gtail[{rr}] = (lane + {64 * jt} < {nc4}) ? *(const oeq_vec16*)(src + {VW} * (lane + {64 * jt})) : "
                  f"oeq_vec16(T(0));")
            s.close()
        s.close()

    def _put_g_tail(self, s: Src, buf: str):
        """The part of the tile's rows that ``_dma_g`` left in registers -> s_g[buf]."""
        VW, rpw = self.vw, RT // WAVES
        nc4 = self.low.L3 // VW
        if nc4 % 64:
            jt = nc4 // 64
            for rr in range(rpw):
                s(f"if (lane + {64 * jt} < {nc4}) *(oeq_vec16*)&s_g[{buf}][wave * {rpw} + {rr}][{VW} * (lane + {64 * jt})] = "
                  f"gtail[{rr}];")

    def _y_regs(self) -> int:
        return (RT * self.low.L2 + 64 * WAVES - 1) // (64 * WAVES)

    def _load_flat_rows(self, s: Src, dst: str, src: str, row0: str):
        """dst[q] = element tid + 256 q of the [16, L2] tile of ``src`` that starts at row ``row0`` (zero past the
        batch)."""
        L2 = self.low.L2
        for q in range(self._y_regs()):
            t = f"(tid + {64 * WAVES * q})"
            inside = f"{t} < {RT * L2} && " if (q + 1) * 64 * WAVES > RT * L2 else ""
            s(f"{dst}[{q}] = ({inside}({row0}) * {L2} + {t} < num_batch * {L2}) ? {src}[({row0}) * {L2} + {t}] : T(0);")

    def _load_x_rows(self, s: Src, dst: str, vp: VPath):
        """X of the wave's 4 rows for a sub-path, lanes = channel u of its input piece (T-compute layout);
        lanes beyond the piece read its last channel (their T values are never multiplied)."""
        low = self.low
        a = self.vin[vp.vi]
        lane = "lane" if a.mul == 64 else f"(lane < {a.mul} ? lane : {a.mul - 1})"
        s.open(f"for (int rr = 0; rr < {RT // WAVES}; ++rr)")
        s(f"i64 row = row0 + wave * {RT // WAVES} + rr; if (row >= num_batch) row = num_batch - 1;")
        s(f"const T* xp = L1_in + row * {low.L1} + {a.off} + {lane} * {a.d};")
        for i in range(a.d):
            s(f"{dst}[rr][{i}] = xp[{i}];")
        if self.t1:
            s(f"const T* ap = L1_alt + row * {low.L1} + {a.off} + {lane} * {a.d};")
            for i in range(a.d):
                s(f"a{dst[1:]}[rr][{i}] = ap[{i}];")
        s.close()

    def _t_compute(self, s: Src, vp: VPath, xsrc: str, buf: str):
        d3 = self.vout[vp.vo].d
        yo = f", {vp.v * self.low.in2[vp.p.i2].d}" if self.multi_v else ""
        s.open(f"for (int rr = 0; rr < {RT // WAVES}; ++rr)")
        s(f"const int r = wave * {RT // WAVES} + rr;")
        s(f"T t[{d3}];")
        if self.t1:
            # contraction of the second-order pass: (a, y) and (x, b)
            s(f"T t2[{d3}];")
            s(f"cg_fwd{vp.p.index}(a{xsrc[1:]}[rr], s_y[r], t{yo});")
            s(f"cg_fwd{vp.p.index}({xsrc}[rr], s_y2[r], t2{yo});")
            for k in range(d3):
                s(f"t[{k}] += t2[{k}];")
        else:
            s(f"cg_fwd{vp.p.index}({xsrc}[rr], s_y[r], t{yo});")
        if self.tlanes < 64:
            s.open(f"if (lane < {self.tlanes})")
        for k in range(d3):
            # (rows of channels beyond the piece are multiplied, with zero weights: they hold zeros, not copies)
            val = f"t[{k}]" if vp.U % 16 == 0 else f"(lane < {vp.U} ? t[{k}] : T(0))"
            s(f"s_T[{buf}][{k}][lane][r] = {val};")
        if self.tlanes < 64:
            s.close()
        s.close()

    def _t_compute_bf3(self, s: Src, vp: VPath, xsrc: str, buf: str, by_row: bool):
        """The contraction T of a sub-path for the wave's 4 rows, lanes = channel u, split into three bf16 parts and
        written to the operand planes s_Tb[buf][k][part]: ``by_row`` [row][channel] (A operand of the forward
        multiply: 8 consecutive channels per lane), else [channel][row] (A operand of the dW multiply: 8 consecutive
        rows). Two rows share every split (the conversions are packed)."""
        d3 = self.vout[vp.vo].d
        yo = f", {vp.v * self.low.in2[vp.p.i2].d}" if self.multi_v else ""
        rpw = RT // WAVES
        s.open("")
        s(f"T t[{rpw}][{d3}];")
        s.open(f"for (int rr = 0; rr < {rpw}; ++rr)")
        s(f"const int r = wave * {rpw} + rr;")
        if self.t1:
            s(f"T t2[{d3}];")
            s(f"cg_fwd{vp.p.index}(a{xsrc[1:]}[rr], s_y[r], t[rr]{yo});")
            s(f"cg_fwd{vp.p.index}({xsrc}[rr], s_y2[r], t2{yo});")
            for k in range(d3):
                s(f"t[rr][{k}] += t2[{k}];")
        else:
            s(f"cg_fwd{vp.p.index}({xsrc}[rr], s_y[r], t[rr]{yo});")
        s.close()
        for k in range(d3):
            if by_row:
                for rp in range(rpw // 2):
                    va, vb = f"t[{2 * rp}][{k}]", f"t[{2 * rp + 1}][{k}]"
                    if vp.U < 64:
                        # (channels beyond the piece are multiplied, with zero weights: they hold zeros)
                        va, vb = f"(lane < {vp.U} ? {va} : T(0))", f"(lane < {vp.U} ? {vb} : T(0))"
                    s(f"{{ unsigned q0, q1, q2; oeq_split2({va}, {vb}, q0, q1, q2);")
                    for c in range(3):
                        s(f"  s_Tb[{buf}][{k}][{c}][wave * {rpw} + {2 * rp}][lane] = (unsigned short)q{c}; "
                          f"s_Tb[{buf}][{k}][{c}][wave * {rpw} + {2 * rp + 1}][lane] = (unsigned short)(q{c} >> 16);")
                    s("}")
            else:
                assert rpw == 4
                s(f"{{ unsigned q0, q1, q2, h0, h1, h2; oeq_split2(t[0][{k}], t[1][{k}], q0, q1, q2); "
                  f"oeq_split2(t[2][{k}], t[3][{k}], h0, h1, h2);")
                for c in range(3):
                    s(f"  *(uint2*)&s_Tb[{buf}][{k}][{c}][lane][wave * {rpw}] = uint2{{q{c}, h{c}}};")
                s("}")
        s.close()

    def _load_wb_forward(self, s: Src, vps: List[VPath], act: str):
        """Weight slices of the forward multiply as bf16 B operands, split in three: for every 32 input channels
        u' = 32 step + 8 (lane / 16) + i and the lane's output channel w = 16 wave + lane % 16, W[u'][w]."""
        for vp in vps:
            steps = (vp.U + 31) // 32
            s(f"oeq_bf8 wb{vp.index}[{steps}][3];")
            s.open("")
            for st in range(steps):
                s("{ float wv[8];")
                for i in range(8):
                    conds = [act]
                    if 32 * st + 8 * 3 + i >= vp.U:
                        conds.append(f"{32 * st} + 8 * lq + {i} < {vp.U}")
                    if vp.Wn % 16:
                        conds.append(f"wave * 16 + l16 < {vp.Wn}")
                    s(f"  wv[{i}] = ({' && '.join(conds)}) ? W[{vp.woff} + ({32 * st} + 8 * lq + {i}) * {vp.ld} + wave * 16 + l16] : 0.0f;")
                s("  unsigned q0[4], q1[4], q2[4];")
                for j in range(4):
                    s(f"  oeq_split2(wv[{2 * j}], wv[{2 * j + 1}], q0[{j}], q1[{j}], q2[{j}]);")
                for c in range(3):
                    s(f"  wb{vp.index}[{st}][{c}] = __builtin_bit_cast(oeq_bf8, oeq_u4{{q{c}[0], q{c}[1], q{c}[2], q{c}[3]}});")
                s("}")
            s.close()

    def _dx_paths(self, s: Src, paths: List[VPath], x: str = "x", dx: str = "dx"):
        """G = dZ W^T of every sub-path on the matrix cores, then its CG part on the vector ALU (in scope:
        x, dx, dy, s_g, s_y, wreg<path>). ``uvw_pipe`` = 0: path after path, operand order left to the
        compiler. 1: the A operands (dZ values from LDS) are fetched one chunk of 4 k-steps ahead of the
        multiplies that use them, and nothing moves across a chunk boundary: left alone, the compiler hoists
        the LDS reads of several paths and spills the weight slices."""
        pipe = self.tune["uvw_pipe"]
        CH = 4

        def cg_rows(vp, G):
            d3 = self.vout[vp.vo].d
            s("#pragma unroll")
            s.open("for (int i = 0; i < 4; ++i)")
            s(f"T Gk[{d3}];")
            for k in range(d3):
                s(f"Gk[{k}] = {G}[{k}][i];")
            yo = f", {vp.v * self.low.in2[vp.p.i2].d}" if self.multi_v else ""
            s(f"cg_bwd{vp.p.index}({x}[i], {self.sy}[{self.row('i')}], Gk, {dx}[i], dy[i]{yo});")
            s.close()

        if pipe == 0:
            for vp in paths:
                bo = self.vout[vp.vo]
                s(f"// path {vp.p.index}, output piece {vp.wb}")
                s.open("")
                # G[k] = sum_w dZ[(r,k), w] * W[u, w]   (A = dZ tile, B = W^T slice in registers)
                s(f"v4t G[{bo.d}];")
                for k in range(bo.d):
                    s(f"G[{k}] = v4t{{}};")
                s("#pragma unroll")
                s.open(f"for (int st = 0; st < {c4(vp.Wn)}; ++st)")
                wcol = "(4 * st + lq)" if vp.Wn % 4 == 0 else f"min(4 * st + lq, {vp.Wn - 1})"
                for k in range(bo.d):
                    s(f"G[{k}] = {MFMA}({self.g_at('l16', f'{bo.off} + {wcol} * {bo.d} + {k}')}, "
                      f"wreg{vp.index}[st], G[{k}], 0, 0, 0);")
                s.close()
                cg_rows(vp, "G")
                s.close()
            return
        maxd = max(self.vout[vp.vo].d for vp in paths)
        s(f"T opa[{CH * maxd}], opb[{CH * maxd}];  // A operands of the current and the next chunk")
        if self.lds_w:
            s(f"T wla[{CH}], wlb[{CH}];  // B operands of a path whose weight slice is kept in LDS")
        s(f"v4t G[{maxd}];")
        segs = [(n, c) for n, vp in enumerate(paths) for c in range(c16(vp.Wn))]

        def reads(seg, buf):
            n, c = seg
            bo = self.vout[paths[n].vo]
            for q in range(CH):
                w0 = 4 * (c * CH + q)
                # (columns past the piece meet zero weights; they are read from its last column, which holds
                # finite values, not from whatever lies behind the row)
                wcol = f"({w0} + lq)" if w0 + 4 <= paths[n].Wn else f"min({w0} + lq, {paths[n].Wn - 1})"
                for k in range(bo.d):
                    s(f"{buf}[{q * bo.d + k}] = {self.g_at('l16', f'{bo.off} + {wcol} * {bo.d} + {k}')};")
            if paths[n].index in self.lds_w:
                slot = self.lds_w.index(paths[n].index)
                for q in range(CH):
                    s(f"{'wla' if buf == 'opa' else 'wlb'}[{q}] = s_wl[{slot}][{c * CH + q}][tid];")

        reads(segs[0], "opa")
        for t, (n, c) in enumerate(segs):
            vp = paths[n]
            bo = self.vout[vp.vo]
            cur, nxt = ("opa", "opb") if t % 2 == 0 else ("opb", "opa")
            if c == 0:
                s(f"// path {vp.p.index}, output piece {vp.wb}")
                for k in range(bo.d):
                    s(f"G[{k}] = v4t{{}};")
            if t + 1 < len(segs):
                reads(segs[t + 1], nxt)
            for q in range(CH):
                wop = (f"{'wla' if cur == 'opa' else 'wlb'}[{q}]" if vp.index in self.lds_w
                       else f"wreg{vp.index}[{c * CH + q}]")
                for k in range(bo.d):
                    s(f"G[{k}] = {MFMA}({cur}[{q * bo.d + k}], {wop}, G[{k}], 0, 0, 0);")
            s("__builtin_amdgcn_sched_barrier(0);")
            if c == c16(vp.Wn) - 1:
                cg_rows(vp, "G")

    def _reduce_dy(self, s: Src):
        """Sum of dy[i][j] (4 rows x L2 values per lane) over the 16 lanes of a lane group, into
        s_dy[wave][row][j]. Each step pairs every lane with one partner through a DPP lane permutation
        (mirror of the 16, mirror of each 8, mirror of each quad, neighbour); a lane keeps one half of its
        values and adds the partner's copies of that half, so the count of values halves with the count of
        lanes that hold them: 45 permuted adds instead of four per value."""
        low = self.low
        n = 4 * low.L2
        cur = (n + 15) // 16 * 16
        s.open("")
        s(f"T rv[{cur}];")
        for o in range(cur):
            s(f"rv[{o}] = {f'dy[{o // low.L2}][{o % low.L2}]' if o < n else 'T(0)'};")
        s("int at = 0;  // index of rv[0] in the lane group's value list")
        for ctrl, bit in (("0x140", 8), ("0x141", 4), ("0x1B", 2), ("0xB1", 1)):
            half = cur // 2
            s.open("")
            s(f"const bool hi = (l16 & {bit}) != 0;")
            for j in range(half):
                s(f"{{ const T keep = hi ? rv[{j + half}] : rv[{j}]; const T send = hi ? rv[{j}] : rv[{j + half}]; "
                  f"rv[{j}] = keep + oeq_dpp<{ctrl}>(send); }}")
            s(f"at += hi ? {half} : 0;")
            s.close()
            cur = half
        for t in range(cur):
            s(f"if (at + {t} < {n}) {self.sdy}[{self.row(f'((at + {t}) / {low.L2})')}][(at + {t}) % {low.L2}] = rv[{t}];")
        s.close()

    # ------------------------------------------------------------- forward
    def _load_wreg(self, s: Src, vps: List[VPath], transposed: bool, act: str = "act", u: str = "u"):
        """Weight slices in MFMA B-operand layout, 1 register per 4 k-steps... per k-step of 4: forward
        B[k = u' = 4 st + lq][n = l16] = W[u'][w = 16 wave + l16] (U / 4 registers); backward (transposed)
        B[k = w = 4 st + lq][n = l16] = W[u][w] (Wn / 4 registers). Waves without channels in the piece load
        nothing (``act`` is in scope)."""
        for vp in vps:
            # (k-steps and channels beyond the corner of the weight matrix: zeros)
            n = 4 * c16(vp.Wn) if transposed else c4(vp.U)
            s(f"T wreg{vp.index}[{n}];")
            s("#pragma unroll")
            if transposed:
                cond = act if vp.Wn % 16 == 0 else f"({act} && 4 * st + lq < {vp.Wn})"
                s(f"for (int st = 0; st < {n}; ++st) wreg{vp.index}[st] = {cond} ? "
                  f"W[{vp.woff} + {u} * {vp.ld} + 4 * st + lq] : T(0);")
            else:
                more = ("" if vp.U % 4 == 0 else f" && 4 * st + lq < {vp.U}") + \
                    ("" if vp.Wn % 16 == 0 else f" && wave * 16 + l16 < {vp.Wn}")
                cond = f"({act}{more})" if more else act
                s(f"for (int st = 0; st < {n}; ++st) wreg{vp.index}[st] = {cond} ? "
                  f"W[{vp.woff} + (4 * st + lq) * {vp.ld} + wave * 16 + l16] : T(0);")

    FWD_SIG = ("(i64 num_batch, const T* __restrict__ L1_in, const T* __restrict__ L2_in, "
               "const T* __restrict__ W, T* __restrict__ L3_out)")
    BWD_SIG = ("(i64 num_batch, const T* __restrict__ L1_in, T* __restrict__ L1_grad, "
               "const T* __restrict__ L2_in, T* __restrict__ L2_grad, const T* __restrict__ W, "
               "T* __restrict__ W_grad, const T* __restrict__ L3_grad, T* __restrict__ wpartial)")

    def _kernel_open(self, s: Src, name: str, sig: str, waves_per_eu: int = 0):
        attr = f"__launch_bounds__({64 * WAVES})"
        if waves_per_eu:
            attr += f" __attribute__((amdgpu_waves_per_eu({waves_per_eu}, {waves_per_eu})))"
        s.open(f'extern "C" __global__ {attr} void {name}{sig}')
        for line in self.alias:
            s(line)

    def _zero_kernel(self, s: Src, ptr: str, row_len: int, blk: VBlock):
        """A piece that no path touches: zeros."""
        self._prologue(s)
        s.open("for (i64 tile = blockIdx.x; tile < ntiles; tile += gridDim.x)")
        s(f"const i64 row0 = tile * {RT};")
        s.open(f"for (int t = tid; t < {RT * blk.mul * blk.d}; t += {64 * WAVES})")
        s(f"const int r = t / {blk.mul * blk.d}, c = t % {blk.mul * blk.d};")
        s(f"if (row0 + r < num_batch) {ptr}[(row0 + r) * {row_len} + {blk.off} + c] = T(0);")
        s.close()
        s.close()
        s.close()

    def _merge(self, groups, cost, limit, blocks):
        """Consecutive (piece, sub-paths, first) groups that share a kernel: a group joins the kernel before
        it while the kernel's estimated registers stay within ``limit``. Kernels of narrow output irreps
        (l = 0: one multiply per k-step) are dominated by what every kernel pays per tile - staging, barriers,
        the X loads - so they ride along with a neighbour. Groups without paths stay alone."""
        kernels = []
        for g in groups:
            prev = kernels[-1][-1] if kernels else None
            # only neighbours in the row share a kernel (one dZ tile then covers their columns)
            adjacent = prev is not None and prev[0] != g[0] and \
                blocks[prev[0]].off + blocks[prev[0]].mul * blocks[prev[0]].d == blocks[g[0]].off
            if adjacent and g[1] and prev[1] and self.tune["uvw_merge"] and cost(kernels[-1] + [g]) <= limit:
                kernels[-1].append(g)
            else:
                kernels.append([g])
        return kernels

    def emit_forward(self, s: Src) -> List[str]:
        """Kernels per piece of an output irrep and piece index of the input side (launched back to back;
        pieces with few paths share a kernel), so that only the weight slices of the sub-paths it multiplies
        are resident and register allocation is per kernel. Returns the kernel names in launch order."""
        low = self.low
        names = []
        # (the summed contraction of the second-order pass holds the rows of two operand pairs)
        xrows = (2 if self.t1 else 1) * 2 * (RT // WAVES) * self.max_d1
        cost = lambda ker: (sum(_slice_regs(vp, "forward", self.bf3) for g in ker for vp in g[1])
                            + sum(4 * self.vout[g[0]].d for g in ker) + xrows + 64)
        # (what the accumulators, the X rows and the rest leave for weight slices, at least two 64-channel slices)
        limit = lambda vo, sub: max(32, self.tune["uvw_fregs"] - (4 * self.vout[vo].d + xrows + 64))
        for ker in self._merge(_groups(self.vpaths, "vo", len(self.vout), "forward", limit, self.bf3), cost,
                               self.tune["uvw_fregs"], self.vout):
            vo0, order0, _ = ker[0]
            if not order0 and self.accumulate:
                continue  # nothing to add to a piece no path writes
            name = (self.prefix + "forward") if not names else f"{self.prefix}forward_o{vo0}_{order0[0].tag('vo') if order0 else 0}"
            names.append(name)
            s("// ======== out pieces " + ", ".join(f"{vo}: {self.vout[vo].mul} x l={self.vout[vo].l}" for vo, _, _ in ker))
            self._kernel_open(s, name, self.sig_f, self.tune["uvw_wf"])
            if not order0:
                self._zero_kernel(s, "L3_out", low.L3, self.vout[vo0])
                continue
            maxd = max(self.vout[vo].d for vo, _, _ in ker)
            if self.bf3:
                s(f"__shared__ __attribute__((aligned(16))) unsigned short s_Tb[2][{maxd}][3][{RT}][{BF3_ROW}];")
            else:
                s(f"__shared__ T s_T[2][{maxd}][{self.tlanes}][{TPAD}];")
            s(f"__shared__ T s_y[{RT}][{low.L2}];")
            if self.t1:
                s(f"__shared__ T s_y2[{RT}][{low.L2}];")
            self._prologue(s)
            s(f"T xa[{RT // WAVES}][{self.max_d1}], xb[{RT // WAVES}][{self.max_d1}];")
            if self.t1:
                s(f"T aa[{RT // WAVES}][{self.max_d1}], ab[{RT // WAVES}][{self.max_d1}];")
            for vo, order, _ in ker:
                s(f"const bool act{vo} = wave * 16 < {self.vout[vo].mul};  // this wave has output channels in the piece")
            order_all = [vp for _, order, _ in ker for vp in order]
            for vo, order, _ in ker:
                if self.bf3:
                    self._load_wb_forward(s, order, f"act{vo}")
                else:
                    self._load_wreg(s, order, transposed=False, act=f"act{vo}")
            s.open("for (i64 tile = blockIdx.x; tile < ntiles; tile += gridDim.x)")
            s(f"const i64 row0 = tile * {RT};")
            s("__syncthreads();  // all reads of the previous tile's LDS data are done")
            self._stage_y(s)
            self._load_x_rows(s, "xa", order_all[0])
            s("__syncthreads();")
            for vo, _, _ in ker:
                s(f"v4t acc{vo}[{self.vout[vo].d}];")
                for k in range(self.vout[vo].d):
                    s(f"acc{vo}[{k}] = v4t{{}};")
            cur, nxt = "xa", "xb"
            for n, vp in enumerate(order_all):
                buf = n % 2
                p = vp.p
                bo = self.vout[vp.vo]
                s(f"// path {p.index}: l=({low.in1[p.i1].l},{low.in2[p.i2].l},{bo.l}), input piece {vp.ub}")
                if self.bf3:
                    self._t_compute_bf3(s, vp, cur, str(buf), by_row=True)
                else:
                    self._t_compute(s, vp, cur, str(buf))
                if n + 1 < len(order_all):
                    self._load_x_rows(s, nxt, order_all[n + 1])
                s("__syncthreads();")
                s.open(f"if (act{vp.vo})")
                if self.bf3:
                    for st in range((vp.U + 31) // 32):
                        for k in range(bo.d):
                            s.open("")
                            for c in range(3):
                                s(f"const oeq_bf8 a{c} = *(const oeq_bf8*)&s_Tb[{buf}][{k}][{c}][l16][{32 * st} + 8 * lq];")
                            for ca, cb in BF3_TERMS:
                                s(f"acc{vp.vo}[{k}] = oeq_mfma_bf(a{ca}, wb{vp.index}[{st}][{cb}], acc{vp.vo}[{k}], 0, 0, 0);")
                            s.close()
                else:
                    s("#pragma unroll")
                    s.open(f"for (int st = 0; st < {c4(vp.U)}; ++st)")
                    for k in range(bo.d):
                        s(f"acc{vp.vo}[{k}] = {MFMA}(s_T[{buf}][{k}][4 * st + lq][l16], wreg{vp.index}[st], "
                          f"acc{vp.vo}[{k}], 0, 0, 0);")
                    s.close()
                s.close()
                cur, nxt = nxt, cur
            # D layout: rows 4*lq + i, column (channel) l16 of the wave's slice
            for vo, _, first in ker:
                bo = self.vout[vo]
                s("#pragma unroll")
                s.open("for (int i = 0; i < 4; ++i)")
                s(f"const i64 row = row0 + {self.row('i')};")
                wok = "" if bo.mul % 16 == 0 else f" && wave * 16 + l16 < {bo.mul}"
                s.open(f"if (act{vo} && row < num_batch{wok})")
                s(f"T* zp = L3_out + row * {low.L3} + {bo.off} + (wave * 16 + l16) * {bo.d};")
                for k in range(bo.d):
                    s(f"zp[{k}] {'=' if first and not self.accumulate else '+='} acc{vo}[{k}][i];")
                s.close()
                s.close()
            s.close()
            s.close()
        return names

    # ------------------------------------------------------------ backward
    sig_f = FWD_SIG
    sig_b = BWD_SIG

    def emit_backward(self, s: Src, parts=("dx", "dw")) -> List[str]:
        """Kernels per piece of an input irrep (dX of the piece and the dY contributions of its sub-paths)
        and per piece of an output irrep (dW of the sub-paths feeding it), launched back to back. A tile is
        always handled by the same block and thread, so what successive kernels add to dY (and to dX, with
        several output pieces) arrives in a fixed order with plain read-modify-writes. Returns the names."""
        low = self.low
        names = []
        # ---------------- dX, dY ------------------------------------------------
        first_dy = True
        # registers per lane: one per 4 k-steps of a resident weight slice, the 4 rows' x / dx per piece, dy, G
        # and the operand chunks
        fixed = lambda ker: (sum(8 * self.vin[g[0]].d for g in ker) + 4 * low.L2
                             + 6 * max(self.vout[vp.vo].d for g in ker for vp in g[1]) + 48)
        cost = lambda ker: sum(4 * c16(vp.Wn) for g in ker for vp in g[1]) + fixed(ker)
        # (a slice of the kernel may live in LDS instead: 16 registers' worth; more of them, which the kernels
        # below still allow, cost more in operand traffic than a kernel more)
        limit = lambda vi, sub: max(32, self.tune["uvw_regs"] + 16 - (
            8 * self.vin[vi].d + 4 * low.L2 + 6 * max(self.vout[vp.vo].d for vp in sub) + 48))
        dx_kernels = self._merge(_groups(self.vpaths, "vi", len(self.vin), "dx", limit), cost, self.tune["uvw_xregs"],
                                 self.vin)
        for ker in (dx_kernels if "dx" in parts else []):
            vi0, paths0, _ = ker[0]
            if not paths0 and self.accumulate:
                continue  # nothing to add to a piece no path reads
            name = (self.prefix + "backward") if not names else f"{self.prefix}backward_x{vi0}_{paths0[0].tag('vi') if paths0 else 0}"
            names.append(name)
            s("// ======== in1 pieces " + ", ".join(f"{vi}: {self.vin[vi].mul} x l={self.vin[vi].l}" for vi, _, _ in ker))
            self._kernel_open(s, name, self.sig_b, self.tune["uvw_wx"])
            if not paths0:
                self._zero_kernel(s, "L1_grad", low.L1, self.vin[vi0])
                continue
            paths_all = [vp for _, ps, _ in ker for vp in ps]
            uok = lambda vi: f"act{vi}" if self.vin[vi].mul % 16 == 0 else f"uok{vi}"
            self._prologue(s)
            for vi, _, _ in ker:
                s(f"const bool act{vi} = wave * 16 < {self.vin[vi].mul};  // this wave has input channels in the piece")
                if self.vin[vi].mul % 16 == 0:
                    s(f"const int u{vi} = act{vi} ? wave * 16 + l16 : 0;  // channel of this lane in the MFMA result layout")
                else:
                    # lanes past the piece's channels compute on channel 0 with zero weights and store nothing
                    s(f"const bool uok{vi} = wave * 16 + l16 < {self.vin[vi].mul};")
                    s(f"const int u{vi} = uok{vi} ? wave * 16 + l16 : 0;  // channel of this lane in the MFMA result layout")
            # Where the registers exceed the budget of two waves per SIMD, the weight slices of the paths with
            # the fewest multiplies are kept in LDS instead (read like the A operands, one chunk ahead): spilled
            # slices would come back from scratch memory in the middle of the multiply sequence.
            by_cost = sorted(paths_all, key=lambda vp: (self.vout[vp.vo].d, vp.index))
            self.lds_w = []
            if self.tune["uvw_pipe"]:
                resident = lambda: sum(4 * c16(vp.Wn) for vp in paths_all if vp.index not in self.lds_w)
                # (what LDS has room for beside the dZ tile: a slice takes 16 x 256 elements)
                room = (LDS_BUDGET - (RT * self.gstride + (1 + WAVES) * RT * low.L2) * low.elem_size) // \
                    (16 * 64 * WAVES * low.elem_size)
                while len(paths_all) - len(self.lds_w) > 1 and len(self.lds_w) < min(3, room) and \
                        resident() + fixed(ker) > self.tune["uvw_regs"]:
                    self.lds_w.append(by_cost[len(self.lds_w)].index)
            if self.lds_w:
                s(f"__shared__ T s_wl[{len(self.lds_w)}][16][{64 * WAVES}];")
            # Two copies of the tile's LDS data (dZ, Y, partial dY), where two blocks per CU still fit (80 KB each):
            # the next tile's dZ arrives by direct global-to-LDS loads while this one is multiplied, its Y through
            # registers, and the partial dY of a tile are summed after the next tile's barrier, so a tile costs one
            # barrier. Else one copy, staged through registers, three barriers per tile.
            lds_two = 2 * (RT * self.gstride + (1 + WAVES) * RT * low.L2) * low.elem_size + \
                len(self.lds_w) * 16 * 64 * WAVES * low.elem_size
            # (rows of whole 64-vector instructions, or rows shorter than one, which then travel through registers
            # like Y and still gain from the single barrier: DiffDock 0.54 -> 0.49 ms, e3tools 0.60 -> 0.54. Rows
            # with whole instructions and a rest keep the one-copy form: with the rest in registers config 4's kernels
            # spill and lose what the direct loads gain, 1.95 against 1.85 ms.)
            nvec = low.L3 // self.vw
            dma = (bool(self.tune["uvw_gdma"]) and low.L3 % self.vw == 0 and lds_two <= 80 * 1024 and not self.t1
                   and (nvec % 64 == 0 or nvec < 64))
            if dma:
                self.g_at = lambda row, col: f"s_g[gb][{row}][{col}]"
                self.sy, self.sdy = "s_y[gb]", "s_dy[gb][wave]"
                s(f"__shared__ __attribute__((aligned(16))) T s_g[2][{RT}][{self.gstride}];")
                s(f"__shared__ T s_y[2][{RT}][{low.L2}];")
                s(f"__shared__ T s_dy[2][{WAVES}][{RT}][{low.L2}];")
            else:
                self.g_at = lambda row, col: f"s_g[{row}][{col}]"
                self.sy, self.sdy = "s_y", "s_dy[wave]"
                s(f"__shared__ __attribute__((aligned(16))) T s_g[{RT}][{self.gstride}];")
                s(f"__shared__ T s_y[{RT}][{low.L2}];")
                s(f"__shared__ T s_dy[{WAVES}][{RT}][{low.L2}];")
            for vi, ps, _ in ker:
                self._load_wreg(s, [vp for vp in ps if vp.index not in self.lds_w], transposed=True,
                                act=uok(vi), u=f"u{vi}")
            for n, pi in enumerate(self.lds_w):
                vp = next(q for q in paths_all if q.index == pi)
                s("#pragma unroll")
                wcond = "" if vp.Wn % 16 == 0 else f" && 4 * st + lq < {vp.Wn}"
                cond = f"({uok(vp.vi)}{wcond})" if wcond else uok(vp.vi)
                s(f"for (int st = 0; st < {4 * c16(vp.Wn)}; ++st) s_wl[{n}][st][tid] = "
                  f"{cond} ? W[{vp.woff} + u{vp.vi} * {vp.ld} + 4 * st + lq] : T(0);")
            rmw_dy = not (first_dy and not self.accumulate)
            ny = self._y_regs()
            if dma:
                # first tile: dZ on its way to copy 0, Y through registers
                def put_y(buf):
                    for q in range(ny):
                        guard = f"if (tid + {64 * WAVES * q} < {RT * low.L2}) " if (q + 1) * 64 * WAVES > RT * low.L2 else ""
                        s(f"{guard}(&s_y[{buf}][0][0])[tid + {64 * WAVES * q}] = ynext[{q}];")

                def finish_dy(buf):
                    """dY of the tile before (rows from prow0): the four waves' partial sums, in wave order, on top
                    of what the earlier kernels left there."""
                    for q in range(ny):
                        tq = f"(tid + {64 * WAVES * q})"
                        inside = f"{tq} < {RT * low.L2} && " if (q + 1) * 64 * WAVES > RT * low.L2 else ""
                        s.open(f"if ({inside}prow0 * {low.L2} + {tq} < num_batch * {low.L2})")
                        s(f"const int r = {tq} / {low.L2}, c = {tq} % {low.L2};")
                        s(f"const T tot = ((s_dy[{buf}][0][r][c] + s_dy[{buf}][1][r][c]) + s_dy[{buf}][2][r][c]) + "
                          f"s_dy[{buf}][3][r][c];")
                        s(f"L2_grad[prow0 * {low.L2} + {tq}] = {f'dyold[{q}] + tot' if rmw_dy else 'tot'};")
                        s.close()

                s("int gb = 0;")
                s("i64 prow0 = -1;  // first row of the tile whose dY is still to be written")
                s(f"T ynext[{ny}];")
                if (low.L3 // self.vw) % 64:
                    s(f"oeq_vec16 gtail[{RT // WAVES}];")
                if rmw_dy:
                    s(f"T dyold[{ny}];")
                s.open("if ((i64)blockIdx.x < ntiles)")
                self._dma_g(s, "(i64)blockIdx.x", "0")
                self._load_flat_rows(s, "ynext", "L2_in", f"(i64)blockIdx.x * {RT}")
                put_y("0")
                self._put_g_tail(s, "0")
                s.close()
                s.open("for (i64 tile = blockIdx.x; tile < ntiles; tile += gridDim.x, gb ^= 1)")
                s(f"const i64 row0 = tile * {RT};")
                # This tile's dZ has landed (each wave waits for its own loads, the barrier for everybody's) and its
                # Y rows are written; the waves' partial dY of the tile before are complete; all reads of the other
                # copies (two tiles back) are done.
                s('asm volatile("s_waitcnt vmcnt(0)" ::: "memory");')
                s("__syncthreads();")
                s('asm volatile("" ::: "memory");')
                s("const bool more = tile + gridDim.x < ntiles;")
                s.open("if (prow0 >= 0)")
                finish_dy("gb ^ 1")
                s.close()
                s("prow0 = row0;")
            else:
                s.open("for (i64 tile = blockIdx.x; tile < ntiles; tile += gridDim.x)")
                s(f"const i64 row0 = tile * {RT};")
                s("__syncthreads();")
                self._stage_g(s)
                self._stage_y(s)
            # X of the lane's 4 (row, channel) pairs: issued before the barrier and the MFMA loop
            s(f"T dy[4][{low.L2}];")
            for vi, _, _ in ker:
                s(f"T x{vi}[4][{self.max_d1}], dx{vi}[4][{self.vin[vi].d}];")
            s("#pragma unroll")
            s.open("for (int i = 0; i < 4; ++i)")
            s(f"i64 row = row0 + {self.row('i')}; if (row >= num_batch) row = num_batch - 1;")
            for vi, _, _ in ker:
                b1 = self.vin[vi]
                s.open("")
                s(f"const T* xp = L1_in + row * {low.L1} + {b1.off} + u{vi} * {b1.d};")
                for c in range(b1.d):
                    s(f"x{vi}[i][{c}] = xp[{c}]; dx{vi}[i][{c}] = T(0);")
                s.close()
            s(f"for (int j = 0; j < {low.L2}; ++j) dy[i][j] = T(0);")
            s.close()
            if not dma:
                s("__syncthreads();")
            else:
                # Requested after the X rows: loads return in order, so the wait for X does not include these.
                if rmw_dy:
                    # what the earlier kernels left in this tile's dY
                    self._load_flat_rows(s, "dyold", "L2_grad", "row0")
                s.open("if (more)")
                self._load_flat_rows(s, "ynext", "L2_in", f"(tile + gridDim.x) * {RT}")
                self._dma_g(s, "tile + gridDim.x", "gb ^ 1")
                s.close()
            for vi, ps, first in ker:
                b1 = self.vin[vi]
                s.open(f"if (act{vi})")
                self._dx_paths(s, ps, f"x{vi}", f"dx{vi}")
                s("#pragma unroll")
                s.open("for (int i = 0; i < 4; ++i)")
                s(f"const i64 row = row0 + {self.row('i')};")
                s.open("if (row < num_batch)" if b1.mul % 16 == 0 else f"if (row < num_batch && uok{vi})")
                s(f"T* dp = L1_grad + row * {low.L1} + {b1.off} + u{vi} * {b1.d};")
                for c in range(b1.d):
                    s(f"dp[{c}] {'=' if first and not self.accumulate else '+='} dx{vi}[i][{c}];")
                s.close()
                s.close()
                s.close()
            # dY: sum over the 16 channels of the lane group, then over the 4 waves through LDS
            self._reduce_dy(s)
            if dma:
                # Y of the next tile into the other copy (last read two barriers ago)
                s.open("if (more)")
                put_y("gb ^ 1")
                self._put_g_tail(s, "gb ^ 1")
                s.close()
                s.close()  # tiles
                s("__syncthreads();")
                s.open("if (prow0 >= 0)")
                finish_dy("gb ^ 1")  # (gb was flipped on leaving the last tile)
                s.close()
                s.close()  # kernel
                first_dy = False
                continue
            s("__syncthreads();")
            s.open(f"for (int t = tid; t < {RT * low.L2}; t += {64 * WAVES})")
            s(f"const int r = t / {low.L2}, c = t % {low.L2};")
            s("const T tot = ((s_dy[0][r][c] + s_dy[1][r][c]) + s_dy[2][r][c]) + s_dy[3][r][c];")
            s(f"if (row0 + r < num_batch) L2_grad[(row0 + r) * {low.L2} + c] {'+=' if rmw_dy else '='} tot;")
            s.close()
            s.close()
            s.close()
            first_dy = False
        if first_dy and "dx" in parts:
            raise AssertionError("no path")
        if "dw" not in parts:
            return names

        # ---------------- dW ----------------------------------------------------
        xrows = (2 if self.t1 else 1) * 2 * (RT // WAVES) * self.max_d1
        regs = lambda ker: (sum(4 * c16(vp.Wn) for g in ker for vp in g[1]) + xrows
                            + 4 * max(c16(self.vout[g[0]].mul) for g in ker) + 64)

        def dw_lds(ker, nbuf):
            """Bytes of LDS of a dW kernel: the dZ columns of its pieces, the T tile (one or two copies), Y."""
            first, last = self.vout[ker[0][0]], self.vout[ker[-1][0]]
            ncols = last.off + last.mul * last.d - first.off
            maxd = max(self.vout[g[0]].d for g in ker)
            return (RT * self._tile_stride(ncols) + nbuf * maxd * self.tlanes * TPAD + 2 * RT * low.L2) * low.elem_size

        # a kernel that would not fit the 160 KB of LDS with its pieces merged stays split (the register estimate
        # is replaced by one beyond any limit)
        cost = lambda ker: regs(ker) if dw_lds(ker, 1) <= LDS_BUDGET else 1 << 30
        limit = lambda vo, sub: max(32, self.tune["uvw_wregs"] - (xrows + 4 * c16(self.vout[vo].mul) + 64))
        groups = [g for g in _groups(self.vpaths, "vo", len(self.vout), "dw", limit) if g[1]]
        for ker in self._merge(groups, cost, self.tune["uvw_wregs"], self.vout):
            # pieces that share a kernel must be neighbours in the row: one dZ tile covers their columns
            pieces = [self.vout[vo] for vo, _, _ in ker]
            if any(a.off + a.mul * a.d != b.off for a, b in zip(pieces, pieces[1:])):
                raise AssertionError("merged output pieces are not contiguous")
            order_all = [vp for _, order, _ in ker for vp in order]
            col0 = pieces[0].off
            ncols = pieces[-1].off + pieces[-1].mul * pieces[-1].d - col0
            maxd = max(b.d for b in pieces)
            name = f"{self.prefix}backward_w{ker[0][0]}_{order_all[0].tag('vo')}"
            names.append(name)
            s("// ======== dW of the sub-paths into out pieces " + ", ".join(str(vo) for vo, _, _ in ker))
            self._kernel_open(s, name, self.sig_b, self.tune["uvw_ww"])
            # only these pieces' columns of the dZ tile are needed (and kept)
            # two copies of the T tile let a path's contraction be written while the previous path's is still
            # being multiplied; where they do not fit (fp64, l = 3 outputs) one copy and a barrier more per path
            nbuf = 2 if dw_lds(ker, 2) <= LDS_BUDGET else 1
            if dw_lds(ker, nbuf) > LDS_BUDGET:
                raise ValueError(f"the dW kernel of output piece {ker[0][0]} needs {dw_lds(ker, nbuf)} bytes of LDS")
            s(f"__shared__ __attribute__((aligned(16))) T s_g[{RT}][{self._tile_stride(ncols)}];")
            s(f"__shared__ T s_T[{nbuf}][{maxd}][{self.tlanes}][{TPAD}];")
            s(f"__shared__ T s_y[{RT}][{low.L2}];")
            if self.t1:
                s(f"__shared__ T s_y2[{RT}][{low.L2}];")
            self._prologue(s)
            s("const int u = wave * 16 + l16;")
            s(f"T* prow = wpartial + (i64)blockIdx.x * {low.WN};")
            s(f"T xa[{RT // WAVES}][{self.max_d1}], xb[{RT // WAVES}][{self.max_d1}];")
            if self.t1:
                s(f"T aa[{RT // WAVES}][{self.max_d1}], ab[{RT // WAVES}][{self.max_d1}];")
            # dw<path>[n]: D tile rows = channels u of the wave's slice, columns = w in 16 n .. 16 n + 15
            for vp in order_all:
                ntile = c16(vp.Wn)
                s(f"v4t dw{vp.index}[{ntile}];")
                s(f"for (int n = 0; n < {ntile}; ++n) dw{vp.index}[n] = v4t{{}};")
            s.open("for (i64 tile = blockIdx.x; tile < ntiles; tile += gridDim.x)")
            s(f"const i64 row0 = tile * {RT};")
            s("__syncthreads();")
            self._stage_g(s, col0, ncols, local=True)
            self._stage_y(s)
            self._load_x_rows(s, "xa", order_all[0])
            s("__syncthreads();")
            cur, nxt = "xa", "xb"
            for n, vp in enumerate(order_all):
                p = vp.p
                bo = self.vout[vp.vo]
                buf = n % nbuf
                s(f"// path {p.index}: l=({low.in1[p.i1].l},{low.in2[p.i2].l},{bo.l})")
                if nbuf == 1 and n > 0:
                    s("__syncthreads();  // the previous path's T tile has been multiplied")
                self._t_compute(s, vp, cur, str(buf))
                if n + 1 < len(order_all):
                    self._load_x_rows(s, nxt, order_all[n + 1])
                s("__syncthreads();")
                # dW[u, w] += sum_(k,r) T[(k,r), u] * dZ[(k,r), w]   (A = T^T, B = dZ tile)
                s.open(f"if (wave * 16 < {vp.U})")
                s("#pragma unroll")
                s.open(f"for (int st = 0; st < {4 * bo.d}; ++st)")
                s("const int kq = 4 * st + lq;")
                s("const int kk = kq >> 4, rr = kq & 15;")
                s(f"const T a = s_T[{buf}][kk][u][rr];")
                for nn in range(c16(vp.Wn)):
                    # (columns past the piece: its last column again; what they give is not stored)
                    wcol = f"({16 * nn} + l16)" if 16 * nn + 16 <= vp.Wn else f"min({16 * nn} + l16, {vp.Wn - 1})"
                    s(f"dw{vp.index}[{nn}] = {MFMA}(a, s_g[rr][{bo.off - col0} + {wcol} * {bo.d} + kk], "
                      f"dw{vp.index}[{nn}], 0, 0, 0);")
                s.close()
                s.close()
                cur, nxt = nxt, cur
            s.close()
            for vp in order_all:
                s.open(f"if (wave * 16 < {vp.U})")
                for nn in range(c16(vp.Wn)):
                    s("#pragma unroll")
                    s.open("for (int i = 0; i < 4; ++i)")
                    conds = ([] if vp.U % 16 == 0 else [f"wave * 16 + {self.row('i')} < {vp.U}"]) + \
                        ([] if 16 * nn + 16 <= vp.Wn else [f"{16 * nn} + l16 < {vp.Wn}"])
                    guard = f"if ({' && '.join(conds)}) " if conds else ""
                    s(f"{guard}prow[{vp.woff} + (wave * 16 + {self.row('i')}) * {vp.ld} + {16 * nn} + l16] = dw{vp.index}[{nn}][i];")
                    s.close()
                s.close()
            s.close()
        return names


    # ------------------------------------------------------- second order
    SIG_A = ("(i64 num_batch, const T* __restrict__ p_x, const T* __restrict__ p_a, const T* __restrict__ p_y, "
             "const T* __restrict__ p_b, const T* __restrict__ p_w, const T* __restrict__ p_c, T* __restrict__ p_gg)")
    SIG_B = ("(i64 num_batch, const T* __restrict__ p_x, const T* __restrict__ p_a, const T* __restrict__ p_y, "
             "const T* __restrict__ p_b, const T* __restrict__ p_w, const T* __restrict__ p_c, "
             "const T* __restrict__ p_g, T* __restrict__ p_dx, T* __restrict__ p_dy, T* __restrict__ p_dw, "
             "T* __restrict__ wpartial)")

    def second_order_kernels(self, s: Src):
        """The kernels of ``double_backward_A`` / ``double_backward_B`` for the matrix-core path, as variants of the
        first-order ones (reference: templates/loop_unroll_batch.cuh:148-317). With cotangents (a, b, c) of
        (dX, dY, dW):

        A  d/d(dZ) = [T(a, y) + T(x, b)] W + T(x, y) C: the forward kernels with the summed contraction, then the
           plain forward kernels on (x, y, C) adding to the result - two channel mixes where composing first-order
           calls runs three;
        B  G = dZ W^T and H = dZ C^T: the dX kernels on (a, b, W), which give dX += c b G and dY += c a G, then on
           (x, y, C) adding c y H and c x H; dW = [T(a, y) + T(x, b)]^T dZ by the dW kernels with the summed
           contraction - two dX passes and one dW pass instead of three of each.

        Returns (names of A, names of B) in launch order."""
        ptr = lambda name, src, const=True: f"{'const ' if const else ''}T* __restrict__ {name} = {src}; (void){name};"
        names_a, names_b = [], []

        def variant(prefix, sig_f=None, sig_b=None, alias=(), accumulate=False, t1=False):
            self.prefix, self.alias, self.accumulate, self.t1 = prefix, list(alias), accumulate, t1
            self.sig_f, self.sig_b = sig_f or self.FWD_SIG, sig_b or self.BWD_SIG

        try:
            variant("dda1_", sig_f=self.SIG_A, t1=True,
                    alias=[ptr("L1_in", "p_x"), ptr("L1_alt", "p_a"), ptr("L2_in", "p_y"), ptr("L2_alt", "p_b"),
                           ptr("W", "p_w"), ptr("L3_out", "p_gg", False)])
            names_a += self.emit_forward(s)
            variant("dda2_", sig_f=self.SIG_A, accumulate=True,
                    alias=[ptr("L1_in", "p_x"), ptr("L2_in", "p_y"), ptr("W", "p_c"), ptr("L3_out", "p_gg", False)])
            names_a += self.emit_forward(s)
            outs = [ptr("L1_grad", "p_dx", False), ptr("L2_grad", "p_dy", False), ptr("L3_grad", "p_g")]
            variant("ddb1_", sig_b=self.SIG_B, alias=[ptr("L1_in", "p_a"), ptr("L2_in", "p_b"), ptr("W", "p_w")] + outs)
            names_b += self.emit_backward(s, parts=("dx",))
            variant("ddb2_", sig_b=self.SIG_B, accumulate=True,
                    alias=[ptr("L1_in", "p_x"), ptr("L2_in", "p_y"), ptr("W", "p_c")] + outs)
            names_b += self.emit_backward(s, parts=("dx",))
            variant("ddb3_", sig_b=self.SIG_B, t1=True,
                    alias=[ptr("L1_in", "p_x"), ptr("L1_alt", "p_a"), ptr("L2_in", "p_y"), ptr("L2_alt", "p_b"),
                           ptr("L3_grad", "p_g")])
            names_b += self.emit_backward(s, parts=("dw",))
        finally:
            variant("")
        return names_a, names_b


def tp_module(low: Lowered, compute_units: int = 256):
    from .. import runtime as rt

    em = MfmaEmitter(low)
    s = Src()
    s(prelude(low.ctype))
    s("typedef T v4t __attribute__((ext_vector_type(4)));")
    s(f"typedef T oeq_vec16 __attribute__((ext_vector_type({16 // low.elem_size})));  // 16 bytes")
    if low.elem_size == 4:
        s("#define oeq_mfma __builtin_amdgcn_mfma_f32_16x16x4f32")
        s("#define oeq_mfma_bf __builtin_amdgcn_mfma_f32_16x16x32_bf16")
        s("typedef __bf16 oeq_bf8 __attribute__((ext_vector_type(8)));")
        s("typedef __bf16 oeq_bf2 __attribute__((ext_vector_type(2)));")
        s("typedef float oeq_f2 __attribute__((ext_vector_type(2)));")
        s("typedef unsigned oeq_u4 __attribute__((ext_vector_type(4)));")
        # a and b as sums of three bf16 numbers each (round to nearest, the remainders are exact in fp32); q<i> holds
        # the i-th parts, a's in the low half
        s("OEQ_DEV unsigned oeq_pk_bf16(float a, float b) { const oeq_f2 v = {a, b}; "
          "return __builtin_bit_cast(unsigned, __builtin_convertvector(v, oeq_bf2)); }")
        s("OEQ_DEV void oeq_split2(float a, float b, unsigned& q0, unsigned& q1, unsigned& q2) { "
          "q0 = oeq_pk_bf16(a, b); "
          "a -= __builtin_bit_cast(float, q0 << 16); b -= __builtin_bit_cast(float, q0 & 0xffff0000u); "
          "q1 = oeq_pk_bf16(a, b); "
          "a -= __builtin_bit_cast(float, q1 << 16); b -= __builtin_bit_cast(float, q1 & 0xffff0000u); "
          "q2 = oeq_pk_bf16(a, b); }")
    else:
        s("#define oeq_mfma __builtin_amdgcn_mfma_f64_16x16x4f64")
        s("template <int CTRL> OEQ_DEV double oeq_dpp(double v) { const long long b = __builtin_bit_cast(long long, v); "
          "const int lo = __builtin_amdgcn_update_dpp(0, (int)b, CTRL, 0xf, 0xf, true); "
          "const int hi = __builtin_amdgcn_update_dpp(0, (int)(b >> 32), CTRL, 0xf, 0xf, true); "
          "return __builtin_bit_cast(double, ((long long)hi << 32) | (unsigned)lo); }")
    # value of the lane that a DPP control word pairs this lane with (row_mirror 0x140, row_half_mirror 0x141,
    # quad_perm otherwise)
    s("template <int CTRL> OEQ_DEV float oeq_dpp(float v) { return __builtin_bit_cast(float, "
      "__builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true)); }")
    s(utility_kernels())
    em._emit_path_fns(s)
    fwd_names = em.emit_forward(s)
    bwd_names = em.emit_backward(s)
    max_blocks = compute_units * em.tune["uvw_blocks"]
    descs = [(rt.ROLE_TP_FORWARD, n, 64 * WAVES, RT, max_blocks) for n in fwd_names]
    descs += [(rt.ROLE_TP_BACKWARD, n, 64 * WAVES, RT, max_blocks) for n in bwd_names]
    if em.tune["uvw_mfma_dd"]:
        names_a, names_b = em.second_order_kernels(s)
        descs += [(rt.ROLE_DOUBLE_BACKWARD_A, n, 64 * WAVES, RT, max_blocks) for n in names_a]
        descs += [(rt.ROLE_DOUBLE_BACKWARD_B, n, 64 * WAVES, RT, max_blocks) for n in names_b]
    descs += [
        (rt.ROLE_FILL_ZERO, "oeq_fill_zero", 256, 256 * 16, compute_units * 16),
        (rt.ROLE_TP_BACKWARD_WREDUCE, "oeq_wreduce", 256, 64, 0),
    ]
    dims = dict(L1_dim=low.L1, L2_dim=low.L2, L3_dim=low.L3, weight_numel=low.WN, elem_size=low.elem_size,
                shared_weights=1, deterministic=0, wpartial_per_block=1)
    return s.text(), dims, descs
