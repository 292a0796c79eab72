"""HIP source generator for per-channel ('uvu') tensor products and the fused
graph convolution built on them (forward and backward).

Replaces the reference's Jinja templates for this mode
(openequivariance/openequivariance/templates/loop_unroll_tp.cuh:18-312,
loop_unroll_batch.cuh:25-142, loop_unroll_conv_atomic.cuh:52-180,
loop_unroll_conv_det.cuh:96-293) with a different decomposition:

* lane <-> channel ``u``; the CG contraction of one channel is straight-line
  code with the sparse coefficients folded into constants; the operand shared
  by all channels (the row's Y) is wave-uniform when a row fills a wave, and so
  is the row's base pointer: accesses are "uniform base + 32-bit lane offset";
* a row's arithmetic is one basic block: lanes without a channel load through a
  clamped index and drop the value, stores are unconditional where every lane
  has a channel, and weight gradients that need a condition wait in registers
  until the last path (a branch inside the chain of paths makes the compiler
  postpone the dX/dY accumulations and keep every path's operands alive);
* the convolution walks each receiver's edges (CSR order given by the caller,
  or an edge index grouped by receiver on the device) and keeps the receiver's
  output (forward) or output gradient (backward) in registers across them, so Z
  and dZ move once per node instead of once per edge; the next edge's operands
  arrive in an LDS staging buffer by direct global->LDS loads meanwhile;
  problems too large for one wave's registers are shared between the waves of
  the node's block by output segment / output block;
* dY is accumulated per lane over all paths and reduced once per row with a
  halving butterfly; no kernel of the walk uses atomics on node data (dX goes
  through per-edge terms and a sender-ordered reduction).
"""

from __future__ import annotations

import os
import re
from typing import Callable, Dict, List, Optional, Sequence, Tuple

from .common import Src, fixup_backward_kernel, prelude, utility_kernels
from .lower import Lowered, Path, float_literal

UNROLL_V_LIMIT = 8


def _pow2ceil(n: int) -> int:
    return 1 << max(0, (n - 1).bit_length())


def tuning(defaults: dict) -> dict:
    """Kernel-shape knobs; ``OEQ_AMD_TUNE="key=value,..."`` overrides them
    (integers), which is how the defaults below were chosen on the GPU."""
    out = dict(defaults)
    for item in os.environ.get("OEQ_AMD_TUNE", "").split(","):
        if "=" in item:
            k, v = item.split("=", 1)
            if k.strip() in out:
                out[k.strip()] = int(v)
    return out


class UvuEmitter:
    def __init__(self, low: Lowered, *, acc_budget_words: int = 128, g_resident_words: int = 128,
                 kahan: bool = False):
        assert low.mode == "uvu"
        assert low.n_chunks <= 16, "blocks of more than 1024 channels are cut into pieces by codegen.lower"
        self.low = low
        self.ir_mul = low.ir_mul
        self.kahan = kahan  # conv forward: compensated (Kahan) summation over a receiver's edges
        # Streaming hints, so that single-use data does not displace the gathered sender rows from the
        # caches: bit 0 = per-row weights loaded non-temporally; bit 1 = per-row results (dW, dX terms)
        # stored non-temporally; bit 2 = the sender-side reduction reads the dX terms non-temporally;
        # bit 3 = output rows stored / output-gradient rows loaded non-temporally; bit 4 = X rows loaded
        # non-temporally (batch kernels only: the convolution re-reads them).
        self.nt = 0
        self.mask_loads = False  # zero X and W values in lanes without a channel (see _operand)
        self.forms = True  # per path, put the CG coefficient on the factor with the fewest distinct products
        self.sched_fence = False
        self.fence_words = 0  # gradient registers between two scheduling fences (0: a fence after every path)
        self.prefetch_runs = False  # request the next run's gradients and weights while a run computes
        self.seg_waves = 1  # conv forward: waves per node that share its output segments between them
        self.bwd_groups: Optional[List[List[int]]] = None  # conv backward: output blocks owned by each wave
        self.group_budget = 0  # gradient words per wave when a node is shared between waves (0: default)
        self.group_count = 0  # that many waves share a node in the backward kernel, whatever their registers (0: by budget)
        self.fit_words = 300  # estimate of backward_words up to which one wave keeps a node's whole gradient
        # plain stores of [64 x d] channel blocks go through the s_tr tile as well: bit 0 = forward outputs,
        # bit 1 = backward dX (kernels that use it declare the tile)
        self.tr_stores = 0
        self.T = low.ctype
        self.words = 1 if low.elem_size == 4 else 2
        self.LPR = low.lanes_per_row
        self.R = low.rows_per_wave
        self.NCH = low.n_chunks
        self.used_in1 = sorted({p.i1 for p in low.paths})
        self.used_out = sorted({p.io for p in low.paths})
        # Blocks of different multiplicity in a row wider than a wave: chunk c only has channels of the blocks
        # with mul > 64 c. The row bodies are then generated once per chunk (the chunk index is wave-uniform),
        # each without the paths, loads and stores of the blocks it has no channel of; cur_chunk is the chunk
        # being generated (None: one body for all chunks).
        used_muls = {low.in1[b].mul for b in self.used_in1} | {low.out[io].mul for io in self.used_out}
        self.chunk_split = self.R == 1 and self.NCH > 1 and any(m != 64 * self.NCH for m in used_muls)
        self.cur_chunk: Optional[int] = None
        # output segments (register-resident accumulators of the conv forward)
        budget = max(1, acc_budget_words // self.words)
        self.segments: List[List[int]] = []
        cur, cur_sz = [], 0
        for io in self.used_out:
            d = low.out[io].d
            if cur and cur_sz + d > budget:
                self.segments.append(cur)
                cur, cur_sz = [], 0
            cur.append(io)
            cur_sz += d
        if cur:
            self.segments.append(cur)
        self.seg_in1 = [sorted({p.i1 for p in low.paths if p.io in seg}) for seg in self.segments]
        self.untouched_out = [io for io in range(len(low.out)) if io not in self.used_out]
        self.g_resident = sum(low.out[io].d for io in self.used_out) * self.words <= g_resident_words
        self.l2_pad = _pow2ceil(low.L2)
        # per-lane weight slots: one per (path, v), in path order
        self.wslot: Dict[int, int] = {}
        n = 0
        for p in low.paths:
            self.wslot[p.index] = n
            n += low.in2[p.i2].mul
        self.n_wslots = n
        # operands of an edge can be fetched ahead into registers when every index is a constant
        self.can_preload = (
            all(low.in2[p.i2].mul <= UNROLL_V_LIMIT for p in low.paths) and low.L2 <= 32 and self.n_wslots <= 128
        )

        self.tr_atomics = False  # set by the conv kernels that declare the s_tr tile
        # Products |c| * y_j of a CG coefficient and a component of the row's second operand are the
        # same for every channel. With ``use_q`` the lanes of a wave compute them once per edge, one
        # product per lane and 64-entry slab, into a wave-private LDS table that the contraction reads
        # back as broadcasts, instead of every lane forming every product in the vector ALU (a third of
        # the forward's and an eighth of the backward's vector instructions at the MACE shape).
        self.use_q = False
        self.q_pin = True
        self.q_ahead = (64, 64)  # multiply-adds between the request of a path's products and their use (fwd, bwd)
        self.q_entries: List[Tuple[int, float]] = []  # table slot -> (index into the Y row, coefficient)
        self.q_slot: Dict[Tuple[int, int, str, int], int] = {}  # (path, v, |c| literal, j) -> slot
        self.stage = self._stage_layout()
        self.stage3 = self._stage3_layout()

    def _stage_layout(self):
        """Layout of one wave's LDS staging buffer for the operands of an edge
        (the wave's 64-channel slice of X[sender] and of W[edge]), filled by
        direct global->LDS loads of 16 B per lane. None when the problem does not
        have the regular shape this needs."""
        low = self.low
        if not (self.R == 1 and self.can_preload and self.words == 1 and len(self.segments) == 1
                and not low.shared_weights):
            return None
        U = 64 * self.NCH
        if any(low.in1[b].mul != U or low.in1[b].off % 4 for b in self.used_in1):
            return None
        if any(low.in2[p.i2].mul != 1 or p.woff != p.index * U for p in low.paths):
            return None
        if low.L1 % 4 or low.WN % 4:
            return None
        xl, units = {}, 0
        for b in self.used_in1:
            xl[b] = units * 4
            units += 16 * low.in1[b].d
        nqx = (units + 63) // 64
        nuw = 16 * len(low.paths)
        nqw = (nuw + 63) // 64
        return dict(U=U, xl=xl, nux=units, nqx=nqx, nuw=nuw, nqw=nqw, XF=nqx * 256, floats=(nqx + nqw) * 256)

    def _stage_src(self, blk, first_unit: int) -> str:
        """Row offset of the 16-byte unit ``t`` of the wave's slice of a block (units in LDS order)."""
        if self.ir_mul:
            # component i = 16 units of 4 channels each; the components of a piece of a folded block lie the
            # whole block's multiplicity apart
            return (f"{blk.off} + ((t - {first_unit}) >> 4) * {blk.cstride or blk.mul} + chunk * 64 + "
                    f"((t - {first_unit}) & 15) * 4")
        return f"{blk.off} + chunk * {64 * blk.d} + (t - {first_unit}) * 4"

    def _stage_x(self, blk, base: int, i: int) -> str:
        """Index of (lane's channel, component i) in a staged block starting at ``base``."""
        return f"{base + i * 64} + ul" if self.ir_mul else f"{base} + ul * {blk.d} + {i}"

    def _emit_stage_offsets(self, s: Src):
        """Per-lane source offsets (in elements) of the staging loads; loop invariant."""
        low, st = self.low, self.stage
        for q in range(st["nqx"]):
            s(f"int xoff{q};")
            s.open("")
            s(f"int t = {q * 64} + lane; if (t > {st['nux'] - 1}) t = {st['nux'] - 1};")
            expr, pu = None, 0
            terms = []
            for b in self.used_in1:
                blk = low.in1[b]
                n = 16 * blk.d
                terms.append((pu, pu + n, self._stage_src(blk, pu)))
                pu += n
            code = terms[-1][2]
            for lo, hi, ex in reversed(terms[:-1]):
                code = f"(t < {hi}) ? ({ex}) : ({code})"
            s(f"xoff{q} = {code};")
            s.close()
        for q in range(st["nqw"]):
            s(f"int woff{q};")
            s.open("")
            s(f"int t = {q * 64} + lane; if (t > {st['nuw'] - 1}) t = {st['nuw'] - 1};")
            s(f"woff{q} = (t >> 4) * {st['U']} + chunk * 64 + (t & 15) * 4;")
            s.close()

    def _emit_stage_issue(self, s: Src, e: str, x: bool = True, w: bool = True, wbuf: Optional[str] = None):
        """Request the operands of edge ``e``: ``x`` = the sender's X slice and the edge's Y, ``w`` = the
        edge's weights, into the second weight buffer of the wave where ``wbuf`` (an expression, 0 or 1)
        says so."""
        low, st = self.low, self.stage
        s.open("")
        s(f"const i64 eid = OEQ_EDGE({e});")
        if x:
            s(f"const T* sx = L1_in + oeq_idx(cols[eid], node_count) * {low.L1};")
            for q in range(st["nqx"]):
                s(f"__builtin_amdgcn_global_load_lds((const OEQ_GPTR)(sx + xoff{q}), "
                  f"(OEQ_LPTR)(&s_stage[wave][{q * 256}]), 16, 0, 0);")
            if self.use_q:
                for r in range(self.q_slabs):
                    s(f"yn[{r}] = L2_in[eid * {low.L2} + qt.j[{r}]];")
            else:
                for j in range(low.L2):
                    s(f"yn[{j}] = L2_in[eid * {low.L2} + {j}];")
        if w:
            s(f"const T* sw = W + eid * {low.WN};")
            base = f"{st['XF']}" if wbuf is None else f"{st['XF']} + ({wbuf}) * {st['nqw'] * 256}"
            for q in range(st["nqw"]):
                s(f"__builtin_amdgcn_global_load_lds((const OEQ_GPTR)(sw + woff{q}), "
                  f"(OEQ_LPTR)(&s_stage[wave][{base} + {q * 256}]), 16, 0, {2 if self.nt & 1 else 0});")
        s.close()

    def _emit_stage_read(self, s: Src, buf: str, wbuf: Optional[str] = None):
        low, st = self.low, self.stage
        wbase = f"{st['XF']}" if wbuf is None else f"{st['XF']} + ({wbuf}) * {st['nqw'] * 256}"
        for b in self.used_in1:
            blk = low.in1[b]
            for i in range(blk.d):
                s(f"{buf}.x.b{b}[{i}] = s_stage[wave][{self._stage_x(blk, st['xl'][b], i)}];")
        for p in low.paths:
            s(f"{buf}.w[{self.wslot[p.index]}] = s_stage[wave][{wbase} + {p.index * 64} + ul];")
        if self.use_q:
            for r in range(self.q_slabs):
                s(f"{buf}.yq[{r}] = yn[{r}];")
        else:
            for j in range(low.L2):
                s(f"{buf}.y[{j}] = yn[{j}];")

    # ---- double-buffered staging: X, W and Y of an edge live only in LDS ------------
    def _stage3_layout(self):
        """Two LDS buffers per wave (separate arrays, so that reads of one do not
        wait for loads into the other); the contraction reads its operands from
        LDS where it uses them, so no register copy of an edge's operands exists."""
        if self.stage is None or self.low.L2 % 4:
            return None
        st = dict(self.stage)
        npaths = len(self.low.paths)
        # Both parts are whole 64-lane instructions (the lanes beyond the data repeat its last unit into padding):
        # a direct load under a lane condition sits in divergent control flow, where one compiler version has been
        # seen to merge two of them into one instruction with the LDS base of the first active lane.
        st["XF"] = st["nqx"] * 256
        st["YOFF"] = st["XF"] + 64 * npaths
        st["nuwy"] = 16 * npaths + self.low.L2 // 4
        st["nqw"] = (st["nuwy"] + 63) // 64
        st["floats"] = st["XF"] + st["nqw"] * 256
        return st

    def _emit_stage3_offsets(self, s: Src):
        low, st = self.low, self.stage3
        for q in range(st["nqx"]):
            s(f"int xoff{q};")
            s.open("")
            s(f"int t = {q * 64} + lane; if (t > {st['nux'] - 1}) t = {st['nux'] - 1};")
            terms, pu = [], 0
            for b in self.used_in1:
                blk = low.in1[b]
                n = 16 * blk.d
                terms.append((pu + n, self._stage_src(blk, pu)))
                pu += n
            code = terms[-1][1]
            for hi, ex in reversed(terms[:-1]):
                code = f"(t < {hi}) ? ({ex}) : ({code})"
            s(f"xoff{q} = {code};")
            s.close()
        nuw = 16 * len(low.paths)
        for q in range(st["nqw"]):
            # units below nuw are weights (16 per path), the rest is the edge's Y row
            s(f"int woff{q}; bool wsel{q};")
            s.open("")
            s(f"int t = {q * 64} + lane; if (t > {st['nuwy'] - 1}) t = {st['nuwy'] - 1};")
            s(f"wsel{q} = t < {nuw};")
            s(f"woff{q} = wsel{q} ? ((t >> 4) * {st['U']} + chunk * 64 + (t & 15) * 4) : ((t - {nuw}) * 4);")
            s.close()

    def _emit_stage3_issue(self, s: Src, buf: str, e: str):
        low, st = self.low, self.stage3
        s.open("")
        s(f"const i64 eid = OEQ_EDGE({e});")
        s(f"const T* sx = L1_in + oeq_idx(cols[eid], node_count) * {low.L1};")
        s(f"const T* sw = W + eid * {low.WN};")
        s(f"const T* sy = L2_in + eid * {low.L2};")
        for q in range(st["nqx"]):
            s(f"__builtin_amdgcn_global_load_lds((const OEQ_GPTR)(sx + xoff{q}), "
              f"(OEQ_LPTR)(&s_stage{buf}[wave][{q * 256}]), 16, 0, 0);")
        for q in range(st["nqw"]):
            s(f"__builtin_amdgcn_global_load_lds((const OEQ_GPTR)((wsel{q} ? sw : sy) + woff{q}), "
              f"(OEQ_LPTR)(&s_stage{buf}[wave][{st['XF'] + q * 256}]), 16, 0, 0);")
        s.close()

    def _acc_staged3(self, sb: str):
        low, st = self.low, self.stage3

        def x(b: int, i: int) -> str:
            return f"{sb}[{self._stage_x(low.in1[b], st['xl'][b], i)}]"

        def y(p: Path, v: str, j: int) -> str:
            return f"{sb}[{st['YOFF'] + low.in2[p.i2].off + j}]"

        def w(p: Path, v: str) -> str:
            return f"{sb}[{st['XF'] + p.index * 64} + ul]"

        return x, y, w

    def _lane_ptr(self, blk) -> Tuple[str, int]:
        """(pointer-offset expression of channel ``u``'s first component within a row, stride between
        components) of a block: [mul, 2l+1] rows keep a channel's components together, [2l+1, mul] rows keep
        a component's channels together (then a wave's accesses are contiguous without any per-lane vector).
        The expression is applied with :meth:`_ptr`."""
        if self.ir_mul:
            return (blk.off, 1), (blk.cstride or blk.mul)
        return (blk.off, blk.d), 1

    def _ptr(self, rowexpr: str, where, mul: Optional[int] = None) -> str:
        """Pointer to element ``const + u * stride`` of a row. When a row fills the wave the row pointer is
        wave-uniform and the lane part is a 32-bit byte offset shared by all blocks of the same stride.
        With ``mul`` given and lanes beyond it, the lane index is clamped (loads stay in bounds and need no
        branch; the caller discards their values)."""
        const, stride = where
        u = "u" if mul is None or self._full(mul) else f"(u < {mul} ? u : {mul - 1})"
        if self.R == 1:
            return f"oeq_at({rowexpr} + {const}, (unsigned){u} * {stride * self.low.elem_size}u)"
        return f"({rowexpr} + {const} + {u} * {stride})"

    def _gptr(self, rowexpr: str, where, mul: int) -> str:
        """Pointer through which a lane reads its channel of an output-gradient block. Lanes without a
        channel are pointed at a row of zeros: every sum across lanes has a factor from the output
        gradient, so this is what keeps their terms out of it, and the loaded values need no select
        (a select after each load has made the compiler wait for the loads one by one)."""
        if self._full(mul):
            return self._ptr(rowexpr, where, mul)
        return f"(u < {mul} ? {self._ptr(rowexpr, where)} : (const T*)oeq_zero_row)"

    def _full(self, mul: int) -> bool:
        """Every lane's channel index is a channel of such a block (over all chunks, or in the chunk being
        generated)."""
        if self.cur_chunk is not None:
            return mul >= 64 * (self.cur_chunk + 1)
        return mul == self.LPR * self.NCH

    def _has(self, mul: int) -> bool:
        """The chunk being generated has channels of a block of this multiplicity."""
        return self.cur_chunk is None or mul > 64 * self.cur_chunk

    def _paths(self, paths: Optional[List[Path]] = None) -> List[Path]:
        base = self.low.paths if paths is None else paths
        return [p for p in base if self._has(self.low.in1[p.i1].mul)]

    def _in1_of(self, blocks: List[int]) -> List[int]:
        return [b for b in blocks if self._has(self.low.in1[b].mul)]

    def _out_of(self, ios: List[int]) -> List[int]:
        return [io for io in ios if self._has(self.low.out[io].mul)]

    def _sfx(self) -> str:
        return "" if self.cur_chunk is None else f"_c{self.cur_chunk}"

    def _per_chunk(self, s: Src, body: Callable[[], None], in_kernel: bool = True):
        """Emit ``body`` once, or once per chunk (inside ``if (chunk == c)`` when in a kernel)."""
        if not self.chunk_split:
            body()
            return
        for c in range(self.NCH):
            self.cur_chunk = c
            try:
                if in_kernel:
                    s.open(f"if (chunk == {c})")
                body()
                if in_kernel:
                    s.close()
            finally:
                self.cur_chunk = None

    def _val(self, mul: int, loaded: str, extra: Optional[str] = None) -> str:
        """A value loaded through a clamped pointer, zeroed for lanes without a channel (and when
        ``extra`` is false)."""
        conds = [c for c in (None if self._full(mul) else f"u < {mul}", extra) if c]
        return f"oeq_sel({' && '.join(conds)}, {loaded})" if conds else loaded

    @staticmethod
    def _guarded(loaded: str, guard: Optional[str]) -> str:
        return f"oeq_sel({guard}, {loaded})" if guard else loaded

    def _operand(self, mul: int, loaded: str) -> str:
        """A per-row operand (X or W value) loaded through a clamped pointer. Lanes without a channel
        read the block's last channel and keep that value: nothing they compute is stored, and every sum
        across lanes (the gradients with respect to Y) has a factor from the output gradient, which
        ``_val`` zeroes for them. Leaving the select off the loads lets the compiler issue them back to
        back; with it, chains of load, wait, select through one register have been seen."""
        return self._val(mul, loaded) if self.mask_loads else loaded

    def _store_cond(self, mul: int, *guards) -> Optional[str]:
        conds = [g for g in guards if g and g != "true"]
        if not self._full(mul):
            conds.append(f"u < {mul}")
        return " && ".join(conds) if conds else None

    @staticmethod
    def _dump_unless(cond: Optional[str], ptr: str) -> str:
        """Pointer of a store inside the chain of paths that only some lanes (or rows) may perform: the others
        are pointed at a scratch array nobody reads, so the store itself is unconditional. A branch around it
        would split the chain into basic blocks; the compiler then sinks the value's computation into the
        conditional block and, when registers are short, spills values that live across it from inside that
        block - with part of the lanes switched off, which leaves those lanes' copies stale. Wrong gradients
        were measured from exactly this (rows of mixed multiplicity whose weight gradients could not be kept
        in registers until the end of the row)."""
        return ptr if not cond else f"(({cond}) ? {ptr} : oeq_dump + ((blockIdx.x & 63u) * 64u + (threadIdx.x & 63u)))"

    def _open_if(self, s: Src, cond: Optional[str], values: Sequence[str] = ()):
        """Open the block of a (possibly conditional) store of ``values``. Values that only a
        conditional store uses are first passed through an empty asm statement: the compiler would
        otherwise move the whole chain of operations that computes them into the conditional block,
        and with it keep every operand of that chain alive until there."""
        if cond:
            for v in values:
                s(f'asm volatile("" : "+v"({v}));')
        s.open(f"if ({cond})" if cond else "")

    def _y_index(self, b2, v: str, j: int) -> str:
        if self.ir_mul:
            return f"{b2.off + j * b2.mul} + ({v})"
        return f"{b2.off} + ({v}) * {b2.d} + {j}"

    @staticmethod
    def _xv(xname, b: int, i: int) -> str:
        return xname(b, i) if callable(xname) else f"{xname}.b{b}[{i}]"

    # ------------------------------------------------------------------ utils
    def lit(self, v: float) -> str:
        return float_literal(v, self.T)

    # operand accessors -------------------------------------------------------
    def _acc_pointer(self):
        low = self.low

        def y(p: Path, v: str, j: int) -> str:
            return f"yrow[{self._y_index(low.in2[p.i2], v, j)}]"

        def w(p: Path, v: str) -> str:
            mul = low.in1[p.i1].mul
            wp = self._ptr("wrow", (f"{p.woff} + ({v})", low.in2[p.i2].mul), mul)
            ld = f"__builtin_nontemporal_load({wp})" if (self.nt & 1) and not low.shared_weights else f"*{wp}"
            return self._operand(mul, ld)

        return y, w

    def _acc_preloaded(self, name: str = "d"):
        low = self.low

        def y(p: Path, v: str, j: int) -> str:
            b2 = low.in2[p.i2]
            return f"{name}.y[{b2.off + (j * b2.mul + int(v) if self.ir_mul else int(v) * b2.d + j)}]"

        def w(p: Path, v: str) -> str:
            return f"{name}.w[{self.wslot[p.index] + int(v)}]"

        return y, w

    def _qarg(self) -> str:
        return ", qt" if self.use_q else ""

    def q_supported(self) -> bool:
        """The product table needs the second operand to be the same for the whole wave (a row that
        fills the wave) and every index a generation-time constant."""
        return self.R == 1 and self.can_preload

    def build_q_table(self):
        """Slots 0..L2-1 hold the raw Y row, the rest the distinct products of every (path, v) in path
        order (so the slots a path reads are contiguous and can be fetched as 16-byte vectors)."""
        low = self.low
        self.q_entries = [(j, 1.0) for j in range(low.L2)]
        self.q_slot = {}
        for p in low.paths:
            b2 = low.in2[p.i2]
            for v in range(b2.mul):
                for (i, j, k, c) in p.nnz:
                    key = (p.index, v, self.lit(abs(c)), j)
                    if key not in self.q_slot:
                        self.q_slot[key] = len(self.q_entries)
                        yidx = b2.off + (j * b2.mul + v if self.ir_mul else v * b2.d + j)
                        self.q_entries.append((yidx, abs(c)))
        self.q_slabs = -(-len(self.q_entries) // 64)
        self.q_floats = self.q_slabs * 64

    def emit_q_tables(self, s: Src):
        """Module-scope constants: for table slot t, which Y component it multiplies and by what."""
        pad = self.q_floats - len(self.q_entries)
        js = [j for j, _ in self.q_entries] + [0] * pad
        cs = [self.lit(c) for _, c in self.q_entries] + [self.lit(0.0)] * pad
        s(f"__device__ const int OEQ_QJ[{self.q_floats}] = {{{', '.join(map(str, js))}}};")
        s(f"__device__ const T OEQ_QC[{self.q_floats}] = {{{', '.join(f'T({c})' for c in cs)}}};")
        s(f"struct __attribute__((aligned({4 * self.low.elem_size}))) oeq_q4 {{ T v[4]; }};")
        s(f"struct Q_t {{ int j[{self.q_slabs}]; T c[{self.q_slabs}]; }};")

    def _emit_q_prologue(self, s: Src, waves: int):
        s(f"__shared__ __attribute__((aligned(16))) T s_q[{waves}][{self.q_floats}];")
        s("Q_t qt;")
        for r in range(self.q_slabs):
            s(f"qt.j[{r}] = OEQ_QJ[{r * 64} + lane]; qt.c[{r}] = OEQ_QC[{r * 64} + lane];")
        s("T* const sq = &s_q[wave][0];")

    def _emit_q_build(self, s: Src, src: str):
        """Fill the wave's table from the Y values its lanes fetched (``src[r]``). The wave-scope fences
        keep the table reads of the previous edge above the writes and those of this edge below."""
        s("oeq_wave_sync();")
        for r in range(self.q_slabs):
            s(f"sq[{r * 64} + lane] = qt.c[{r}] * {src}[{r}];")
        s("oeq_wave_sync();")

    def _q_slots_of(self, p: Path, v: int) -> List[int]:
        return [self.q_slot[(p.index, v, self.lit(abs(c)), j)] for (i, j, k, c) in p.nnz]

    def _q_fetch_plan(self, ordered: List[Path], ahead: int = 64):
        """Which table vectors to request before each path of ``ordered``: those of the paths that
        start within the next ``ahead`` multiply-adds (and were not requested yet), so that a path's
        products have arrived by the time its first instruction needs them. Returns a list, per path,
        of vector indices; the caller declares them at the scope of the whole contraction."""
        low = self.low
        groups = []
        for p in ordered:
            gs = set()
            for v in range(low.in2[p.i2].mul):
                sl = self._q_slots_of(p, v)
                gs |= set(range(min(sl) // 4, max(sl) // 4 + 1))
            groups.append(sorted(gs))
        plan, declared, reach = [], set(), 0
        for k in range(len(ordered)):
            work, m = 0, k
            want = []
            while m < len(ordered) and (m == k or work < ahead):
                want += [g for g in groups[m] if g not in declared and g not in want]
                work += len(ordered[m].nnz) * low.in2[ordered[m].i2].mul
                m += 1
            declared |= set(want)
            plan.append(want)
        return plan

    def _emit_q_fetch(self, s: Src, want: List[int]):
        for g in want:
            s(f"const oeq_q4 qg{g} = *(const oeq_q4*)(sq + {4 * g});")
        if want and self.q_pin:
            # keep the requests here: the scheduler would otherwise sink them to their first use
            s("__builtin_amdgcn_sched_barrier(0);")

    def _emit_q_raw_y(self, s: Src):
        """The raw Y row (table slots 0..L2-1), for the contractions that use it beside the products."""
        for g in range(-(-self.low.L2 // 4)):
            s(f"const oeq_q4 qy{g} = *(const oeq_q4*)(sq + {4 * g});")

    def _products(self, s: Src, p: Path, v: str, yacc) -> Dict[int, Tuple[str, bool]]:
        """Emit the distinct |c|*y_j products of a path. Returns nnz index ->
        (operand name, negative)."""
        if self.use_q:
            b2 = self.low.in2[p.i2]
            for j in sorted({j for _, j, _, _ in p.nnz}):
                yidx = b2.off + (j * b2.mul + int(v) if self.ir_mul else int(v) * b2.d + j)
                s(f"const T y{j} = qy{yidx // 4}.v[{yidx % 4}];")
            slots = self._q_slots_of(p, int(v))
            return {n: (f"qg{t // 4}.v[{t % 4}]", p.nnz[n][3] < 0) for n, t in enumerate(slots)}
        for j in sorted({j for _, j, _, _ in p.nnz}):
            s(f"const T y{j} = {yacc(p, v, j)};")
        names: Dict[Tuple[str, int], str] = {}
        out = {}
        for n, (i, j, k, c) in enumerate(p.nnz):
            key = (self.lit(abs(c)), j)
            if key not in names:
                names[key] = f"q{len(names)}"
                s(f"const T {names[key]} = T({key[0]}) * y{j};")
            out[n] = (names[key], c < 0)
        return out

    def _form_counts(self, p: Path):
        """Distinct (|c|, j), (|c|, i), (|c|, k) pairs and distinct |c| of a path: what it costs to carry
        the coefficient on the Y value, on the X value, on the output, and to fold the weight into it."""
        mag = lambda c: self.lit(abs(c))
        cj = len({(mag(c), j) for _, j, _, c in p.nnz})
        ci = len({(mag(c), i) for i, _, _, c in p.nnz})
        ck = len({(mag(c), k) for _, _, k, c in p.nnz})
        nc = len({mag(c) for _, _, _, c in p.nnz})
        return cj, ci, ck, nc

    def _y_values(self, s: Src, p: Path, v: str, yacc):
        for j in sorted({j for _, j, _, _ in p.nnz}):
            s(f"const T y{j} = {yacc(p, v, j)};")

    def _scaled(self, s: Src, p: Path, which: int, operand, prefix: str, weight: Optional[str] = None):
        """Emit the distinct products |c| * operand(index) of a path, index = component ``which`` of an
        nnz entry (0: i, 1: j, 2: k); with ``weight`` the coefficient is |c| * weight, formed once per
        distinct |c|. Returns nnz index -> (name, negative)."""
        cw = {}
        if weight is not None:
            for _, _, _, c in p.nnz:
                m = self.lit(abs(c))
                if m not in cw:
                    cw[m] = f"cw{len(cw)}"
                    s(f"const T {cw[m]} = T({m}) * {weight};")
        names, out = {}, {}
        for n, ent in enumerate(p.nnz):
            key = (self.lit(abs(ent[3])), ent[which])
            if key not in names:
                names[key] = f"{prefix}{len(names)}"
                coef = cw[key[0]] if weight is not None else f"T({key[0]})"
                s(f"const T {names[key]} = {coef} * {operand(ent[which])};")
            out[n] = (names[key], ent[3] < 0)
        return out

    def _load_x(self, s: Src, rowexpr: str, blocks: List[int], dst: str = "x"):
        low = self.low
        for b in self._in1_of(blocks):
            blk = low.in1[b]
            s.open("")
            base, st = self._lane_ptr(blk)
            s(f"const T* xp = {self._ptr(rowexpr, base, blk.mul)};")
            for i in range(blk.d):
                ld = f"__builtin_nontemporal_load(xp + {i * st})" if self.nt & 16 else f"xp[{i * st}]"
                s(f"{dst}.b{b}[{i}] = {self._operand(blk.mul, ld)};")
            s.close()

    def _for_v(self, s: Src, p: Path, body: Callable[[str], None]):
        V = self.low.in2[p.i2].mul
        if V <= UNROLL_V_LIMIT:
            for v in range(V):
                s.open("")
                body(str(v))
                s.close()
        else:
            s("#pragma unroll 1")
            s.open(f"for (int v = 0; v < {V}; ++v)")
            body("v")
            s.close()

    # ------------------------------------------------------- shared structs
    def emit_structs(self, s: Src):
        low = self.low
        s("struct X_t {")
        for b in self.used_in1:
            s(f"    T b{b}[{low.in1[b].d}];")
        s("};")
        s("struct G_t {")
        for io in self.used_out:
            s(f"    T o{io}[{low.out[io].d}];")
        s("};")
        partial = [low.out[io] for io in self.used_out if low.out[io].mul % (self.LPR * self.NCH)]
        if partial:
            # what lanes without a channel read in place of an output-gradient block (see _gptr)
            extent = max((b.d - 1) * self._lane_ptr(b)[1] + 1 for b in partial)
            s(f"__device__ const T oeq_zero_row[{extent}] = {{}};")
        # where lanes (or rows) that must not store point their store inside a chain of paths (see _dump_unless)
        s("__device__ T oeq_dump[4096];")
        if self.can_preload and self.q_entries:
            # y: the edge's Y row; yq: the Y values this lane multiplies for the wave's product table
            # (a kernel uses one of the two)
            self.emit_q_tables(s)
            s(f"struct E_t {{ X_t x; T w[{self.n_wslots}]; T y[{low.L2}]; T yq[{self.q_slabs}]; }};")
        elif self.can_preload:
            s(f"struct E_t {{ X_t x; T w[{self.n_wslots}]; T y[{low.L2}]; }};")
        for si, seg in enumerate(self.segments):
            s(f"struct A{si}_t {{")
            for io in seg:
                s(f"    T o{io}[{low.out[io].d}];")
            s("};")
            s.open(f"OEQ_DEV void zero_seg{si}(A{si}_t& a)")
            for io in seg:
                for k in range(low.out[io].d):
                    s(f"a.o{io}[{k}] = T(0);")
            s.close()
            if self.kahan:
                # c holds one edge's contribution plus the rounding error carried from the previous
                # addition; afterwards it holds the part of it that did not fit into a
                s.open(f"OEQ_DEV void kahan_seg{si}(A{si}_t& c, A{si}_t& a)")
                for io in seg:
                    for k in range(low.out[io].d):
                        e = f"o{io}[{k}]"
                        s(f"{{ const T y = c.{e}; const T t = a.{e} + y; c.{e} = y - (t - a.{e}); a.{e} = t; }}")
                s.close()

    def _emit_load_edge(self, s: Src, name: str, in1_blocks: List[int], paths: List[Path]):
        """load_edge: fetch X[cols[e]] (the listed blocks), the weights of the
        listed paths and the edge's Y into an E_t."""
        low = self.low
        paths = self._paths(paths)
        s.open(
            f"OEQ_DEV void {name}{self._sfx()}(E_t& d, const i64 e, const T* __restrict__ L1_in, "
            "const T* __restrict__ L2_in, "
f"const T* __restrict__ W, const i64* __restrict__ cols, const i64 node_count, const int u"
            f"{', const Q_t& qt' if self.use_q else ''})"
        )
        s("const i64 c = oeq_idx(cols[e], node_count);")
        s(f"const T* xrow = L1_in + c * {low.L1};")
        s(f"const T* yrow = L2_in + e * {low.L2};")
        s(f"const T* wrow = W{'' if low.shared_weights else f' + e * {low.WN}'};")
        _, wptr = self._acc_pointer()
        for p in paths:
            for v in range(low.in2[p.i2].mul):
                s(f"d.w[{self.wslot[p.index] + v}] = {wptr(p, str(v))};")
        self._load_x(s, "xrow", in1_blocks, "d.x")
        if self.use_q:
            for r in range(self.q_slabs):
                s(f"d.yq[{r}] = yrow[qt.j[{r}]];")
        else:
            for j in range(low.L2):
                s(f"d.y[{j}] = yrow[{j}];")
        s.close()

    # --------------------------------------------------------- forward cores
    def _emit_fwd_seg(self, s: Src, si: int, preloaded):
        if self.use_q and preloaded is not True:
            # only the register-operand variant reads the product table
            self.use_q = False
            try:
                return self._emit_fwd_seg(s, si, preloaded)
            finally:
                self.use_q = True
        low = self.low
        seg = self.segments[si]
        if preloaded == "lds":
            xname, yacc, wacc = self._acc_staged3("sb")
            s.open(f"OEQ_DEV void fwd_seg{si}_lds{self._sfx()}(const T* sb, const int ul, A{si}_t& a)")
        elif preloaded:
            yacc, wacc = self._acc_preloaded("d")
            s.open(f"OEQ_DEV void fwd_seg{si}_pre{self._sfx()}(const E_t& d, {'const T* sq, ' if self.use_q else ''}"
                   f"A{si}_t& a)")
            xname = "d.x"
        else:
            yacc, wacc = self._acc_pointer()
            s.open(
                f"OEQ_DEV void fwd_seg{si}{self._sfx()}(const X_t& x, const T* __restrict__ yrow, "
                f"const T* __restrict__ wrow, const int u, A{si}_t& a)"
            )
            xname = "x"
        seg_paths = [p for p in self._paths() if p.io in seg]
        if self.use_q:
            qplan = self._q_fetch_plan(seg_paths, self.q_ahead[0])
            self._emit_q_raw_y(s)
        for n_p, p in enumerate(seg_paths):
            b1, b2, bo = low.in1[p.i1], low.in2[p.i2], low.out[p.io]
            s(f"// path {p.index}: l=({b1.l},{b2.l},{bo.l}) in1[{p.i1}] x in2[{p.i2}] -> out[{p.io}], nnz={len(p.nnz)}")
            if self.use_q:
                self._emit_q_fetch(s, qplan[n_p])

            def body(v, p=p, bo=bo):
                # The coefficient of a term rides on whichever factor has the fewest distinct (|c|, index)
                # pairs in this path: the Y value, the X value, or - summing the +-x_i*y_j of equal |c| first -
                # the output, where it is folded into the weight (no separate scaling of the outputs then).
                cj, ci, ck, nc = self._form_counts(p)
                n = len(p.nnz)
                form = 0
                if self.forms and not self.use_q:
                    costs = [cj + n + bo.d, ci + n + bo.d, n + nc + ck]
                    form = costs.index(min(costs))
                if form == 2:
                    self._y_values(s, p, v, yacc)
                    sums = {}
                    for i, j, k, c in p.nnz:
                        key = (self.lit(abs(c)), k)
                        term = f"{self._xv(xname, p.i1, i)} * y{j}"
                        if key not in sums:
                            sums[key] = f"s{len(sums)}"
                            s(f"T {sums[key]} = {'-' if c < 0 else ''}{term};")
                        else:
                            s(f"{sums[key]} {'-=' if c < 0 else '+='} {term};")
                    s(f"const T wv = {wacc(p, v)};")
                    cw = {}
                    for (m, k), name in sums.items():
                        if m not in cw:
                            cw[m] = f"cw{len(cw)}"
                            s(f"const T {cw[m]} = T({m}) * wv;")
                        s(f"a.o{p.io}[{k}] += {cw[m]} * {name};")
                    return
                if form == 1:
                    self._y_values(s, p, v, yacc)
                    prods = self._scaled(s, p, 0, lambda i: self._xv(xname, p.i1, i), "qx")
                    other = lambda i, j: f"y{j}"
                else:
                    prods = self._products(s, p, v, yacc)
                    other = lambda i, j: self._xv(xname, p.i1, i)
                started = set()
                for n_, (i, j, k, c) in enumerate(p.nnz):
                    q, neg = prods[n_]
                    if k not in started:
                        s(f"T t{k} = {'-' if neg else ''}{q} * {other(i, j)};")
                        started.add(k)
                    else:
                        s(f"t{k} {'-=' if neg else '+='} {q} * {other(i, j)};")
                s(f"const T wv = {wacc(p, v)};")
                for k in sorted(started):
                    s(f"a.o{p.io}[{k}] += wv * t{k};")

            self._for_v(s, p, body)
        s.close()

    def emit_forward_cores(self, s: Src, preloaded: bool):
        def emit():
            for si in range(len(self.segments)):
                self._emit_fwd_seg(s, si, False)
                if preloaded and self.can_preload:
                    paths = [p for p in self.low.paths if p.io in self.segments[si]]
                    self._emit_load_edge(s, f"load_edge_f{si}", self.seg_in1[si], paths)
                    self._emit_fwd_seg(s, si, True)
                if preloaded and self.stage3 is not None:
                    self._emit_fwd_seg(s, si, "lds")

        self._per_chunk(s, emit, in_kernel=False)
        if self.chunk_split:
            emit()  # chunk-agnostic versions, used by the float-atomics kernels

    def _regular_wave(self) -> bool:
        """Every used block is exactly 64 channels per wave-chunk and a row fills the wave."""
        low = self.low
        U = 64 * self.NCH
        return (self.R == 1 and all(low.in1[b].mul == U for b in self.used_in1)
                and all(low.out[io].mul == U for io in self.used_out))

    def _atomics_coalesce(self) -> bool:
        """The sender-gradient atomics of the backward kernel can go through the LDS transpose: rows that fill the
        wave's chunks, or rows of one chunk (or less: several rows to a wave) whatever the multiplicities of their
        blocks."""
        return self._regular_wave() or self.NCH == 1

    def _atomic_block_transposed(self, s: Src, rowexpr: str, off: int, d: int, val: Callable[[int], str],
                                 mul: Optional[int] = None):
        """Atomic accumulation of one [64 x d] channel block. The lane-per-channel registers go
        through a wave-private LDS tile so that every atomic instruction of the wave covers 64
        consecutive elements (two cache lines) instead of 64 elements ``d`` apart. ``mul`` < 64 (rows of one
        chunk only): a block of that many channels, whose mul * d values are consecutive as well."""
        # lanes exchange data through the tile: the wave-scope fences keep the compiler from
        # reordering one lane's reads against its own (different-address) writes
        s("oeq_wave_sync();")
        if self.R == 1 and (mul is None or mul == 64 * self.NCH):
            for k in range(d):
                s(f"s_tr[wave][ul * {d} + {k}] = {val(k)};")
            s("oeq_wave_sync();")
            for t in range(d):
                s(f"oeq_atomic_add({rowexpr} + {off} + chunk * {64 * d} + {t * 64} + ul, s_tr[wave][{t * 64} + ul]);")
            return
        # (rows narrower than the wave: each group of lanes has its own row and its own part of the tile)
        assert self.NCH == 1 and mul <= self.LPR
        lpr = self.LPR
        mine = f"r * {lpr * d} + " if self.R > 1 else ""
        s.open(f"if (ul < {mul})")
        for k in range(d):
            s(f"s_tr[wave][{mine}ul * {d} + {k}] = {val(k)};")
        s.close()
        s("oeq_wave_sync();")
        n = mul * d
        for t in range((n + lpr - 1) // lpr):
            guard = f"if ({t * lpr} + ul < {n}) " if (t + 1) * lpr > n else ""
            s(f"{guard}oeq_atomic_add({rowexpr} + {off} + {t * lpr} + ul, s_tr[wave][{mine}{t * lpr} + ul]);")

    def _store_block_transposed(self, s: Src, rowexpr: str, off: int, d: int, val: Callable[[int], str],
                                nt: bool = False):
        """Store of one [64 x d] channel block through the wave-private LDS tile: every store instruction
        of the wave then writes 64 consecutive elements. Per-lane stores of d contiguous values split into
        16-byte and smaller pieces whose instructions each leave holes in the cache lines they touch."""
        s("oeq_wave_sync();")
        for k in range(d):
            s(f"s_tr[wave][ul * {d} + {k}] = {val(k)};")
        s("oeq_wave_sync();")
        for t in range(d):
            dst = f"{rowexpr} + {off} + chunk * {64 * d} + {t * 64} + ul"
            s(f"__builtin_nontemporal_store(s_tr[wave][{t * 64} + ul], {dst});" if nt
              else f"*({dst}) = s_tr[wave][{t * 64} + ul];")

    def _can_transpose(self, blk, bit: int) -> bool:
        return bool(self.tr_stores & bit) and self.R == 1 and not self.ir_mul and blk.d > 1 \
            and self._full(blk.mul)

    def _store_seg(self, s: Src, si: int, rowexpr: str, guard: str, atomic: bool = False):
        low = self.low
        if atomic and self.tr_atomics:
            for io in self._out_of(self.segments[si]):
                bo = low.out[io]
                self._atomic_block_transposed(s, rowexpr, bo.off, bo.d, lambda k, io=io: f"a.o{io}[{k}]")
            return
        for io in self._out_of(self.segments[si]):
            bo = low.out[io]
            if not atomic and guard == "true" and self._can_transpose(bo, 1):
                self._store_block_transposed(s, rowexpr, bo.off, bo.d, lambda k, io=io: f"a.o{io}[{k}]",
                                             bool(self.nt & 8))
                continue
            self._open_if(s, self._store_cond(bo.mul, guard), [f"a.o{io}[{k}]" for k in range(bo.d)])
            base, st = self._lane_ptr(bo)
            s(f"T* zp = {self._ptr(rowexpr, base)};")
            for k in range(bo.d):
                if atomic:
                    s(f"oeq_atomic_add(zp + {k * st}, a.o{io}[{k}]);")
                elif self.nt & 8:
                    s(f"__builtin_nontemporal_store(a.o{io}[{k}], zp + {k * st});")
                else:
                    s(f"zp[{k * st}] = a.o{io}[{k}];")
            s.close()

    def _zero_untouched_out(self, s: Src, rowexpr: str, guard: str):
        """Output blocks no instruction writes are still part of the row."""
        low = self.low
        for io in self.untouched_out:
            bo = low.out[io]
            s.open(f"if ({guard})")
            s(f"for (int t = ul + chunk * 64; t < {bo.mul * bo.d}; t += {self.LPR} * {self.NCH}) "
              f"({rowexpr})[{bo.off} + t] = T(0);")
            s.close()

    def _lane_prologue(self, s: Src, seg_waves: int = 1):
        """``seg_waves`` > 1: the waves of a node are (chunk, sg) pairs, ``sg`` naming the output segments
        the wave owns."""
        s("const int lane = oeq_lane();")
        s("const int wave = oeq_wave();")
        s(f"const int chunk = wave % {self.NCH};")
        if seg_waves > 1:
            s(f"const int sg = (wave / {self.NCH}) % {seg_waves};")
            s(f"const int g = wave / {self.NCH * seg_waves};")
        else:
            s(f"const int g = wave / {self.NCH};")
        if self.R > 1:
            s(f"const int r = lane / {self.LPR};")
            s(f"const int ul = lane % {self.LPR};")
        else:
            s("const int r = 0;")
            s("const int ul = lane;")
        s("const int u = chunk * 64 + ul;")
        s("(void)r; (void)g; (void)lane;")

    @staticmethod
    def _attrs(block: int, waves_per_eu: int) -> str:
        a = f"__launch_bounds__({block})"
        if waves_per_eu >= 10:
            # two digits: the register budget of the first, at most as many waves as the second
            a += f" __attribute__((amdgpu_waves_per_eu({waves_per_eu // 10}, {waves_per_eu % 10})))"
        elif waves_per_eu > 0:
            # exactly that many waves per SIMD: the register budget of that occupancy, and no more waves than that
            a += f" __attribute__((amdgpu_waves_per_eu({waves_per_eu}, {waves_per_eu})))"
        elif waves_per_eu < 0:
            # at least that many: the same register budget, but a kernel that needs fewer registers runs more waves
            a += f" __attribute__((amdgpu_waves_per_eu({-waves_per_eu})))"
        return a

    # ---------------------------------------------------------- TP forward
    def emit_tp_forward(self, s: Src, G: int, waves_per_eu: int = 0):
        low = self.low
        block = 64 * self.NCH * G
        s.open(
            f'extern "C" __global__ {self._attrs(block, waves_per_eu)} void forward(i64 num_batch, '
            "const T* __restrict__ L1_in, const T* __restrict__ L2_in, const T* __restrict__ W, T* __restrict__ L3_out)"
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
        s(f"const T* yrow = L2_in + rowc * {low.L2};")
        s(f"const T* wrow = W{'' if low.shared_weights else f' + rowc * {low.WN}'};")
        s(f"T* zrow = L3_out + rowc * {low.L3};")
        # a row that fills the wave is live or not for the whole wave: one uniform branch around the body
        # instead of a guard on every store
        live = "live"
        if self.R == 1:
            s.open("if (live)")
            live = "true"
        def row_body():
            s("X_t x;")
            self._load_x(s, "xrow", self.used_in1)
            for si in range(len(self.segments)):
                s.open("")
                s(f"A{si}_t a; zero_seg{si}(a);")
                s(f"fwd_seg{si}{self._sfx()}(x, yrow, wrow, u, a);")
                self._store_seg(s, si, "zrow", live)
                s.close()

        self._per_chunk(s, row_body)
        self._zero_untouched_out(s, "zrow", live)
        if self.R == 1:
            s.close()
        s.close()
        s.close()
        return block

    # ---------------------------------------------------------- conv forward
    def _edge_loop(self, s: Src, first: str, last: str, load: Callable[[str, str], None],
                   compute: Callable[[str, str], None], pipelined: int, before_edge: Callable[[str], None] = None):
        """Walk edges ``first, first+R, ... < last``. Pipelined: two operand
        sets (A, B); the next edge's loads are issued before the current edge is
        computed. ``load(buf, e)`` / ``compute(buf, e)`` emit code."""
        R = self.R
        # The compiler takes a direct global->LDS load to write only the bytes at the pointer it is given,
        # not the 64 lanes' worth behind it, so it would move reads of the staging buffer across the load
        # or across the wait for it. The empty asm statements pin them: no memory access crosses one.
        fence = 'asm volatile("" ::: "memory");'

        def vmcnt(n: int) -> str:
            # s_waitcnt with only vmcnt set (gfx9 encoding: vmcnt = simm16[3:0] | simm16[15:14] << 4)
            return f"__builtin_amdgcn_s_waitcnt({(n & 15) | 0x0F70 | ((n >> 4) << 14)}); /* vmcnt({n}) */ {fence}"

        # lgkmcnt(0): LDS reads retired before the buffer is refilled
        lgkm0 = f"{fence} __builtin_amdgcn_s_waitcnt(0xC07F); {fence}"
        if pipelined == 3:
            # Two LDS buffers per wave, loads one edge ahead. Stores and atomics of the loop body share
            # the vector-memory counter, so the wait before an edge is for everything outstanding.
            s(f"i64 e = {first};")
            s.open(f"if (e < {last})")
            self._emit_stage3_issue(s, "A", "e")
            s.close()
            s.open(f"while (e < {last})")
            s("const i64 en = e + 1;")
            s(vmcnt(0))
            s.open(f"if (en < {last})")
            self._emit_stage3_issue(s, "B", "en")
            s.close()
            if before_edge:
                before_edge("e")
            compute("A", "e")
            s(lgkm0)
            s.open(f"if (en < {last})")
            s(vmcnt(0))
            s.open(f"if (e + 2 < {last})")
            self._emit_stage3_issue(s, "A", "e + 2")
            s.close()
            if before_edge:
                before_edge("en")
            compute("B", "en")
            s(lgkm0)
            s.close()
            s("e += 2;")
            s.close()
            return
        if pipelined == 4:
            # As below (one staging buffer, copied to registers), with the weights two edges ahead in a second
            # weight buffer: while edge e is computed, X / Y of e+1 and the weights of e+1 and e+2 are in
            # flight, 16 KB per wave at the MACE shape instead of 10. With 8 waves per CU one edge of prefetch
            # keeps too few bytes in flight to fill the memory system (the forward with its arithmetic taken
            # out ran no faster). Vector-memory results return in issue order, so waiting until only the
            # youngest weight loads are outstanding means everything of edge e has arrived.
            nqw = self.stage["nqw"]
            s(f"T yn[{self.q_slabs if self.use_q else self.low.L2}];")
            s(f"i64 e = {first};")
            s("int wpar = 0;")
            s.open(f"if (e < {last})")
            self._emit_stage_issue(s, "e", x=True, w=True, wbuf="0")
            s.open(f"if (e + 1 < {last})")
            self._emit_stage_issue(s, "e + 1", x=False, w=True, wbuf="1")
            s.close()
            s.close()
            s.open(f"while (e < {last})")
            s.open(f"if (e + 1 < {last})")
            s(vmcnt(nqw))
            s.close()
            s.open("else")
            s(vmcnt(0))
            s.close()
            self._emit_stage_read(s, "A", wbuf="wpar")
            s(lgkm0)
            s.open(f"if (e + 1 < {last})")
            self._emit_stage_issue(s, "e + 1", x=True, w=False)
            s.open(f"if (e + 2 < {last})")
            self._emit_stage_issue(s, "e + 2", x=False, w=True, wbuf="wpar")
            s.close()
            s.close()
            if before_edge:
                before_edge("e")
            compute("A", "e")
            s("++e; wpar ^= 1;")
            s.close()
            return
        if pipelined == 2:
            # one LDS buffer per wave, copied to registers before the next edge's loads are issued
            s(f"T yn[{self.q_slabs if self.use_q else self.low.L2}];")
            s(f"i64 e = {first};")
            s.open(f"if (e < {last})")
            self._emit_stage_issue(s, "e")
            s.close()
            s.open(f"while (e < {last})")
            s(vmcnt(0))
            self._emit_stage_read(s, "A")
            s(lgkm0)
            s.open(f"if (e + 1 < {last})")
            self._emit_stage_issue(s, "e + 1")
            s.close()
            if before_edge:
                before_edge("e")
            compute("A", "e")
            s("++e;")
            s.close()
            return
        if not pipelined:
            s.open(f"for (i64 e = {first}; e < {last}; e += {R})")
            if before_edge:
                before_edge("e")
            load("A", "e")
            compute("A", "e")
            s.close()
            return
        s(f"i64 e = {first};")
        s.open(f"if (e < {last})")
        load("A", "e")
        s.close()
        s.open(f"while (e < {last})")
        s(f"const i64 en = e + {R};")
        s.open(f"if (en < {last})")
        load("B", "en")
        s.close()
        if before_edge:
            before_edge("e")
        compute("A", "e")
        s.open(f"if (en < {last})")
        s(f"const i64 en2 = en + {R};")
        s.open(f"if (en2 < {last})")
        load("A", "en2")
        s.close()
        if before_edge:
            before_edge("en")
        compute("B", "en")
        s.close()
        s(f"e += {2 * R};")
        s.close()

    def _edge_mode(self, pipelined: int) -> int:
        """0: load, then compute; 1: next edge's operands prefetched into a second register set;
        2: next edge's operands prefetched into the wave's LDS staging buffer."""
        if pipelined == 3 and self.stage3 is not None and not self.use_q:
            return 3
        if pipelined == 4 and self.stage is not None and self.R == 1:
            return 4
        if pipelined >= 2 and self.stage is not None:
            return 2
        if pipelined and self.can_preload:
            return 1
        return 0

    # Trailing parameters of every kernel that walks receivers: the table of long edge segments cut into
    # chunks (see _node_loop_open). Forward-shaped kernels also take the rows that the extra chunks write.
    HUB_PARAMS = (", const i64* __restrict__ hubptr, const i64* __restrict__ hubnode, i64 hub_limit, "
                  "i64 hub_units")
    HUB_ROWS_PARAM = ", T* __restrict__ hub_rows"

    def _node_loop_open(self, s: Src, G: int, xcd: int):
        """One wave group per walk position. A position is a receiver node with its edge segment, or, for
        a node with more than ``hub_limit`` edges, one chunk of that many edges: the first chunk is the
        node's own position, the others are listed in ``hubnode`` (``hubptr[v]`` = first extra position of
        node v, ``hubptr[node_count]`` = their number) and take the first ``hub_units`` positions of the
        grid, so that a hub's chunks start early and run side by side instead of one wave walking tens of
        thousands of edges (the role of the reference's fixup_forward scheme,
        templates/loop_unroll_conv_det.cuh:34-66, 96-179, which cuts the edge list into equal ranges).
        Leaves ``node``, ``e0``, ``e1`` and ``hubpos`` (the extra position, -1 for a node's own) in scope.
        Workgroups are handed to the XCDs round-robin; with ``xcd`` > 1 (grid a multiple of it, and so is
        the number of blocks the extra positions take) block ids are remapped so that each XCD walks one
        contiguous range of nodes and neighbouring receivers share their senders' rows through that
        XCD's L2."""
        # ``order`` (may be NULL) lists the nodes in the order in which they are to be walked: nodes that
        # share senders next to each other, so that the blocks resident on one XCD gather from a small set
        # of sender rows (the library derives it from the graph at every index build).
        s("const i64 walk_end = hub_units + node_count;")
        if xcd > 1:
            s(f"const i64 hub_blocks = hub_units / {G};")
            s(f"const i64 vper = ((i64)gridDim.x - hub_blocks) / {xcd};")
            s(f"const i64 nblk = (i64)blockIdx.x - hub_blocks;")
            s(f"const i64 vblk = (nblk % {xcd}) * vper + nblk / {xcd};")
            s(f"const i64 wpos0 = (nblk < 0 ? (i64)blockIdx.x : hub_blocks + vblk) * {G} + g;")
            s.open("for (i64 wpos = wpos0; wpos < walk_end; wpos += walk_end + 1)")
        else:
            s.open(f"for (i64 wpos = (i64)blockIdx.x * {G} + g; wpos < walk_end; wpos += (i64)gridDim.x * {G})")
        s("i64 node, e0, e1, hubpos = -1;")
        s.open("if (wpos < hub_units)")
        s("if (wpos >= hubptr[node_count]) continue;")
        s("hubpos = wpos;")
        s("node = oeq_idx(hubnode[wpos], node_count);")
        s("e0 = oeq_pos(rowptr[node] + (wpos - hubptr[node] + 1) * hub_limit, nnz);")
        s("e1 = oeq_pos(rowptr[node + 1], nnz);")
        s("if (e1 - e0 > hub_limit) e1 = e0 + hub_limit;")
        s.close()
        s.open("else")
        s("const i64 vnode = wpos - hub_units;")
        s("node = order ? order[vnode] : vnode;")
        s("e0 = oeq_pos(rowptr[node], nnz);")
        s("e1 = oeq_pos(rowptr[node + 1], nnz);")
        s("if (hub_limit > 0 && e1 - e0 > hub_limit) e1 = e0 + hub_limit;")
        s.close()

    def emit_conv_forward(self, s: Src, G: int, deterministic: bool, pipelined: bool, waves_per_eu: int = 0,
                          xcd: int = 1, tr_atomics: bool = True, name: str = "forward"):
        low = self.low
        # With several output segments the waves of a node can each own some of them (their accumulators
        # stay in registers) and walk the node's edges side by side, instead of one wave walking the edges
        # once per segment.
        segw = self.seg_waves if deterministic else 1
        block = 64 * self.NCH * G * segw
        R = self.R
        # weights two edges ahead: only where the loop body issues no stores or atomics (they share the
        # vector-memory counter with the loads the loop waits for by count)
        mode = self._edge_mode(pipelined if (deterministic or pipelined != 4) else 2)
        s.open(
            f'extern "C" __global__ {self._attrs(block, waves_per_eu)} void {name}(i64 node_count, i64 nnz, '
            "const T* __restrict__ L1_in, const T* __restrict__ L2_in, const T* __restrict__ W, "
            "T* __restrict__ L3_out, const i64* __restrict__ rows, const i64* __restrict__ cols, "
            f"const i64* __restrict__ rowptr, const i64* __restrict__ eperm, const i64* __restrict__ order"
            f"{self.HUB_PARAMS}{self.HUB_ROWS_PARAM})"
        )
        self._lane_prologue(s, segw)
        if self.use_q:
            self._emit_q_prologue(s, block // 64)
        if self.can_preload:
            s("E_t A, B;")
        if mode in (2, 4):
            floats = self.stage["floats"] + (self.stage["nqw"] * 256 if mode == 4 else 0)
            s(f"__shared__ __attribute__((aligned(16))) T s_stage[{self.NCH * G}][{floats}];")
            self._emit_stage_offsets(s)
        if mode == 3:
            for b in "AB":
                s(f"__shared__ __attribute__((aligned(16))) T s_stage{b}[{self.NCH * G}][{self.stage3['floats']}];")
            self._emit_stage3_offsets(s)
        self.tr_atomics = (not deterministic) and tr_atomics and self._regular_wave() and not self.ir_mul
        if self.tr_atomics or (self.tr_stores & 1 and self.R == 1):
            s(f"__shared__ T s_tr[{self.NCH * G * segw}][{64 * max(low.out[io].d for io in self.used_out)}];")

        def make_load(si):
            def load(buf, e):
                if self.can_preload:
                    s(f"load_edge_f{si}{self._sfx()}({buf}, OEQ_EDGE({e}), L1_in, L2_in, W, cols, node_count, u{self._qarg()});")
            return load

        kahan = self.kahan and deterministic
        acc = "c" if kahan else "a"

        def make_compute(si):
            def compute(buf, e):
                inner(si, buf, e)
                if kahan:
                    s(f"kahan_seg{si}(c, a);")
            return compute

        def inner(si, buf, e):
            if mode == 3:
                s(f"fwd_seg{si}_lds{self._sfx()}(&s_stage{buf}[wave][0], ul, {acc});")
            elif self.can_preload:
                if self.use_q:
                    self._emit_q_build(s, f"{buf}.yq")
                s(f"fwd_seg{si}_pre{self._sfx()}({buf}, {'sq, ' if self.use_q else ''}{acc});")
            else:
                s.open("")
                s(f"const i64 eid = OEQ_EDGE({e});")
                s(f"const T* xrow = L1_in + oeq_idx(cols[eid], node_count) * {low.L1};")
                s(f"const T* yrow = L2_in + eid * {low.L2};")
                s(f"const T* wrow = W{'' if low.shared_weights else f' + eid * {low.WN}'};")
                s("X_t x;")
                self._load_x(s, "xrow", self.seg_in1[si])
                s(f"fwd_seg{si}{self._sfx()}(x, yrow, wrow, u, {acc});")
                s.close()

        if deterministic:
            self._node_loop_open(s, G, xcd)
            s(f"T* zrow = hubpos >= 0 ? hub_rows + hubpos * {low.L3} : L3_out + node * {low.L3};")
            for si in range(len(self.segments)):
                s.open(f"if (sg == {si % segw})" if segw > 1 else "")

                def node_body(si=si):
                    if self.cur_chunk is not None and not self._out_of(self.segments[si]):
                        return  # this chunk has no channel of the segment's blocks
                    s(f"A{si}_t a; zero_seg{si}(a);")
                    if kahan:
                        s(f"A{si}_t c; zero_seg{si}(c);")
                    self._edge_loop(s, "e0 + r", "e1", make_load(si), make_compute(si), mode)
                    if R > 1:
                        # fold the R lane groups (fixed order) into group 0
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
        else:
            # contiguous edge range per wave group; flush with atomics whenever the receiver changes
            s(f"const i64 ngrp = (i64)gridDim.x * {G};")
            s("const i64 per = (nnz + ngrp - 1) / ngrp;")
            s(f"const i64 eb = ((i64)blockIdx.x * {G} + g) * per;")
            s("const i64 ee = (eb + per < nnz) ? eb + per : nnz;")
            for si in range(len(self.segments)):
                s.open("")
                s(f"A{si}_t a; zero_seg{si}(a);")
                s("i64 cur = -1;")

                def before_edge(e, si=si):
                    s.open("")
                    s(f"const i64 row = oeq_idx(rows[OEQ_EDGE({e})], node_count);")
                    s.open("if (row != cur)")
                    s.open("if (cur >= 0)")
                    s(f"T* zrow = L3_out + cur * {low.L3};")
                    self._store_seg(s, si, "zrow", "true", atomic=True)
                    s.close()
                    s(f"zero_seg{si}(a);")
                    s("cur = row;")
                    s.close()
                    s.close()

                self._edge_loop(s, "eb + r", "ee", make_load(si), make_compute(si), mode, before_edge)
                s.open("if (cur >= 0)")
                s(f"T* zrow = L3_out + cur * {low.L3};")
                self._store_seg(s, si, "zrow", "true", atomic=True)
                s.close()
                s.close()
        s.close()
        return block

    # ------------------------------------------------------- backward pieces
    def _load_g(self, s: Src, rowexpr: str, ios: List[int], dst: str = "gr"):
        low = self.low
        for io in self._out_of(ios):
            bo = low.out[io]
            s.open("")
            base, st = self._lane_ptr(bo)
            s(f"const T* gp = {self._gptr(rowexpr, base, bo.mul)};")
            for k in range(bo.d):
                ld = f"__builtin_nontemporal_load(gp + {k * st})" if self.nt & 8 else f"gp[{k * st}]"
                s(f"{dst}.o{io}[{k}] = {ld};")
            s.close()

    def _bwd_paths(self, s: Src, *, xname: str, yacc, wacc, g_on_demand_row: Optional[str] = None,
                   dw_mode: str = "store", g_guard: Optional[str] = None, dw_guard: Optional[str] = None,
                   paths: Optional[List[Path]] = None):
        """Straight-line backward of all paths. In scope: ``xname`` (X_t), dx (X_t),
        dy[], u, and either gr (G_t, resident) or a row pointer to load output
        gradients from. dw_mode 'store': dwrow[...] = v; 'acc': dwacc[slot] += v."""
        low = self.low
        ordered = sorted(self._paths(paths), key=lambda q: (q.io, q.index))
        since_fence = 0
        # On-demand gradients with fences: the paths between two fences form a run. With prefetch_runs the
        # gradient (and weight) values of run k+1 are requested at the start of run k, into variables named
        # per path, so that a run computes while the next one's loads are in flight; without it every run
        # starts with an exposed memory round trip.
        prefetch = (self.prefetch_runs and self.sched_fence and g_on_demand_row is not None
                    and all(low.in2[q.i2].mul <= UNROLL_V_LIMIT for q in ordered))
        runs: List[List[Path]] = []
        if prefetch:
            cur, words = [], 0
            for q in ordered:
                dq = low.out[q.io].d * self.words
                if cur and words + dq > self.fence_words:
                    runs.append(cur)
                    cur, words = [], 0
                cur.append(q)
                words += dq
            runs.append(cur)

        def emit_run_loads(run):
            for q in run:
                bo_q = low.out[q.io]
                s(f"T gk{q.index}[{bo_q.d}];")
                s.open("")
                base, st = self._lane_ptr(bo_q)
                s(f"const T* gp = {self._gptr(g_on_demand_row, base, bo_q.mul)};")
                for k in range(bo_q.d):
                    ld = f"__builtin_nontemporal_load(gp + {k * st})" if self.nt & 8 else f"gp[{k * st}]"
                    s(f"gk{q.index}[{k}] = {self._guarded(ld, g_guard)};")
                s.close()
                for v in range(low.in2[q.i2].mul):
                    s(f"const T wv{q.index}_{v} = {wacc(q, str(v))};")

        run_of = {q.index: ri for ri, run in enumerate(runs) for q in run}
        if prefetch:
            emit_run_loads(runs[0])
        if self.use_q:
            qplan = self._q_fetch_plan(ordered, self.q_ahead[1])
            self._emit_q_raw_y(s)
        for n_path, p in enumerate(ordered):
            b1, b2, bo = low.in1[p.i1], low.in2[p.i2], low.out[p.io]
            V = b2.mul
            s(f"// path {p.index}: l=({b1.l},{b2.l},{bo.l})")
            if self.use_q:
                self._emit_q_fetch(s, qplan[n_path])
            if prefetch and runs[run_of[p.index]][0] is p and run_of[p.index] + 1 < len(runs):
                emit_run_loads(runs[run_of[p.index] + 1])
            s.open("")
            if prefetch:
                gname = lambda k, idx=p.index: f"gk{idx}[{k}]"
            elif g_on_demand_row is not None:
                s(f"T gk[{bo.d}];")
                s.open("")
                base, st = self._lane_ptr(bo)
                s(f"const T* gp = {self._gptr(g_on_demand_row, base, bo.mul)};")
                for k in range(bo.d):
                    ld = f"__builtin_nontemporal_load(gp + {k * st})" if self.nt & 8 else f"gp[{k * st}]"
                    s(f"gk[{k}] = {self._guarded(ld, g_guard)};")
                s.close()
                gname = lambda k: f"gk[{k}]"
            else:
                gname = lambda k, io=p.io: f"gr.o{io}[{k}]"
            base_slot = self.wslot[p.index]

            def body(v, p=p, b1=b1, b2=b2, V=V, gname=gname, base_slot=base_slot):
                ks = sorted({k for _, _, k, _ in p.nnz})
                js = sorted({j for _, j, _, _ in p.nnz})
                # dX: dx_i += c * y_j * g_k * w. As in the forward pass the coefficient rides on the factor
                # with the fewest distinct (|c|, index) pairs - Y, the weighted gradient, or (after summing the
                # +-y_j*g_k of equal |c|) the result - and the weight on the gradient values or on the coefficient.
                cj, ci, ck, nc = self._form_counts(p)
                nz = len(p.nnz)
                form = 0
                if self.forms and not self.use_q:
                    costs = [cj + min(len(ks), nc) + nz, ck + min(len(ks), nc) + nz, nz + nc + ci]
                    form = costs.index(min(costs))
                    if form < 2 and nc < len(ks):
                        form += 3  # weight folded into the coefficient instead of into the gradient values
                wv_expr = f"wv{p.index}_{v}" if prefetch else wacc(p, v)
                if form == 0:
                    prods = self._products(s, p, v, yacc)
                    s(f"const T wv = {wv_expr};")
                    for k in ks:
                        s(f"const T gw{k} = {gname(k)} * wv;")
                    for n, (i, j, k, c) in enumerate(p.nnz):
                        q, neg = prods[n]
                        s(f"dx.b{p.i1}[{i}] {'-=' if neg else '+='} {q} * gw{k};")
                else:
                    self._y_values(s, p, v, yacc)
                    s(f"const T wv = {wv_expr};")
                    if form == 1:
                        for k in ks:
                            s(f"const T gw{k} = {gname(k)} * wv;")
                        prods = self._scaled(s, p, 2, lambda k: f"gw{k}", "qg")
                        other = lambda j, k: f"y{j}"
                    elif form == 3:
                        prods = self._scaled(s, p, 1, lambda j: f"y{j}", "q", weight="wv")
                        other = lambda j, k: gname(k)
                    elif form == 4:
                        prods = self._scaled(s, p, 2, gname, "qg", weight="wv")
                        other = lambda j, k: f"y{j}"
                    if form == 2:
                        sums = {}
                        for i, j, k, c in p.nnz:
                            key = (self.lit(abs(c)), i)
                            term = f"y{j} * {gname(k)}"
                            if key not in sums:
                                sums[key] = f"sx{len(sums)}"
                                s(f"T {sums[key]} = {'-' if c < 0 else ''}{term};")
                            else:
                                s(f"{sums[key]} {'-=' if c < 0 else '+='} {term};")
                        cw = {}
                        for (m, i), name in sums.items():
                            if m not in cw:
                                cw[m] = f"cw{len(cw)}"
                                s(f"const T {cw[m]} = T({m}) * wv;")
                            s(f"dx.b{p.i1}[{i}] += {cw[m]} * {name};")
                    else:
                        for n, (i, j, k, c) in enumerate(p.nnz):
                            q, neg = prods[n]
                            s(f"dx.b{p.i1}[{i}] {'-=' if neg else '+='} {q} * {other(j, k)};")
                # h_j = sum_ik c x_i g_k is the unweighted dY term of this lane; it also gives
                # dW = sum_j y_j h_j, so the forward contraction need not be recomputed
                pair, hstart = {}, set()
                for n, (i, j, k, c) in enumerate(p.nnz):
                    if (i, k) not in pair:
                        pair[(i, k)] = f"xg{len(pair)}"
                        s(f"const T {pair[(i, k)]} = {self._xv(xname, p.i1, i)} * {gname(k)};")
                    if j not in hstart:
                        s(f"T h{j} = T({self.lit(c)}) * {pair[(i, k)]};")
                        hstart.add(j)
                    else:
                        s(f"h{j} += T({self.lit(c)}) * {pair[(i, k)]};")
                s(f"T dwv = y{js[0]} * h{js[0]};")
                for j in js[1:]:
                    s(f"dwv += y{j} * h{j};")
                if dw_mode == "store" and self._dw_deferred(dw_guard):
                    s(f"dwkeep[{base_slot} + {v}] = dwv;")
                elif dw_mode == "store":
                    dwp = self._dump_unless(self._store_cond(b1.mul, dw_guard),
                                            self._ptr("dwrow", (f"{p.woff} + ({v})", V)))
                    s(f"__builtin_nontemporal_store(dwv, {dwp});" if self.nt & 2 else f"*{dwp} = dwv;")
                else:
                    s(f"dwacc[{base_slot} + {v}] += dwv;")
                for j in js:
                    s(f"dy[{self._y_index(b2, v, j)}] += wv * h{j};")

            self._for_v(s, p, body)
            s.close()
            if prefetch:
                if runs[run_of[p.index]][-1] is p:
                    s("__builtin_amdgcn_sched_barrier(0);")
            elif self.sched_fence and g_on_demand_row is not None:
                # keep the scheduler from hoisting all later paths' gradient loads over this path (with
                # many paths that costs more registers than a wave has): a fence after every run of
                # paths whose gradients take about ``fence_words`` registers, so that each run's loads
                # still go out together
                since_fence += bo.d * self.words
                nxt = ordered[n_path + 1] if n_path + 1 < len(ordered) else None
                if nxt is None or since_fence + low.out[nxt.io].d * self.words > self.fence_words:
                    s("__builtin_amdgcn_sched_barrier(0);")
                    since_fence = 0

    def _dw_deferred(self, dw_guard: Optional[str]) -> bool:
        """Per-row weight gradients whose store needs a condition are kept in registers (``dwkeep``) and
        stored after the last path: a conditional store inside the chain of paths splits it into many
        basic blocks, and the compiler then moves the dY/dX accumulations to the end of the row, keeping
        every path's operands alive until there (hundreds of registers for problems with many paths)."""
        needs_cond = any(self._store_cond(self.low.in1[p.i1].mul, dw_guard) for p in self._paths())
        return needs_cond and self.can_preload

    def _pin_gradients(self, s: Src, blocks: List[int], deferred: bool, paths: Optional[List[Path]] = None):
        """After the last path of a row / edge: pass every gradient accumulator through an empty asm
        statement. What follows (conditional stores, the dY reduction) has branches, and the compiler
        would otherwise move the accumulation chains below them, keeping every path's operands alive
        until there."""
        low = self.low
        vals = [f"dx.b{b}[{i}]" for b in self._in1_of(blocks) for i in range(low.in1[b].d)]
        vals += [f"dy[{t}]" for t in range(self.l2_pad)]
        if deferred:
            for p in self._paths(paths):
                vals += [f"dwkeep[{self.wslot[p.index] + v}]" for v in range(low.in2[p.i2].mul)]
        for v in vals:
            s(f'asm volatile("" : "+v"({v}));')

    def _flush_dwkeep(self, s: Src, dw_guard: Optional[str]):
        low = self.low
        for p in self._paths():
            b1, V = low.in1[p.i1], low.in2[p.i2].mul
            self._open_if(s, self._store_cond(b1.mul, dw_guard),
                          [f"dwkeep[{self.wslot[p.index] + v}]" for v in range(V)])
            for v in range(V):
                dwp = self._ptr("dwrow", (f"{p.woff} + {v}", V))
                val = f"dwkeep[{self.wslot[p.index] + v}]"
                s(f"__builtin_nontemporal_store({val}, {dwp});" if self.nt & 2 else f"*{dwp} = {val};")
            s.close()

    def _dy_reduce(self, s: Src):
        """Halving butterfly over the lanes of one row. Leaves, in every lane,
        ``rv[0..cur)`` = totals of dy indices ``dyidx + j``; lanes with
        ``(ul & dup) != 0`` hold copies. Returns (cur, dup)."""
        n = self.l2_pad
        s(f"T rv[{n}];")
        for j in range(n):
            s(f"rv[{j}] = dy[{j}];")
        s("int dyidx = 0;")
        cur, dup = n, 0
        m = self.LPR // 2
        while m >= 1:
            if cur > 1:
                half = cur // 2
                s.open("")
                s(f"const bool hi = (ul & {m}) != 0;")
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
        return cur, dup

    def _dy_finish(self, s: Src, dst_row: str, live: str):
        """Cross-lane (and cross-chunk) reduction of dy, then write of the row."""
        low = self.low
        s.open("")
        cur, dup = self._dy_reduce(s)
        if self.NCH == 1:
            s.open(f"if ({live} && (ul & {dup}) == 0)")
            for j in range(cur):
                s(f"if (dyidx + {j} < {low.L2}) ({dst_row})[dyidx + {j}] = rv[{j}];")
            s.close()
        else:
            assert self.R == 1
            s.open(f"if ((ul & {dup}) == 0)")
            for j in range(cur):
                s(f"s_dy[g][chunk][dyidx + {j}] = rv[{j}];")
            s.close()
            s("__syncthreads();")
            s.open(f"if (chunk == 0 && {live})")
            s.open(f"for (int j = lane; j < {low.L2}; j += 64)")
            s("T tot = s_dy[g][0][j];")
            s(f"for (int cc = 1; cc < {self.NCH}; ++cc) tot += s_dy[g][cc][j];")
            s(f"({dst_row})[j] = tot;")
            s.close()
            s.close()
            s("__syncthreads();")
        s.close()

    def _store_dx(self, s: Src, rowexpr: str, guard: str, atomic: bool = False, nt: bool = False):
        low = self.low
        if atomic and self.tr_atomics:
            for b in self._in1_of(self.used_in1):
                blk = low.in1[b]
                self._atomic_block_transposed(s, rowexpr, blk.off, blk.d, lambda i, b=b: f"dx.b{b}[{i}]", blk.mul)
            return
        for b in self._in1_of(self.used_in1):
            blk = low.in1[b]
            if not atomic and guard == "true" and self._can_transpose(blk, 2):
                self._store_block_transposed(s, rowexpr, blk.off, blk.d, lambda i, b=b: f"dx.b{b}[{i}]", nt)
                continue
            self._open_if(s, self._store_cond(blk.mul, guard), [f"dx.b{b}[{i}]" for i in range(blk.d)])
            base, st = self._lane_ptr(blk)
            s(f"T* dp = {self._ptr(rowexpr, base)};")
            for i in range(blk.d):
                if atomic:
                    s(f"oeq_atomic_add(dp + {i * st}, dx.b{b}[{i}]);")
                elif nt:
                    s(f"__builtin_nontemporal_store(dx.b{b}[{i}], dp + {i * st});")
                else:
                    s(f"dp[{i * st}] = dx.b{b}[{i}];")
            s.close()

    def _term_slots(self):
        """Position of (input block, component) in a wave's lane-major slice of a per-edge dX term row:
        value (b, i) of lane ``ul`` sits at ``chunk * 64 * n + slot * 64 + ul`` (n = number of slots), so
        every store or load instruction of the wave covers 64 consecutive elements."""
        slots, n = {}, 0
        for b in self.used_in1:
            for i in range(self.low.in1[b].d):
                slots[(b, i)] = n
                n += 1
        return slots, n

    def _term_ptr(self, rowexpr: str, slot: int, n: int) -> str:
        return f"oeq_at({rowexpr} + chunk * {64 * n} + {slot * 64}, (unsigned)ul * {self.low.elem_size}u)"

    def _store_terms(self, s: Src, rowexpr: str):
        slots, n = self._term_slots()
        for (b, i), slot in slots.items():
            ptr = self._term_ptr(rowexpr, slot, n)
            s(f"*{ptr} = dx.b{b}[{i}];")

    def _load_terms(self, s: Src, rowexpr: str, dst: str):
        slots, n = self._term_slots()
        for (b, i), slot in slots.items():
            ptr = self._term_ptr(rowexpr, slot, n)
            s(f"{dst}.b{b}[{i}] = *{ptr};")

    def _arrivals(self, s: Src):
        """After a wave has stored the dX terms of its node's edges: make them visible to the device,
        count one arrival per edge at the edge's sender (one counter per sender and channel chunk), and
        for every sender whose count is now complete sum its terms in ``sperm`` order and write its row.
        The last arrival is whichever wave happens to come last; the sum it forms does not depend on that."""
        low = self.low
        s("__threadfence();")  # release: this wave's terms before its arrivals
        s.open("for (i64 eb = e0; eb < e1; eb += 64)")
        s("const i64 ea = eb + lane;")
        s("i64 sn = 0; bool last = false;")
        s.open("if (ea < e1)")
        s("sn = oeq_idx(cols[OEQ_EDGE(ea)], node_count);")
        s(f"const int seen = __hip_atomic_fetch_add(arrivals + sn * {self.NCH} + chunk, 1, __ATOMIC_RELAXED, "
          "__HIP_MEMORY_SCOPE_AGENT) + 1;")
        s("last = seen == (int)(colptr[sn + 1] - colptr[sn]);")
        s.close()
        s("unsigned long long todo = __ballot(last);")
        s.open("while (todo)")
        s("const int src_lane = __ffsll((long long)todo) - 1;")
        s("todo &= todo - 1;")
        s("const i64 snd = ((i64)__builtin_amdgcn_readlane((int)(sn >> 32), src_lane) << 32) | "
          "(unsigned)__builtin_amdgcn_readlane((int)sn, src_lane);")
        s("__threadfence();")  # acquire: the other waves' terms after their arrivals
        s("X_t tot;")
        self._zero_x(s, "tot")
        s("const i64 j0 = oeq_pos(colptr[snd], nnz), j1 = oeq_pos(colptr[snd + 1], nnz);")
        # the additions stay in list order; unrolling only lets several rows be in flight at a time
        s("#pragma unroll 4")
        s.open("for (i64 j = j0; j < j1; ++j)")
        s(f"const T* trow = dx_tmp + oeq_idx(sperm[j], nnz) * {low.L1};")
        s("X_t t;")
        self._load_terms(s, "trow", "t")
        for b in self._in1_of(self.used_in1):
            for i in range(low.in1[b].d):
                s(f"tot.b{b}[{i}] += t.b{b}[{i}];")
        s.close()
        s(f"T* orow = L1_grad + snd * {low.L1};")
        s.open("")
        s("X_t& dx = tot;")
        self._store_dx(s, "orow", "true")
        s.close()
        s.close()
        s.close()

    def _zero_untouched_in1(self, s: Src, rowexpr: str, guard: str):
        low = self.low
        for b in range(len(low.in1)):
            if b in self.used_in1:
                continue
            blk = low.in1[b]
            s.open(f"if ({guard})")
            s(f"for (int t = ul + chunk * 64; t < {blk.mul * blk.d}; t += {self.LPR} * {self.NCH}) "
              f"({rowexpr})[{blk.off} + t] = T(0);")
            s.close()

    def _zero_x(self, s: Src, name: str):
        for b in self._in1_of(self.used_in1):
            for i in range(self.low.in1[b].d):
                s(f"{name}.b{b}[{i}] = T(0);")

    def _dw_slots(self):
        return [(p, self.wslot[p.index]) for p in self.low.paths]

    # ---------------------------------------------------------- TP backward
    def emit_tp_backward(self, s: Src, G: int, waves_per_eu: int = 0, g_resident: bool = False):
        low = self.low
        if self.NCH > 1:
            G = 1  # one row per block: the dY reduction across chunk waves uses block barriers
        block = 64 * self.NCH * G
        shared = low.shared_weights
        s.open(
            f'extern "C" __global__ {self._attrs(block, waves_per_eu)} void backward(i64 num_batch, '
            "const T* __restrict__ L1_in, T* __restrict__ L1_grad, const T* __restrict__ L2_in, "
            "T* __restrict__ L2_grad, const T* __restrict__ W, T* __restrict__ W_grad, "
            "const T* __restrict__ L3_grad, T* __restrict__ wpartial)"
        )
        self._lane_prologue(s)
        if self.NCH > 1:
            s(f"__shared__ T s_dy[{G}][{self.NCH}][{self.l2_pad}];")
        if self.tr_stores & 2 and self.R == 1:
            s(f"__shared__ T s_tr[{self.NCH * G}][{64 * max(b.d for b in low.in1)}];")
        if shared:
            s(f"T dwacc[{self.n_wslots}];")
            s(f"for (int t = 0; t < {self.n_wslots}; ++t) dwacc[t] = T(0);")
        s(f"const i64 ngroups = (num_batch + {self.R - 1}) / {self.R};")
        # uniform trip count per block: the dY reduction contains block barriers
        s.open(f"for (i64 base = (i64)blockIdx.x * {G}; base < ngroups; base += (i64)gridDim.x * {G})")
        s("const i64 grp = base + g;")
        s(f"const i64 row = grp * {self.R} + r;")
        s("const bool live = row < num_batch;")
        s("const i64 rowc = live ? row : num_batch - 1;")
        s(f"const T* xrow = L1_in + rowc * {low.L1};")
        s(f"const T* yrow = L2_in + rowc * {low.L2};")
        s(f"const T* wrow = W{'' if shared else f' + rowc * {low.WN}'};")
        s(f"const T* grow = L3_grad + rowc * {low.L3};")
        if not shared:
            s(f"T* dwrow = W_grad + rowc * {low.WN};")
        # Rows past the end of the batch are clamped duplicates. A row that fills the wave is live or not
        # for the whole wave (and, with one row per block, for the whole block, barriers included): one
        # uniform branch around the body. Packed rows keep per-lane guards: gradients zeroed (shared
        # weights) and no result stored.
        live = "live"
        if self.R == 1:
            s.open("if (live)")
            live = "true"
        def row_body():
            s("X_t x, dx;")
            self._load_x(s, "xrow", self.used_in1)
            self._zero_x(s, "dx")
            s(f"T dy[{self.l2_pad}];")
            s(f"for (int t = 0; t < {self.l2_pad}; ++t) dy[t] = T(0);")
            yacc, wacc = self._acc_pointer()
            deferred = not shared and self._dw_deferred(live)
            if deferred:
                s(f"T dwkeep[{self.n_wslots}];")
            if g_resident and not shared:
                # the whole output-gradient slice is requested up front, together with X and W: one long
                # burst of loads per row instead of a load-wait-compute round per path
                s("G_t gr;")
                self._load_g(s, "grow", self.used_out)
                self._bwd_paths(s, xname="x", yacc=yacc, wacc=wacc, dw_mode="store", dw_guard=live)
            else:
                self._bwd_paths(s, xname="x", yacc=yacc, wacc=wacc, g_on_demand_row="grow",
                                dw_mode="acc" if shared else "store",
                                g_guard="live" if shared and self.R > 1 else None, dw_guard=live)
            self._pin_gradients(s, self.used_in1, deferred)
            if deferred:
                self._flush_dwkeep(s, live)
            s(f"T* dxrow = L1_grad + rowc * {low.L1};")
            self._store_dx(s, "dxrow", live, nt=bool(self.nt & 2))
            self._zero_untouched_in1(s, "dxrow", live)
            # every chunk's body ends with the same block barriers of the dY reduction
            self._dy_finish(s, f"L2_grad + rowc * {low.L2}", live)

        self._per_chunk(s, row_body)
        if self.R == 1:
            s.close()
        s.close()
        if shared:
            # fold the R row groups of the wave, then every wave group writes one partial row
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

    # -------------------------------------------------------- conv backward
    def ragged(self) -> bool:
        """Some used block has lanes without a channel (guards, clamped loads, deferred dW stores)."""
        low = self.low
        full = self.LPR * self.NCH
        return any(low.in1[b].mul != full for b in self.used_in1) or any(low.out[io].mul != full
                                                                          for io in self.used_out)

    def backward_words(self, g_resident: bool) -> int:
        """Rough count of 32-bit registers a lane needs in a backward row / edge body."""
        low = self.low
        x = sum(low.in1[b].d for b in self.used_in1)
        g = sum(low.out[io].d for io in self.used_out) if g_resident else 8
        w = self.n_wslots * (2 if self.ragged() else 1)  # weights, and weight gradients waiting for their store
        return self.words * (g + 2 * x + self.l2_pad + w + low.L2) + 40

    def plan_backward_groups(self, max_waves: int) -> Optional[List[List[int]]]:
        """When a node's output gradient does not fit one wave's registers, share the output blocks (and
        with them the paths) between several waves of the node so that each keeps its share resident.
        Returns the blocks per wave, or None when that is not possible or not needed.

        The estimate of ``backward_words`` decides, for the whole gradient and for a wave's share of it alike.
        Up to about 285 words the one-wave kernel compiles to at most 256 registers with no or a few words of
        scratch memory (35 problems compiled: mixed multiplicities 207..285 none, uniform ones 28 B at 277) and
        beats the shared node (config-5 graph, backward: NequiX main layer 7.52 -> 5.89 ms; 64 / 128 channels with
        harmonics up to l = 4 -15 % .. -30 %; an estimate of 285 -19 %); at 318 (80 B of scratch) the two are
        level, from 330 on it loses by far (SevenNet main layer 25.6 against 10.1 ms). Of the group counts 1, 2, 3,
        4, 6 and 8, forced on 24 problems with estimates from 266 to 643, the best was always the smallest of 1, 2
        and 4 whose share stays under that same limit (shares of 273 and 281 words: two waves, -54 % and -16 %
        against the four and five that a fixed share of 64 gradient words gave; 311 and more: four waves); three,
        six and eight waves never won, and five or seven cost up to 2x."""
        low = self.low
        if low.shared_weights or not self.can_preload or self.R != 1:
            return None
        sizes = [low.out[io].d for io in self.used_out]

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

        def share_words(n: int) -> int:
            """backward_words with a wave's share, 1 / n, of the gradient and of the weights."""
            x = sum(low.in1[b].d for b in self.used_in1)
            w = self.n_wslots * (2 if self.ragged() else 1)
            return self.words * (-(-sum(sizes) // n) + 2 * x + self.l2_pad + -(-w // n) + low.L2) + 40

        if self.group_count:  # forced
            return balanced(max(1, min(self.group_count, max_waves, len(sizes))))
        if self.backward_words(True) <= self.fit_words:
            # one wave: the ordinary kernel where it keeps the gradient in registers by its own rule, else the
            # shared-node kernel with a single owner (which always does)
            return None if self.g_resident else [list(self.used_out)]
        if not self.group_budget:
            for n in (2, 4, 8):
                if n <= max_waves and n <= len(sizes) and share_words(n) <= self.fit_words:
                    return balanced(n)
        # a fixed share of gradient words per wave (group_budget; or nothing above fitted)
        budget = max(1, (self.group_budget or (96 if not self.ragged() else 64)) // self.words)
        n = max(2 if self.g_resident else 1, -(-sum(sizes) // budget))
        while n <= max_waves:
            groups = balanced(n)
            if all(sum(low.out[io].d for io in grp) <= budget for grp in groups):
                return groups
            n += 1
        # No count brings a wave's share under the limit (double precision with many output blocks: NequIP benzene
        # and eight synthetic shapes of 276 problems in both precisions). The unshared kernel, which reads a node's
        # gradient per edge, is the slowest choice there: as many waves as allowed (config-5 graph, fp64, backward:
        # benzene 103.5 -> 61.8 ms; six other shapes -11 % .. -28 %, one +2 %; four waves instead of eight:
        # -35 % .. +20 %).
        n = min(8, max_waves, len(sizes))
        return balanced(n) if n >= 2 else None

    def emit_conv_backward_split(self, s: Src, waves_per_eu: int = 0, xcd: int = 1, dx_atomic: bool = False) -> int:
        """Deterministic-walk backward for problems whose output gradient exceeds one wave's registers:
        the waves of a block all walk the edges of one node; wave ``sg`` keeps the gradient of its output
        blocks resident and handles the paths into them (their dW is final); the partial dX and dY of an
        edge are summed over the waves through LDS, in a fixed order. ``dx_atomic``: the summed sender gradient of
        an edge is added to the sender's row with float atomics (64 consecutive values per instruction, read
        across the LDS copy) instead of being written to ``dx_tmp`` for the ordered reduction."""
        low = self.low
        groups = self.bwd_groups
        SW = len(groups)
        block = 64 * self.NCH * SW
        xoff, XW = {}, 0
        for b in self.used_in1:
            xoff[b] = XW
            XW += low.in1[b].d
        gpaths = [[p for p in low.paths if p.io in grp] for grp in groups]
        gin1 = [sorted({p.i1 for p in ps}) for ps in gpaths]
        for si in range(SW):
            self._per_chunk(s, lambda si=si: self._emit_load_edge(s, f"load_edge_b{si}", gin1[si], gpaths[si]),
                            in_kernel=False)
        s.open(
            f'extern "C" __global__ {self._attrs(block, waves_per_eu)} void backward(i64 node_count, i64 nnz, '
            "const T* __restrict__ L1_in, T* __restrict__ L1_grad, const T* __restrict__ L2_in, "
            "T* __restrict__ L2_grad, const T* __restrict__ W, T* __restrict__ W_grad, "
            "const T* __restrict__ L3_grad, const i64* __restrict__ rows, const i64* __restrict__ cols, "
            "const i64* __restrict__ rowptr, T* __restrict__ dx_tmp, const i64* __restrict__ eperm, "
            "T* __restrict__ wpartial, const i64* __restrict__ colptr, const i64* __restrict__ sperm, "
            f"int* __restrict__ arrivals, const i64* __restrict__ order{self.HUB_PARAMS})"
        )
        self._lane_prologue(s, SW)
        if self.use_q:
            self._emit_q_prologue(s, block // 64)
        if SW == 1:
            s("const int sg = 0;")
        s(f"__shared__ T s_dy[{SW * self.NCH}][{self.l2_pad}];")
        s(f"__shared__ T s_dx[{SW}][{self.NCH}][{XW}][64];")
        s("E_t A;")
        self._node_loop_open(s, 1, xcd)
        for si in range(SW):
            s.open(f"if (sg == {si})")

            def sg_body(si=si):
                s("G_t gr;")
                self._load_g(s, f"L3_grad + node * {low.L3}", groups[si])
                # every wave of the block runs the same number of edges, so the block barriers match up
                s.open("for (i64 e = e0; e < e1; ++e)")
                s("const i64 eid = OEQ_EDGE(e);")
                s(f"load_edge_b{si}{self._sfx()}(A, eid, L1_in, L2_in, W, cols, node_count, u{self._qarg()});")
                yacc, wacc = self._acc_preloaded("A")
                if self.use_q:
                    self._emit_q_build(s, "A.yq")
                s(f"T* dwrow = W_grad + eid * {low.WN};")
                s("X_t dx;")
                self._zero_x(s, "dx")
                s(f"T dy[{self.l2_pad}];")
                s(f"for (int t = 0; t < {self.l2_pad}; ++t) dy[t] = T(0);")
                deferred = self._dw_deferred(None)
                if deferred:
                    s(f"T dwkeep[{self.n_wslots}];")
                self._bwd_paths(s, xname="A.x", yacc=yacc, wacc=wacc, dw_mode="store", paths=gpaths[si])
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
                if dx_atomic:
                    s(f"T* dxrow = L1_grad + oeq_idx(cols[eid], node_count) * {low.L1};")
                else:
                    s(f"T* dxrow = dx_tmp + eid * {low.L1};")
                for n, b in enumerate(self.used_in1):
                    if n % SW != si or not self._has(low.in1[b].mul):
                        continue
                    blk = low.in1[b]
                    contributors = [c for c in range(SW) if b in gin1[c]]
                    if dx_atomic:
                        # the chunk's channels of the block, channel-major in memory: value f of them is component
                        # f % d of channel f / d
                        if not contributors:
                            continue
                        ch = min(64, blk.mul - 64 * self.cur_chunk) if self.cur_chunk is not None else min(64, blk.mul)
                        first = f"chunk * {64 * blk.d}" if self.NCH > 1 else "0"
                        for tt in range((ch * blk.d + 63) // 64):
                            s.open(f"if ({tt * 64} + ul < {ch * blk.d})" if (tt + 1) * 64 > ch * blk.d else "")
                            s(f"const int f = {tt * 64} + ul, fu = f / {blk.d}, fi = f % {blk.d};")
                            terms = " + ".join(f"s_dx[{c}][chunk][{xoff[b]} + fi][fu]" for c in contributors)
                            s(f"oeq_atomic_add(dxrow + {blk.off} + {first} + f, {terms});")
                            s.close()
                        continue
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
                    if not dx_atomic:  # (the library clears the sender rows before a launch that adds to them)
                        self._zero_untouched_in1(s, "dxrow", "true")
                    s.open(f"if (chunk == 0)")
                    s.open(f"for (int j = lane; j < {low.L2}; j += 64)")
                    s("T tot = s_dy[0][j];")
                    s(f"for (int cc = 1; cc < {SW * self.NCH}; ++cc) tot += s_dy[cc][j];")
                    s(f"L2_grad[eid * {low.L2} + j] = tot;")
                    s.close()
                    s.close()
                s("__syncthreads();")
                s.close()

            self._per_chunk(s, sg_body)
            s.close()
        s.close()
        s.close()
        return block

    DX_TERMS, DX_ATOMIC, DX_ARRIVAL, DX_SENDER_WALK = 0, 1, 2, 3

    def emit_conv_backward(self, s: Src, deterministic: bool, G: int, pipelined: bool, waves_per_eu: int = 0,
                           g_resident: Optional[bool] = None, xcd: int = 1, tr_atomics: bool = True,
                           dx_mode: int = 0):
        """``deterministic``: the kernel walks each receiver's edge segment. What happens to the per-edge
        dX terms of the walk is ``dx_mode``: DX_TERMS writes them to ``dx_tmp`` for the sender-ordered
        reduction of ``fixup_backward``; DX_ATOMIC adds them into the (cleared) sender rows with float
        atomics; DX_ARRIVAL writes them to ``dx_tmp`` and counts, per sender and channel chunk, the terms
        that have arrived: the wave that delivers a sender's last term sums that sender's terms in the
        order of ``sperm`` and writes the row, so the reduction needs no kernel of its own and stays
        bit-identical to ``fixup_backward``. (At the MACE shape the walk kernel is bound by its memory
        traffic, the in-kernel reduction adds the same 13 GB of reads to it, and the sum comes out slower
        than the separate kernel: 15.0 against 14.6 ms. Hence opt-in, ``conv_dxm=2``.) DX_SENDER_WALK: this kernel
        leaves dX alone (nothing of it is computed); a second, forward-shaped kernel walks the senders' edge
        segments and forms dX from dZ, Y and W (``conv_module``)."""
        low = self.low
        shared = low.shared_weights
        if self.NCH > 1:
            G = 1  # one node (or edge range) per block: the per-edge dY reduction uses block barriers
        block = 64 * self.NCH * G
        mode = self._edge_mode(2 if pipelined == 4 else pipelined)  # the body stores: see emit_conv_forward
        if self.can_preload:
            self._emit_load_edge(s, "load_edge_b", self.used_in1, low.paths)
            if self.chunk_split and deterministic:
                self._per_chunk(s, lambda: self._emit_load_edge(s, "load_edge_b", self.used_in1, low.paths),
                                in_kernel=False)
        s.open(
            f'extern "C" __global__ {self._attrs(block, waves_per_eu)} void backward(i64 node_count, i64 nnz, '
            "const T* __restrict__ L1_in, T* __restrict__ L1_grad, const T* __restrict__ L2_in, "
            "T* __restrict__ L2_grad, const T* __restrict__ W, T* __restrict__ W_grad, "
            "const T* __restrict__ L3_grad, const i64* __restrict__ rows, const i64* __restrict__ cols, "
            "const i64* __restrict__ rowptr, T* __restrict__ dx_tmp, const i64* __restrict__ eperm, "
            "T* __restrict__ wpartial, const i64* __restrict__ colptr, const i64* __restrict__ sperm, "
            f"int* __restrict__ arrivals, const i64* __restrict__ order{self.HUB_PARAMS})"
        )
        self._lane_prologue(s)
        if self.use_q:
            self._emit_q_prologue(s, block // 64)
        if self.NCH > 1:
            s(f"__shared__ T s_dy[{G}][{self.NCH}][{self.l2_pad}];")
        if shared:
            s(f"T dwacc[{self.n_wslots}];")
            s(f"for (int t = 0; t < {self.n_wslots}; ++t) dwacc[t] = T(0);")
        if self.can_preload:
            s("E_t A, B;")
        if mode in (2, 4):
            floats = self.stage["floats"] + (self.stage["nqw"] * 256 if mode == 4 else 0)
            s(f"__shared__ __attribute__((aligned(16))) T s_stage[{self.NCH * G}][{floats}];")
            self._emit_stage_offsets(s)
        if mode == 3:
            for b in "AB":
                s(f"__shared__ __attribute__((aligned(16))) T s_stage{b}[{self.NCH * G}][{self.stage3['floats']}];")
            self._emit_stage3_offsets(s)
        dx_atomic = (not deterministic) or dx_mode == self.DX_ATOMIC
        self.tr_atomics = dx_atomic and tr_atomics and self._atomics_coalesce() and not self.ir_mul
        if self.tr_atomics or (self.tr_stores & 2 and self.R == 1):
            s(f"__shared__ T s_tr[{self.NCH * G}][{64 * max(low.in1[b].d for b in self.used_in1)}];")
        resident = deterministic and (self.g_resident if g_resident is None else g_resident)
        if dx_mode == self.DX_ARRIVAL:
            assert deterministic and self.R == 1, "arrival counting needs the receiver walk and rows that fill a wave"

        def load(buf, e):
            if self.can_preload:
                s(f"load_edge_b{self._sfx()}({buf}, OEQ_EDGE({e}), L1_in, L2_in, W, cols, node_count, u{self._qarg()});")

        def make_compute(grow_expr_of):
            def compute(buf, pos):
                s.open("")
                s(f"const i64 eid = OEQ_EDGE({pos});")
                e = "eid"
                if mode == 3:
                    s(f"const T* sb = &s_stage{buf}[wave][0];")
                    xname, yacc, wacc = self._acc_staged3("sb")
                elif self.can_preload:
                    yacc, wacc = self._acc_preloaded(buf)
                    xname = f"{buf}.x"
                    if self.use_q:
                        self._emit_q_build(s, f"{buf}.yq")
                else:
                    yacc, wacc = self._acc_pointer()
                    xname = "x"
                    s(f"const T* xrow = L1_in + oeq_idx(cols[{e}], node_count) * {low.L1};")
                    s(f"const T* yrow = L2_in + {e} * {low.L2};")
                    s(f"const T* wrow = W{'' if shared else f' + {e} * {low.WN}'};")
                    s("X_t x;")
                    self._load_x(s, "xrow", self.used_in1)
                if not shared:
                    s(f"T* dwrow = W_grad + {e} * {low.WN};")
                s("X_t dx;")
                self._zero_x(s, "dx")
                s(f"T dy[{self.l2_pad}];")
                s(f"for (int t = 0; t < {self.l2_pad}; ++t) dy[t] = T(0);")
                deferred = not shared and self._dw_deferred(None)
                if deferred:
                    s(f"T dwkeep[{self.n_wslots}];")
                if resident:
                    self._bwd_paths(s, xname=xname, yacc=yacc, wacc=wacc, dw_mode="acc" if shared else "store")
                else:
                    s(f"const T* grow = {grow_expr_of(e)};")
                    if deterministic:
                        # The receiver's gradient row is the same for all its edges: without this the compiler
                        # hoists every load of it out of the edge loop, i.e. makes the whole row register
                        # resident, which is exactly what did not fit.
                        s(f'asm volatile("" : "+{"s" if self.R == 1 else "v"}"(grow));')
                    self._bwd_paths(s, xname=xname, yacc=yacc, wacc=wacc, g_on_demand_row="grow",
                                    dw_mode="acc" if shared else "store")
                self._pin_gradients(s, [] if dx_mode == self.DX_SENDER_WALK else self.used_in1, deferred)
                if deferred:
                    self._flush_dwkeep(s, None)
                if dx_mode == self.DX_SENDER_WALK:
                    pass  # (dx is dead: the compiler drops its arithmetic)
                elif not dx_atomic:
                    s(f"T* dxrow = dx_tmp + {e} * {low.L1};")
                    # terms the arrival scheme re-reads soon are stored plainly, so that they stay cached
                    if dx_mode == self.DX_ARRIVAL:
                        self._store_terms(s, "dxrow")
                    else:
                        self._store_dx(s, "dxrow", "true", nt=bool(self.nt & 2))
                        self._zero_untouched_in1(s, "dxrow", "true")
                else:
                    s(f"T* dxrow = L1_grad + oeq_idx(cols[{e}], node_count) * {low.L1};")
                    self._store_dx(s, "dxrow", "true", atomic=True)
                self._dy_finish(s, f"L2_grad + {e} * {low.L2}", "true")
                s.close()
            return compute

        if deterministic:
            self._node_loop_open(s, G, xcd)

            def node_body():
                if resident:
                    s("G_t gr;")
                    self._load_g(s, f"L3_grad + node * {low.L3}", self.used_out)
                # with more than one chunk all waves of the block walk the same edges, so the
                # block barriers of the dY reduction are reached uniformly (also across per-chunk bodies)
                self._edge_loop(s, "e0 + r", "e1", load, make_compute(lambda e: f"L3_grad + node * {low.L3}"),
                                mode)
                if dx_mode == self.DX_ARRIVAL:
                    self._arrivals(s)

            self._per_chunk(s, node_body)
            s.close()
        else:
            s(f"const i64 ngrp = (i64)gridDim.x * {G};")
            s("const i64 per = (nnz + ngrp - 1) / ngrp;")
            s(f"const i64 eb = ((i64)blockIdx.x * {G} + g) * per;")
            s("const i64 ee = (eb + per < nnz) ? eb + per : nnz;")
            self._edge_loop(s, "eb + r", "ee", load, make_compute(lambda e: f"L3_grad + oeq_idx(rows[{e}], node_count) * {low.L3}"),
                            mode)
        if shared and deterministic:
            # shared weights, walk kernels: every wave group writes the sum over its nodes as one partial
            # row (lane groups of packed rows folded first); the rows are added up in order afterwards
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
        elif shared:
            # float-atomics kernels: one atomic add per weight per wave
            for p, slot in self._dw_slots():
                b1, V = low.in1[p.i1], low.in2[p.i2].mul
                s.open(f"if (u < {b1.mul})")
                s(f"for (int v = 0; v < {V}; ++v) oeq_atomic_add(W_grad + {p.woff} + u * {V} + v, dwacc[{slot} + v]);")
                s.close()
        s.close()
        self.backward_groups_per_block = G
        return block


# ---------------------------------------------------------------------------
# module assembly
# ---------------------------------------------------------------------------


def tp_module(low: Lowered, compute_units: int = 256):
    """Source + launch descriptors for the batch tensor product (forward, backward)."""
    from .. import runtime as rt

    # Measured on MI355X. Forward: 2 waves/SIMD (fp32), fp64 left to the compiler. Backward: the row's whole
    # output-gradient slice is requested up front with X and W (one long burst of loads per row) at 2
    # waves/SIMD; when that slice alone would take more than 256 registers per lane the gradients are
    # loaded per path instead, with scheduling fences between paths, at 3 waves/SIMD. Forward outputs of
    # full 64-channel blocks are stored through an LDS transpose (tp_trs bit 0): fp64 forward 45 % -> 66 %
    # of HBM peak at the MACE shape, fp32 within noise; the same for dX (bit 1) measured neutral.
    f32 = low.elem_size == 4
    wide = low.n_chunks > 1
    g_words = sum(low.out[io].d for io in {p.io for p in low.paths}) * (1 if f32 else 2)
    probe = UvuEmitter(low)
    big = g_words > 256
    on_demand = big or probe.backward_words(True) > (250 if f32 else 420)
    # the next run's gradients can be requested ahead when every path's v loop is unrolled
    pf_ok = all(low.in2[p.i2].mul <= UNROLL_V_LIMIT for p in low.paths)
    t = tuning(dict(tp_acc=48, tp_gf=1 if wide else 4, tp_gb=1 if wide else 4,
                    tp_wf=2 if f32 else 0, tp_wb=3 if (big and not pf_ok) else 2, tp_nt=0,
                    tp_gres=0 if on_demand else 1,
                    tp_sb=1 if on_demand else 0, tp_trs=1, tp_fw=64, tp_pf=1,
                    tp_dd=1, dd_wa=2, dd_wb=2, tp_mask=0, tp_forms=1))
    em = UvuEmitter(low, acc_budget_words=t["tp_acc"])
    em.nt = t["tp_nt"]
    em.mask_loads = bool(t["tp_mask"])
    em.forms = bool(t["tp_forms"])
    em.sched_fence = bool(t["tp_sb"])
    em.fence_words = t["tp_fw"]
    em.prefetch_runs = bool(t["tp_pf"])
    em.tr_stores = t["tp_trs"]
    s = Src()
    s(prelude(low.ctype))
    s(utility_kernels())
    em.emit_structs(s)
    em.emit_forward_cores(s, preloaded=False)
    G_f, G_b = t["tp_gf"], (1 if em.NCH > 1 else t["tp_gb"])
    blk_f = em.emit_tp_forward(s, G_f, t["tp_wf"])
    blk_b = em.emit_tp_backward(s, G_b, t["tp_wb"], bool(t["tp_gres"]))
    max_blocks_b = compute_units * 8
    descs = [
        (rt.ROLE_TP_FORWARD, "forward", blk_f, G_f * em.R, 0),
        (rt.ROLE_TP_BACKWARD, "backward", blk_b, G_b * em.R, max_blocks_b if low.shared_weights else 0),
        (rt.ROLE_FILL_ZERO, "oeq_fill_zero", 256, 256 * 16, compute_units * 16),
        (rt.ROLE_TP_BACKWARD_WREDUCE, "oeq_wreduce", 256, 64, 0),
    ]
    from . import uvu_double
    if t["tp_dd"] and uvu_double.supported(low):
        descs += uvu_double.add_tp_kernels(s, low, em, t, G_b, compute_units)
    dims = dict(L1_dim=low.L1, L2_dim=low.L2, L3_dim=low.L3, weight_numel=low.WN, elem_size=low.elem_size,
                shared_weights=int(low.shared_weights), deterministic=0,
                wpartial_per_block=G_b if low.shared_weights else 0)
    return s.text(), dims, descs


def _forward_plan(low: Lowered, first_budget: int) -> Tuple[UvuEmitter, bool]:
    """(emitter, two operand sets in flight?) for a walk kernel without LDS staging: the accumulators of an output
    segment, the edge's operands (X blocks, the weights of the segment's paths, Y) once or twice, within the registers
    of two waves per SIMD. The segment budget shrinks until that fits; the prefetch goes when 48-word segments do
    not fit with it."""
    words = 1 if low.elem_size == 4 else 2

    def plan(budget, sets):
        e = UvuEmitter(low, acc_budget_words=budget)
        need = max(sets * words * (sum(low.in1[b].d for b in e.seg_in1[si]) + low.L2 +
                                   sum(low.in2[p.i2].mul for p in low.paths if p.io in seg))
                   + words * sum(low.out[io].d for io in seg) for si, seg in enumerate(e.segments))
        return e, need + (40 if e.ragged() else 0)

    e = UvuEmitter(low, acc_budget_words=first_budget)
    if e.stage is not None or not e.can_preload:
        return e, True
    budgets = (first_budget, 96, 64, 48)
    for budget in budgets:
        e, need = plan(budget, 2)
        if need <= 170:
            return e, True
    for budget in budgets:
        e, need = plan(budget, 1)
        if need <= 190:
            break
    return e, False


def conv_module(low: Lowered, deterministic: bool, compute_units: int = 256, kahan: bool = False,
                override: Optional[Dict[str, int]] = None):
    """Source + launch descriptors for the fused convolution (forward, backward).

    ``deterministic``: the caller passes receiver-sorted edges and the sender-major permutation; the
    kernels walk each node's edge segment (no atomics on node data, fixed summation order). Otherwise
    the edge order is arbitrary and, by default, the library groups the edge indices by receiver and
    by sender on the device and runs the same kernels through that index (``conv_sort=0`` in
    ``OEQ_AMD_TUNE`` selects the kernels that walk contiguous edge ranges and flush with float atomics
    instead, the scheme of the reference's templates/loop_unroll_conv_atomic.cuh).

    ``kahan`` (deterministic mode only): compensated summation where rows are summed over edges, i.e.
    the receiver's output in `forward` and the sender's gradient in `fixup_backward`, as in the
    reference (templates/loop_unroll_conv_det.cuh:70-94, 135-160, 227-271).

    ``override``: knob values that take precedence over ``OEQ_AMD_TUNE`` (the function's own second attempt,
    see the end)."""
    from .. import runtime as rt

    assert not (deterministic and low.shared_weights), "deterministic convolution needs per-edge weights"
    t = tuning(dict(conv_acc=128, conv_gf=max(1, 4 // low.n_chunks), conv_gb=4, conv_pipe_f=2, conv_pipe_b=0,
                    conv_wf=23, conv_wb=2, conv_wx=0, conv_gres=-1, conv_xcd=8, conv_tra=1, conv_nt=15, conv_epw=8,
                    conv_sort=1, conv_trs=3 if low.elem_size == 8 else 0, conv_sb=-1,
                    conv_segw=4, conv_split=1, conv_dd=1, dd_acc=0, dd_g=2, dd_wa=2, dd_wb=2, dd_fp=0, dd_fw=32,
                    dd_gres=-1, dd_split=1, dd_segw=4, dd_merge=0, dd_need=200, dd_ngrp=0, conv_gbud=0, conv_ngrp=0, conv_fit=300, conv_fw=0, conv_pf=0,
                    conv_dxm=-1, conv_q=0, conv_hops=2, conv_qpin=1, conv_qaf=48, conv_qab=24, tp_mask=0, tp_forms=1,
                    conv_hub=256, conv_dxs=-1))
    assert deterministic or not kahan, "kahan=True requires deterministic=True"
    # knobs somebody set: the rules below leave those alone
    user_tune = os.environ.get("OEQ_AMD_TUNE", "")
    if override:
        t.update(override)
        user_tune = ",".join([user_tune, *override])
    if kahan:  # the compensation terms double the accumulator registers: walk the outputs in more passes
        t["conv_acc"] = min(t["conv_acc"], 48)
    if deterministic:
        mode = rt.CONV_SORTED
    else:
        mode = rt.CONV_GROUPED if t["conv_sort"] else rt.CONV_ATOMIC
    walk = mode != rt.CONV_ATOMIC  # kernels walk per-node edge segments
    em = UvuEmitter(low, acc_budget_words=t["conv_acc"], kahan=kahan)
    # fp64 with rows that fill the wave: when everything a node needs (accumulators or gradient slice, one
    # operand set) fits the 512 registers a lane has at one wave per SIMD, that beats walking the edges once
    # per output segment / sharing the node between waves (MACE shape, fp64: forward 18.4 -> 12.5 ms,
    # backward 42.1 -> 26.4 ms). The same plan loses for every fp32 problem tried.
    wide64 = low.elem_size == 8 and em.R == 1 and not kahan and walk and not low.shared_weights
    wide64_forward = False
    if low.elem_size == 8 and "conv_wf" not in user_tune:
        # fp64 forward kernels get the plain budget of two waves per SIMD: allowed a third, the compiler stays
        # under 256 registers without reaching 168 and the kernel runs at half speed (config-5 graph, forward:
        # 128x{0e,1o,2e} with l <= 3 harmonics, 216 registers, 10.5 against 5.4 ms; 128x{0e..3o} 12.9 / 7.5 and
        # 36.2 / 19.4); the zoo's eleven fp64 kernels of this kind are within -4.3 % .. +1.4 % either way.
        t["conv_wf"] = 2
    if wide64 and "conv_acc" not in user_tune and "conv_wf" not in user_tune:
        x_all = sum(low.in1[b].d for b in em.used_in1)
        need_f = 2 * (sum(low.out[io].d for io in em.used_out) + x_all + em.n_wslots + low.L2) + 40
        if len(em.segments) > 1 and need_f <= 480:
            t["conv_acc"], t["conv_wf"] = 1 << 20, 1
            t["conv_trs"] &= ~1
            em = UvuEmitter(low, acc_budget_words=t["conv_acc"], kahan=kahan)
            wide64_forward = True
    if wide64 and not any(k in user_tune for k in ("conv_wb", "conv_gres", "conv_split")):
        if 240 < em.backward_words(True) <= 480:
            t["conv_wb"], t["conv_gres"], t["conv_split"] = 1, 1, 0
    if em.stage is None and em.can_preload and "conv_acc" not in user_tune and t["conv_acc"] < (1 << 20):
        # Forward without LDS staging keeps two operand sets of an edge (X blocks, the weights of the
        # output segment's paths, Y) beside the accumulators: shrink the segments until that fits, and
        # give up the prefetch when even 48-word segments do not.
        words = 1 if low.elem_size == 4 else 2

        def plan(budget, sets):
            e = UvuEmitter(low, acc_budget_words=budget, kahan=kahan)
            need = max(sets * words * (sum(low.in1[b].d for b in e.seg_in1[si]) + low.L2 +
                                       sum(low.in2[p.i2].mul for p in low.paths if p.io in seg))
                       + words * sum(low.out[io].d for io in seg) for si, seg in enumerate(e.segments))
            return e, need + (40 if e.ragged() else 0)  # clamped indices and select masks of ragged blocks

        budgets = (t["conv_acc"], 96, 64, 48)
        for budget in budgets:
            em, need = plan(budget, 2)
            if need <= 170:
                break
        else:
            t["conv_pipe_f"] = 0
            for budget in budgets:
                em, need = plan(budget, 1)
                if need <= 190:
                    break
    em.nt = t["conv_nt"]
    em.mask_loads = bool(t["tp_mask"])
    em.forms = bool(t["tp_forms"])
    q_fwd = q_bwd = False
    if t["conv_q"] and em.q_supported():
        # bit 0: forward, bit 1: backward. Backward gains nothing at the MACE shape (it is bound by its
        # memory traffic, and the table's vectors compete with the resident gradient slice for registers)
        q_fwd, q_bwd = bool(t["conv_q"] & 1), bool(t["conv_q"] & 2)
        em.q_pin = bool(t["conv_qpin"])
        em.q_ahead = (t["conv_qaf"], t["conv_qab"])
        em.build_q_table()
    if walk and len(em.segments) > 1 and t["conv_segw"] and em.stage is None and em.R == 1:
        em.seg_waves = max(1, min(len(em.segments), t["conv_segw"], max(1, 8 // em.NCH)))
        t["conv_gf"] = max(1, min(t["conv_gf"], 8 // (em.NCH * em.seg_waves)))
    if walk and (len(em.segments) > 1 or low.elem_size == 8) and "conv_gf" not in user_tune:
        # Several output segments (a wave walks the node's edges once per segment it owns): one node per block.
        # Blocks of several nodes hold all their wave slots until the slowest wave is through; over 118 problems
        # on the config-5 graph one node per block is never slower (+0.3 % at worst) and up to 30 % faster
        # (forward: SevenNet main layer 4.36 -> 3.09 ms, NequiX main layer 2.51 -> 2.21, NequIP benzene
        # 8.33 -> 7.98). fp64 kernels likewise, whatever their segments (18 problems: 0 .. -12 %).
        t["conv_gf"] = 1
    em.tr_stores = t["conv_trs"]
    # output gradients that do not fit the register budget are loaded per path: fence the paths then
    em.sched_fence = (not em.g_resident) if t["conv_sb"] < 0 else bool(t["conv_sb"])
    em.fence_words = t["conv_fw"]
    em.prefetch_runs = bool(t["conv_pf"])
    s = Src()
    s(prelude(low.ctype))
    s(utility_kernels(kahan))
    # position in the walk -> edge index: through the library's grouping when there is one
    s("#define OEQ_EDGE(j) (eperm ? eperm[(j)] : (j))")
    em.emit_structs(s)
    em.use_q = q_fwd
    em.emit_forward_cores(s, preloaded=True)
    # Kernels with few words per lane (output segment, X blocks, weights: first and last layers of a network,
    # narrow models) need well under 128 registers. The register budget of two waves per SIMD is then no help
    # and the limit of two waves a loss: they get that budget as a minimum and run as many waves as their
    # registers allow (config-5 graph, step: SevenNet first layer 3.96 -> 2.58 ms, last layers 3.85 -> 3.49,
    # NequiX first layer 2.58 -> 2.30, MACE-medium 5.99 -> 5.68, NequIP water 2.18 -> 2.05). Larger kernels keep
    # the budget of two: without a limit the scheduler aims for an occupancy they cannot use (SevenNet main layer
    # 15.3 -> 21.2 ms); the forward kernel may run a third wave where its registers allow (conv_wf=23: NequiX /
    # SevenNet main layers' forward -10 % / -16 %, nothing else moves), the backward kernel not (SevenNet main
    # layer +30 %).
    per_lane = (1 if low.elem_size == 4 else 2) * (max(sum(low.out[io].d for io in seg) for seg in em.segments)
                                                   + sum(low.in1[b].d for b in em.used_in1) + em.n_wslots)
    if walk and per_lane <= 48:
        for knob in ("conv_wf", "conv_wb"):
            if knob not in user_tune:
                t[knob] = -2
    elif walk and not low.shared_weights and "conv_gb" not in user_tune:
        # One node per block for the backward kernel as well where a row fits one wave and the kernel is not a
        # small one (blocks of four nodes keep their wave slots until the slowest is through; same 118 problems,
        # fp32: -8 % .. +0.3 %, mean -1.7 %; NequiX main layer 6.13 -> 5.77 ms; small kernels: up to +1.4 %; 18
        # problems in fp64: -8 % .. +1 %)
        t["conv_gb"] = 1
    G_f = t["conv_gf"]
    G_b = 1 if em.NCH > 1 else t["conv_gb"]
    xcd = max(1, t["conv_xcd"])
    xcd_b = 1 if (walk and low.shared_weights) else xcd  # bounded grid: one partial dW row per wave group
    blk_f = em.emit_conv_forward(s, G_f, walk, t["conv_pipe_f"], t["conv_wf"], xcd, bool(t["conv_tra"]))
    em.use_q = q_bwd
    gres = None if t["conv_gres"] < 0 else bool(t["conv_gres"])
    dx_mode = 0
    em.group_budget = t["conv_gbud"]
    em.fit_words = t["conv_fit"]
    em.group_count = t["conv_ngrp"]
    em.bwd_groups = em.plan_backward_groups(max(1, 8 // em.NCH)) if (walk and t["conv_split"] and gres is None) else None
    if em.bwd_groups:
        G_b = 1
        wpb = em.NCH * len(em.bwd_groups)
        if 8 % wpb and 12 % wpb == 0 and "conv_wb" not in user_tune:
            # blocks of 3 waves leave a quarter of the wave slots empty at 2 waves per SIMD (8 per CU); at 3
            # per SIMD they fill them (SevenNet main layer: 14.6 -> 10.1 ms)
            t["conv_wb"] = 3
        # deterministic=False, on request (conv_dxm=1): the edge's summed sender gradient leaves as float atomics
        # from the LDS copy it is summed in. Against the per-edge terms and their ordered reduction, backward op on
        # the config-5 graph: SevenNet main layer 9.47 -> 8.96 ms and a 512-word row -6 %, but rows of 864 words
        # and more +21 % .. +41 % (NequIP benzene 21.9 -> 26.5 ms): the one-wave kernel's rule does not carry over.
        split_atomic = (mode == rt.CONV_GROUPED and not kahan and not em.ir_mul and t["conv_dxm"] == em.DX_ATOMIC)
        dx_mode = em.DX_ATOMIC if split_atomic else em.DX_TERMS
        blk_b = em.emit_conv_backward_split(s, t["conv_wb"], xcd, split_atomic)
    else:
        # what becomes of the walk's per-edge dX terms (UvuEmitter.emit_conv_backward)
        if walk and not kahan:
            # deterministic=False may use float atomics, and adding the terms straight into the sender
            # rows saves their round trip through scratch memory and the second kernel; the caller-sorted
            # mode promises the same bits on every run and keeps the ordered reduction
            # (only where a row fills the wave and the atomics go through the LDS transpose, 64 consecutive
            # floats per instruction: per-lane atomics of packed or ragged rows are several times slower than
            # the ordered reduction)
            coalesced = bool(t["conv_tra"]) and em._atomics_coalesce() and not em.ir_mul
            dx_mode = t["conv_dxm"] if t["conv_dxm"] >= 0 else (
                em.DX_ATOMIC if (mode == rt.CONV_GROUPED and coalesced) else em.DX_TERMS)
            # arrival counting keeps an edge's terms lane-major, 64 values per (block, component) and chunk: they
            # fit the edge's row of dx_tmp only when no used block has lanes without a channel
            if dx_mode == em.DX_ARRIVAL and (em.R != 1 or 64 * em.NCH * em._term_slots()[1] > low.L1):
                dx_mode = em.DX_TERMS
            # Rows of X that are long against an edge's weights and an output row (the last layer of a network:
            # many irreps in, a few scalars out; few paths per input irrep): the per-edge dX terms, written and read
            # back, are then most of the backward's traffic (2 L1 words per edge). A second walk over the SENDERS'
            # edge segments that reads W and Y again and gathers the dZ rows moves WN + L2 + L3 words per edge
            # instead (the gathered rows mostly from the L2) and sums in the same list order. It is the forward
            # kernel of the adjoint problem (lower.adjoint). Measured over 128 problems on the config-5 graph,
            # backward op: ratio (WN + L2 + L3) / L1 of 1.1 .. 3.5: -16 % .. -57 %; 4.0 (NequIP aspirin, water):
            # -5 %; 4.6: -2 % .. -6 %; 5.1: +-3 %; 5.3 and more: slower, +27 % at config 5 (7.6).
            auto = 9 * low.L1 >= 2 * (low.WN + low.L2 + low.L3) and not low.shared_weights and t["conv_dxm"] < 0
            if (t["conv_dxs"] > 0) or (t["conv_dxs"] < 0 and auto):
                dx_mode = em.DX_SENDER_WALK
        blk_b = em.emit_conv_backward(s, walk, G_b, t["conv_pipe_b"], t["conv_wb"], gres, xcd_b,
                                      bool(t["conv_tra"]), dx_mode)
        G_b = em.backward_groups_per_block
    descs = [
        (rt.ROLE_FILL_ZERO, "oeq_fill_zero", 256, 256 * 16, compute_units * 16),
        (rt.ROLE_SEGMENT_PTR, "oeq_segment_ptr", 256, 256, compute_units * 16),
    ]
    if walk:
        s(fixup_backward_kernel(low.L1, kahan, bool(em.nt & 4)))
        descs += [
            (rt.ROLE_CONV_FORWARD, "forward", blk_f, G_f, 0, xcd),
            (rt.ROLE_CONV_BACKWARD, "backward", blk_b, G_b, compute_units * 8 if low.shared_weights else 0, xcd_b),
            (rt.ROLE_CONV_FIXUP_BACKWARD, "fixup_backward", 256, 1, 0),
        ]
        if low.shared_weights:
            descs.append((rt.ROLE_TP_BACKWARD_WREDUCE, "oeq_wreduce", 256, 64, 0))
        if dx_mode == UvuEmitter.DX_SENDER_WALK:
            from .lower import adjoint
            low_x = adjoint(low)
            ex, pipe_x = _forward_plan(low_x, t["conv_acc"])
            ex.nt, ex.mask_loads, ex.forms, ex.tr_stores = t["conv_nt"], bool(t["tp_mask"]), bool(t["tp_forms"]), t["conv_trs"]
            words_x = (1 if low.elem_size == 4 else 2) * (
                max(sum(low_x.out[io].d for io in seg) for seg in ex.segments)
                + sum(low_x.in1[b].d for b in ex.used_in1) + ex.n_wslots)
            # (its structs and contraction functions have the names of the forward kernel's: a namespace of its own)
            s("namespace oeq_dx {")
            ex.emit_structs(s)
            ex.use_q = False
            ex.emit_forward_cores(s, preloaded=True)
            G_x = max(1, 4 // low_x.n_chunks)
            waves_x = t["conv_wx"] if t["conv_wx"] else (-2 if words_x <= 48 else 2)
            blk_x = ex.emit_conv_forward(s, G_x, True, t["conv_pipe_f"] if pipe_x else 0, waves_x,
                                         xcd, bool(t["conv_tra"]), name="backward_dx")
            s("}  // namespace oeq_dx")
            descs.append((rt.ROLE_CONV_BACKWARD_DX, "backward_dx", blk_x, G_x, 0, xcd))
        from . import uvu_double
        if t["conv_dd"] and uvu_double.supported(low, conv=True):
            descs += uvu_double.add_conv_kernels(s, low, em, t, xcd, G_b, compute_units, kahan)
        # counting sort: of the edge indices by node (GROUPED mode) and of the nodes by cluster (walk order)
        descs += [
            (rt.ROLE_GROUP_COUNT, "oeq_group_count", 256, 256 * 4, compute_units * 16),
            (rt.ROLE_GROUP_SCAN, "oeq_group_scan", 1024, 1, 1),
            (rt.ROLE_GROUP_SCATTER, "oeq_group_scatter", 256, 256 * 4, compute_units * 16),
            (rt.ROLE_GROUP_ORDER, "oeq_group_order", 256, 4, compute_units * 32),
            (rt.ROLE_ORDER_HOP, "oeq_order_hop", 256, 256, compute_units * 16),
            # long edge segments in chunks: table of the extra walk positions, and the sum of their rows
            (rt.ROLE_HUB_COUNT, "oeq_hub_count", 256, 256, compute_units * 16),
            (rt.ROLE_HUB_FILL, "oeq_hub_fill", 256, 256, compute_units * 16),
            (rt.ROLE_CONV_FIXUP_FORWARD, "fixup_forward", 256, 1, compute_units * 32),
        ]
    else:
        # edge ranges: about conv_epw consecutive edges per wave group
        epw = max(1, t["conv_epw"])
        descs += [
            (rt.ROLE_CONV_FORWARD, "forward", blk_f, G_f * em.R * epw, compute_units * 32),
            (rt.ROLE_CONV_BACKWARD, "backward", blk_b, G_b * em.R * epw, compute_units * 32),
        ]
    # Segments longer than conv_hub edges are walked in chunks of that many (0: whole). Not with Kahan
    # summation (its compensation terms belong to one running sum) nor where the second-order kernel B also
    # forms kernel A's result.
    hub_limit = max(0, t["conv_hub"]) if (walk and not kahan and not t["dd_merge"]) else 0
    dims = dict(L1_dim=low.L1, L2_dim=low.L2, L3_dim=low.L3, weight_numel=low.WN, elem_size=low.elem_size,
                shared_weights=int(low.shared_weights), deterministic=mode,
                wpartial_per_block=G_b if (walk and low.shared_weights) else 0, dx_mode=dx_mode,
                n_chunks=em.NCH, order_hops=max(0, t["conv_hops"]) if walk else 0, hub_limit=hub_limit)
    src = s.text()
    if dx_mode == UvuEmitter.DX_SENDER_WALK and t["conv_dxs"] < 0:
        # the sender walk was chosen by its rule, not asked for: not with a kernel that does not fit its registers
        # (forced on shapes beyond the rule, adjoint kernels with 200 - 320 B of scratch ran 3x slower than the terms)
        _lds, scratch = rt.kernel_resources(rt.compile_source(src)).get("backward_dx", (0, 0))
        if scratch > 64:
            return conv_module(low, deterministic, compute_units, kahan, dict(override or {}, conv_dxs=0))
    if em.seg_waves > 1 and "conv_segw" not in user_tune:
        # Waves that share a node's output segments: with two operand sets in flight and three or more segments
        # the compiler has been seen to need more registers for the kernel that selects a wave's segments by
        # branches than for the one that walks them one after the other (64x{0e,1e,2e,3e} with l <= 3 harmonics:
        # 256 registers and 280 B of scratch memory per lane against 227 and none; forward 14.5 against 4.0 ms).
        # The code object says so (compiled here, cached like any other): then one wave owns the node.
        _lds, scratch = rt.kernel_resources(rt.compile_source(src)).get("forward", (0, 0))
        if scratch > 64:
            return conv_module(low, deterministic, compute_units, kahan, dict(override or {}, conv_segw=0))
    if wide64_forward:
        # fp64 with a node's whole output row in one wave's 512 registers: the estimate that admits this plan is
        # optimistic for rows of 96 channels (two waves' lanes, the second half empty). With scratch memory the
        # kernel loses to the output segments it was meant to beat (config-5 graph, forward, 96x{0e..3o}: 484 B,
        # 25.9 against 8.3 ms; 228 B, 15.4 / 8.7; 96x{0e,1o,2e}: 196 B, 11.3 / 6.8).
        _lds, scratch = rt.kernel_resources(rt.compile_source(src)).get("forward", (0, 0))
        if scratch > 64:
            return conv_module(low, deterministic, compute_units, kahan, dict(override or {}, conv_wf=2))
    if walk and t["conv_wf"] == 23 and "conv_wf" not in user_tune and low.elem_size == 4:
        # A forward kernel that the compiler gave more than a third of a SIMD's registers runs two waves there.
        # Held to a third it runs three, which pays where the compiler manages that without scratch memory (fp32,
        # config-5 graph, forward: 96 channels of l <= 3 with l <= 3 harmonics 176 -> 168 registers, -18 %; 64
        # channels of l <= 3, l <= 2 harmonics 197 -> 160, -10 %; all five such shapes of 128 tried gained 9 - 19 %)
        # and costs where it does not (12 B of scratch: +21 % and +28 %; 100 B and more: +40 % .. +144 %).
        # The code objects say which it is (compiled here, cached like any other; of the second form only the
        # forward kernel).
        if rt.kernel_registers(rt.compile_source(src)).get("forward", 0) > 168:
            third = conv_module(low, deterministic, compute_units, kahan, dict(override or {}, conv_wf=3))
            if _forward_scratch(third[0]) == 0:
                return third
    return src, dims, descs


def _forward_scratch(source: str) -> int:
    """Bytes of scratch memory per lane of a convolution module's forward kernel, compiled without the module's
    other kernels."""
    from .. import runtime as rt
    common, kernels = rt.split_kernels(source)
    own = [k for k in kernels if re.search(r"\bvoid\s+forward\s*\(", k)]
    blob = rt.compile_source(common + "\n" + own[0] if len(own) == 1 else source)
    return rt.kernel_resources(blob).get("forward", (0, 0))[1]
