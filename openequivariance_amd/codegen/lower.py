"""Lower a TPProblem to the flat tables the HIP emitters work from.

This is the planner of this package. Where the reference splits
multiplicities into warp-sized chunks and packs instructions into shared-memory
segments (openequivariance/openequivariance/core/ComputationSchedule.py:185-649),
the gfx950 plan is: lanes of a wave64 are channels ``u`` of one row; rows narrower
than a wave are packed several to a wave; rows wider than a wave are split into
64-channel chunks owned by different waves of the same block; outputs that are
accumulated over many edges stay in registers, grouped into "segments" that fit
a register budget.
"""

from __future__ import annotations

import math
from dataclasses import dataclass, replace
from typing import List, Tuple

import numpy as np

from ..core.cg import sparse_cg
from ..core.spec import TPProblem


def filter_and_analyze_problem(problem: TPProblem) -> dict:
    """Reject what the kernels do not cover; same rules and messages as the
    reference (openequivariance/openequivariance/core/utils.py:81-117)."""
    first = problem.instructions[0].connection_mode if len(problem.instructions) else None
    for i, inst in enumerate(problem.instructions):
        assert inst.connection_mode == first, (
            f"All instructions must have the same connection mode, got {inst.connection_mode} and {first}"
        )
        assert inst.has_weight, f"All instructions must have trainable weights, got {inst.has_weight} at index {i}"
    assert len(problem.instructions) > 0, "Tensor product has no valid instructions!"
    assert first in ["uvu", "uvw"], f"Connection mode must be 'uvu' or 'uvw', got {first}"
    if problem.layout == "ir_mul":
        assert first == "uvu", "layout='ir_mul' is only supported for pure 'uvu' problems"
    assert problem.irrep_dtype == problem.weight_dtype, (
        f"irrep_dtype and weight_dtype must be the same, got {problem.irrep_dtype} and {problem.weight_dtype}"
    )
    assert not problem.internal_weights, (
        f"Openequivariance does not support internal weights, got {problem.internal_weights}"
    )
    return {"is_uvw": first == "uvw"}


@dataclass
class Block:
    off: int
    mul: int
    l: int
    # [2l+1, mul] layout only: distance between two components of a channel when it is not ``mul`` (a
    # piece of a wider block keeps the stride of the block it was cut from)
    cstride: int = 0

    @property
    def d(self) -> int:
        return 2 * self.l + 1


@dataclass
class Path:
    index: int
    i1: int
    i2: int
    io: int
    woff: int
    coeff: float
    nnz: List[Tuple[int, int, int, float]]  # (i, j, k, coeff * C[i,j,k]) sorted by (j, i, k)
    l: Tuple[int, int, int] = (0, 0, 0)


@dataclass
class Lowered:
    mode: str
    ctype: str
    elem_size: int
    shared_weights: bool
    in1: List[Block]
    in2: List[Block]
    out: List[Block]
    paths: List[Path]
    L1: int
    L2: int
    L3: int
    WN: int
    label: str = ""
    # lane mapping
    lanes_per_row: int = 64
    rows_per_wave: int = 1
    n_chunks: int = 1
    max_u: int = 1
    total_nnz: int = 0
    # True: every irrep block of a row is stored [2l+1, mul] (component-major) instead of [mul, 2l+1]
    ir_mul: bool = False

    def flops(self, direction: str) -> int:
        """Reference FLOP convention (benchmark/metrics.py:49-94,
        core/ConvolutionBase.py:14-54): 3 per CG non-zero forward, 9 backward,
        times mul1*mul2, plus the weight application."""
        per_nz = 3 if direction == "forward" else 9
        total = 0
        for p in self.paths:
            a, b, o = self.in1[p.i1], self.in2[p.i2], self.out[p.io]
            total += per_nz * len(p.nnz) * a.mul * b.mul
            if direction == "forward":
                if self.mode == "uvu":
                    total += o.mul * o.d
                else:
                    total += a.mul * b.mul * o.d * o.mul
        return total


def _blocks(irreps) -> List[Block]:
    out, off = [], 0
    for mul, ir in irreps:
        out.append(Block(off, mul, ir.l))
        off += mul * ir.dim
    return out


def _pow2ceil(n: int) -> int:
    return 1 << max(0, (n - 1).bit_length())


def lower(problem: TPProblem) -> Lowered:
    info = filter_and_analyze_problem(problem)
    dtype = np.dtype(problem.irrep_dtype)
    if dtype == np.float32:
        ctype, es = "float", 4
    elif dtype == np.float64:
        ctype, es = "double", 8
    else:
        raise AssertionError(f"unsupported irrep dtype {dtype}")

    in1, in2, out = _blocks(problem.irreps_in1), _blocks(problem.irreps_in2), _blocks(problem.irreps_out)
    mode = "uvw" if info["is_uvw"] else "uvu"
    paths, woff = [], 0
    for idx, ins in enumerate(problem.instructions):
        a, b, o = in1[ins.i_in1], in2[ins.i_in2], out[ins.i_out]
        if mode == "uvu":
            assert o.mul == a.mul, "'uvu' needs mul_out == mul_in1"
        nnz = sparse_cg(a.l, b.l, o.l, scale=ins.path_weight)
        paths.append(Path(idx, ins.i_in1, ins.i_in2, ins.i_out, woff, ins.path_weight, nnz, (a.l, b.l, o.l)))
        woff += math.prod(ins.path_shape)
    assert woff == problem.weight_numel

    low = Lowered(
        mode=mode, ctype=ctype, elem_size=es, shared_weights=bool(problem.shared_weights),
        in1=in1, in2=in2, out=out, paths=paths,
        L1=problem.irreps_in1.dim, L2=problem.irreps_in2.dim, L3=problem.irreps_out.dim,
        WN=problem.weight_numel, label=problem.label,
    )
    low.ir_mul = problem.layout == "ir_mul"
    _lane_mapping(low)
    if mode == "uvu" and low.n_chunks > MAX_CHUNKS:
        # One wave per 64-channel chunk, all in one block of at most 1024 threads: blocks of more than 1024
        # channels are cut into pieces of that many, each an ordinary block further into the row, and every
        # path into one path per piece (the reference chunks any multiplicity into warp-sized children,
        # core/ComputationSchedule.py:185-343).
        low = _fold_wide_blocks(low, piece=64 * MAX_CHUNKS)
    elif mode == "uvu" and 1 < low.n_chunks <= 4 and any(in1[p.i1].mul != 64 * low.n_chunks for p in paths):
        low = _fold_wide_blocks(low)
    return low


MAX_CHUNKS = 16  # 64-channel chunks of a row that one block of 1024 threads covers


def _lane_mapping(low: Lowered) -> None:
    in1, paths = low.in1, low.paths
    used_mul = [in1[p.i1].mul for p in paths]
    low.max_u = max(used_mul)
    low.lanes_per_row = 64 if low.max_u > 32 else _pow2ceil(low.max_u)
    low.rows_per_wave = 64 // low.lanes_per_row
    low.n_chunks = (low.max_u + 63) // 64
    low.total_nnz = sum(len(p.nnz) for p in paths)


def _fold_wide_blocks(low: Lowered, piece: int = 64) -> Lowered:
    """'uvu' rows wider than a wave whose irreps have different multiplicities (128x0e+64x1o+32x2e,
    89x0e, ...): cut every block into pieces of at most ``piece`` = 64 channels and every path into the paths
    between matching pieces. In the [mul, 2l+1] layout a piece is just a block that starts further into
    the row (in the [2l+1, mul] layout: 64 channels further into each component, with the components
    still ``mul`` apart), and its weights start ``64 * mul_v`` further into the path's weights, so the
    result is an ordinary problem with at most 64 channels per block: one wave then owns the whole row and walks the
    pieces one after the other, where waves that each owned one 64-channel slice of every block would
    mostly have idle lanes or nothing to do. With ``piece`` = 1024 the same cut brings blocks of more than
    1024 channels down to what one block of threads covers; the pieces then still span several waves."""
    def cut(blocks: List[Block], used):
        pieces, index = [], {}
        for b, blk in enumerate(blocks):
            if low.ir_mul and b not in used:
                # [2l+1, mul] layout: the channels of a piece are not one contiguous range; a block no path
                # touches (it is only cleared) stays whole
                index[(b, 0)] = len(pieces)
                pieces.append(blk)
                continue
            for c in range((blk.mul + piece - 1) // piece):
                index[(b, c)] = len(pieces)
                n = min(piece, blk.mul - c * piece)
                if low.ir_mul:  # component i of channel u sits at off + i * mul + u
                    pieces.append(Block(blk.off + c * piece, n, blk.l, cstride=blk.cstride or blk.mul))
                else:
                    pieces.append(Block(blk.off + c * piece * blk.d, n, blk.l))
        return pieces, index

    in1, index1 = cut(low.in1, {p.i1 for p in low.paths})
    out, index3 = cut(low.out, {p.io for p in low.paths})
    paths = []
    for p in low.paths:
        v_mul = low.in2[p.i2].mul
        for c in range((low.in1[p.i1].mul + piece - 1) // piece):
            paths.append(Path(len(paths), index1[(p.i1, c)], p.i2, index3[(p.io, c)], p.woff + c * piece * v_mul,
                              p.coeff, p.nnz, p.l))
    folded = Lowered(mode=low.mode, ctype=low.ctype, elem_size=low.elem_size, shared_weights=low.shared_weights,
                     in1=in1, in2=low.in2, out=out, paths=paths, L1=low.L1, L2=low.L2, L3=low.L3, WN=low.WN,
                     label=low.label)
    folded.ir_mul = low.ir_mul
    _lane_mapping(folded)
    return folded


def float_literal(v: float, ctype: str) -> str:
    """Exact C++17 hex-float literal of ``v`` rounded to ``ctype``."""
    if ctype == "float":
        return float(np.float32(v)).hex() + "f"
    return float(v).hex()


def adjoint(low: Lowered) -> Lowered:
    """The 'uvu' problem whose forward map is the X-gradient of ``low``: the roles of the first operand and the
    output swapped, every structural non-zero (i, j, k, c) as (k, j, i, c), same weights (a 'uvu' path has one
    weight per channel, whichever side the channel is read from) and same second operand. With dZ as its
    first operand, ``forward(dZ, Y, W)`` of this problem is dX of the original."""
    assert low.mode == "uvu"
    paths = [Path(p.index, p.io, p.i2, p.i1, p.woff, p.coeff,
                  sorted(((k, j, i, c) for (i, j, k, c) in p.nnz), key=lambda q: (q[1], q[0], q[2])),
                  (p.l[2], p.l[1], p.l[0])) for p in low.paths]
    return replace(low, in1=low.out, out=low.in1, paths=paths, L1=low.L3, L3=low.L1, label=f"{low.label}-adjoint")

