"""Ready-made tensor-product problems.

Constructors with the same names and instruction/irrep ordering as the
reference's problem zoo (openequivariance/openequivariance/benchmark/problems.py:14-33,
122-196, 292-330), plus the five benchmark configurations of this package.
"""

from __future__ import annotations

from typing import Optional

import numpy as np

from .spec import Irreps, TPProblem


class FullyConnectedTPProblem(TPProblem):
    """Every allowed (in1, in2, out) triple gets one 'uvw' path
    (problems.py:14-33): ``i_1`` outer, ``i_2`` middle, ``i_out`` inner."""

    def __init__(self, irreps_in1, irreps_in2, irreps_out, **kwargs) -> None:
        a, b, o = Irreps(irreps_in1), Irreps(irreps_in2), Irreps(irreps_out)
        paths = []
        for i1, (_, ir1) in enumerate(a):
            for i2, (_, ir2) in enumerate(b):
                allowed = list(ir1 * ir2)
                for io, (_, iro) in enumerate(o):
                    if iro in allowed:
                        paths.append((i1, i2, io, "uvw", True, 1.0))
        super().__init__(a, b, o, paths, **kwargs)


class ChannelwiseTPP(TPProblem):
    """MACE/NequIP-style per-channel ('uvu') product (problems.py:122-170).

    A path (i, j -> ir_out) is kept iff ``ir_out`` occurs in the target
    ``irreps_out``; every kept path owns a separate output block of
    multiplicity ``mul_i``. Blocks are then stably sorted by ``(l, p)`` and
    the instruction list by output index, which also fixes the weight order.
    """

    def __init__(
        self,
        irreps_in1,
        irreps_in2,
        irreps_out,
        label: Optional[str] = None,
        irrep_dtype=np.float32,
        weight_dtype=np.float32,
    ):
        a, b, target = Irreps(irreps_in1), Irreps(irreps_in2), Irreps(irreps_out)
        blocks, paths = [], []
        for i, (mul, ir_in) in enumerate(a):
            for j, (_, ir_edge) in enumerate(b):
                for ir_out in ir_in * ir_edge:
                    if ir_out in target:
                        paths.append((i, j, len(blocks), "uvu", True))
                        blocks.append((mul, ir_out))
        ordered, new_index, _ = Irreps(blocks).sort()
        paths = sorted(((i, j, new_index[k], m, t) for i, j, k, m, t in paths), key=lambda t: t[2])
        super().__init__(
            a,
            b,
            ordered,
            paths,
            internal_weights=False,
            shared_weights=False,
            label=label,
            irrep_dtype=irrep_dtype,
            weight_dtype=weight_dtype,
        )


class SingleInstruction(TPProblem):
    """One instruction ``(0, 0, 0, mode, True)`` (problems.py:173-196)."""

    def __init__(self, irreps_in1, irreps_in2, irreps_in3, mode: str, label: Optional[str] = None, **kwargs):
        kwargs.setdefault("internal_weights", False)
        kwargs.setdefault("shared_weights", False)
        super().__init__(
            Irreps(irreps_in1), Irreps(irreps_in2), Irreps(irreps_in3), [(0, 0, 0, mode, True)], label=label, **kwargs
        )


FCTPP = FullyConnectedTPProblem
CTPP = ChannelwiseTPP


def mace_problems():
    """problems.py:292-309."""
    return [
        CTPP("128x0e+128x1o+128x2e", "1x0e+1x1o+1x2e+1x3o", "128x0e+128x1o+128x2e+128x3o", "mace-large"),
        CTPP("128x0e+128x1o", "1x0e+1x1o+1x2e+1x3o", "128x0e+128x1o+128x2e", "mace-medium"),
    ]


def nequip_problems():
    """problems.py:312-345."""
    return [
        CTPP(
            "32x0o + 32x0e + 32x1o + 32x1e + 32x2o + 32x2e",
            "0e + 1o + 2e",
            "32x0o + 32x0e + 32x1o + 32x1e + 32x2o + 32x2e",
            "nequip-lips",
        ),
        CTPP("64x0o + 64x0e + 64x1o + 64x1e", "0e + 1o", "64x0o + 64x0e + 64x1o + 64x1e", "nequip-revmd17-aspirin"),
        CTPP(
            "64x0o + 64x0e + 64x1o + 64x1e + 64x2o + 64x2e",
            "0e + 1o + 2e",
            "64x0o + 64x0e + 64x1o + 64x1e + 64x2o + 64x2e",
            "nequip-revmd17-toluene",
        ),
        CTPP(
            "64x0o + 64x0e + 64x1o + 64x1e + 64x2o + 64x2e + 64x3o + 64x3e",
            "0e + 1o + 2e + 3o",
            "64x0o + 64x0e + 64x1o + 64x1e + 64x2o + 64x2e + 64x3o + 64x3e",
            "nequip-revmd17-benzene",
        ),
        CTPP("32x0o + 32x0e + 32x1o + 32x1e", "0e + 1o", "32x0o + 32x0e + 32x1o + 32x1e", "nequip-water"),
    ]


def tetris_poly_problems():
    """The two fully connected products of e3nn's tetris polynomial example (problems.py:253-270);
    default (shared) weights."""
    return [
        FCTPP("1x0e + 1x1o + 1x2e + 1x3o", "1x0e + 1x1o + 1x2e + 1x3o", "64x0e + 24x1e + 24x1o + 16x2e + 16x2o",
              label="tetris-poly-1"),
        FCTPP("64x0e + 24x1e + 24x1o + 16x2e + 16x2o", "1x0e + 1x1o + 1x2e", "0o + 6x0e", label="tetris-poly-2"),
    ]


def nequix_problems():
    """NequiX MP-1 layers: mixed multiplicities per irrep, one with 89 channels (problems.py:351-372)."""
    sh = "1x0e+1x1o+1x2e+1x3o"
    mid = "128x0e+64x1o+32x2e+32x3o"
    return [
        CTPP("89x0e", sh, "89x0e+89x1o+89x2e+89x3o", "nequix-mp-1-first_layer"),
        CTPP(mid, sh, "128x0e+128x1o+128x2e+128x3o+64x1o+64x0e+64x2e+64x1o+64x3o+64x2e+32x2e+32x1o+32x3o+32x0e+32x2e"
                      "+32x1o+32x3o+32x3o+32x2e+32x1o+32x3o+32x0e+32x2e", "nequix-mp-1-main_layers"),
        CTPP(mid, sh, "128x0e+64x0e+32x0e+32x0e", "nequix-mp-1-last_layer"),
    ]


def seven_net_problems():
    """SevenNet l3i5 layers, even-parity harmonics (problems.py:375-395)."""
    sh = "1x0e+1x1e+1x2e+1x3e"
    mid = "128x0e+64x1e+32x2e+32x3e"
    return [
        CTPP("128x0e", sh, "128x0e+128x1e+128x2e+128x3e", "SevenNet_l3i5-first-layer"),
        CTPP(mid, sh, "128x0e+64x0e+32x0e+32x0e+128x1e+64x1e+64x1e+64x1e+32x1e+32x1e+32x1e+32x1e+32x1e+128x2e+64x2e"
                      "+64x2e+64x2e+32x2e+32x2e+32x2e+32x2e+32x2e+32x2e+32x2e+128x3e+64x3e+64x3e+32x3e+32x3e+32x3e"
                      "+32x3e+32x3e+32x3e+32x3e", "SevenNet_l3i5-main-layers"),
        CTPP(mid, sh, "128x0e+64x0e+32x0e+32x0e", "SevenNet_l3i5-last-layer"),
    ]


def diffdock_problems():
    """Fully connected DiffDock score-model layers with per-row weights (problems.py:273-289)."""
    feats = "10x1o + 10x1e + 48x0e + 48x0o"
    return [
        FCTPP(feats, "1x0e + 1x1o", feats, shared_weights=False, label="DiffDock-L=1"),
        FCTPP(feats, "1x0e + 1x1o + 1x2e", feats, shared_weights=False, label="DiffDock-L=2"),
    ]


def e3tools_problems():
    """e3tools convolution / transformer blocks (problems.py:398-419); the second shares its weights."""
    return [
        FCTPP("64x0e+16x1o", "1x0e+1x1o", "80x0e+16x1o", label="e3tools_conv", shared_weights=False,
              internal_weights=False),
        FCTPP("64x0e+16x1o", "1x0e+1x1o", "64x0e+16x1o", label="e3tools_transformer", shared_weights=True,
              internal_weights=False),
    ]


# ---------------------------------------------------------------------------
# The five benchmark configurations
# ---------------------------------------------------------------------------

_DT = {"float32": np.float32, "float64": np.float64, np.float32: np.float32, np.float64: np.float64}


def _natural_parity_target(lmax: int) -> str:
    return "+".join(f"{l}{'e' if l % 2 == 0 else 'o'}" for l in range(lmax + 1))


def config1_single_uvu(dtype=np.float32) -> TPProblem:
    """1x2e (x) 1x3e -> 1x2e, one 'uvu' instruction, per-row weights."""
    return TPProblem(
        "1x2e", "1x3e", "1x2e", [(0, 0, 0, "uvu", True)],
        shared_weights=False, internal_weights=False, label="cfg1-single-uvu",
        irrep_dtype=_DT[dtype], weight_dtype=_DT[dtype],
    )


def config2_nequip_uvu(dtype=np.float32) -> TPProblem:
    """32x{0e,1o,2e} (x) SH(lmax 3) -> all natural-parity outputs with l<=2
    (13 'uvu' paths, one output block per path)."""
    return CTPP("32x0e+32x1o+32x2e", "1x0e+1x1o+1x2e+1x3o", _natural_parity_target(2),
                "cfg2-nequip-uvu", _DT[dtype], _DT[dtype])


def config3_mace_uvu(dtype=np.float32) -> TPProblem:
    """128x{0e,1o,2e,3o} (x) SH(lmax 3) -> all natural-parity outputs with
    l<=3 (23 'uvu' paths; L1=2048, L3=12672, weight_numel=2944)."""
    return CTPP("128x0e+128x1o+128x2e+128x3o", "1x0e+1x1o+1x2e+1x3o", _natural_parity_target(3),
                "cfg3-mace-uvu", _DT[dtype], _DT[dtype])


def config4_uvw_shared(dtype=np.float32) -> TPProblem:
    """64x{0e,1o,2e} (x) {0e,1o,2e} -> 64x{0e,1o,2e}, fully connected 'uvw',
    one shared weight tensor (11 paths, weight_numel=45056)."""
    return FCTPP("64x0e+64x1o+64x2e", "1x0e+1x1o+1x2e", "64x0e+64x1o+64x2e",
                 shared_weights=True, internal_weights=False, label="cfg4-uvw-shared",
                 irrep_dtype=_DT[dtype], weight_dtype=_DT[dtype])


def config5_mace_conv(dtype=np.float32) -> TPProblem:
    """The config-3 problem, used as a fused graph convolution."""
    p = config3_mace_uvu(dtype)
    p.label = "cfg5-mace-conv"
    return p


def factor_shared_uvw(problem: TPProblem):
    """A fully connected ('uvw') problem with ONE weight tensor for all rows and single-channel second
    operands, written as two problems: ``A`` = the CG contraction without the channel mix, one output block
    ``U x l3`` per path ('uvu', weights all one), and ``B`` = the channel mix of those blocks ('uvw' against a
    scalar one, same weight tensor as the original, same order). ``TP(x, y, W) = B(A(x, y, 1), 1, W)`` for one
    row; over a graph the sum over a receiver's edges commutes with the mix, because the weights do not
    depend on the edge: ``sum_e B(A(x_e, y_e), W) = B(sum_e A(x_e, y_e), W)``. So the convolution is the
    fused 'uvu' convolution of ``A`` followed by ``B`` on one row per NODE: the channel mix runs once per node
    instead of once per edge and nothing of size [edges, L3] exists. (The reference mixes per edge inside its
    edge loop, templates/loop_unroll_conv_atomic.cuh:52-180 with loop_unroll_tp.cuh:55-84.) None when the
    problem does not have this shape."""
    ins = problem.instructions
    if not problem.shared_weights or not ins or any(i.connection_mode != "uvw" or not i.has_weight for i in ins):
        return None
    in1, in2, out = problem.irreps_in1, problem.irreps_in2, problem.irreps_out
    if any(in2[i.i_in2].mul != 1 for i in ins):
        return None
    mid = Irreps([(in1[i.i_in1].mul, out[i.i_out].ir) for i in ins])
    common = dict(irrep_normalization="none", path_normalization="none", shared_weights=True, internal_weights=False,
                  irrep_dtype=problem.irrep_dtype, weight_dtype=problem.weight_dtype)
    # stored coefficient = sqrt(path weight given here). The scalar second operand of B brings the factor
    # wigner_3j(l, 0, l) = identity / sqrt(2l+1), which A's coefficient makes up for.
    a = TPProblem(in1, in2, mid, [(i.i_in1, i.i_in2, n, "uvu", True, i.path_weight ** 2 * out[i.i_out].ir.dim)
                                  for n, i in enumerate(ins)], label=f"{problem.label}-contraction", **common)
    b = TPProblem(mid, "1x0e", out, [(n, 0, i.i_out, "uvw", True, 1.0) for n, i in enumerate(ins)],
                  label=f"{problem.label}-mix", **common)
    assert b.weight_numel == problem.weight_numel
    return a, b
