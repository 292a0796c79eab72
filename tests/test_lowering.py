"""Planner invariants that need no GPU: folding of wide rows with mixed multiplicities, which kernel
sets carry the fused second-order kernels, and that the generated sources compile for gfx950."""

import numpy as np
import pytest

import openequivariance_amd as oeq
from openequivariance_amd import runtime as rt
from openequivariance_amd.codegen import lower as L
from openequivariance_amd.codegen import uvu_double
from openequivariance_amd.core import problems as P


def _unfolded(problem):
    """The tables before folding (what lower() would return for a row that needs none)."""
    low = L.lower(problem)
    in1, in2, out = (L._blocks(ir) for ir in (problem.irreps_in1, problem.irreps_in2, problem.irreps_out))
    return low, in1, in2, out


@pytest.mark.parametrize("problem", P.nequix_problems() + P.seven_net_problems(), ids=lambda p: p.label)
def test_folding_preserves_the_problem(problem):
    low, in1, in2, out = _unfolded(problem)
    wide = max(in1[i.i_in1].mul for i in problem.instructions) > 64
    ragged = any(in1[i.i_in1].mul != 64 * ((max(b.mul for b in in1) + 63) // 64) for i in problem.instructions)
    assert (low.n_chunks == 1) == (not wide or ragged)
    assert (low.L1, low.L2, low.L3, low.WN) == (problem.irreps_in1.dim, problem.irreps_in2.dim,
                                                problem.irreps_out.dim, problem.weight_numel)
    # pieces tile their blocks exactly: same elements, at most 64 channels each
    for pieces, blocks in ((low.in1, in1), (low.out, out)):
        covered = sorted((b.off, b.off + b.mul * b.d) for b in pieces)
        assert covered[0][0] == 0 and covered[-1][1] == sum(b.mul * b.d for b in blocks)
        assert all(a[1] == b[0] for a, b in zip(covered, covered[1:]))
        if low.n_chunks == 1 and wide:
            assert max(b.mul for b in pieces) <= 64
    # every weight belongs to exactly one folded path
    spans = sorted((p.woff, p.woff + low.in1[p.i1].mul * low.in2[p.i2].mul) for p in low.paths)
    assert spans[0][0] == 0 and spans[-1][1] == low.WN and all(a[1] == b[0] for a, b in zip(spans, spans[1:]))
    # same arithmetic: the reference's FLOP count does not change
    plain = sum(3 * len(p.nnz) * low.in1[p.i1].mul * low.in2[p.i2].mul + low.out[p.io].mul * low.out[p.io].d
                for p in low.paths)
    assert low.flops("forward") == plain
    assert sum(low.in1[p.i1].mul for p in low.paths) == sum(in1[i.i_in1].mul for i in problem.instructions)


def test_uniform_wide_rows_are_not_folded():
    low = L.lower(P.config3_mace_uvu())
    assert low.n_chunks == 2 and len(low.paths) == 23 and max(b.mul for b in low.in1) == 128


def test_folding_in_component_major_layout():
    problem = P.seven_net_problems()[1].clone()
    problem.layout = "ir_mul"
    low = L.lower(problem)
    assert low.ir_mul and low.n_chunks == 1 and max(b.mul for b in low.in1) <= 64
    whole = L._blocks(problem.irreps_in1)
    # the two pieces of 128x0e: 64 channels apart, components a whole block's multiplicity apart
    first, second = [b for b in low.in1 if whole[0].off <= b.off < whole[0].off + whole[0].mul * whole[0].d][:2]
    assert (second.off - first.off, first.cstride, second.cstride) == (64, 128, 128)


def test_which_sets_carry_fused_second_order_kernels():
    assert uvu_double.supported(L.lower(P.config3_mace_uvu()))
    assert uvu_double.supported(L.lower(P.config3_mace_uvu()), conv=True)
    seven = L.lower(P.seven_net_problems()[1])
    assert uvu_double.supported(seven) and uvu_double.supported(seven, conv=True)  # 38 paths: within the limit of 96
    assert len(seven.paths) <= uvu_double.CONV_MAX_PATHS < 200
    shared = P.config2_nequip_uvu().clone()
    shared.shared_weights = True
    # shared weights: batch and (device-grouped) convolution
    assert uvu_double.supported(L.lower(shared)) and uvu_double.supported(L.lower(shared), conv=True)
    assert not uvu_double.supported(L.lower(P.config4_uvw_shared()))  # 'uvw' has its own second-order kernels


@pytest.mark.parametrize("make,conv", [(lambda: P.nequix_problems()[1], False), (lambda: P.seven_net_problems()[0], True),
                                       (lambda: P.config2_nequip_uvu(np.float64), True),
                                       (lambda: P.diffdock_problems()[0], False), (lambda: P.tetris_poly_problems()[0], False),
                                       (lambda: P.e3tools_problems()[1], False)],
                         ids=["nequix-main-tp", "sevennet-first-conv", "cfg2-f64-conv", "diffdock-tp", "tetris-tp",
                              "e3tools-transformer-tp"])
def test_generated_sources_compile_for_gfx950(make, conv):
    from openequivariance_amd._torch.tensor_product import build_tp_module
    from openequivariance_amd._torch.tensor_product_conv import build_conv_module
    problem = make()
    src, dims, descs = build_conv_module(problem, True) if conv else build_tp_module(problem)
    blob = rt.compile_source(src, use_disk_cache=False)
    assert all(part[:4] == b"\x7fELF" for part in rt.unpack_code(blob))
    names = {d[1] for d in descs}
    assert {"forward", "backward"} <= names
    if problem.instructions[0].connection_mode == "uvu":
        assert {"double_backward_A", "double_backward_B"} <= names
        assert {d[0] for d in descs} >= {rt.ROLE_DOUBLE_BACKWARD_A, rt.ROLE_DOUBLE_BACKWARD_B}


@pytest.mark.parametrize("mul", [1088, 2048, 2500])
@pytest.mark.parametrize("layout", ["mul_ir", "ir_mul"])
def test_blocks_wider_than_1024_channels_are_cut_into_pieces(mul, layout):
    """One wave per 64-channel chunk and one block of threads per row: 1024 channels is what a block covers,
    so wider irrep blocks are lowered as several pieces of at most 1024 channels, each with its own path
    (the reference chunks any multiplicity, core/ComputationSchedule.py:185-343). The pieces tile the
    block, the paths tile the weights, and the kernels generate and compile."""
    import openequivariance_amd as oeq
    from openequivariance_amd import runtime as rt
    from openequivariance_amd._torch.tensor_product import build_tp_module
    from openequivariance_amd._torch.tensor_product_conv import build_conv_module
    from openequivariance_amd.codegen.lower import lower
    problem = oeq.TPProblem(f"{mul}x1o", "1x1o", f"{mul}x0e+{mul}x2e", [(0, 0, 0, "uvu", True), (0, 0, 1, "uvu", True)],
                            shared_weights=False, internal_weights=False, layout=layout)
    low = lower(problem)
    n_pieces = (mul + 1023) // 1024
    assert low.n_chunks <= 16 and len(low.paths) == 2 * n_pieces
    assert [b.mul for b in low.in1] == [min(1024, mul - 1024 * c) for c in range(n_pieces)]
    assert sorted(p.woff for p in low.paths) == sorted(i * mul + 1024 * c for i in range(2) for c in range(n_pieces))
    if layout == "mul_ir":
        assert [b.off for b in low.in1] == [1024 * 3 * c for c in range(n_pieces)]
    else:
        assert [(b.off, b.cstride) for b in low.in1] == [(1024 * c, mul) for c in range(n_pieces)]
    for src, _dims, _descs in (build_tp_module(problem), build_conv_module(problem, True)):
        assert all(part[:4] == b"\x7fELF" for part in rt.unpack_code(rt.compile_source(src, use_disk_cache=False)))


def test_matrix_core_path_accepts_only_what_its_kernels_can_hold():
    """Every shared-weight problem the matrix-core path accepts generates (its LDS checks raise otherwise): single
    paths up to l = 7 in both precisions. fp64 outputs with l >= 5 exceed the LDS and must be refused, not raise."""
    import numpy as np

    import openequivariance_amd as oeq
    from openequivariance_amd._torch.tensor_product import build_tp_module
    from openequivariance_amd.codegen import uvw_mfma
    from openequivariance_amd.codegen.lower import lower
    accepted = refused_f64 = 0
    for l1 in (0, 3, 5, 7):
        for l2 in (0, 1, 3):
            for l3 in range(abs(l1 - l2), min(l1 + l2, 7) + 1):
                for dt in (np.float32, np.float64):
                    p = oeq.TPProblem(f"64x{l1}e", f"1x{l2}e", f"40x{l3}e", [(0, 0, 0, "uvw", True)], shared_weights=True,
                                      internal_weights=False, irrep_dtype=dt, weight_dtype=dt)
                    if uvw_mfma.supported(lower(p)):
                        src, dims, descs = build_tp_module(p)
                        assert "oeq_mfma" in src
                        accepted += 1
                    else:
                        assert dt == np.float64 and l3 >= 5, (l1, l2, l3, dt)
                        refused_f64 += 1
    assert accepted > 40 and refused_f64 > 5


def test_matrix_core_kernel_plan_covers_every_sub_path_once():
    """The kernels of each pass of the matrix-core path partition the sub-paths (piece of the input block x piece of
    the output block x channel of the second operand): every sub-path in exactly one kernel, exactly one kernel per
    piece that stores instead of adding, weight corners inside the path's weight block and disjoint, parts within
    the register budget."""
    import openequivariance_amd as oeq
    from openequivariance_amd.codegen import uvw_mfma as M
    from openequivariance_amd.codegen.lower import lower
    sh3 = "1x0e+1x1o+1x2e+1x3o"
    problems = [
        P.config4_uvw_shared(),
        P.FullyConnectedTPProblem("64x0e+64x1o+64x2e+64x3o", sh3, "64x0e+64x1o+64x2e+64x3o", shared_weights=True,
                                  internal_weights=False),
        P.FullyConnectedTPProblem("70x0e+20x1o", "2x0e+3x1o", "100x0e+33x1o", shared_weights=True, internal_weights=False),
        P.FullyConnectedTPProblem("130x1o", "1x1o", "5x0e+17x1e+130x2e", shared_weights=True, internal_weights=False),
    ]
    for problem in problems:
        low = lower(problem)
        assert M.supported(low)
        vin, vout, vpaths = M._split(low)
        # the corners of a path tile its weight block
        for p in low.paths:
            U, V, W = low.in1[p.i1].mul, low.in2[p.i2].mul, low.out[p.io].mul
            seen = set()
            for vp in (q for q in vpaths if q.p is p):
                assert vp.ld == V * W
                for u in range(vp.U):
                    for w in (0, vp.Wn - 1):
                        at = vp.woff + u * vp.ld + w
                        assert p.woff <= at < p.woff + U * V * W and at not in seen
                        seen.add(at)
            assert sum(q.U * q.Wn for q in vpaths if q.p is p) == U * V * W
        for side, blocks, which in (("vo", vout, "forward"), ("vi", vin, "dx"), ("vo", vout, "dw")):
            groups = M._groups(vpaths, side, len(blocks), which)
            listed = [vp.index for _, sub, _ in groups for vp in sub]
            assert sorted(listed) == list(range(len(vpaths)))
            for b in range(len(blocks)):
                mine = [g for g in groups if g[0] == b]
                assert sum(1 for g in mine if g[2]) == 1 and mine[0][2]
            for _, sub, _ in groups:
                assert sum(M._slice_regs(vp, which) for vp in sub) <= M.SLICE_REGS[which]


def test_adjoint_problem_gives_the_first_operand_gradient():
    """lower.adjoint: g . F(x, y, w) == x . F_adjoint(g, y, w) for every x and g, i.e. the adjoint problem's forward map
    applied to the output gradient is the gradient with respect to the first operand (evaluated from the lowered
    non-zeros, one row; folded mixed-multiplicity rows included)."""
    import numpy as np
    from openequivariance_amd.codegen.lower import adjoint, lower
    from openequivariance_amd.core import problems as P

    def forward(lw, x, y, w):
        z = np.zeros(lw.L3)
        for p in lw.paths:
            b1, b2, bo = lw.in1[p.i1], lw.in2[p.i2], lw.out[p.io]
            for u in range(b1.mul):
                for (i, j, k, c) in p.nnz:
                    z[bo.off + u * bo.d + k] += c * x[b1.off + u * b1.d + i] * y[b2.off + j] * w[p.woff + u]
        return z

    rng = np.random.default_rng(0)
    for problem in (P.nequix_problems()[2], P.config2_nequip_uvu(), P.seven_net_problems()[0]):
        low = lower(problem)
        adj = adjoint(low)
        assert (adj.L1, adj.L3, adj.WN, adj.L2) == (low.L3, low.L1, low.WN, low.L2)
        x, y, w, g = (rng.normal(size=n) for n in (low.L1, low.L2, low.WN, low.L3))
        lhs, rhs = g @ forward(low, x, y, w), x @ forward(adj, g, y, w)
        assert abs(lhs - rhs) <= 1e-12 * max(1.0, abs(lhs))


def test_backward_wave_count_per_node():
    """Waves that share a node's output gradient in the convolution's backward kernel: one where the register
    estimate fits, else the smallest of two and four whose share fits, and all eight where none does."""
    from openequivariance_amd.codegen import uvu

    def count(problem):
        em = uvu.UvuEmitter(L.lower(problem))
        groups = em.plan_backward_groups(max(1, 8 // em.NCH))
        if groups is not None:  # every output block once, in order
            assert [io for grp in groups for io in grp] == list(em.used_out)
        return 0 if groups is None else len(groups)

    def f64(problem):
        out = problem.clone()
        out.irrep_dtype = out.weight_dtype = np.float64
        return out

    assert count(P.config5_mace_conv()) == 0                      # fits one wave's registers by the ordinary rule
    assert count(P.seven_net_problems()[1]) == 2
    assert count(P.nequip_problems()[3]) == 4                     # benzene
    assert count(f64(P.nequip_problems()[3])) == 8                # ... whose shares in double precision never fit
