"""GPU parity of the batched tensor product against the CPU oracle, through
the torch ops and directly through the C ABI. Tolerances: max normalised error
<= 1e-5 (fp32) and <= 1e-12 (fp64) against the float64 oracle."""

import numpy as np
import pytest
import torch

import openequivariance_amd as oeq
from openequivariance_amd._torch import ops
from openequivariance_amd.core import problems as P
from oracle import e3nn_ref as R
from gpu_util import err, to_gpu, tol_of, tp_inputs

pytestmark = pytest.mark.gpu


def _odd_uvu(shared):
    return oeq.TPProblem("5x1e+3x2e", "2x1e+1x0e", "5x1e+3x2e+5x0e",
                         [(0, 0, 0, "uvu", True), (0, 1, 0, "uvu", True), (1, 0, 1, "uvu", True),
                          (0, 0, 2, "uvu", True)], shared_weights=shared, internal_weights=False, label="odd-uvu")


def _odd_uvw(shared):
    return oeq.TPProblem("5x1e+3x2e+70x0e", "2x1e+1x0e", "7x1e+3x2e+100x0e",
                         [(0, 0, 0, "uvw", True), (0, 1, 0, "uvw", True), (1, 0, 1, "uvw", True),
                          (0, 0, 2, "uvw", True), (2, 1, 2, "uvw", True, 0.3)], shared_weights=shared,
                         internal_weights=False, label="odd-uvw")


def _single_channel_uvw(shared):
    # first operand with one channel per irrep (lanes = output channels in backward), outputs wider than a wave
    return oeq.TPProblem("1x1o+1x0e+1x2e", "1x1o+2x0e", "70x1o+24x0e+130x1e+3x2e",
                         [(0, 1, 0, "uvw", True), (1, 1, 1, "uvw", True), (0, 0, 2, "uvw", True),
                          (2, 1, 3, "uvw", True), (1, 0, 0, "uvw", True, 0.5)], shared_weights=shared,
                         internal_weights=False, label="single-channel-uvw")


def _very_wide_ragged():
    # wider than four waves with a different multiplicity per irrep: not folded, the chunk waves run
    # bodies specialised per chunk
    return oeq.TPProblem("300x0e+70x1o+20x2e", "1x0e+1x1o", "300x0e+70x1o+300x1o+20x1o",
                         [(0, 0, 0, "uvu", True), (1, 0, 1, "uvu", True), (0, 1, 2, "uvu", True),
                          (2, 1, 3, "uvu", True)], shared_weights=False, internal_weights=False,
                         label="very-wide-ragged")


def _folded_with_gaps():
    # a row wider than a wave with a different multiplicity per irrep (folded into 64-channel pieces), one
    # input block no instruction reads, one output block no instruction writes, second operand with mul 2
    return oeq.TPProblem("100x0e+70x1o+40x2e+96x1e", "1x0e+2x1o", "100x0e+70x1o+100x1o+40x1o+33x2e",
                         [(0, 0, 0, "uvu", True), (1, 0, 1, "uvu", True), (0, 1, 2, "uvu", True),
                          (2, 1, 3, "uvu", True, 0.7)], shared_weights=False, internal_weights=False,
                         label="folded-gaps")


def _fc_shared(in1, in2, out):
    return P.FullyConnectedTPProblem(in1, in2, out, shared_weights=True, internal_weights=False,
                                     label=f"fc-shared {in1}")


def _shared(problem):
    q = problem.clone()
    q.shared_weights = True
    return q


def _as_f64(problem):
    q = problem.clone()
    q.irrep_dtype, q.weight_dtype = np.float64, np.float64
    return q


CASES = [
    ("cfg1-b1000", P.config1_single_uvu, 1000),
    ("cfg1-b37", P.config1_single_uvu, 37),
    ("cfg1-f64", lambda: P.config1_single_uvu(np.float64), 129),
    ("cfg2", P.config2_nequip_uvu, 301),
    ("cfg3-f32", P.config3_mace_uvu, 203),
    ("cfg3-f64", lambda: P.config3_mace_uvu(np.float64), 101),
    ("cfg4-shared", P.config4_uvw_shared, 257),
    ("cfg4-f64", lambda: P.config4_uvw_shared(np.float64), 50),
    ("mace-large", lambda: P.mace_problems()[0], 99),
    ("nequip-aspirin", lambda: P.nequip_problems()[1], 99),
    ("odd-uvu", lambda: _odd_uvu(False), 77),
    ("odd-uvu-shared", lambda: _odd_uvu(True), 77),
    ("wide-uvu-shared", lambda: oeq.TPProblem(
        "100x1e+70x2e", "1x1e+1x0e", "100x1e+70x2e+100x0e",
        [(0, 0, 0, "uvu", True), (0, 1, 0, "uvu", True), (1, 0, 1, "uvu", True), (0, 0, 2, "uvu", True)],
        shared_weights=True, internal_weights=False), 77),
    ("uvu-l5", lambda: P.SingleInstruction("33x5e", "1x3e", "33x5e", "uvu"), 40),
    ("uvu-mul2", lambda: P.SingleInstruction("19x2e", "3x1e", "19x2e", "uvu"), 40),
    ("uvu-mul2-big", lambda: P.SingleInstruction("4x1e", "12x1e", "4x1e", "uvu"), 40),
    ("uvw-unshared", lambda: P.FullyConnectedTPProblem("16x0e+16x1o", "1x0e+1x1o", "16x0e+16x1o",
                                                      shared_weights=False, internal_weights=False), 33),
    # production layers with a different multiplicity per irrep (rows wider than a wave: the chunks of a
    # row then run different code), one with 89 channels
    ("single-channel-uvw", lambda: _single_channel_uvw(False), 45),
    ("single-channel-uvw-shared", lambda: _single_channel_uvw(True), 45),
    ("single-channel-uvw-f64", lambda: _as_f64(_single_channel_uvw(False)), 23),
    ("very-wide-ragged", _very_wide_ragged, 37),
    ("folded-gaps", _folded_with_gaps, 61),
    ("folded-gaps-f64", lambda: _as_f64(_folded_with_gaps()), 37),
    ("nequix-first", lambda: P.nequix_problems()[0], 53),
    ("nequix-main", lambda: P.nequix_problems()[1], 53),
    ("nequix-last", lambda: P.nequix_problems()[2], 53),
    ("sevennet-main", lambda: P.seven_net_problems()[1], 53),
    ("sevennet-main-f64", lambda: _as_f64(P.seven_net_problems()[1]), 29),
    ("tetris-1", lambda: P.tetris_poly_problems()[0], 53),
    ("tetris-2", lambda: P.tetris_poly_problems()[1], 53),
    ("odd-uvw", lambda: _odd_uvw(False), 21),
    ("odd-uvw-shared", lambda: _odd_uvw(True), 21),
    # shared-weight 'uvw' on the matrix cores: 32 channels (half the waves sit out the multiplies), 128 channels
    # (two pieces per irrep, four sub-paths per path, later kernels add to the first one's rows), a different
    # multiplicity per irrep, an input irrep no path reads and an output irrep no path writes
    ("mfma-32", lambda: _fc_shared("32x0e+32x1o+32x2e", "1x0e+1x1o+1x2e", "32x0e+32x1o+32x2e"), 75),
    ("mfma-128", lambda: _fc_shared("128x0e+128x1o", "1x0e+1x1o", "128x0e+128x1o"), 45),
    ("mfma-mixed", lambda: _fc_shared("64x0e+32x1o+16x2e", "1x0e+1x1o", "48x0e+80x1o+16x2e"), 50),
    ("mfma-gaps", lambda: oeq.TPProblem(
        "32x0e+16x1o+48x2e", "1x0e+1x1o", "32x0e+16x1e+64x1o",
        [(0, 0, 0, "uvw", True), (0, 1, 2, "uvw", True), (1, 0, 2, "uvw", True, 0.6), (1, 1, 0, "uvw", True)],
        shared_weights=True, internal_weights=False, label="mfma-gaps"), 50),
    # the same kernels in fp64 (v_mfma_f64_16x16x4_f64, whose result rows are laid out differently)
    ("mfma-128-f64", lambda: _as_f64(_fc_shared("128x0e+128x1o", "1x0e+1x1o", "128x0e+128x1o")), 45),
    ("mfma-mixed-f64", lambda: _as_f64(_fc_shared("64x0e+32x1o+16x2e", "1x0e+1x1o", "48x0e+80x1o+16x2e")), 50),
    # fp64 with l = 3 outputs: two copies of the 64 x 7 x 17 T tile beside the dZ columns exceed the 160 KB of LDS;
    # the dW kernels then keep one copy, and pieces whose columns would not fit together stay in separate kernels
    ("mfma-l3-f64", lambda: _as_f64(oeq.TPProblem(
        "64x1e+64x0e", "1x2o+1x2e+1x0o", "48x1e+80x3o", [(0, 0, 1, "uvw", True, 0.8), (0, 1, 0, "uvw", True)],
        shared_weights=True, internal_weights=False, label="mfma-l3")), 50),
    ("mfma-l3-wide-f64", lambda: _as_f64(oeq.TPProblem(
        "16x1o+128x3o", "1x2o", "96x3e", [(0, 0, 0, "uvw", True), (1, 0, 0, "uvw", True, 0.6)],
        shared_weights=True, internal_weights=False, label="mfma-l3-wide")), 40),
    # multiplicities that are no multiples of 16 (or of 4): tiles padded with zero weights. Channels past a piece are
    # neither loaded nor stored; 70 and 100 channels leave a narrow second piece; a block no path reads or writes
    ("mfma-pad-diffdock", lambda: _shared(P.diffdock_problems()[0]), 50),
    ("mfma-pad-mid", lambda: _fc_shared("40x0e+30x1o", "1x0e+1x1o", "50x0e+20x1o+10x2e"), 67),
    ("mfma-pad-mid-f64", lambda: _as_f64(_fc_shared("40x0e+30x1o", "1x0e+1x1o", "50x0e+20x1o+10x2e")), 35),
    ("mfma-pad-wide", lambda: _fc_shared("100x0e+70x1o", "1x0e+1x1o", "33x0e+20x1o"), 50),
    ("mfma-pad-wide-f64", lambda: _as_f64(_fc_shared("70x0e+20x1o", "1x0e+1x1o", "70x0e+20x1o")), 33),
    ("mfma-pad-gaps", lambda: oeq.TPProblem(
        "30x0e+13x1o+45x2e", "1x0e+1x1o", "27x0e+15x1e+61x1o",
        [(0, 0, 0, "uvw", True), (0, 1, 2, "uvw", True), (1, 0, 2, "uvw", True, 0.6), (1, 1, 0, "uvw", True)],
        shared_weights=True, internal_weights=False, label="mfma-pad-gaps"), 50),
    # second operands with several channels: one sub-path per channel (rows of its weight matrix V * W words apart)
    ("mfma-mul2-pad", lambda: _fc_shared("40x0e+30x1o", "2x0e+1x1o", "25x0e+10x1o+5x2e"), 50),
    ("mfma-mul3-f64", lambda: _as_f64(_fc_shared("64x0e+64x1o", "3x0e+2x1o", "64x0e+64x1o")), 33),
    ("mfma-mul2-mixed", lambda: oeq.TPProblem(
        "32x0e+20x1o", "1x0e+3x1o+2x1e", "16x0e+40x1o+24x1e",
        [(0, 0, 0, "uvw", True), (0, 1, 1, "uvw", True, 0.7), (1, 1, 0, "uvw", True), (1, 2, 1, "uvw", True),
         (1, 0, 1, "uvw", True), (0, 2, 2, "uvw", True)],
        shared_weights=True, internal_weights=False, label="mfma-mul2-mixed"), 50),
    # irreps fed by more paths than one kernel holds weight slices for (seven 64-channel paths into l = 3; six per
    # irrep with both parities): the group of sub-paths is cut into parts, later parts add to the first one's rows
    ("mfma-64-l3", lambda: _fc_shared("64x0e+64x1o+64x2e+64x3o", "1x0e+1x1o+1x2e+1x3o", "64x0e+64x1o+64x2e+64x3o"), 40),
    # second operands of 35 to 64 values (many channels; spherical harmonics up to l = 6 and 7)
    ("mfma-in2-35", lambda: _fc_shared("20x0e+10x1o", "20x0e+5x1o", "12x0e+6x1o"), 45),
    ("mfma-sh6-f64", lambda: _as_f64(_fc_shared("64x0e+64x1o+64x2e", "1x0e+1x1o+1x2e+1x3o+1x4e+1x5o+1x6e",
                                                "64x0e+64x1o+64x2e")), 35),
    ("mfma-sh7", lambda: _fc_shared("32x0e+32x1o+32x2e+32x3o", "1x0e+1x1o+1x2e+1x3o+1x4e+1x5o+1x6e+1x7o",
                                    "32x0e+32x1o+32x2e+32x3o"), 35),
    # l = 7 on either side (15 components per channel)
    ("mfma-l7", lambda: oeq.TPProblem("64x7e", "1x1e", "40x7e", [(0, 0, 0, "uvw", True)], shared_weights=True,
                                      internal_weights=False, label="mfma-l7"), 37),
    ("mfma-l7-in-f64", lambda: _as_f64(oeq.TPProblem("20x7e", "1x4e", "70x3e", [(0, 0, 0, "uvw", True)],
                                                    shared_weights=True, internal_weights=False, label="mfma-l7-in")), 37),
    # (rows of 2 048 values: the dZ tile of the dX kernels is staged in two rounds)
    ("mfma-128-l3", lambda: _fc_shared("128x0e+128x1o+128x2e+128x3o", "1x0e+1x1o+1x2e+1x3o",
                                       "128x0e+128x1o+128x2e+128x3o"), 21),
    ("mfma-50-l3-f64", lambda: _as_f64(_fc_shared("50x0e+50x1o+50x2e+50x3o", "1x0e+1x1o+1x2e+1x3o",
                                                   "50x0e+50x1o+50x2e+50x3o")), 35),
    ("mfma-64-l2-both-parities", lambda: _fc_shared("64x0e+64x0o+64x1e+64x1o+64x2e+64x2o", "1x0e+1x1o+1x2e",
                                                    "64x0e+64x0o+64x1e+64x1o+64x2e+64x2o"), 40),
    ("mfma-pad-l3", lambda: oeq.TPProblem(
        "14x1o+90x3o", "1x2o", "75x3e+11x1e", [(0, 0, 0, "uvw", True), (1, 0, 0, "uvw", True, 0.6), (1, 0, 1, "uvw", True)],
        shared_weights=True, internal_weights=False, label="mfma-pad-l3"), 40),
]
MFMA_CASES = {"cfg4-shared", "cfg4-f64", "mfma-32", "mfma-128", "mfma-mixed", "mfma-gaps", "mfma-128-f64",
              "mfma-mixed-f64", "mfma-l3-f64", "mfma-l3-wide-f64", "mfma-pad-diffdock", "mfma-pad-mid",
              "mfma-pad-mid-f64", "mfma-pad-wide", "mfma-pad-wide-f64", "mfma-pad-gaps", "mfma-pad-l3", "mfma-mul2-pad",
              "mfma-mul3-f64", "mfma-mul2-mixed", "mfma-64-l3", "mfma-50-l3-f64",
              "mfma-64-l2-both-parities", "mfma-128-l3", "mfma-l7", "mfma-l7-in-f64", "mfma-in2-35",
              "mfma-sh6-f64", "mfma-sh7"}
# shared weights off the matrix cores (second operand of more than 64 values): the general kernels' weight gradient
# in an LDS copy per wave and in partial rows in global memory
# irrep blocks of more than 1024 channels, cut into pieces of 1024 by the planner (one block of 1024
# threads covers 16 chunks of 64): two pieces, a ragged last piece, a second operand with two channels (the
# component-major layout of such blocks: tests/test_ir_mul_gpu.py)
CASES += [
    ("uvu-2048", lambda: oeq.TPProblem("2048x1o", "1x1o", "2048x0e+2048x1e+2048x2e",
                                       [(0, 0, 0, "uvu", True), (0, 0, 1, "uvu", True), (0, 0, 2, "uvu", True)],
                                       shared_weights=False, internal_weights=False, label="uvu-2048"), 21),
    ("uvu-1500-mixed", lambda: oeq.TPProblem("1500x1o+70x0e", "2x1o+1x0e", "1500x2e+70x0e+1500x1o",
                                             [(0, 0, 0, "uvu", True), (1, 1, 1, "uvu", True), (0, 1, 2, "uvu", True)],
                                             shared_weights=False, internal_weights=False, label="uvu-1500"), 19),
    ("uvu-2048-shared-f64", lambda: _as_f64(oeq.TPProblem(
        "2048x1o", "1x1o", "2048x0e", [(0, 0, 0, "uvu", True)], shared_weights=True, internal_weights=False,
        label="uvu-2048-shared")), 33),
]

CASES += [
    ("uvw-shared-lds", lambda: _fc_shared("20x0e+10x1o", "40x0e+10x1o", "12x0e+6x1o"), 77),
    ("uvw-shared-lds-wide", lambda: _fc_shared("70x0e+3x1o", "1x0e+1x1o+1x2e+1x3o+1x4e+1x5o+1x6e+1x7o+1x8e", "3x0e+2x1o"), 77),
    ("uvw-shared-global-f64", lambda: _as_f64(_fc_shared("20x0e+10x1o", "40x0e+10x1o", "40x0e+20x1o")), 41),
]


@pytest.mark.parametrize("name,make,B", CASES, ids=[c[0] for c in CASES])
def test_forward_backward_match_oracle(name, make, B):
    problem = make()
    tol = tol_of(problem)
    x, y, w, g = tp_inputs(problem, B, seed=12345)
    ref = R.Problem.from_spec(problem)
    z_ref = R.tp_forward(ref, x, y, w)
    dx_ref, dy_ref, dw_ref = R.tp_backward(ref, x, y, w, g)
    tp = oeq.TensorProduct(problem)
    if name in MFMA_CASES:
        from openequivariance_amd.codegen import uvw_mfma
        from openequivariance_amd.codegen.lower import lower
        assert uvw_mfma.supported(lower(problem)), "this case is meant to run on the MFMA kernels"
    tx, ty, tw = to_gpu(x, y, w, requires_grad=True)
    (tg,) = to_gpu(g)
    z = tp(tx, ty, tw)
    assert z.shape == (B, problem.irreps_out.dim)
    assert err(z, z_ref) <= tol
    z.backward(tg)
    assert err(tx.grad, dx_ref) <= tol
    assert err(ty.grad, dy_ref) <= tol
    # a shared weight gradient sums `B` same-sign terms (the inputs are uniform[0,1)); it still has to meet
    # the tolerance of every other result
    assert err(tw.grad, dw_ref) <= tol


BF3_CASES = [c for c in CASES if c[0] in ("cfg4-shared", "mfma-mixed", "mfma-pad-diffdock", "mfma-mul2-pad", "mfma-64-l3",
                                          "mfma-l7")]


@pytest.mark.parametrize("name,make,B", BF3_CASES, ids=[c[0] for c in BF3_CASES])
def test_split_operand_forward(name, make, B, monkeypatch):
    """uvw_bf3=1: the forward channel mix with every fp32 operand split into three bf16 parts and the six leading
    cross products on the bf16 matrix instruction (the opt-in form of the matrix-core forward kernels). It meets the
    same bound as the fp32 instruction; second order as well (its kernel A is made of forward kernels). A problem
    whose operand planes exceed the LDS (l = 7) keeps the fp32 form."""
    monkeypatch.setenv("OEQ_AMD_TUNE", "uvw_bf3=1")
    problem = make()
    x, y, w, g = tp_inputs(problem, B, seed=4321)
    ref = R.Problem.from_spec(problem)
    tp = oeq.TensorProduct(problem)
    src = ops.get_entry(tp.kid).build_fn()[0]
    assert ("oeq_mfma_bf(" in src) == (name != "mfma-l7")
    tx, ty, tw = to_gpu(x, y, w, requires_grad=True)
    z = tp(tx, ty, tw)
    assert err(z, R.tp_forward(ref, x, y, w)) <= tol_of(problem)
    (tg,) = to_gpu(g)
    first = torch.autograd.grad(z, (tx, ty, tw), tg, create_graph=True)
    second = torch.autograd.grad(sum((t ** 2).sum() for t in first), (tx, ty, tw))
    monkeypatch.setenv("OEQ_AMD_TUNE", "")
    tp0 = oeq.TensorProduct(problem)
    ux, uy, uw = to_gpu(x, y, w, requires_grad=True)
    first0 = torch.autograd.grad(tp0(ux, uy, uw), (ux, uy, uw), tg, create_graph=True)
    second0 = torch.autograd.grad(sum((t ** 2).sum() for t in first0), (ux, uy, uw))
    for a_, b_ in zip(second, second0):
        assert float((a_ - b_).abs().max() / b_.abs().max()) <= 1e-5


def test_same_precision_reference_is_not_closer_by_accident():
    """fp32 kernel vs the oracle evaluated in fp32: same order of error."""
    problem = P.config3_mace_uvu()
    x, y, w, g = tp_inputs(problem, 64, seed=1)
    ref = R.Problem.from_spec(problem)
    z32 = R.tp_forward(ref, x, y, w, dtype=np.float32)
    tp = oeq.TensorProduct(problem)
    z = tp(*to_gpu(x, y, w))
    assert err(z, z32) <= 1e-5


def test_c_abi_direct_call():
    """Call oeq_tp_forward / oeq_tp_backward through ctypes with raw pointers."""
    from openequivariance_amd import runtime as rt
    from openequivariance_amd._torch.tensor_product import build_tp_module
    problem = P.config2_nequip_uvu()
    src, dims, descs = build_tp_module(problem)
    ks = rt.get_kernel_set(src, dims, descs)
    B = 123
    x, y, w, g = tp_inputs(problem, B, seed=7)
    tx, ty, tw, tg = to_gpu(x, y, w, g)
    out = torch.empty(B, problem.irreps_out.dim, device="cuda")
    dx, dy, dw = torch.empty_like(tx), torch.empty_like(ty), torch.empty_like(tw)
    stream = torch.cuda.current_stream().cuda_stream
    ks.tp_forward(B, tx.data_ptr(), ty.data_ptr(), tw.data_ptr(), out.data_ptr(), stream)
    ks.tp_backward(B, tx.data_ptr(), dx.data_ptr(), ty.data_ptr(), dy.data_ptr(), tw.data_ptr(), dw.data_ptr(),
                   tg.data_ptr(), 0, 0, stream)
    torch.cuda.synchronize()
    ref = R.Problem.from_spec(problem)
    assert err(out, R.tp_forward(ref, x, y, w)) <= 1e-5
    dx_ref, dy_ref, dw_ref = R.tp_backward(ref, x, y, w, g)
    assert err(dx, dx_ref) <= 1e-5 and err(dy, dy_ref) <= 1e-5 and err(dw, dw_ref) <= 1e-5
    # NULL buffers are refused with an error code, not a fault
    with pytest.raises(rt.OeqError, match="NULL buffer"):
        ks.tp_forward(B, 0, ty.data_ptr(), tw.data_ptr(), out.data_ptr(), stream)


def test_empty_batch():
    """No rows: empty results, nothing launched; through autograd too (the empty gradients have no address).
    With shared weights the weight gradient is a sum over no rows: zeros."""
    tp = oeq.TensorProduct(P.config1_single_uvu())
    xs = [torch.zeros(0, n, device="cuda", requires_grad=True) for n in (5, 7, 1)]
    z = tp(*xs)
    assert z.shape == (0, 5)
    z.backward(torch.zeros(0, 5, device="cuda"))
    assert [tuple(t.grad.shape) for t in xs] == [(0, 5), (0, 7), (0, 1)]
    shared = P.config1_single_uvu().clone()
    shared.shared_weights = True
    tps = oeq.TensorProduct(shared)
    xs = [torch.zeros(0, 5, device="cuda", requires_grad=True), torch.zeros(0, 7, device="cuda", requires_grad=True),
          torch.ones(1, device="cuda", requires_grad=True)]
    tps(*xs).backward(torch.zeros(0, 5, device="cuda"))
    assert float(xs[2].grad.abs().max()) == 0.0 and xs[0].grad.shape == (0, 5)


def test_full_size_properties_cfg3():
    """At the benchmark batch the oracle is too slow: check size-independent
    properties instead (agreement of a row sample with the oracle, linearity in
    each argument, independence of rows from their neighbours)."""
    problem = P.config3_mace_uvu()
    B = 100000
    gen = torch.Generator(device="cuda").manual_seed(0)
    x = torch.randn(B, 2048, device="cuda", generator=gen)
    y = torch.randn(B, 16, device="cuda", generator=gen)
    w = torch.randn(B, 2944, device="cuda", generator=gen)
    tp = oeq.TensorProduct(problem)
    z = tp(x, y, w)
    idx = torch.tensor([0, 1, 63, 64, 4097, B // 2, B - 2, B - 1], device="cuda")
    ref = R.Problem.from_spec(problem)
    z_ref = R.tp_forward(ref, x[idx].cpu().numpy(), y[idx].cpu().numpy(), w[idx].cpu().numpy())
    assert err(z[idx], z_ref) <= 1e-5
    assert torch.equal(tp(x[idx], y[idx], w[idx]), z[idx])  # a row does not depend on its position
    z2 = tp(2.0 * x, y, w)
    assert torch.equal(z2, 2.0 * z)  # scaling by 2 is exact in binary floating point
    z3 = tp(x, y, -w)
    assert torch.equal(z3, -z)
    assert torch.isfinite(z).all()


def test_double_backward_matches_autograd_of_oracle_formula():
    """Second derivatives come from compositions of the forward/backward ops;
    compare with torch autograd through an einsum restatement in float64."""
    problem = P.config1_single_uvu(np.float64)
    B = 16
    x, y, w, g = tp_inputs(problem, B, seed=3)
    C = torch.tensor(R.wigner_3j_ref(2, 3, 2) * np.sqrt(5.0))

    def ref_fn(tx, ty, tw):
        return torch.einsum("ijk,zi,zj,z->zk", C, tx, ty, tw[:, 0])

    tp = oeq.TensorProduct(problem)
    outs = []
    for fn, dev in ((ref_fn, "cpu"), (tp, "cuda")):
        tx, ty, tw = (torch.tensor(a, device=dev, requires_grad=True) for a in (x, y, w))
        tg = torch.tensor(g, device=dev, requires_grad=True)
        z = fn(tx, ty, tw) if dev == "cuda" else fn(tx, ty, tw)
        dx, dy, dw = torch.autograd.grad(z, (tx, ty, tw), tg, create_graph=True)
        loss = (dx ** 2).sum() + (dy ** 2).sum() + (dw ** 2).sum()
        second = torch.autograd.grad(loss, (tx, ty, tw, tg))
        outs.append([t.detach().cpu().numpy() for t in second])
    for a, b in zip(outs[1], outs[0]):
        assert R.normalized_error(a, b) <= 1e-12


def test_input_validation_messages():
    tp = oeq.TensorProduct(P.config1_single_uvu())
    x, y, w = (torch.rand(8, n, device="cuda") for n in (5, 7, 1))
    tp(x, y, w)
    with pytest.raises(RuntimeError, match="Shape mismatch"):
        tp(x.unsqueeze(1), y, w)
    with pytest.raises(RuntimeError, match="Shape mismatch"):
        tp(x, y[:, :6], w)
    with pytest.raises(RuntimeError, match="Shape mismatch"):
        tp(x, y, torch.rand(9, 1, device="cuda"))
    with pytest.raises(RuntimeError, match="Dtype mismatch"):
        tp(x, y.to(torch.bfloat16), w)
    with pytest.raises(RuntimeError, match="Dtype mismatch"):
        tp(x.double(), y, w)


def test_module_to_dtype_respecialises():
    tp = oeq.TensorProduct(P.config2_nequip_uvu())
    tp = tp.to(torch.float64)
    problem = P.config2_nequip_uvu(np.float64)
    x, y, w, _ = tp_inputs(problem, 9, seed=5)
    z = tp(*to_gpu(x, y, w))
    assert z.dtype == torch.float64
    assert err(z, R.tp_forward(R.Problem.from_spec(problem), x, y, w)) <= 1e-12


def test_runs_on_a_side_stream():
    tp = oeq.TensorProduct(P.config2_nequip_uvu())
    problem = P.config2_nequip_uvu()
    x, y, w, _ = tp_inputs(problem, 64, seed=9)
    tx, ty, tw = to_gpu(x, y, w)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        z = tp(tx, ty, tw)
    side.synchronize()
    assert err(z, R.tp_forward(R.Problem.from_spec(problem), x, y, w)) <= 1e-5


@pytest.mark.parametrize("knobs", ["tp_gres=0,tp_wb=2,tp_gb=2", "tp_nt=31,tp_acc=24", "tp_wf=0,tp_wb=0,tp_gf=2,tp_gb=2"])
def test_kernel_shape_knobs_keep_results(knobs, monkeypatch):
    """The alternatives selectable through OEQ_AMD_TUNE (gradient slice on demand, streaming hints,
    output segmentation, occupancy and rows per block) compute the same tensor product."""
    monkeypatch.setenv("OEQ_AMD_TUNE", knobs)
    for make in (P.config3_mace_uvu, P.config2_nequip_uvu, lambda: _odd_uvu(True)):
        problem = make()
        x, y, w, g = tp_inputs(problem, 45, seed=6)
        ref = R.Problem.from_spec(problem)
        z_ref = R.tp_forward(ref, x, y, w)
        grads_ref = R.tp_backward(ref, x, y, w, g)
        tx, ty, tw = to_gpu(x, y, w, requires_grad=True)
        z = oeq.TensorProduct(problem)(tx, ty, tw)
        z.backward(torch.tensor(g, device="cuda"))
        assert err(z, z_ref) <= 1e-5
        for got, want in zip((tx.grad, ty.grad, tw.grad), grads_ref):
            assert err(got, want) <= 1e-5, knobs


def test_autotune_keeps_results():
    """`TensorProduct.autotune` times the alternative kernel shapes (also the occupancy forms that the knob test
    above does not name) and may adopt one: the module computes the same product afterwards, and the knob string it
    returns is the one in its kernel-set description."""
    import json
    for make in (lambda: P.seven_net_problems()[0], P.config2_nequip_uvu):
        problem = make()
        x, y, w, g = tp_inputs(problem, 500, seed=9)
        ref = R.Problem.from_spec(problem)
        z_ref = R.tp_forward(ref, x, y, w)
        grads_ref = R.tp_backward(ref, x, y, w, g)
        tp = oeq.TensorProduct(problem)
        tune = tp.autotune(*to_gpu(x, y, w), repeats=2)
        assert set(filter(None, tune.split(","))) <= set(tp.AUTOTUNE_FORWARD) | set(tp.AUTOTUNE_BACKWARD)
        assert json.loads(bytes(tp.spec.tolist()).decode())["tune"] == tune
        tx, ty, tw = to_gpu(x, y, w, requires_grad=True)
        z = tp(tx, ty, tw)
        z.backward(torch.tensor(g, device="cuda"))
        assert err(z, z_ref) <= 1e-5
        for got, want in zip((tx.grad, ty.grad, tw.grad), grads_ref):
            assert err(got, want) <= 1e-5
    shared = oeq.TensorProduct(P.config4_uvw_shared())
    before = shared.kid
    assert shared.autotune(*[torch.zeros(1, device="cuda")] * 3) == "" and shared.kid == before


@pytest.mark.parametrize("knobs", ["tp_wf=-2,tp_wb=-2", "tp_wf=23,tp_wb=23,tp_gres=1"])
def test_occupancy_forms_keep_results(knobs, monkeypatch):
    """The occupancy forms that `autotune` may adopt (a minimum only; a minimum and a maximum) on a small, a large and
    a shared-weight problem."""
    monkeypatch.setenv("OEQ_AMD_TUNE", knobs)
    for make in (P.config3_mace_uvu, lambda: P.seven_net_problems()[2], lambda: _odd_uvu(True)):
        problem = make()
        x, y, w, g = tp_inputs(problem, 45, seed=6)
        ref = R.Problem.from_spec(problem)
        z_ref = R.tp_forward(ref, x, y, w)
        grads_ref = R.tp_backward(ref, x, y, w, g)
        tx, ty, tw = to_gpu(x, y, w, requires_grad=True)
        z = oeq.TensorProduct(problem)(tx, ty, tw)
        z.backward(torch.tensor(g, device="cuda"))
        assert err(z, z_ref) <= 1e-5
        for got, want in zip((tx.grad, ty.grad, tw.grad), grads_ref):
            assert err(got, want) <= 1e-5, knobs
