"""Host-side API: Irreps / TPProblem behave like the reference front-end
(openequivariance/openequivariance/core/e3nn_lite.py) and unsupported problems
are rejected with the reference's messages (core/utils.py:81-117,
tests/input_validation_test.py:143-155)."""

import io

import numpy as np
import pytest

import openequivariance_amd as oeq
from openequivariance_amd.core import problems as P
from openequivariance_amd.core.spec import Irrep, Irreps, TPProblem


def test_irrep_parsing():
    assert Irrep("2e") == (2, 1) and Irrep("1o") == (1, -1) and Irrep("3y") == (3, -1) and Irrep("2y") == (2, 1)
    assert Irrep("1o").dim == 3 and repr(Irrep(4, 1)) == "4e"
    with pytest.raises(ValueError):
        Irrep("x")
    assert [repr(i) for i in Irrep("1o") * Irrep("2e")] == ["1o", "2o", "3o"]


def test_irreps_api():
    ir = Irreps("32x0e + 32x1o+2e")
    assert ir.dim == 32 + 96 + 5 and len(ir) == 3 and ir[2].mul == 1
    assert ir.slices() == [slice(0, 32), slice(32, 128), slice(128, 133)]
    assert str(ir) == "32x0e+32x1o+1x2e"
    assert "1o" in ir and "1e" not in ir and ir.count("0e") == 32
    assert str(Irreps("2x1o+3x1o+0x2e").simplify()) == "5x1o"
    s = Irreps("1x2e+1x0e+1x1o+1x1e+1x0e").sort()
    assert str(s.irreps) == "1x0e+1x0e+1x1o+1x1e+1x2e"
    assert s.p == (4, 0, 2, 3, 1) and s.inv == (1, 4, 2, 3, 0)
    assert str(Irreps.spherical_harmonics(3)) == "1x0e+1x1o+1x2e+1x3o"
    assert Irreps([(2, (1, -1)), (1, "0e")]).dim == 7
    assert Irreps("4x0e").lmax == 0 and Irreps("2x3o").ls == [3, 3]


def test_tpproblem_attributes():
    p = TPProblem("1x2e", "1x3e", "1x2e", [(0, 0, 0, "uvu", True)], shared_weights=False, internal_weights=False)
    assert p.weight_numel == 1 and p.shared_weights is False and p.layout == "mul_ir"
    assert p.irrep_dtype == np.float32 and p.weight_dtype == np.float32
    assert len(p.instructions[0]) == 7 and p.instructions[0].path_shape == (1, 1)
    q = p.clone()
    q.irrep_dtype = np.float64
    assert p.irrep_dtype == np.float32
    assert TPProblem("1x0e", "1x0e", "1x0e", [(0, 0, 0, "uvw", True)]).shared_weights is True
    assert "1x2e" in str(p) and "uvu" in repr(p)


def test_tpproblem_rejects_bad_paths():
    with pytest.raises(AssertionError):
        TPProblem("1x1o", "1x1o", "1x1o", [(0, 0, 0, "uvu", True)])  # parity
    with pytest.raises(AssertionError):
        TPProblem("1x1o", "1x1o", "1x3e", [(0, 0, 0, "uvu", True)])  # triangle


def test_unsupported_problems_rejected():
    with pytest.raises(AssertionError, match="layout='ir_mul'"):
        oeq.TensorProduct(TPProblem("5x5e", "1x3e", "5x5e", [(0, 0, 0, "uvw", True)], shared_weights=False,
                                    internal_weights=False, layout="ir_mul"))
    with pytest.raises(AssertionError, match="same connection mode"):
        oeq.TensorProduct(TPProblem("2x1o", "1x1o", "2x0e+2x0e", [(0, 0, 0, "uvu", True), (0, 0, 1, "uvw", True)],
                                    shared_weights=False, internal_weights=False))
    with pytest.raises(AssertionError, match="trainable weights"):
        oeq.TensorProduct(TPProblem("2x1o", "1x1o", "2x0e", [(0, 0, 0, "uvu", False)], shared_weights=False,
                                    internal_weights=False))
    with pytest.raises(AssertionError, match="Connection mode"):
        oeq.TensorProduct(TPProblem("2x1o", "2x1o", "2x0e", [(0, 0, 0, "uuu", True)], shared_weights=False,
                                    internal_weights=False))
    with pytest.raises(AssertionError, match="must be the same"):
        oeq.TensorProduct(TPProblem("2x1o", "1x1o", "2x0e", [(0, 0, 0, "uvu", True)], shared_weights=False,
                                    internal_weights=False, irrep_dtype=np.float64))
    with pytest.raises(AssertionError, match="shared weights"):
        oeq.TensorProductConv(P.config4_uvw_shared(), deterministic=True)


def test_modules_construct_and_pickle_without_gpu():
    import torch
    tp = oeq.TensorProduct(P.config1_single_uvu())
    assert tp.L3_dim == 5 and tp.weight_numel == 1
    buf = io.BytesIO()
    torch.save(tp, buf)
    buf.seek(0)
    tp2 = torch.load(buf, weights_only=True)
    assert tp2.L3_dim == 5 and str(tp2.config.irreps_in2) == "1x3e"
    conv = oeq.TensorProductConv(P.config2_nequip_uvu(), deterministic=True)
    assert conv.L3_dim == 1376
    tp64 = oeq.TensorProduct(P.config1_single_uvu()).to(torch.float64)
    assert tp64.config.irrep_dtype == np.float64
    w = torch.zeros(3, 1)
    assert tp.reorder_weights_to_e3nn(tp.reorder_weights_from_e3nn(w)) is w
    assert oeq.torch_to_oeq_dtype(torch.float64) == np.float64


def test_ops_reject_cpu_tensors():
    import torch
    tp = oeq.TensorProduct(P.config1_single_uvu())
    with pytest.raises((RuntimeError, NotImplementedError)):
        tp(torch.zeros(2, 5), torch.zeros(2, 7), torch.zeros(2, 1))


def test_graph_npz_round_trip(tmp_path):
    from openequivariance_amd.core.graph import CoordGraph, periodic_radius_graph
    coords, rows, cols, _ = periodic_radius_graph(50, 6, 5.0, 1)
    g = CoordGraph(coords, rows, cols, "toy")
    g.save_npz(tmp_path / "g.npz")
    h = CoordGraph.from_npz(tmp_path / "g.npz", "toy")
    assert h.node_count == g.node_count and h.nnz == g.nnz
    assert np.array_equal(h.rows, g.rows) and np.array_equal(h.cols, g.cols)
    assert np.array_equal(h.transpose_perm, g.transpose_perm)
    # rows are receiver-sorted and the permutation lists the edges sender-major
    assert np.all(np.diff(h.rows) >= 0) and np.all(np.diff(h.cols[h.transpose_perm]) >= 0)
