"""The C ABI driven by a stand-alone C++ program (tests/cabi/cabi_roundtrip.cpp): hiprtc compile,
kernel-set creation, forward and backward on plain hipMalloc'ed buffers, no Python or torch in that
process. This test only writes the kernel bundle and the oracle's expected values, then runs it."""

import subprocess
from pathlib import Path

import numpy as np
import pytest

from openequivariance_amd.core import problems as P
from oracle import e3nn_ref as R

pytestmark = pytest.mark.gpu

ROOT = Path(__file__).resolve().parent.parent
BINARY = ROOT / "tests" / "cabi" / "cabi_roundtrip"


@pytest.mark.parametrize("make", [P.config2_nequip_uvu, P.config4_uvw_shared], ids=["cfg2-uvu", "cfg4-uvw-mfma"])
def test_standalone_program(make, tmp_path):
    from openequivariance_amd._torch.tensor_product import build_tp_module
    if not BINARY.exists():
        pytest.fail(f"{BINARY} is not built; run `python __graft_entry__.py build`")
    problem = make()
    src, dims, descs = build_tp_module(problem)
    B = 77
    rng = np.random.default_rng(5)
    x = rng.uniform(size=(B, problem.irreps_in1.dim)).astype(np.float32)
    y = rng.uniform(size=(B, problem.irreps_in2.dim)).astype(np.float32)
    w = rng.uniform(size=(problem.weight_numel,) if problem.shared_weights else (B, problem.weight_numel)).astype(
        np.float32)
    g = rng.uniform(size=(B, problem.irreps_out.dim)).astype(np.float32)
    ref = R.Problem.from_spec(problem)
    z = R.tp_forward(ref, x, y, w)
    dx, dy, dw = R.tp_backward(ref, x, y, w, g)
    (tmp_path / "kernels.hip").write_text(src)
    lines = [" ".join(str(int(dims[k])) for k in ("L1_dim", "L2_dim", "L3_dim", "weight_numel", "elem_size",
                                                    "shared_weights", "deterministic", "wpartial_per_block")),
             f"{B} {len(descs)}"]
    for d in descs:
        d = tuple(d) + (0,) * (6 - len(d))
        lines.append(f"{d[0]} {d[1]} {d[2]} {d[3]} {d[4]} {d[5]}")
    (tmp_path / "bundle.txt").write_text("\n".join(lines) + "\n")
    for name, arr in (("x", x), ("y", y), ("w", w), ("g", g), ("z", z), ("dx", dx), ("dy", dy), ("dw", dw)):
        np.asarray(arr, dtype=np.float32).tofile(tmp_path / f"{name}.bin")
    res = subprocess.run([str(BINARY), str(tmp_path)], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0 and "OK" in res.stdout, res.stdout + res.stderr
    # both sets carry the fused second-order kernels (the shared-weight one with a workspace for kernel B)
    assert "second order: d/d(dZ)=" in res.stdout, res.stdout
