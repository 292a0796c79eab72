"""Writes the golden fixtures of this directory from the reference's numpy-only
specification modules. Run once in the build container:

    OEQ_NOTORCH=1 python tests/golden/make_golden.py /root/reference/openequivariance

What is dumped is what no closed form or invariant fixes: the overall sign and
component ordering convention of each real-basis CG tensor (equivariance and
unit norm determine it only up to a sign per (l1, l2, l3)), and the ordering
conventions of the problem constructors (output-block order, instruction order,
weight offsets) together with the normalised path coefficients.

Outputs (data only): wigner_3j.npz, problems.json.
"""

import json
import os
import sys

import numpy as np

os.environ["OEQ_NOTORCH"] = "1"
sys.path.insert(0, sys.argv[1] if len(sys.argv) > 1 else "/root/reference/openequivariance")

from openequivariance.core.e3nn_lite import TPProblem, wigner_3j  # noqa: E402
from openequivariance.benchmark.problems import ChannelwiseTPP, FullyConnectedTPProblem  # noqa: E402

here = os.path.dirname(os.path.abspath(__file__))

LMAX = 4
tensors = {}
for l1 in range(LMAX + 1):
    for l2 in range(LMAX + 1):
        for l3 in range(abs(l1 - l2), min(LMAX, l1 + l2) + 1):
            tensors[f"{l1}_{l2}_{l3}"] = wigner_3j(l1, l2, l3)
for t in [(5, 3, 4), (6, 6, 6), (7, 1, 7), (7, 5, 3)]:
    tensors["%d_%d_%d" % t] = wigner_3j(*t)
np.savez_compressed(os.path.join(here, "wigner_3j.npz"), **tensors)


def dump(p):
    return {
        "irreps_in1": str(p.irreps_in1), "irreps_in2": str(p.irreps_in2), "irreps_out": str(p.irreps_out),
        "weight_numel": int(p.weight_numel), "shared_weights": bool(p.shared_weights),
        "instructions": [
            [int(i.i_in1), int(i.i_in2), int(i.i_out), i.connection_mode, bool(i.has_weight), float(i.path_weight),
             [int(s) for s in i.path_shape]] for i in p.instructions
        ],
        "weight_ranges": [[int(a), int(b)] for a, b, _ in
                          (p.weight_range_and_shape_for_instruction(n) for n in range(len(p.instructions)))],
    }


def nat(lmax):
    return "+".join(f"{l}{'e' if l % 2 == 0 else 'o'}" for l in range(lmax + 1))


problems = {
    "cfg1": TPProblem("1x2e", "1x3e", "1x2e", [(0, 0, 0, "uvu", True)], shared_weights=False, internal_weights=False),
    "cfg2": ChannelwiseTPP("32x0e+32x1o+32x2e", "1x0e+1x1o+1x2e+1x3o", nat(2)),
    "cfg3": ChannelwiseTPP("128x0e+128x1o+128x2e+128x3o", "1x0e+1x1o+1x2e+1x3o", nat(3)),
    "cfg4": FullyConnectedTPProblem("64x0e+64x1o+64x2e", "1x0e+1x1o+1x2e", "64x0e+64x1o+64x2e",
                                    shared_weights=True, internal_weights=False),
    "mace_large": ChannelwiseTPP("128x0e+128x1o+128x2e", "1x0e+1x1o+1x2e+1x3o", "128x0e+128x1o+128x2e+128x3o"),
    "nequip_lips": ChannelwiseTPP("32x0o + 32x0e + 32x1o + 32x1e + 32x2o + 32x2e", "0e + 1o + 2e",
                                  "32x0o + 32x0e + 32x1o + 32x1e + 32x2o + 32x2e"),
    "mixed_norm": TPProblem("3x1o+2x2e", "2x1o+1x0e", "3x1o+2x2e+4x0e",
                            [(0, 0, 2, "uvw", True, 0.5), (0, 1, 0, "uvw", True), (1, 0, 0, "uvw", True, 2.0),
                             (1, 1, 1, "uvw", True)], irrep_normalization="norm", path_normalization="path",
                            in1_var=[1.0, 2.0], in2_var=[0.5, 1.0], out_var=[1.0, 3.0, 2.0],
                            shared_weights=False, internal_weights=False),
}
with open(os.path.join(here, "problems.json"), "w") as f:
    json.dump({k: dump(v) for k, v in problems.items()}, f, indent=1)
print("wrote", len(tensors), "tensors and", len(problems), "problems")
