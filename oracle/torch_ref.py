"""CPU baseline: the e3nn-equivalent tensor product / convolution in torch on
the host (einsum per instruction + index_add scatter, backward by autograd),
which is how e3nn's ``o3.TensorProduct`` evaluates. e3nn itself is not
installed in this image, so this restatement is what gets timed.

TEST / BENCHMARK INFRASTRUCTURE ONLY (see oracle/e3nn_ref.py). Follows
openequivariance/openequivariance/_torch/E3NNTensorProduct.py:39-95 and
_torch/E3NNConv.py:41-75 of the reference.
"""

from __future__ import annotations

import torch

from . import e3nn_ref as R


class TorchTP:
    def __init__(self, prob: R.Problem, dtype=torch.float32):
        self.prob = prob
        self.dtype = dtype
        self.cg = [torch.tensor(R.wigner_3j_ref(*p["l"]) * p["coeff"], dtype=dtype) for p in prob.paths]
        self.o1, self.o2, self.oo = (R.block_offsets(b) for b in (prob.in1, prob.in2, prob.out))

    def __call__(self, x, y, w):
        prob = self.prob
        Z = x.shape[0]
        outs = [None] * len(prob.out)
        for p, C in zip(prob.paths, self.cg):
            m1, l1, _ = prob.in1[p["i1"]]
            m2, l2, _ = prob.in2[p["i2"]]
            xi = x[:, self.o1[p["i1"]]:self.o1[p["i1"]] + m1 * (2 * l1 + 1)].reshape(Z, m1, 2 * l1 + 1)
            yj = y[:, self.o2[p["i2"]]:self.o2[p["i2"]] + m2 * (2 * l2 + 1)].reshape(Z, m2, 2 * l2 + 1)
            n = 1
            for s in p["shape"]:
                n *= s
            if prob.shared_weights:
                wp = w[p["woff"]:p["woff"] + n].reshape(p["shape"])
                zw = ""
            else:
                wp = w[:, p["woff"]:p["woff"] + n].reshape((Z,) + tuple(p["shape"]))
                zw = "z"
            if p["mode"] == "uvu":
                r = torch.einsum(f"{zw}uv,ijk,zui,zvj->zuk", wp, C, xi, yj)
            else:
                r = torch.einsum(f"{zw}uvw,ijk,zui,zvj->zwk", wp, C, xi, yj)
            r = r.reshape(Z, -1)
            outs[p["io"]] = r if outs[p["io"]] is None else outs[p["io"]] + r
        cols = []
        for io, (mo, lo, _) in enumerate(prob.out):
            cols.append(outs[io] if outs[io] is not None else x.new_zeros(Z, mo * (2 * lo + 1)))
        return torch.cat(cols, dim=1)


class TorchConv:
    def __init__(self, prob: R.Problem, dtype=torch.float32):
        self.tp = TorchTP(prob, dtype)
        self.prob = prob

    def __call__(self, X, Y, W, rows, cols):
        msg = self.tp(X[cols], Y, W)
        out = X.new_zeros(X.shape[0], self.prob.dims[2])
        return out.index_add(0, rows, msg)
