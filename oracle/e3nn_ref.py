"""CPU oracle: a restatement of e3nn ``o3.TensorProduct`` (+ scatter-sum for the
graph convolution) in numpy.

TEST INFRASTRUCTURE ONLY. Nothing in the shipped package imports this module;
it is used by tests/, by ``__graft_entry__.smoke()`` and by the CPU-baseline
leg of ``bench.py`` as the checker / the thing timed on the host, never as a
fallback for the GPU path.

What it restates (all citations into the reference tree):

* ``wigner_3j_ref``      - openequivariance/openequivariance/core/e3nn_lite.py:656-733
                           (real-basis CG tensor, Frobenius-normalised). The SU(2)
                           coefficients here come from ``sympy.physics.wigner`` rather
                           than from a re-typed Racah sum, so they are independent of
                           the package's own generator.
* ``path_coefficients``  - e3nn_lite.py:451-565 (path_shape, element/path/none
                           normalisation, sqrt(alpha)).
* ``tp_forward/backward``- the e3nn einsum semantics used by the reference's oracle
                           wrapper, openequivariance/openequivariance/_torch/E3NNTensorProduct.py:39-95
                           ('uvu': zuv,ijk,zui,zvj->zuk; 'uvw': zuvw,ijk,zui,zvj->zwk;
                           weights in instruction order, each block row-major over
                           path_shape, e3nn_lite.py:643-650).
* ``conv_forward/backward`` - openequivariance/openequivariance/_torch/E3NNConv.py:41-75 and
                           core/ConvolutionBase.py:292-301: tensor product on gathered
                           sender rows followed by a scatter-add over receivers.
* ``sorted_graph``       - core/ConvolutionBase.py:57-82 (row-major sort and the
                           transpose permutation).

Pins (see tests/test_oracle.py): closed forms of the CG tensor, unit norm,
permutation symmetry, structural non-zero counts, equivariance under random
rotations, brute-force triple loops on tiny problems, special cases that reduce
to dot/cross products, finite differences and the adjoint identity for the
backward pass. No golden vectors exist in the reference for this path.
"""

from __future__ import annotations

import functools
import math

import numpy as np

# --------------------------------------------------------------------------
# irreps / instructions (minimal, independent of the package's parser)
# --------------------------------------------------------------------------


def parse_irreps(irreps):
    """-> list of (mul, l, p). Accepts 'AxLp+...' strings or iterables of
    (mul, (l, p)) pairs."""
    out = []
    if isinstance(irreps, str):
        for tok in irreps.split("+"):
            tok = tok.strip()
            if not tok:
                continue
            mul, ir = (tok.split("x") + [None])[:2] if "x" in tok else ("1", tok)
            ir = ir.strip()
            l = int(ir[:-1])
            p = {"e": 1, "o": -1, "y": (-1) ** l}[ir[-1]]
            out.append((int(mul), l, p))
        return out
    for mul, ir in irreps:
        l, p = ir
        out.append((int(mul), int(l), int(p)))
    return out


def irreps_dim(blocks):
    return sum(mul * (2 * l + 1) for mul, l, _ in blocks)


def block_offsets(blocks):
    offs, s = [], 0
    for mul, l, _ in blocks:
        offs.append(s)
        s += mul * (2 * l + 1)
    return offs


class Problem:
    """Plain-data view of a tensor-product problem for the oracle."""

    def __init__(self, irreps_in1, irreps_in2, irreps_out, instructions, shared_weights,
                 irrep_normalization="component", path_normalization="element",
                 in1_var=None, in2_var=None, out_var=None):
        self.in1 = parse_irreps(irreps_in1)
        self.in2 = parse_irreps(irreps_in2)
        self.out = parse_irreps(irreps_out)
        self.shared_weights = bool(shared_weights)
        raw = [tuple(t) if len(t) == 6 else tuple(t) + (1.0,) for t in instructions]
        self.paths = path_coefficients(self.in1, self.in2, self.out, raw, irrep_normalization,
                                       path_normalization, in1_var, in2_var, out_var)
        self.weight_numel = sum(int(np.prod(p["shape"])) for p in self.paths if p["has_weight"])
        self.dims = (irreps_dim(self.in1), irreps_dim(self.in2), irreps_dim(self.out))

    @classmethod
    def from_spec(cls, spec):
        """Build from any object with the reference's TPProblem attributes
        (uses the *raw* instructions and recomputes the normalisation)."""
        return cls(
            [(m, (ir[0], ir[1])) for m, ir in spec.irreps_in1],
            [(m, (ir[0], ir[1])) for m, ir in spec.irreps_in2],
            [(m, (ir[0], ir[1])) for m, ir in spec.irreps_out],
            spec.instructions_raw, spec.shared_weights, spec.irrep_normalization,
            spec.path_normalization, spec.in1_var, spec.in2_var, spec.out_var,
        )


def path_coefficients(in1, in2, out, raw, irrep_normalization, path_normalization,
                      in1_var=None, in2_var=None, out_var=None):
    """e3nn_lite.py:451-565: one dict per instruction with the final
    coefficient sqrt(alpha), the weight block shape and its offset."""
    v1 = [1.0] * len(in1) if in1_var is None else [float(v) for v in in1_var]
    v2 = [1.0] * len(in2) if in2_var is None else [float(v) for v in in2_var]
    vo = [1.0] * len(out) if out_var is None else [float(v) for v in out_var]

    def shape(mode, m1, m2, mo):
        return {"uvw": (m1, m2, mo), "uvu": (m1, m2)}[mode]

    def fan(mode, m1, m2):
        return {"uvw": m1 * m2, "uvu": m2}[mode]

    paths, woff = [], 0
    for (i1, i2, io, mode, has_w, pw) in raw:
        m1, l1, p1 = in1[i1]
        m2, l2, p2 = in2[i2]
        mo, lo, po = out[io]
        assert p1 * p2 == po and abs(l1 - l2) <= lo <= l1 + l2
        alpha = {"component": 2 * lo + 1, "norm": (2 * l1 + 1) * (2 * l2 + 1), "none": 1}[irrep_normalization]
        sib = [r for r in raw if r[2] == io]
        if path_normalization == "element":
            x = sum(v1[r[0]] * v2[r[1]] * fan(r[3], in1[r[0]][0], in2[r[1]][0]) for r in sib)
        elif path_normalization == "path":
            x = v1[i1] * v2[i2] * fan(mode, m1, m2) * len(sib)
        else:
            x = 1
        if x > 0:
            alpha /= x
        alpha *= vo[io] * pw
        shp = shape(mode, m1, m2, mo)
        paths.append(dict(i1=i1, i2=i2, io=io, mode=mode, has_weight=has_w, coeff=math.sqrt(alpha),
                          shape=shp, woff=woff, l=(l1, l2, lo)))
        if has_w:
            woff += int(np.prod(shp))
    return paths


# --------------------------------------------------------------------------
# real-basis CG tensor
# --------------------------------------------------------------------------


def _complex_from_real(l):
    """Matrix A with  Y^complex_m = sum_a A[m, a] Y^real_a  (textbook real
    spherical harmonics), times (-i)^l as in e3nn_lite.py:656-674."""
    n = 2 * l + 1
    A = np.zeros((n, n), dtype=np.complex128)
    r = 1 / math.sqrt(2)
    for m in range(-l, l + 1):
        row = l + m
        if m < 0:
            A[row, l + (-m)] = r          # cosine-type component |m|
            A[row, l - (-m)] = -1j * r    # sine-type component -|m|
        elif m == 0:
            A[row, l] = 1
        else:
            A[row, l + m] = (-1) ** m * r
            A[row, l - m] = 1j * (-1) ** m * r
    return (-1j) ** l * A


@functools.lru_cache(maxsize=None)
def wigner_3j_ref(l1, l2, l3):
    from sympy import S
    from sympy.physics.wigner import clebsch_gordan

    A1, A2, A3 = _complex_from_real(l1), _complex_from_real(l2), _complex_from_real(l3)
    C = np.zeros((2 * l1 + 1, 2 * l2 + 1, 2 * l3 + 1), dtype=np.complex128)
    for m1 in range(-l1, l1 + 1):
        for m2 in range(-l2, l2 + 1):
            m3 = m1 + m2
            if abs(m3) > l3:
                continue
            cg = float(clebsch_gordan(S(l1), S(l2), S(l3), S(m1), S(m2), S(m3)).evalf(40))
            if cg == 0.0:
                continue
            # real[a,b,c] += A1[m1,a] A2[m2,b] conj(A3[m3,c]) <l1 m1 l2 m2|l3 m3>
            C += cg * np.einsum("a,b,c->abc", A1[l1 + m1], A2[l2 + m2], np.conj(A3[l3 + m3]))
    assert np.abs(C.imag).max() < 1e-12
    C = C.real.copy()
    C /= np.sqrt((C * C).sum())
    return C


# --------------------------------------------------------------------------
# tensor product forward / backward (float64 unless told otherwise)
# --------------------------------------------------------------------------


def _views(prob, x, y, w):
    o1, o2 = block_offsets(prob.in1), block_offsets(prob.in2)
    Z = x.shape[0]
    xs = [x[:, o:o + m * (2 * l + 1)].reshape(Z, m, 2 * l + 1) for o, (m, l, _) in zip(o1, prob.in1)]
    ys = [y[:, o:o + m * (2 * l + 1)].reshape(Z, m, 2 * l + 1) for o, (m, l, _) in zip(o2, prob.in2)]
    ws = []
    for p in prob.paths:
        n = int(np.prod(p["shape"]))
        if prob.shared_weights:
            ws.append(w[p["woff"]:p["woff"] + n].reshape(p["shape"]))
        else:
            ws.append(w[:, p["woff"]:p["woff"] + n].reshape((Z,) + tuple(p["shape"])))
    return xs, ys, ws


def tp_forward(prob, x, y, w, dtype=np.float64):
    x, y, w = (np.asarray(a, dtype=dtype) for a in (x, y, w))
    Z = x.shape[0]
    xs, ys, ws = _views(prob, x, y, w)
    oo = block_offsets(prob.out)
    out = np.zeros((Z, prob.dims[2]), dtype=dtype)
    zw = "" if prob.shared_weights else "z"
    for p, wp in zip(prob.paths, ws):
        C = wigner_3j_ref(*p["l"]).astype(dtype) * dtype(p["coeff"])
        xi, yj = xs[p["i1"]], ys[p["i2"]]
        mo, lo, _ = prob.out[p["io"]]
        if p["mode"] == "uvu":
            r = np.einsum(f"{zw}uv,ijk,zui,zvj->zuk", wp, C, xi, yj, optimize=True)
        else:
            r = np.einsum(f"{zw}uvw,ijk,zui,zvj->zwk", wp, C, xi, yj, optimize=True)
        s = oo[p["io"]]
        out[:, s:s + mo * (2 * lo + 1)] += r.reshape(Z, -1)
    return out


def tp_backward(prob, x, y, w, g, dtype=np.float64):
    """Vector-Jacobian products (dx, dy, dw) for output gradient ``g``."""
    x, y, w, g = (np.asarray(a, dtype=dtype) for a in (x, y, w, g))
    Z = x.shape[0]
    xs, ys, ws = _views(prob, x, y, w)
    o1, o2, oo = block_offsets(prob.in1), block_offsets(prob.in2), block_offsets(prob.out)
    dx, dy, dw = np.zeros_like(x), np.zeros_like(y), np.zeros_like(w)
    zw = "" if prob.shared_weights else "z"
    for p, wp in zip(prob.paths, ws):
        C = wigner_3j_ref(*p["l"]).astype(dtype) * dtype(p["coeff"])
        xi, yj = xs[p["i1"]], ys[p["i2"]]
        m1, l1, _ = prob.in1[p["i1"]]
        m2, l2, _ = prob.in2[p["i2"]]
        mo, lo, _ = prob.out[p["io"]]
        gk = g[:, oo[p["io"]]:oo[p["io"]] + mo * (2 * lo + 1)].reshape(Z, mo, 2 * lo + 1)
        if p["mode"] == "uvu":
            gx = np.einsum(f"{zw}uv,ijk,zvj,zuk->zui", wp, C, yj, gk, optimize=True)
            gy = np.einsum(f"{zw}uv,ijk,zui,zuk->zvj", wp, C, xi, gk, optimize=True)
            gw = np.einsum(f"ijk,zui,zvj,zuk->{zw}uv", C, xi, yj, gk, optimize=True)
        else:
            gx = np.einsum(f"{zw}uvw,ijk,zvj,zwk->zui", wp, C, yj, gk, optimize=True)
            gy = np.einsum(f"{zw}uvw,ijk,zui,zwk->zvj", wp, C, xi, gk, optimize=True)
            gw = np.einsum(f"ijk,zui,zvj,zwk->{zw}uvw", C, xi, yj, gk, optimize=True)
        dx[:, o1[p["i1"]]:o1[p["i1"]] + m1 * (2 * l1 + 1)] += gx.reshape(Z, -1)
        dy[:, o2[p["i2"]]:o2[p["i2"]] + m2 * (2 * l2 + 1)] += gy.reshape(Z, -1)
        n = int(np.prod(p["shape"]))
        if prob.shared_weights:
            dw[p["woff"]:p["woff"] + n] += gw.reshape(-1)
        else:
            dw[:, p["woff"]:p["woff"] + n] += gw.reshape(Z, -1)
    return dx, dy, dw


def tp_forward_loops(prob, x, y, w):
    """Pure-Python element loops (tiny problems only): the definition itself,
    used to pin the vectorised einsum version."""
    x, y, w = (np.asarray(a, dtype=np.float64) for a in (x, y, w))
    Z = x.shape[0]
    o1, o2, oo = block_offsets(prob.in1), block_offsets(prob.in2), block_offsets(prob.out)
    out = np.zeros((Z, prob.dims[2]))
    for p in prob.paths:
        C = wigner_3j_ref(*p["l"])
        m1, l1, _ = prob.in1[p["i1"]]
        m2, l2, _ = prob.in2[p["i2"]]
        mo, lo, _ = prob.out[p["io"]]
        d1, d2, d3 = 2 * l1 + 1, 2 * l2 + 1, 2 * lo + 1
        for z in range(Z):
            wrow = w if prob.shared_weights else w[z]
            for u in range(m1):
                for v in range(m2):
                    for i in range(d1):
                        for j in range(d2):
                            for k in range(d3):
                                c = C[i, j, k]
                                if c == 0.0:
                                    continue
                                t = p["coeff"] * c * x[z, o1[p["i1"]] + u * d1 + i] * y[z, o2[p["i2"]] + v * d2 + j]
                                if p["mode"] == "uvu":
                                    out[z, oo[p["io"]] + u * d3 + k] += wrow[p["woff"] + u * m2 + v] * t
                                else:
                                    for ww in range(mo):
                                        out[z, oo[p["io"]] + ww * d3 + k] += wrow[p["woff"] + (u * m2 + v) * mo + ww] * t
    return out


# --------------------------------------------------------------------------
# fused graph convolution
# --------------------------------------------------------------------------


def conv_forward(prob, X, Y, W, rows, cols, dtype=np.float64, chunk=4096):
    """Z[r] = sum over edges e with rows[e]==r of TP(X[cols[e]], Y[e], W[e])."""
    X, Y, W = (np.asarray(a, dtype=dtype) for a in (X, Y, W))
    rows, cols = np.asarray(rows), np.asarray(cols)
    out = np.zeros((X.shape[0], prob.dims[2]), dtype=dtype)
    E = rows.shape[0]
    for s in range(0, E, chunk):
        e = slice(s, min(E, s + chunk))
        msg = tp_forward(prob, X[cols[e]], Y[e], W if prob.shared_weights else W[e], dtype)
        np.add.at(out, rows[e], msg)
    return out


def conv_backward(prob, X, Y, W, G, rows, cols, dtype=np.float64, chunk=4096):
    X, Y, W, G = (np.asarray(a, dtype=dtype) for a in (X, Y, W, G))
    rows, cols = np.asarray(rows), np.asarray(cols)
    dX, dY, dW = np.zeros_like(X), np.zeros_like(Y), np.zeros_like(W)
    E = rows.shape[0]
    for s in range(0, E, chunk):
        e = slice(s, min(E, s + chunk))
        gx, gy, gw = tp_backward(prob, X[cols[e]], Y[e], W if prob.shared_weights else W[e], G[rows[e]], dtype)
        np.add.at(dX, cols[e], gx)
        dY[e] = gy
        if prob.shared_weights:
            dW += gw
        else:
            dW[e] = gw
    return dX, dY, dW


def sorted_graph(rows, cols):
    """Row-major (receiver, sender) sort and the permutation that lists the
    sorted edges in column-major (sender, receiver) order
    (core/ConvolutionBase.py:57-82). Returns (rows, cols, order, transpose_perm)."""
    rows, cols = np.asarray(rows), np.asarray(cols)
    order = np.lexsort((cols, rows))
    r, c = rows[order], cols[order]
    tperm = np.lexsort((r, c))
    return r, c, order, tperm


def normalized_error(a, b):
    """max|a-b| / max|b| (b is the oracle)."""
    a, b = np.asarray(a, dtype=np.float64), np.asarray(b, dtype=np.float64)
    denom = np.abs(b).max()
    if denom == 0:
        return float(np.abs(a).max())
    return float(np.abs(a - b).max() / denom)


# --------------------------------------------------------------------------
# real spherical harmonics (inputs only; component normalisation)
# --------------------------------------------------------------------------


def spherical_harmonics(lmax, vecs):
    """Component-normalised real spherical harmonics of unit vectors, l=0..lmax,
    built by the CG recursion Y^{l+1} ~ C(l,1,l+1)(Y^l (x) Y^1) with
    Y^1 = sqrt(3)*(x,y,z); |Y^l|^2 = 2l+1. These are *inputs* to the tensor
    product; agreement with e3nn's own harmonics is not claimed."""
    v = np.asarray(vecs, dtype=np.float64)
    v = v / np.linalg.norm(v, axis=1, keepdims=True)
    ys = [np.ones((v.shape[0], 1)), math.sqrt(3.0) * v]
    for l in range(1, lmax):
        nxt = np.einsum("ijk,zi,zj->zk", wigner_3j_ref(l, 1, l + 1), ys[l], ys[1])
        nxt *= math.sqrt(2 * l + 3) / np.linalg.norm(nxt, axis=1, keepdims=True)
        ys.append(nxt)
    return np.concatenate(ys[: lmax + 1], axis=1)
