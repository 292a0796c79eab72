"""Real-basis Clebsch-Gordan ("Wigner 3j") tensors, generated in float64.

These are the constants that get baked into every generated kernel. The
convention follows the reference (e3nn_lite.py:656-733): complex SU(2)
coupling coefficients from the Racah sum in exact rational arithmetic, a
real<->complex change of basis carrying a ``(-i)^l`` phase so the result is
real, and normalisation of the whole tensor to unit Frobenius norm.
"""

from __future__ import annotations

import functools
from fractions import Fraction
from math import factorial, isqrt

import numpy as np


def _sqrt_fraction(q: Fraction) -> float:
    """sqrt of a non-negative rational, exact when both parts are squares."""
    n, d = q.numerator, q.denominator
    rn, rd = isqrt(n), isqrt(d)
    if rn * rn == n and rd * rd == d:
        return rn / rd
    return float(np.sqrt(np.longdouble(n) / np.longdouble(d)))


def su2_coupling(j1: int, m1: int, j2: int, m2: int, j3: int, m3: int) -> float:
    """<j1 m1; j2 m2 | j3 m3> for integer spins (Racah's formula,
    cf. e3nn_lite.py:807-864)."""
    if m1 + m2 != m3 or not (abs(j1 - j2) <= j3 <= j1 + j2):
        return 0.0
    if abs(m1) > j1 or abs(m2) > j2 or abs(m3) > j3:
        return 0.0
    f = factorial
    pref = Fraction(
        (2 * j3 + 1) * f(j3 + j1 - j2) * f(j3 - j1 + j2) * f(j1 + j2 - j3) * f(j3 + m3) * f(j3 - m3),
        f(j1 + j2 + j3 + 1) * f(j1 - m1) * f(j1 + m1) * f(j2 - m2) * f(j2 + m2),
    )
    lo = max(-j1 + j2 + m3, -j1 + m1, 0)
    hi = min(j2 + j3 + m1, j3 - j1 + j2, j3 + m3)
    total = Fraction(0)
    for v in range(lo, hi + 1):
        sign = -1 if (v + j2 + m2) % 2 else 1
        total += sign * Fraction(
            f(j2 + j3 + m1 - v) * f(j1 - m1 + v),
            f(v) * f(j3 - j1 + j2 - v) * f(j3 + m3 - v) * f(v + j1 - j2 - m3),
        )
    # value = sqrt(pref) * total, kept exact as sign * sqrt(pref * total^2)
    if total == 0:
        return 0.0
    mag = _sqrt_fraction(pref * total * total)
    return mag if total > 0 else -mag


def real_to_complex(l: int) -> np.ndarray:
    """Unitary taking real spherical-harmonic components (index l+m, m=-l..l)
    to complex ones, times ``(-i)^l`` (e3nn_lite.py:656-674)."""
    q = np.zeros((2 * l + 1, 2 * l + 1), dtype=np.complex128)
    s = 2.0**-0.5
    q[l, l] = 1.0
    for m in range(1, l + 1):
        # row for -m
        q[l - m, l + m] = s
        q[l - m, l - m] = -1j * s
        # row for +m
        q[l + m, l + m] = (-1) ** m * s
        q[l + m, l - m] = 1j * (-1) ** m * s
    return (-1j) ** l * q


@functools.lru_cache(maxsize=None)
def _wigner_3j_cached(l1: int, l2: int, l3: int) -> np.ndarray:
    su2 = np.zeros((2 * l1 + 1, 2 * l2 + 1, 2 * l3 + 1), dtype=np.complex128)
    for m1 in range(-l1, l1 + 1):
        for m2 in range(-l2, l2 + 1):
            m3 = m1 + m2
            if abs(m3) <= l3:
                su2[l1 + m1, l2 + m2, l3 + m3] = su2_coupling(l1, m1, l2, m2, l3, m3)
    q1, q2, q3 = real_to_complex(l1), real_to_complex(l2), real_to_complex(l3)
    c = np.einsum("ij,kl,mn,ikn->jlm", q1, q2, np.conj(q3.T), su2)
    assert np.all(np.abs(c.imag) < 1e-5)
    c = np.ascontiguousarray(c.real)
    c /= np.linalg.norm(c.ravel())
    c.setflags(write=False)
    return c


def wigner_3j(l1: int, l2: int, l3: int, dtype=np.float64) -> np.ndarray:
    """Real CG tensor of shape ``(2l1+1, 2l2+1, 2l3+1)`` with unit Frobenius
    norm (e3nn_lite.py:677-733)."""
    assert isinstance(l1, int) and isinstance(l2, int) and isinstance(l3, int)
    assert abs(l2 - l3) <= l1 <= l2 + l3
    return np.array(_wigner_3j_cached(l1, l2, l3), dtype=dtype)


def sparse_cg(l1: int, l2: int, l3: int, scale: float = 1.0, tol: float = 1e-10):
    """Structural non-zeros of ``scale * wigner_3j`` as a list of
    ``(i, j, k, value)`` sorted by ``(j, i, k)``. Entries below ``tol`` are
    round-off from the basis change and are dropped."""
    c = _wigner_3j_cached(l1, l2, l3)
    out = []
    for j in range(c.shape[1]):
        for i in range(c.shape[0]):
            for k in range(c.shape[2]):
                if abs(c[i, j, k]) > tol:
                    out.append((i, j, k, float(c[i, j, k] * scale)))
    return out
