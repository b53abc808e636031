"""Oracle: real-basis Wigner 3j tensors (test infrastructure, numpy only).

Restates openequivariance/implementations/e3nn_lite.py:573-771 of the
reference: SU(2) coupling coefficients from Racah's formula (:719-771), the
real-to-complex change of basis with the (-i)^l phase (:573-591), contraction
and Frobenius normalisation (:635-649).  Floating-point factorials are used
here on purpose (the product side works in exact rationals), so the two
implementations do not share a failure mode.
"""
from __future__ import annotations

import functools
from math import factorial as fact

import numpy as np


def su2_cg_coeff(j1, m1, j2, m2, j3, m3) -> float:
    """<j1 m1 j2 m2 | j3 m3>, integer spins (e3nn_lite.py:719-771)."""
    if m3 != m1 + m2:
        return 0.0
    vmin = max(-j1 + j2 + m3, -j1 + m1, 0)
    vmax = min(j2 + j3 + m1, j3 - j1 + j2, j3 + m3)
    num = (2.0 * j3 + 1.0) * fact(j3 + j1 - j2) * fact(j3 - j1 + j2) * fact(j1 + j2 - j3) \
        * fact(j3 + m3) * fact(j3 - m3)
    den = float(fact(j1 + j2 + j3 + 1) * fact(j1 - m1) * fact(j1 + m1) * fact(j2 - m2) * fact(j2 + m2))
    total = 0.0
    for v in range(vmin, vmax + 1):
        sign = -1.0 if (v + j2 + m2) % 2 else 1.0
        total += sign * fact(j2 + j3 + m1 - v) * fact(j1 - m1 + v) / (
            fact(v) * fact(j3 - j1 + j2 - v) * fact(j3 + m3 - v) * fact(v + j1 - j2 - m3))
    return (num / den) ** 0.5 * total


def su2_cg(j1: int, j2: int, j3: int) -> np.ndarray:
    """Dense coupling tensor indexed [j1+m1, j2+m2, j3+m3] (e3nn_lite.py:688-716)."""
    mat = np.zeros((2 * j1 + 1, 2 * j2 + 1, 2 * j3 + 1))
    if abs(j1 - j2) <= j3 <= j1 + j2:
        for m1 in range(-j1, j1 + 1):
            for m2 in range(-j2, j2 + 1):
                if abs(m1 + m2) <= j3:
                    mat[j1 + m1, j2 + m2, j3 + m1 + m2] = su2_cg_coeff(j1, m1, j2, m2, j3, m1 + m2)
    return mat


def change_basis_real_to_complex(l: int) -> np.ndarray:
    """e3nn_lite.py:573-591."""
    q = np.zeros((2 * l + 1, 2 * l + 1), dtype=np.complex128)
    r = 2 ** -0.5
    for m in range(-l, 0):
        q[l + m, l + abs(m)] = r
        q[l + m, l - abs(m)] = -1j * r
    q[l, l] = 1.0
    for m in range(1, l + 1):
        q[l + m, l + abs(m)] = (-1) ** m * r
        q[l + m, l - abs(m)] = 1j * (-1) ** m * r
    return (-1j) ** l * q


@functools.lru_cache(maxsize=None)
def _wigner_3j(l1: int, l2: int, l3: int) -> np.ndarray:
    q1 = change_basis_real_to_complex(l1)
    q2 = change_basis_real_to_complex(l2)
    q3 = change_basis_real_to_complex(l3)
    c = su2_cg(l1, l2, l3).astype(np.complex128)
    c = np.einsum("ij,kl,mn,ikn->jlm", q1, q2, np.conj(q3.T), c)   # e3nn_lite.py:641
    assert np.all(np.abs(c.imag) < 1e-5)
    c = c.real
    return c / np.linalg.norm(c)


def wigner_3j(l1: int, l2: int, l3: int) -> np.ndarray:
    assert abs(l2 - l3) <= l1 <= l2 + l3
    return _wigner_3j(l1, l2, l3).copy()
