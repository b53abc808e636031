"""Real-basis Clebsch-Gordan (Wigner 3j) tensors, in e3nn's convention.

``wigner_3j(l1, l2, l3)`` returns the tensor ``C[2l1+1, 2l2+1, 2l3+1]`` that
the tensor-product kernels bake in as compile-time constants.  It has to agree
with the reference to the sign, so it follows the same construction
(reference: openequivariance/implementations/e3nn_lite.py:573-771):

1. the complex (SU(2)) coupling coefficients ``<j1 m1 j2 m2 | j3 m3>`` from
   Racah's closed form, evaluated here in exact rational arithmetic with a
   single square root at the end;
2. the unitary change of basis from real to complex spherical harmonics with
   the extra ``(-i)^l`` phase that makes the result real;
3. Frobenius normalisation ``sum C_ijk^2 = 1``.
"""
from __future__ import annotations

import functools
from fractions import Fraction
from math import factorial, sqrt

import numpy as np


def _racah_cg(j1: int, m1: int, j2: int, m2: int, j3: int, m3: int) -> float:
    """<j1 m1; j2 m2 | j3 m3> for integer spins (Racah's formula)."""
    if m3 != m1 + m2 or not (abs(j1 - j2) <= j3 <= j1 + j2):
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
    acc = Fraction(0)
    for v in range(lo, hi + 1):
        term = Fraction(
            f(j2 + j3 + m1 - v) * f(j1 - m1 + v),
            f(v) * f(j3 - j1 + j2 - v) * f(j3 + m3 - v) * f(v + j1 - j2 - m3),
        )
        acc += term if (v + j2 + m2) % 2 == 0 else -term
    # sign(acc) * sqrt(pref * acc^2) keeps everything exact until the last step
    mag = sqrt(pref * acc * acc)
    return mag if acc >= 0 else -mag


@functools.lru_cache(maxsize=None)
def su2_clebsch_gordan(j1: int, j2: int, j3: int) -> np.ndarray:
    """Dense ``[2j1+1, 2j2+1, 2j3+1]`` array of complex-basis coefficients."""
    out = np.zeros((2 * j1 + 1, 2 * j2 + 1, 2 * j3 + 1), dtype=np.float64)
    for m1 in range(-j1, j1 + 1):
        for m2 in range(-j2, j2 + 1):
            m3 = m1 + m2
            if abs(m3) <= j3:
                out[j1 + m1, j2 + m2, j3 + m3] = _racah_cg(j1, m1, j2, m2, j3, m3)
    out.setflags(write=False)
    return out


@functools.lru_cache(maxsize=None)
def real_to_complex(l: int) -> np.ndarray:
    """Matrix ``Q`` taking real harmonics (index ``l + m``) to complex ones."""
    q = np.zeros((2 * l + 1, 2 * l + 1), dtype=np.complex128)
    s = 1.0 / sqrt(2.0)
    q[l, l] = 1.0
    for m in range(1, l + 1):
        sign = -1.0 if m % 2 else 1.0
        # row for -m
        q[l - m, l + m] = s
        q[l - m, l - m] = -1j * s
        # row for +m
        q[l + m, l + m] = sign * s
        q[l + m, l - m] = 1j * sign * s
    q = (-1j) ** l * q
    q.setflags(write=False)
    return q


@functools.lru_cache(maxsize=None)
def _real_cg(l1: int, l2: int, l3: int) -> np.ndarray:
    q1, q2, q3 = real_to_complex(l1), real_to_complex(l2), real_to_complex(l3)
    c = su2_clebsch_gordan(l1, l2, l3).astype(np.complex128)
    # C_real[j,l,m] = sum_{i,k,n} Q1[i,j] Q2[k,l] conj(Q3)[m,n]^T ... i.e. contract the complex
    # indices of the coupling tensor with Q1, Q2 and Q3^dagger
    c = np.einsum("ij,kl,mn,ikn->jlm", q1, q2, np.conj(q3.T), c)
    if np.abs(c.imag).max() > 1e-10:
        raise ArithmeticError(f"real-basis CG for {(l1, l2, l3)} is not real")
    c = np.ascontiguousarray(c.real)
    c /= np.linalg.norm(c)
    c.setflags(write=False)
    return c


def wigner_3j(l1: int, l2: int, l3: int, dtype=np.float64) -> np.ndarray:
    """Real-basis coupling tensor of shape ``(2l1+1, 2l2+1, 2l3+1)``, norm 1."""
    for l in (l1, l2, l3):
        if not isinstance(l, (int, np.integer)) or l < 0:
            raise ValueError("degrees must be non-negative integers")
    if not abs(l2 - l3) <= l1 <= l2 + l3:
        raise ValueError(f"({l1}, {l2}, {l3}) violates the triangle rule")
    return np.array(_real_cg(int(l1), int(l2), int(l3)), dtype=dtype)


def cg_nonzeros(l1: int, l2: int, l3: int, scale: float = 1.0, tol: float = 1e-12):
    """Sparse list ``[(i, j, k, value)]`` of ``scale * C`` sorted by ``(i, j, k)``."""
    c = _real_cg(l1, l2, l3)
    idx = np.argwhere(np.abs(c) > tol)
    return [(int(i), int(j), int(k), float(c[i, j, k] * scale)) for i, j, k in idx]
