"""Real spherical harmonics of unit vectors, used to synthesise edge features.

The reference has no harmonics of its own (callers bring e3nn's); benchmarks
and tests here need ``Y`` inputs whose basis is consistent with the coupling
tensors of :mod:`openequivariance_amd.wigner`, so they are built by the
recursion ``Y_{l+1} ~ C(l, 1, l+1) . (Y_l (x) Y_1)`` starting from
``Y_0 = 1`` and ``Y_1 = sqrt(3) (x, y, z)`` ("component" normalisation:
``|Y_l|^2 = 2l+1`` on the unit sphere).  Equivariance under rotations follows
from the invariance of ``C``; the overall sign of each degree is fixed by
requiring a positive value at the pole ``(0, 1, 0)``.
"""
from __future__ import annotations

import numpy as np

from .wigner import wigner_3j


def spherical_harmonics(lmax: int, vectors: np.ndarray, normalize: bool = True) -> np.ndarray:
    """``[n, (lmax+1)^2]`` array of component-normalised harmonics of ``vectors[n, 3]``."""
    v = np.asarray(vectors, dtype=np.float64)
    if v.ndim != 2 or v.shape[1] != 3:
        raise ValueError("vectors must have shape [n, 3]")
    if normalize:
        v = v / np.linalg.norm(v, axis=1, keepdims=True)
    pole = np.array([[0.0, 1.0, 0.0]])
    pts = np.concatenate([v, pole], axis=0)

    cols = [np.ones((pts.shape[0], 1))]
    if lmax >= 1:
        y1 = np.sqrt(3.0) * pts
        cols.append(y1)
        prev = y1
        for l in range(1, lmax):
            c = wigner_3j(l, 1, l + 1)
            nxt = np.einsum("ijk,ni,nj->nk", c, prev, y1)
            # on the unit sphere |nxt| is constant; rescale to sqrt(2l+3)
            norm = np.linalg.norm(nxt[-1])
            nxt = nxt * (np.sqrt(2 * (l + 1) + 1) / norm)
            # sign convention: the m=0 component is positive at the pole
            if nxt[-1, l + 1] < 0:
                nxt = -nxt
            cols.append(nxt)
            prev = nxt
    return np.concatenate(cols, axis=1)[:-1]


def random_unit_vectors(n: int, rng: np.random.Generator) -> np.ndarray:
    """Normalised N(0, I3) samples."""
    v = rng.standard_normal((n, 3))
    return v / np.linalg.norm(v, axis=1, keepdims=True)
