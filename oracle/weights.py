"""Oracle: the reference's external ("oeq") weight order, restated procedurally.

Test infrastructure.  Follows
openequivariance/implementations/ComputationSchedule.py:161-230 (every
multiplicity is cut into chunks of <= 32; uvu children enumerate
(u-chunk, v-chunk), uvw children (u-chunk, v-chunk, w-chunk); each child
remembers its sub-range of the parent's weight tensor) and :427-471 (each
child block is the parent's slice transposed (u,v)->(v,u) resp.
(u,v,w)->(v,u,w) and flattened; children are concatenated in creation order).
Written element by element, on purpose, so it shares no code path with the
vectorised permutation the product uses.
"""
from __future__ import annotations

from math import prod

import numpy as np

from .spec import Problem

CHUNK = 32


def _ranges(n):
    return [(s, min(s + CHUNK, n)) for s in range(0, n, CHUNK)]


def e3nn_to_oeq(prob: Problem, w_e3nn: np.ndarray) -> np.ndarray:
    """Reorder the last axis of ``w_e3nn`` into the order the kernels ingest."""
    w_e3nn = np.asarray(w_e3nn)
    out = np.zeros_like(w_e3nn)
    pos = 0
    for p in prob.paths:
        shape = p["shape"]
        parent = w_e3nn[..., p["woff"]: p["woff"] + prod(shape)].reshape(w_e3nn.shape[:-1] + tuple(shape))
        if p["mode"] == "uvu":
            mu, mv = shape
            for (u0, u1) in _ranges(mu):
                for (v0, v1) in _ranges(mv):
                    for v in range(v0, v1):
                        for u in range(u0, u1):
                            out[..., pos] = parent[..., u, v]
                            pos += 1
        else:
            mu, mv, mw = shape
            for (u0, u1) in _ranges(mu):
                for (v0, v1) in _ranges(mv):
                    for (w0, w1) in _ranges(mw):
                        for v in range(v0, v1):
                            for u in range(u0, u1):
                                n = w1 - w0
                                out[..., pos:pos + n] = parent[..., u, v, w0:w1]
                                pos += n
    assert pos == prob.weight_numel
    return out


def oeq_to_e3nn(prob: Problem, w_oeq: np.ndarray) -> np.ndarray:
    """Inverse of :func:`e3nn_to_oeq` (used to bring dW back for comparison)."""
    w_oeq = np.asarray(w_oeq)
    idx = e3nn_to_oeq(prob, np.arange(prob.weight_numel))      # idx[k] = e3nn position stored at oeq slot k
    out = np.zeros_like(w_oeq)
    out[..., idx] = w_oeq
    return out
