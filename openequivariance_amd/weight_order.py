"""The two external weight layouts and the permutation between them.

*e3nn order*: instruction after instruction, each instruction's weights stored
row-major in its ``path_shape`` (``[u][v]`` for uvu, ``[u][v][w]`` for uvw).

*oeq order* (what ``TensorProduct.__call__`` consumes, kept for drop-in
compatibility with the reference): every multiplicity is cut into chunks of at
most 32; for each instruction the chunk combinations are enumerated
lexicographically ``(u-chunk, v-chunk[, w-chunk])`` and each block is stored
``[v_local][u_local]`` (uvu) or ``[v_local][u_local][w_local]`` (uvw)
(reference: openequivariance/implementations/ComputationSchedule.py:161-230
for the chunk enumeration and :427-471 for the transposition).  For uvu
problems whose second operand has multiplicity 1 the two orders coincide.

The map is a pure index permutation; it is computed once per problem as an
int64 array ``perm`` with ``w_oeq[..., k] = w_e3nn[..., perm[k]]``.
"""
from __future__ import annotations

from math import prod

import numpy as np

from .problem import TPProblem

OEQ_CHUNK = 32


def _chunks(n: int, size: int):
    return [(s, min(size, n - s)) for s in range(0, n, size)]


def oeq_from_e3nn_permutation(problem: TPProblem, chunk: int = OEQ_CHUNK) -> np.ndarray:
    """``perm`` with ``w_oeq[k] = w_e3nn[perm[k]]`` (length ``weight_numel``)."""
    perm = np.empty(problem.weight_numel, dtype=np.int64)
    pos = 0
    base = 0
    for t in problem.instructions:
        if not t.has_weight:
            continue
        shape = t.path_shape
        idx = base + np.arange(prod(shape), dtype=np.int64).reshape(shape)
        if t.connection_mode == "uvu":
            mu, mv = shape
            for us, ul in _chunks(mu, chunk):
                for vs, vl in _chunks(mv, chunk):
                    blk = idx[us:us + ul, vs:vs + vl].transpose(1, 0).reshape(-1)
                    perm[pos:pos + blk.size] = blk
                    pos += blk.size
        elif t.connection_mode == "uvw":
            mu, mv, mw = shape
            for us, ul in _chunks(mu, chunk):
                for vs, vl in _chunks(mv, chunk):
                    for ws, wl in _chunks(mw, chunk):
                        blk = idx[us:us + ul, vs:vs + vl, ws:ws + wl].transpose(1, 0, 2).reshape(-1)
                        perm[pos:pos + blk.size] = blk
                        pos += blk.size
        else:
            raise NotImplementedError(f"weight order for mode {t.connection_mode!r}")
        base += prod(shape)
    assert pos == problem.weight_numel
    return perm


def is_identity(perm: np.ndarray) -> bool:
    return bool(np.array_equal(perm, np.arange(perm.size)))


class WeightReorder:
    """Callable pair with the reference's calling convention
    ``f(weights_in, weights_out, has_batch_dim)`` writing into ``weights_out``
    (reference: openequivariance/implementations/LoopUnrollTP.py:65-68)."""

    def __init__(self, problem: TPProblem):
        self.perm = oeq_from_e3nn_permutation(problem)
        self.inv = np.empty_like(self.perm)
        self.inv[self.perm] = np.arange(self.perm.size)

    def e3nn_to_oeq(self, weights_in, weights_out, has_batch_dim: bool = False) -> None:
        weights_out[...] = weights_in[..., self.perm]

    def oeq_to_e3nn(self, weights_in, weights_out, has_batch_dim: bool = False) -> None:
        weights_out[...] = weights_in[..., self.inv]
