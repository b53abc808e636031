"""Work models the harness reports when an implementation has none of its own
(reference: openequivariance/benchmark/perf_metrics_utils.py, e3nn_lite_utils.py)."""
from __future__ import annotations

import functools
import math

import numpy as np

from ..problem import TPProblem
from ..wigner import wigner_3j


@functools.lru_cache(maxsize=None)
def count_cg_non_zero(l1: int, l2: int, l3: int) -> int:
    return int(np.count_nonzero(wigner_3j(l1, l2, l3)))


def sparse_outer_product_work(cg: np.ndarray) -> int:
    """(i, j) pairs that feed at least one nonzero coefficient."""
    return int(np.sum(np.any(cg != 0, axis=2)))


def _ls(tpp: TPProblem, ins):
    return tpp.irreps_in1[ins.i_in1].ir.l, tpp.irreps_in2[ins.i_in2].ir.l, tpp.irreps_out[ins.i_out].ir.l


def calculate_total_nnz(tpp: TPProblem) -> int:
    """Nonzeros of the distinct Clebsch-Gordan tensors the problem uses (each (l1,l2,l3) once)."""
    return sum(count_cg_non_zero(*ls) for ls in {_ls(tpp, ins) for ins in tpp.instructions})


def _streamed(tpp: TPProblem, batch_size: int, parts) -> dict:
    si, sw = np.dtype(tpp.irrep_dtype).itemsize, np.dtype(tpp.weight_dtype).itemsize
    width = {"input 1": (tpp.irreps_in1.dim, si), "input 2": (tpp.irreps_in2.dim, si), "output": (tpp.irreps_out.dim, si),
             "weights": (tpp.weight_numel, sw)}
    out = {}
    for name in parts:
        dim, size = width[name.replace(" grad", "")]
        out[name] = dim * batch_size * size
    out["total"] = sum(out.values())
    return out


def calculate_minimum_memory_streamed_forward(tpp: TPProblem, batch_size: int) -> dict:
    """Bytes of every operand touched once (weights counted per row, as the reference does)."""
    return _streamed(tpp, batch_size, ("input 1", "input 2", "output", "weights"))


def calculate_minimum_memory_streamed_backward(tpp: TPProblem, batch_size: int) -> dict:
    return _streamed(tpp, batch_size, ("input 1", "input 1 grad", "input 2", "input 2 grad", "output grad",
                                       "weights", "weights grad"))


def calculate_minimum_flops_forward(tpp: TPProblem, batch_size: int) -> dict:
    """Outer products formed once per instruction, two flops per nonzero and per weight use."""
    outer = cg = lin = 0
    for ins in tpp.instructions:
        l1, l2, l3 = _ls(tpp, ins)
        outer += sparse_outer_product_work(wigner_3j(l1, l2, l3))
        cg += count_cg_non_zero(l1, l2, l3) * ins.path_shape[0] * ins.path_shape[1]
        lin += (2 * l3 + 1) * math.prod(ins.path_shape) if ins.has_weight else 0
    out = {"outer_products": outer * batch_size, "CG_decomposition": 2 * cg * batch_size,
           "linear_combination": 2 * lin * batch_size}
    out["total"] = sum(out.values())
    return out


def calculate_minimum_flops_backward(tpp: TPProblem, batch_size: int) -> dict:
    raise NotImplementedError("no minimum-flop model for the backward pass (the reference has none either)")
