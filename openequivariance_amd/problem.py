"""Tensor-product problem description (host side, numpy only).

``TPProblem`` mirrors the constructor, attributes and normalisation rules of
the reference's class of the same name
(reference: openequivariance/implementations/e3nn_lite.py:365-571), and the
three problem families used by its benchmarks are provided with the same
instruction ordering (reference: openequivariance/benchmark/tpp_creation_utils.py).
"""
from __future__ import annotations

from math import prod, sqrt
from typing import List, NamedTuple, Optional, Sequence, Tuple

import numpy as np

from .irreps import Irrep, Irreps

CONNECTION_MODES = ("uvw", "uvu", "uvv", "uuw", "uuu", "uvuv", "uvu<v", "u<vw")


class Instruction(NamedTuple):
    i_in1: int
    i_in2: int
    i_out: int
    connection_mode: str
    has_weight: bool
    path_weight: float
    path_shape: tuple


def _path_shape(mode: str, m1: int, m2: int, mo: int) -> tuple:
    if mode == "uvw":
        return (m1, m2, mo)
    if mode in ("uvu", "uvv", "uvuv"):
        return (m1, m2)
    if mode == "uuw":
        return (m1, mo)
    if mode == "uuu":
        return (m1,)
    if mode == "uvu<v":
        return (m1 * (m2 - 1) // 2,)
    if mode == "u<vw":
        return (m1 * (m2 - 1) // 2, mo)
    raise ValueError(f"unknown connection mode {mode!r}")


def _fan_in(mode: str, m1: int, m2: int) -> int:
    """Number of (u, v) pairs summed into one output channel by an instruction."""
    if mode == "uvw":
        return m1 * m2
    if mode == "uvu":
        return m2
    if mode in ("uvv", "uuw"):
        return m1
    if mode in ("uuu", "uvuv", "uvu<v"):
        return 1
    if mode == "u<vw":
        return m1 * (m2 - 1) // 2
    raise ValueError(f"unknown connection mode {mode!r}")


class TPProblem:
    """Specification of a weighted Clebsch-Gordan tensor product.

    After construction ``instructions[t].path_weight`` holds the *final*
    coefficient ``sqrt(alpha_t)`` multiplying path ``t`` where

        alpha = N_irrep / x * out_var[i_out] * user_path_weight
        N_irrep = dim(out) | dim(in1) * dim(in2) | 1   (component | norm | none)
        x = sum over paths into the same output of in1_var * in2_var * fan_in
            (element), or that product for this path times the number of such
            paths (path), or 1 (none)

    (reference: e3nn_lite.py:465-500).
    """

    def __init__(
        self,
        irreps_in1,
        irreps_in2,
        irreps_out,
        instructions: Sequence[tuple],
        in1_var: Optional[Sequence[float]] = None,
        in2_var: Optional[Sequence[float]] = None,
        out_var: Optional[Sequence[float]] = None,
        irrep_normalization: str = "component",
        path_normalization: str = "element",
        internal_weights: Optional[bool] = None,
        shared_weights: Optional[bool] = None,
        label: Optional[str] = None,
        irrep_dtype=np.float32,
        weight_dtype=np.float32,
    ) -> None:
        if irrep_normalization not in ("component", "norm", "none"):
            raise AssertionError(f"bad irrep_normalization {irrep_normalization!r}")
        if path_normalization not in ("element", "path", "none"):
            raise AssertionError(f"bad path_normalization {path_normalization!r}")
        irrep_dtype = np.dtype(irrep_dtype).type
        weight_dtype = np.dtype(weight_dtype).type

        self.irreps_in1 = Irreps(irreps_in1)
        self.irreps_in2 = Irreps(irreps_in2)
        self.irreps_out = Irreps(irreps_out)
        self.instructions_raw = instructions
        self.in1_var, self.in2_var, self.out_var = in1_var, in2_var, out_var
        self.irrep_normalization = irrep_normalization
        self.path_normalization = path_normalization
        self.label = label

        L1, L2, L3 = self.irreps_in1, self.irreps_in2, self.irreps_out
        raw: List[Instruction] = []
        for ins in instructions:
            ins = tuple(ins)
            if len(ins) == 5:
                ins = ins + (1.0,)
            i1, i2, io, mode, has_w, pw = ins
            if mode not in CONNECTION_MODES:
                raise AssertionError(f"unknown connection mode {mode!r}")
            a, b, c = L1[i1], L2[i2], L3[io]
            assert a.ir.p * b.ir.p == c.ir.p, f"parity mismatch in instruction {ins}"
            assert abs(a.ir.l - b.ir.l) <= c.ir.l <= a.ir.l + b.ir.l, f"triangle rule violated in {ins}"
            raw.append(Instruction(i1, i2, io, mode, bool(has_w), float(pw), _path_shape(mode, a.mul, b.mul, c.mul)))

        def _var(v, irreps, name):
            if v is None:
                return [1.0] * len(irreps)
            v = [float(t) for t in v]
            assert len(v) == len(irreps), f"len({name}) must equal the number of irrep blocks"
            return v

        v1 = _var(in1_var, L1, "in1_var")
        v2 = _var(in2_var, L2, "in2_var")
        vo = _var(out_var, L3, "out_var")

        def weight_of(t: Instruction) -> float:
            return v1[t.i_in1] * v2[t.i_in2] * _fan_in(t.connection_mode, L1[t.i_in1].mul, L2[t.i_in2].mul)

        final: List[Instruction] = []
        for t in raw:
            if irrep_normalization == "component":
                alpha = float(L3[t.i_out].ir.dim)
            elif irrep_normalization == "norm":
                alpha = float(L1[t.i_in1].ir.dim * L2[t.i_in2].ir.dim)
            else:
                alpha = 1.0
            siblings = [s for s in raw if s.i_out == t.i_out]
            if path_normalization == "element":
                x = sum(weight_of(s) for s in siblings)
            elif path_normalization == "path":
                x = weight_of(t) * len(siblings)
            else:
                x = 1.0
            if x > 0.0:
                alpha /= x
            alpha *= vo[t.i_out] * t.path_weight
            final.append(t._replace(path_weight=sqrt(alpha)))
        self.instructions = final

        self._in1_dim, self._in2_dim = L1.dim, L2.dim

        if shared_weights is False and internal_weights is None:
            internal_weights = False
        if shared_weights is None:
            shared_weights = True
        if internal_weights is None:
            internal_weights = shared_weights and any(t.has_weight for t in final)
        assert shared_weights or not internal_weights
        self.internal_weights = internal_weights
        self.shared_weights = shared_weights

        self.weight_numel = sum(prod(t.path_shape) for t in final if t.has_weight)
        self.output_mask = None
        self.irrep_dtype = irrep_dtype
        self.weight_dtype = weight_dtype

    # ------------------------------------------------------------------
    def weight_range_and_shape_for_instruction(self, instruction: int) -> Tuple[int, int, tuple]:
        t = self.instructions[instruction]
        if not t.has_weight:
            raise ValueError(f"Instruction {instruction} has no weights.")
        start = sum(prod(s.path_shape) for s in self.instructions[:instruction])
        return start, start + prod(t.path_shape), t.path_shape

    def __str__(self) -> str:
        return (f"{type(self).__name__}({self.irreps_in1.simplify()} x {self.irreps_in2.simplify()})"
                f" -> {self.irreps_out.simplify()}")

    def __repr__(self) -> str:
        lines = [str(self),
                 f"irrep_normalization = {self.irrep_normalization!r}",
                 f"path_normalization = {self.path_normalization!r}",
                 f"internal_weights = {self.internal_weights}",
                 f"shared_weights = {self.shared_weights}",
                 f"num weights {self.weight_numel}",
                 "| in1 | in2 | out |  l1 |  l2 |  l3 | mul1 | mul2 | mulo | mode  | w | coeff"]
        for t in self.instructions:
            a, b, c = self.irreps_in1[t.i_in1], self.irreps_in2[t.i_in2], self.irreps_out[t.i_out]
            lines.append(f"| {t.i_in1:3} | {t.i_in2:3} | {t.i_out:3} | {a.ir.l:3} | {b.ir.l:3} | {c.ir.l:3} |"
                         f" {a.mul:4} | {b.mul:4} | {c.mul:4} | {t.connection_mode:<5} |"
                         f" {int(t.has_weight)} | {t.path_weight:.6f}")
        return "\n".join(lines)


# ----------------------------------------------------------------------------
# Problem families (instruction enumeration rules of the reference benchmarks)
# ----------------------------------------------------------------------------

class FullyConnectedTPProblem(TPProblem):
    """Every allowed (in1, in2, out) triple in nested-loop order, mode ``uvw``
    (reference: benchmark/tpp_creation_utils.py:15-36)."""

    def __init__(self, irreps_in1, irreps_in2, irreps_out, **kwargs) -> None:
        L1, L2, L3 = Irreps(irreps_in1), Irreps(irreps_in2), Irreps(irreps_out)
        instr = []
        for i1, a in enumerate(L1):
            for i2, b in enumerate(L2):
                allowed = set(a.ir * b.ir)
                for io, c in enumerate(L3):
                    if c.ir in allowed:
                        instr.append((i1, i2, io, "uvw", True, 1.0))
        super().__init__(L1, L2, L3, instr, **kwargs)


class ChannelwiseTPP(TPProblem):
    """MACE-style channel-wise product: one ``uvu`` path and one output block
    per allowed (in1, in2, l3) combination whose irrep occurs in ``irreps_out``;
    output blocks stably sorted by (l, p); instructions ordered by output block;
    per-row (non-shared) weights (reference: benchmark/tpp_creation_utils.py:118-162)."""

    def __init__(self, irreps_in1, irreps_in2, irreps_out, label: Optional[str] = None,
                 irrep_dtype=np.float32, weight_dtype=np.float32) -> None:
        L1, L2, target = Irreps(irreps_in1), Irreps(irreps_in2), Irreps(irreps_out)
        blocks, instr = [], []
        for i1, a in enumerate(L1):
            for i2, b in enumerate(L2):
                for ir_out in a.ir * b.ir:
                    if ir_out in target:
                        instr.append((i1, i2, len(blocks), "uvu", True))
                        blocks.append((a.mul, ir_out))
        out_sorted, perm, _ = Irreps(blocks).sort()
        instr = sorted(((i1, i2, perm[io], mode, w) for i1, i2, io, mode, w in instr), key=lambda t: t[2])
        super().__init__(L1, L2, out_sorted, instr, internal_weights=False, shared_weights=False,
                         label=label, irrep_dtype=irrep_dtype, weight_dtype=weight_dtype)


class SingleInstruction(TPProblem):
    """One instruction ``(0, 0, 0, mode)`` with per-row weights
    (reference: benchmark/tpp_creation_utils.py:164-181)."""

    def __init__(self, irreps_in1, irreps_in2, irreps_out, mode: str, label: Optional[str] = None,
                 irrep_dtype=np.float32, weight_dtype=np.float32) -> None:
        super().__init__(Irreps(irreps_in1), Irreps(irreps_in2), Irreps(irreps_out), [(0, 0, 0, mode, True)],
                         internal_weights=False, shared_weights=False, label=label,
                         irrep_dtype=irrep_dtype, weight_dtype=weight_dtype)
