"""Oracle: problem description, normalisation and instruction enumeration.

Test infrastructure; plain Python.  Restates
openequivariance/implementations/e3nn_lite.py:374-523 (path shapes, the
normalisation coefficient, weight count) and
openequivariance/benchmark/tpp_creation_utils.py:15-36, :118-181 (the
fully-connected, channel-wise and single-instruction problem families).

Irreps are lists of ``(mul, l, p)`` triples; ``parse_irreps`` reads the usual
"128x0e+128x1o" strings.
"""
from __future__ import annotations

from math import prod, sqrt
from typing import List, Sequence, Tuple

Irr = Tuple[int, int, int]          # (mul, l, p)


def parse_irreps(text) -> List[Irr]:
    if not isinstance(text, str):
        return [(int(m), int(l), int(p)) for m, l, p in text]
    out = []
    for term in text.replace(" ", "").split("+"):
        if not term:
            continue
        mul, name = term.split("x") if "x" in term else ("1", term)
        l = int(name[:-1])
        p = {"e": 1, "o": -1, "y": (-1) ** l}[name[-1]]
        out.append((int(mul), l, p))
    return out


def dim(irreps: Sequence[Irr]) -> int:
    return sum(m * (2 * l + 1) for m, l, _ in irreps)


def offsets(irreps: Sequence[Irr]) -> List[int]:
    out, s = [], 0
    for m, l, _ in irreps:
        out.append(s)
        s += m * (2 * l + 1)
    return out


def product_irreps(a: Irr, b: Irr):
    """(l, p) pairs allowed by the selection rule for a (x) b."""
    return [(l, a[2] * b[2]) for l in range(abs(a[1] - b[1]), a[1] + b[1] + 1)]


class Problem:
    """Mirror of the reference TPProblem, reduced to what the contraction needs."""

    def __init__(self, irreps_in1, irreps_in2, irreps_out, instructions, *,
                 in1_var=None, in2_var=None, out_var=None,
                 irrep_normalization="component", path_normalization="element",
                 shared_weights=None):
        self.in1, self.in2, self.out = parse_irreps(irreps_in1), parse_irreps(irreps_in2), parse_irreps(irreps_out)
        v1 = [1.0] * len(self.in1) if in1_var is None else list(map(float, in1_var))
        v2 = [1.0] * len(self.in2) if in2_var is None else list(map(float, in2_var))
        vo = [1.0] * len(self.out) if out_var is None else list(map(float, out_var))
        ins = [tuple(t) if len(t) == 6 else tuple(t) + (1.0,) for t in instructions]

        def shape(t):                       # e3nn_lite.py:421-430
            m1, m2, mo = self.in1[t[0]][0], self.in2[t[1]][0], self.out[t[2]][0]
            return {"uvw": (m1, m2, mo), "uvu": (m1, m2)}[t[3]]

        def num_elements(t):                # e3nn_lite.py:453-463
            m1, m2 = self.in1[t[0]][0], self.in2[t[1]][0]
            return {"uvw": m1 * m2, "uvu": m2}[t[3]]

        self.paths = []
        for t in ins:
            i1, i2, io, mode, has_w, pw = t
            assert self.in1[i1][2] * self.in2[i2][2] == self.out[io][2]
            assert abs(self.in1[i1][1] - self.in2[i2][1]) <= self.out[io][1] <= self.in1[i1][1] + self.in2[i2][1]
            if irrep_normalization == "component":      # e3nn_lite.py:474-479
                alpha = 2 * self.out[io][1] + 1
            elif irrep_normalization == "norm":
                alpha = (2 * self.in1[i1][1] + 1) * (2 * self.in2[i2][1] + 1)
            else:
                alpha = 1
            if path_normalization == "element":         # e3nn_lite.py:481-487
                x = sum(v1[s[0]] * v2[s[1]] * num_elements(s) for s in ins if s[2] == io)
            elif path_normalization == "path":
                x = v1[i1] * v2[i2] * num_elements(t) * len([s for s in ins if s[2] == io])
            else:
                x = 1
            if x > 0.0:
                alpha /= x
            alpha *= vo[io] * pw
            self.paths.append(dict(i1=i1, i2=i2, io=io, mode=mode, has_weight=bool(has_w),
                                   coeff=sqrt(alpha), shape=shape(t)))
        woff = 0
        for p in self.paths:                            # e3nn_lite.py:566-571
            p["woff"] = woff
            woff += prod(p["shape"])
        self.weight_numel = woff
        self.shared_weights = True if shared_weights is None else bool(shared_weights)
        self.d1, self.d2, self.d3 = dim(self.in1), dim(self.in2), dim(self.out)


def _sorted_blocks(blocks):
    """Stable sort by (l, p): returns (sorted blocks, perm old->new) (e3nn_lite.py:321-328)."""
    order = sorted(range(len(blocks)), key=lambda i: ((blocks[i][1], blocks[i][2]), i))
    perm = [0] * len(blocks)
    for new, old in enumerate(order):
        perm[old] = new
    return [blocks[i] for i in order], perm


def channelwise(irreps_in1, irreps_in2, irreps_out) -> Problem:
    """tpp_creation_utils.py:118-162."""
    a, b, target = parse_irreps(irreps_in1), parse_irreps(irreps_in2), parse_irreps(irreps_out)
    wanted = {(l, p) for _, l, p in target}
    blocks, ins = [], []
    for i, x in enumerate(a):
        for j, y in enumerate(b):
            for (l, p) in product_irreps(x, y):
                if (l, p) in wanted:
                    ins.append((i, j, len(blocks), "uvu", True))
                    blocks.append((x[0], l, p))
    blocks, perm = _sorted_blocks(blocks)
    ins = sorted([(i, j, perm[k], m, w) for i, j, k, m, w in ins], key=lambda t: t[2])
    return Problem(a, b, blocks, ins, shared_weights=False)


def fully_connected(irreps_in1, irreps_in2, irreps_out, shared_weights=None) -> Problem:
    """tpp_creation_utils.py:15-36."""
    a, b, c = parse_irreps(irreps_in1), parse_irreps(irreps_in2), parse_irreps(irreps_out)
    ins = [(i, j, k, "uvw", True, 1.0)
           for i, x in enumerate(a) for j, y in enumerate(b) for k, z in enumerate(c)
           if (z[1], z[2]) in product_irreps(x, y)]
    return Problem(a, b, c, ins, shared_weights=shared_weights)


def single_instruction(irreps_in1, irreps_in2, irreps_out, mode) -> Problem:
    """tpp_creation_utils.py:164-181."""
    return Problem(irreps_in1, irreps_in2, irreps_out, [(0, 0, 0, mode, True)], shared_weights=False)
