"""Generator of gfx950 HIP source for channel-wise ("uvu") tensor products.

This class holds what every uvu kernel shares - the lane mapping, the unrolled Clebsch-Gordan
arithmetic of one output block (forward and backward), the weight indexing and the launch plans -
and generates the LDS-staged batch product itself, which is the schedule used for *shared* weights
(persistent wavefronts and an ordered dW reduction).  The kernels for per-row weights and for the
convolutions derive from it: ``uvu_direct.py`` (register-direct loads), ``uvu_det.py`` (one node per
wavefront), ``uvu_sorted.py`` (on-the-fly grouping by receiver).  ``kind`` names the operator family
a subclass generates for: ``tp``, ``conv_atomic`` (per-edge kernels, scatter by atomics) or
``conv_det`` (segmented, no atomics).

Mapping to the hardware (the arithmetic follows the reference's kernels,
openequivariance/templates/loop_unroll_tp.cuh:20-97 forward and :107-252 backward, but the
schedule is new):

* a workgroup is ONE 64-lane wavefront; ``__syncthreads`` therefore costs a wait, not a barrier;
* lane <-> multiplicity channel ``u``.  Multiplicities above 64 are walked in chunks of 64;
  multiplicities of at most 32 pack ``R = 64 / P`` rows (edges) into one wavefront,
  ``P`` = the multiplicity rounded up to a power of two;
* global memory is always touched in contiguous runs: rows of X / dZ are copied to LDS with
  consecutive lanes reading consecutive words and are then read back transposed
  (lane ``u`` reads words ``u*(2l+1)+m``; the stride is odd, hence conflict free); Z / dX take the
  opposite route.  Blocks with l = 0 need no transposition and go straight to registers;
* the Clebsch-Gordan coefficients, multiplied by the path normalisation, are emitted as exact
  hexadecimal literals in fully unrolled fused multiply-adds; zero coefficients emit nothing;
* Y (<= 16 words per row) is loaded once per row; with one row per wavefront its address is
  wave-uniform, which lets the compiler keep it in scalar registers.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Tuple

import numpy as np

from ..problem import TPProblem
from ..wigner import wigner_3j
from .common import WAVE, Emitter, jinja_env, literal, next_pow2

MAX_UNROLLED_V = 8


@dataclass
class Block:
    idx: int
    mul: int
    l: int
    off: int

    @property
    def D(self) -> int:
        return 2 * self.l + 1

    @property
    def dim(self) -> int:
        return self.mul * self.D


@dataclass
class Path:
    t: int
    a: Block
    b: Block
    o: Block
    coeff: float
    woff: int
    pairs: Dict[Tuple[int, int], List[Tuple[int, float]]] = field(default_factory=dict)

    @property
    def mu(self) -> int:
        return self.a.mul

    @property
    def mv(self) -> int:
        return self.b.mul

    @property
    def nnz(self) -> int:
        return sum(len(v) for v in self.pairs.values())

    @property
    def looped(self) -> bool:
        """The copies v of the second operand are walked by a run-time loop instead of unrolled code."""
        return self.b.mul > MAX_UNROLLED_V

    def ordered_pairs(self):
        """(i, j) pairs sorted by j then i (the reference sorts its nonzeros by (j, i, k):
        openequivariance/implementations/ComputationSchedule.py:52-66)."""
        return sorted(self.pairs.items(), key=lambda kv: (kv[0][1], kv[0][0]))


def _blocks(irreps) -> List[Block]:
    out, off = [], 0
    for i, mi in enumerate(irreps):
        out.append(Block(i, mi.mul, mi.ir.l, off))
        off += mi.dim
    return out


class UVUGenerator:
    """Builds the source text and the launch plan for one uvu problem."""

    idx_ctype = "i64"        # element type of the convolution's index tensors ("int" for int32 callers)
    # Backward arithmetic per path.  True: t_i = sum_j s_ij y_j with dw = sum_i x_i t_i and dx_i += w t_i, and the
    # products c g_k that several pairs share computed once - two multiply-adds per pair beyond s_ij, a fifth fewer
    # vector instructions than one pair at a time.  The kernels are bound by memory and no faster for it (128 / 256
    # channels, batch and convolution: within 1 %); a kernel that holds a whole dZ row in registers spills more with
    # it and keeps the pair-at-a-time form (False).
    regroup_pairs = True

    def __init__(self, problem: TPProblem, kind: str = "tp", dw_partials: int = 1024):
        if kind not in ("tp", "conv_atomic", "conv_det"):
            raise ValueError(kind)
        if type(self) is UVUGenerator and kind != "tp":
            raise NotImplementedError("the convolution kernels come from uvu_direct / uvu_det / uvu_sorted")
        self.problem, self.kind = problem, kind
        self.T = {np.float32: "float", np.float64: "double"}[problem.irrep_dtype]
        self.itemsize = 4 if self.T == "float" else 8
        self.shared = bool(problem.shared_weights)
        self.in1 = _blocks(problem.irreps_in1)
        self.in2 = _blocks(problem.irreps_in2)
        self.out = _blocks(problem.irreps_out)
        self.D1, self.D2, self.D3 = problem.irreps_in1.dim, problem.irreps_in2.dim, problem.irreps_out.dim
        self.WN = problem.weight_numel

        self.paths: List[Path] = []
        woff = 0
        for t, ins in enumerate(problem.instructions):
            if ins.connection_mode != "uvu":
                raise ValueError("UVUGenerator handles uvu instructions only")
            if not ins.has_weight:
                raise NotImplementedError("instructions without weights are not supported")
            a, b, o = self.in1[ins.i_in1], self.in2[ins.i_in2], self.out[ins.i_out]
            if a.mul != o.mul:
                raise ValueError(f"uvu instruction {t}: mul(in1)={a.mul} must equal mul(out)={o.mul}")
            c = wigner_3j(a.l, b.l, o.l) * ins.path_weight
            p = Path(t, a, b, o, ins.path_weight, woff)
            for i, j, k in np.argwhere(np.abs(c) > 1e-14):
                p.pairs.setdefault((int(i), int(j)), []).append((int(k), float(c[i, j, k])))
            self.paths.append(p)
            woff += a.mul * b.mul
        if not self.paths:
            raise ValueError("Tensor product problem has no valid instructions!")
        if kind != "tp":
            if self.shared:
                raise NotImplementedError("fused convolution requires per-edge weights (shared_weights=False)")
            for b in self.in2:
                if b.mul != 1:
                    raise AssertionError("fused convolution requires multiplicity 1 for every irrep of in2")

        self.used_in1 = sorted({p.a.idx for p in self.paths})
        self.used_out = sorted({p.o.idx for p in self.paths})
        # Y values held in registers: those of the unrolled paths.  A second-operand block with more than
        # MAX_UNROLLED_V copies is walked by a run-time loop over v (reference: loop_unroll_tp.cuh:48-60 and
        # :140-175 loop over the v chunk): its Y values are read inside the loop and its dY sums are kept in LDS
        self.used_y = sorted({p.b.off + v * p.b.D + j for p in self.paths if not p.looped
                              for v in range(p.mv) for (_, j) in p.pairs})
        self.looped_y = {}                   # Y column of a looped block -> slot in the LDS accumulator
        for p in self.paths:
            if p.looped:
                for q in range(p.b.off, p.b.off + p.b.dim):
                    self.looped_y.setdefault(q, len(self.looped_y))
        self.NLY = len(self.looped_y)

        # lanes <-> channels over the widest block of X or Z: blocks that no path touches are zero-filled
        # through the same mapping, so it has to cover them too
        max_mul = max([b.mul for b in self.in1 if b.dim > 0] + [o.mul for o in self.out if o.dim > 0])
        if max_mul <= 32:
            self.P = next_pow2(max_mul)
            self.R = WAVE // self.P
            self.NCH = 1
        else:
            self.P, self.R = WAVE, 1
            self.NCH = (max_mul + WAVE - 1) // WAVE
        self.LOGP = self.P.bit_length() - 1
        # the deterministic convolution spreads chunks over blockIdx.y and stages one chunk of X
        self.chunk_in_grid = (kind == "conv_det")
        self.x_chunk_layout = self.chunk_in_grid and self.NCH > 1
        self.unroll_chunks = (self.NCH <= 2 or self.shared) and not self.chunk_in_grid
        self.dw_partials = dw_partials if self.shared else 0

        # ---- LDS map (in elements of T) --------------------------------------
        self.xl: Dict[int, int] = {}
        if self.x_chunk_layout:
            pos = 0
            for i in self.used_in1:
                self.xl[i] = pos
                pos += WAVE * self.in1[i].D
            self.x_lds = pos
        else:
            self.x_lds = self.R * self.D1
        stage = [WAVE * self.out[i].D for i in self.used_out if self.out[i].D > 1]
        stage += [WAVE * b.D for b in self.in1 if b.D > 1]
        self.ZB = self.x_lds
        self.stage_lds = max(stage) if stage else 0
        self.lds_elems = max(1, self.x_lds + self.stage_lds)

    # ------------------------------------------------------------------ helpers
    def lit(self, v: float) -> str:
        return literal(v, self.T)

    def backward_attr(self) -> str:
        """Extra kernel attributes of the backward kernel: the wavefronts per SIMD the register allocation
        must leave room for, when the schedule sets one (capping the wavefronts per SIMD of the batch
        kernels at 2, 3 or 4 helped plain copies of their shape by up to 5 % and the kernels not at all)."""
        w = getattr(self, "waves_per_eu", 0)
        return f" __attribute__((amdgpu_waves_per_eu({w})))" if w else ""

    def widx(self, p: Path, u: str, v) -> str:
        """oeq-order position of weight (u, v) of path ``p`` (see weight_order.py): chunks of 32 over u
        and v enumerated (u-chunk, v-chunk), each stored [v_local][u_local], which for any v is
        ``(u >> 5) * 32 * mv + width(u-chunk) * v + (u & 31)``.  ``v`` is a number or a C expression."""
        mu, mv = p.mu, p.mv
        if mv == 1:
            return f"{p.woff} + {u}"
        if mu <= 32:
            return (f"{p.woff + v * mu} + {u}" if isinstance(v, int) else f"{p.woff} + ({v}) * {mu} + {u}")
        ulw = "32" if mu % 32 == 0 else f"min(32, {mu} - (({u}) >> 5) * 32)"
        return f"{p.woff} + (({u}) >> 5) * {32 * mv} + {ulw} * ({v}) + (({u}) & 31)"

    def full(self, blk: Block) -> bool:
        """True when every lane of every chunk maps to a valid channel of ``blk``."""
        return blk.mul == self.P * self.NCH

    def act(self, blk: Block) -> str:
        return "rv" if self.full(blk) else f"(rv && u < {blk.mul})"

    def paths_into(self, o_idx: int) -> List[Path]:
        return [p for p in self.paths if p.o.idx == o_idx]

    def chunk_count(self, blk: Block) -> str:
        """Number of valid channels of ``blk`` in chunk ``c`` (C expression)."""
        if self.full(blk):
            return f"{self.P}"
        if self.NCH == 1:
            return f"{blk.mul}"
        return f"max(0, min({self.P}, {blk.mul} - c * {self.P}))"

    # ---------------------------------------------------------------- prologue
    def emit_lane(self, E: Emitter) -> None:
        E("const int lane = threadIdx.x;")
        E(f"const int sub = lane >> {self.LOGP};")
        E(f"const int ul = lane & {self.P - 1};")
        E(f"__shared__ T lds[{self.lds_elems}];")

    def emit_y_load(self, E: Emitter, ptr: str, valid: str) -> None:
        for f in self.used_y:
            E(f"const T y{f} = {valid} ? {ptr}[{f}] : (T)0;")

    # ------------------------------------------------------------- X staging
    def emit_x_stage(self, E: Emitter) -> None:
        """Copy the X rows (or the X chunk) of this tile into LDS.

        Row sources: ``tp`` -> rows row0 .. row0+R-1 (contiguous in memory);
        convolution -> row ``xsrc`` of each sub-row (int, -1 when the sub-row is idle;
        ``xsrc_u`` is its wave-uniform copy when R == 1)."""
        D1, R = self.D1, self.R
        if self.x_chunk_layout:
            E("if (xsrc_u >= 0) {")
            for i in self.used_in1:
                a = self.in1[i]
                E(f"    {{ const T* __restrict__ src = X + (u64)xsrc_u * {D1} + {a.off} + c * {self.P * a.D};")
                E(f"      const int len = {self.chunk_count(a)} * {a.D};")
                E(f"      #pragma unroll")
                E(f"      for (int it = 0; it < {a.D}; ++it) {{ const int q = lane + it * 64; if (q < len) lds[{self.xl[i]} + q] = src[q]; }} }}")
            E("}")
            return
        total = R * D1
        iters = (total + WAVE - 1) // WAVE
        if self.kind == "tp":
            E("{")
            E(f"    const u64 left = n - row0;")
            E(f"    const int avail = (int)(left < {R} ? left : {R}) * {D1};")
            E(f"    const T* __restrict__ src = X + row0 * {D1};")
            E(f"    #pragma unroll")
            E(f"    for (int it = 0; it < {iters}; ++it) {{ const int q = lane + it * 64; if (q < avail) lds[q] = src[q]; }}")
            E("}")
        elif R == 1:
            E("if (xsrc_u >= 0) {")
            E(f"    const T* __restrict__ src = X + (u64)xsrc_u * {D1};")
            E(f"    #pragma unroll")
            E(f"    for (int it = 0; it < {iters}; ++it) {{ const int q = lane + it * 64; if (q < {D1}) lds[q] = src[q]; }}")
            E("}")
        else:
            E(f"#pragma unroll")
            E(f"for (int it = 0; it < {iters}; ++it) {{")
            E(f"    const int q = lane + it * 64;")
            E(f"    const int r = q / {D1};")
            E(f"    const int s = oeq_shfl_i32(xsrc, (r < {R} ? r : 0) << {self.LOGP});")
            E(f"    if (q < {total} && s >= 0) lds[q] = X[(u64)s * {D1} + (q - r * {D1})];")
            E("}")

    def emit_x_regs(self, E: Emitter) -> None:
        for i in self.used_in1:
            a = self.in1[i]
            for m in range(a.D):
                if self.x_chunk_layout:
                    addr = f"{self.xl[i]} + ul * {a.D} + {m}"
                else:
                    addr = f"sub * {self.D1} + {a.off} + u * {a.D} + {m}"
                E(f"const T x{i}_{m} = {self.act(a)} ? lds[{addr}] : (T)0;")

    def emit_weights(self, E: Emitter, p: Path, wptr: str) -> None:
        for v in range(p.mv):
            E(f"const T w{p.t}_{v} = {self.act(p.a)} ? {wptr}[{self.widx(p, 'u', v)}] : (T)0;")

    # --------------------------------------------------------- forward arithmetic
    def emit_forward_block(self, E: Emitter, o: Block, wptr: str, zname: str = "z", declare: bool = True) -> None:
        """z_k (+)= sum over paths into ``o``: w * sum_ij c_ijk x_i y_j."""
        if declare:
            for k in range(o.D):
                E(f"T {zname}{k} = (T)0;")
        for p in self.paths_into(o.idx):
            if p.looped:
                self.emit_forward_looped(E, p, wptr, zname)
                continue
            E(f"{{ // path {p.t}: l = {p.a.l} x {p.b.l} -> {p.o.l}, coefficient {p.coeff:.9g}")
            self.emit_weights(E, p, wptr)
            for v in range(p.mv):
                body, seen = [], []
                for (i, j), ks in p.ordered_pairs():
                    yv = f"y{p.b.off + v * p.b.D + j}"
                    body.append(f"{{ const T t = x{p.a.idx}_{i} * {yv};")
                    for k, val in ks:
                        if k in seen:
                            body.append(f"  p{k} = oeq_fma({self.lit(val)}, t, p{k});")
                        else:
                            body.append(f"  p{k} = {self.lit(val)} * t;")
                            seen.append(k)
                    body.append("}")
                E("{ T " + ", ".join(f"p{k}" for k in sorted(seen)) + ";")
                E.extend("  " + b for b in body)
                for k in sorted(seen):
                    E(f"  {zname}{k} = oeq_fma(w{p.t}_{v}, p{k}, {zname}{k});")
                E("}")
            E("}")

    # ------------------------------------------------- run-time loop over the copies of in2
    def looped_weight(self, p: Path, wptr: str) -> str:
        """Weight (u, v) of a looped path inside its v loop (zero for idle lanes)."""
        return f"({self.act(p.a)} ? {wptr}[{self.widx(p, 'u', 'v')}] : (T)0)"

    def emit_forward_looped(self, E: Emitter, p: Path, wptr: str, zname: str) -> None:
        E(f"// path {p.t}: l = {p.a.l} x {p.b.l} -> {p.o.l}, {p.mv} copies of the second operand walked at run time")
        E(f"for (int v = 0; v < {p.mv}; ++v) {{")
        E.level += 1
        E(f"const T wv = {self.looped_weight(p, wptr)};")
        E(f"const T* __restrict__ yv = Yr + {p.b.off} + v * {p.b.D};")
        for j in sorted({j for (_, j) in p.pairs}):
            E(f"const T yv{j} = yv[{j}];")
        ks_all = sorted({k for ks in p.pairs.values() for (k, _) in ks})
        E("T " + ", ".join(f"p{k} = (T)0" for k in ks_all) + ";")
        seen = ks_all
        for (i, j), ks in p.ordered_pairs():
            E(f"{{ const T t = x{p.a.idx}_{i} * yv{j};")
            for k, val in ks:
                E(f"  p{k} = oeq_fma({self.lit(val)}, t, p{k});")
            E("}")
        for k in sorted(seen):
            E(f"{zname}{k} = oeq_fma(wv, p{k}, {zname}{k});")
        E.level -= 1
        E("}")

    def emit_backward_looped(self, E: Emitter, p: Path, wptr: str, dw_sink) -> None:
        """The v loop of a looped path in the backward: dW per (u, v) goes to ``dw_sink`` with v = "v", dX
        accumulates in registers, and the dY sums of this v (over the lanes of the row) are added to the
        row's LDS accumulator by its writer lane."""
        E(f"// path {p.t}: l = {p.a.l} x {p.b.l} -> {p.o.l}, {p.mv} copies of the second operand walked at run time")
        E("{")
        self._emit_cg_products(E, p)
        E(f"for (int v = 0; v < {p.mv}; ++v) {{")
        E.level += 1
        E(f"const T wv = {self.looped_weight(p, wptr)};")
        E(f"const T* __restrict__ yv = Yr + {p.b.off} + v * {p.b.D};")
        js = sorted({j for (_, j) in p.pairs})
        for j in js:
            E(f"const T yv{j} = yv[{j}]; T dyv{j} = (T)0;")
        self._emit_backward_pairs(E, p, "wv", lambda j: f"yv{j}", lambda j: f"dyv{j}")
        dw_sink(E, p, "v", "dw")
        for j in js:
            if self.P == WAVE:
                E(f"dyv{j} = oeq_wave_sum63(dyv{j});")
            else:
                E(f"dyv{j} = oeq_group_sum<{self.P}>(dyv{j});")
        writer = "lane == 63" if self.P == WAVE else "ul == 0"
        E(f"if ({writer}) {{ T* __restrict__ a_ = ylds + sub * {self.NLY} + {self.looped_y[p.b.off]} + v * {p.b.D}; "
          + " ".join(f"a_[{j}] += dyv{j};" for j in js) + " }")
        E.level -= 1
        E("}")
        E("}")

    def emit_looped_dy_begin(self, E: Emitter) -> None:
        """LDS accumulator of the dY columns of looped blocks: one run of NLY words per row of the wavefront,
        touched by the row's writer lane only."""
        if not self.NLY:
            return
        writer = "lane == 63" if self.P == WAVE else "ul == 0"
        E(f"__shared__ T ylds[{self.R * self.NLY}];")
        E(f"if ({writer}) for (int q = 0; q < {self.NLY}; ++q) ylds[sub * {self.NLY} + q] = (T)0;")

    def looped_dy_value(self, f: int) -> str:
        return f"ylds[sub * {self.NLY} + {self.looped_y[f]}]"

    # -------------------------------------------------------- backward arithmetic
    def emit_backward_block(self, E: Emitter, o: Block, wptr: str, dw_sink) -> None:
        """Given g_k = dZ[o][u, k] (registers g0..), update dx{a}_{i}, dy{f} and hand every
        dW value to ``dw_sink(E, path, v, expr)``.  Formulas: loop_unroll_tp.cuh:167-174 of the
        reference; see ``regroup_pairs`` for the two ways the pairs of a path are evaluated."""
        for p in self.paths_into(o.idx):
            if p.looped:
                self.emit_backward_looped(E, p, wptr, dw_sink)
                continue
            E(f"{{ // path {p.t}: l = {p.a.l} x {p.b.l} -> {p.o.l}")
            self.emit_weights(E, p, wptr)
            self._emit_cg_products(E, p)
            for v in range(p.mv):
                ya = lambda j: f"y{p.b.off + v * p.b.D + j}"
                E("{")
                self._emit_backward_pairs(E, p, f"w{p.t}_{v}", ya, lambda j: f"dy{p.b.off + v * p.b.D + j}")
                dw_sink(E, p, v, "dw")
                E("}")
            E("}")

    def _cg_key(self, k: int, val: float):
        return (k, float(np.float64(abs(val)).round(12)))

    def _emit_cg_products(self, E: Emitter, p: Path) -> None:
        """c * g_k for the pairs of ``p`` with a single output component, once per distinct (k, |c|)."""
        self._cg_names = {}
        if not self.regroup_pairs:
            return
        for (i, j), ks in p.ordered_pairs():
            if len(ks) == 1:
                key = self._cg_key(*ks[0])
                if key not in self._cg_names:
                    self._cg_names[key] = f"cg{len(self._cg_names)}"
                    E(f"  const T {self._cg_names[key]} = {self.lit(abs(ks[0][1]))} * g{ks[0][0]};")

    def _emit_backward_pairs(self, E: Emitter, p: Path, w: str, ya, dya) -> None:
        """The (i, j) pairs of one copy of the second operand: declares and fills ``dw``, updates dx and dy."""
        if not self.regroup_pairs:
            # every pair on its own: dw += s x_i y_j, dx_i += s (w y_j), dy_j += s (w x_i)
            js = sorted({j for (_, j) in p.pairs})
            is_ = sorted({i for (i, _) in p.pairs})
            for j in js:
                E(f"  const T wy{j} = {w} * {ya(j)};")
            for i in is_:
                E(f"  const T wx{i} = {w} * x{p.a.idx}_{i};")
            E("  T dw = (T)0;")
            for (i, j), ks in p.ordered_pairs():
                E("  {")
                for n_, (k, val) in enumerate(ks):
                    E(f"    T s = {self.lit(val)} * g{k};" if n_ == 0 else f"    s = oeq_fma({self.lit(val)}, g{k}, s);")
                E(f"    dw = oeq_fma(s, x{p.a.idx}_{i} * {ya(j)}, dw);")
                E(f"    dx{p.a.idx}_{i} = oeq_fma(s, wy{j}, dx{p.a.idx}_{i});")
                E(f"    {dya(j)} = oeq_fma(s, wx{i}, {dya(j)});")
                E("  }")
            return
        # one component i of the first operand after the other, t_i = sum_j s_ij y_j
        by_i = {}
        for (i, j), ks in sorted(p.pairs.items()):
            by_i.setdefault(i, []).append((j, ks))
        E("  T dw = (T)0;")
        for i, lst in sorted(by_i.items()):
            E("  {")
            E(f"    const T wx = {w} * x{p.a.idx}_{i};")
            E("    T t;")
            for n_, (j, ks) in enumerate(lst):
                shared = len(ks) == 1
                if shared:
                    s = ("-" if ks[0][1] < 0 else "") + self._cg_names[self._cg_key(*ks[0])]
                else:
                    E("    {")
                    for m_, (k, val) in enumerate(ks):
                        E(f"      T s = {self.lit(val)} * g{k};" if m_ == 0 else f"      s = oeq_fma({self.lit(val)}, g{k}, s);")
                    s = "s"
                E(f"      t = {s} * {ya(j)};" if n_ == 0 else f"      t = oeq_fma({s}, {ya(j)}, t);")
                E(f"      {dya(j)} = oeq_fma({s}, wx, {dya(j)});")
                if not shared:
                    E("    }")
            E(f"    dw = oeq_fma(x{p.a.idx}_{i}, t, dw);")
            E(f"    dx{p.a.idx}_{i} = oeq_fma({w}, t, dx{p.a.idx}_{i});")
            E("  }")

    # --------------------------------------------------------------- LDS slots
    def emit_slot_write(self, E: Emitter, blk: Block, name: str, act: str) -> None:
        """registers name0.. -> lds[ZB + lane*D + k]."""
        E("oeq_sync();")
        E(f"if ({act}) {{ " + " ".join(f"lds[{self.ZB} + lane * {blk.D} + {k}] = {name}{k};" for k in range(blk.D)) + " }")
        E("oeq_sync();")

    def emit_slot_read(self, E: Emitter, blk: Block, name: str, act: str) -> None:
        for k in range(blk.D):
            E(f"const T {name}{k} = {act} ? lds[{self.ZB} + lane * {blk.D} + {k}] : (T)0;")

    def emit_slot_to_global(self, E: Emitter, blk: Block, ptr: str, rowdim: int, row_of, op: str = "store",
                            zero: bool = False) -> None:
        """Copy the slot of block ``blk`` (chunk c) from LDS to rows of ``ptr`` (row length
        ``rowdim``).  ``row_of(r)`` -> (row expression, validity expression) for sub-row r;
        op is "store" or "atomic".  With ``zero`` the slot is not read: zeros are stored."""
        D, P, R = blk.D, self.P, self.R
        val = lambda e: "(T)0" if zero else e

        def put(dst: str, v: str) -> str:
            return f"oeq_atomic_add(&{dst}, {v});" if op == "atomic" else f"{dst} = {v};"
        if R == 1:
            row, ok = row_of("0")
            cnt = self.chunk_count(blk)
            E(f"if ({ok}) {{")
            E(f"    T* __restrict__ dst = {ptr} + (u64){row} * {rowdim} + {blk.off} + c * {P * D};")
            E(f"    const int len = {cnt} * {D};")
            E(f"    #pragma unroll")
            E(f"    for (int it = 0; it < {D}; ++it) {{ const int q = lane + it * 64; if (q < len) {{ {put('dst[q]', val(f'lds[{self.ZB} + q]'))} }} }}")
            E("}")
        else:
            L = blk.mul * D                      # NCH == 1 here
            total = R * L
            iters = (total + WAVE - 1) // WAVE
            row, ok = row_of("rr")
            E(f"#pragma unroll")
            E(f"for (int it = 0; it < {iters}; ++it) {{")
            E(f"    const int q = lane + it * 64;")
            E(f"    const int r = q / {L};")
            E(f"    const int rr = r < {R} ? r : 0;")
            E(f"    const int qq = q - r * {L};")
            E(f"    const i64 grow = (i64){row};")
            E(f"    const bool ok = {ok};")
            E(f"    if (q < {total} && ok) {{ {put(f'{ptr}[(u64)grow * {rowdim} + {blk.off} + qq]', val(f'lds[{self.ZB} + rr * {P * D} + qq]'))} }}")
            E("}")

    def emit_global_to_slot(self, E: Emitter, blk: Block, ptr: str, rowdim: int, row_of) -> None:
        """Inverse of emit_slot_to_global (plain loads)."""
        D, P, R = blk.D, self.P, self.R
        E("oeq_sync();")
        if R == 1:
            row, ok = row_of("0")
            cnt = self.chunk_count(blk)
            E(f"if ({ok}) {{")
            E(f"    const T* __restrict__ src = {ptr} + (u64){row} * {rowdim} + {blk.off} + c * {P * D};")
            E(f"    const int len = {cnt} * {D};")
            E(f"    #pragma unroll")
            E(f"    for (int it = 0; it < {D}; ++it) {{ const int q = lane + it * 64; if (q < len) lds[{self.ZB} + q] = src[q]; }}")
            E("}")
        else:
            L = blk.mul * D
            total = R * L
            iters = (total + WAVE - 1) // WAVE
            row, ok = row_of("rr")
            E(f"#pragma unroll")
            E(f"for (int it = 0; it < {iters}; ++it) {{")
            E(f"    const int q = lane + it * 64;")
            E(f"    const int r = q / {L};")
            E(f"    const int rr = r < {R} ? r : 0;")
            E(f"    const int qq = q - r * {L};")
            E(f"    const i64 grow = (i64){row};")
            E(f"    const bool ok = {ok};")
            E(f"    if (q < {total} && ok) lds[{self.ZB} + rr * {P * D} + qq] = {ptr}[(u64)grow * {rowdim} + {blk.off} + qq];")
            E("}")
        E("oeq_sync();")

    # block output: registers -> global, choosing the direct path for l = 0
    def emit_block_out(self, E: Emitter, blk: Block, name: str, ptr: str, rowdim: int, own_row: Tuple[str, str],
                       row_of, op: str = "store") -> None:
        act = self.act(blk)
        if blk.D == 1:
            row, ok = own_row
            dst = f"{ptr}[(u64){row} * {rowdim} + {blk.off} + u]"
            stmt = f"oeq_atomic_add(&{dst}, {name}0);" if op == "atomic" else f"{dst} = {name}0;"
            E(f"if ({act} && {ok}) {{ {stmt} }}")
        else:
            self.emit_slot_write(E, blk, name, act)
            self.emit_slot_to_global(E, blk, ptr, rowdim, row_of, op)

    def emit_block_in(self, E: Emitter, blk: Block, name: str, ptr: str, rowdim: int, own_row: Tuple[str, str],
                      row_of) -> None:
        act = self.act(blk)
        if blk.D == 1:
            row, ok = own_row
            E(f"const T {name}0 = ({act} && {ok}) ? {ptr}[(u64){row} * {rowdim} + {blk.off} + u] : (T)0;")
        else:
            self.emit_global_to_slot(E, blk, ptr, rowdim, row_of)
            self.emit_slot_read(E, blk, name, act)

    def emit_block_zero(self, E: Emitter, blk: Block, ptr: str, rowdim: int, own_row, row_of) -> None:
        """Store zeros over chunk c of a block nothing contributes to."""
        if blk.D == 1:
            row, ok = own_row
            E(f"if ({self.act(blk)} && {ok}) {ptr}[(u64){row} * {rowdim} + {blk.off} + u] = (T)0;")
        else:
            self.emit_slot_to_global(E, blk, ptr, rowdim, row_of, zero=True)

    # ------------------------------------------------------------- dY reduction
    def emit_dy_reduce(self, E: Emitter) -> None:
        """Sum of dy* over the P lanes of each sub-row (fixed order -> deterministic): DPP row
        operations for groups of up to 32 lanes, a shuffle butterfly for a full wavefront."""
        if self.P <= 32:
            for f in self.used_y:
                E(f"dy{f} = oeq_group_sum<{self.P}>(dy{f});")
            return
        m = self.P // 2
        while m >= 1:
            for f in self.used_y:
                E(f"dy{f} += oeq_shfl_xor(dy{f}, {m});")
            m //= 2

    # ------------------------------------------------------------ chunk loops
    def chunk_loop(self, E: Emitter, body) -> None:
        """Run ``body(E)`` once per chunk with ``c`` and ``u`` defined."""
        if self.chunk_in_grid:
            E("{")
            E.level += 1
            E("const int c = blockIdx.y;")
            E(f"const int u = c * {self.P} + ul;")
            body(E)
            E.level -= 1
            E("}")
        elif self.NCH == 1:
            E("{")
            E.level += 1
            E("const int c = 0;")
            E("const int u = ul;")
            body(E)
            E.level -= 1
            E("}")
        else:
            E("#pragma unroll" if self.unroll_chunks else "#pragma unroll 1")
            E(f"for (int c = 0; c < {self.NCH}; ++c) {{")
            E.level += 1
            E(f"const int u = c * {self.P} + ul;")
            body(E)
            E.level -= 1
            E("}")

    # =================================================================== batch TP
    def tp_forward_body(self) -> str:
        E = Emitter()
        self.emit_lane(E)
        R = self.R
        ntiles = f"(n + {R - 1}) / {R}"
        E(f"for (u64 tile = blockIdx.x; tile < {ntiles}; tile += gridDim.x) {{")
        E.level += 1
        E(f"const u64 row0 = tile * {R};")
        E("const u64 row = row0 + sub;")
        E("const bool rv = row < n;")
        E(f"const T* __restrict__ Yr = Y + (rv ? row : 0) * {self.D2};")
        E("const T* __restrict__ Wr = W" + ("" if self.shared else f" + row * {self.WN}") + ";")
        self.emit_y_load(E, "Yr", "rv")
        E("oeq_sync();")
        self.emit_x_stage(E)
        E("oeq_sync();")
        own = ("row", "rv")
        row_of = lambda r: (f"(row0 + {r})", f"(row0 + {r} < n)")

        def body(E):
            self.emit_x_regs(E)
            for o in self.out:
                E("{")
                E.level += 1
                if o.idx in self.used_out:
                    self.emit_forward_block(E, o, "Wr")
                    self.emit_block_out(E, o, "z", "Z", self.D3, own, row_of)
                elif o.dim > 0:
                    if o.D > 1:
                        E("oeq_sync();")
                    self.emit_block_zero(E, o, "Z", self.D3, own, row_of)
                E.level -= 1
                E("}")
        self.chunk_loop(E, body)
        E.level -= 1
        E("}")
        return E.text()

    def tp_backward_body(self) -> str:
        E = Emitter()
        self.emit_lane(E)
        R = self.R
        ntiles = f"(n + {R - 1}) / {R}"
        if self.shared:
            # per-workgroup dW partial sums live in registers across the tile loop; those of looped paths
            # (one value per copy of the second operand) are accumulated in the workgroup's partial row itself
            E(f"T* __restrict__ part = (T*)ws + (u64)blockIdx.x * {self.WN};")
            for p in self.paths:
                for c in range(self.NCH):
                    if p.looped:
                        E(f"{{ const int u = {c * self.P} + ul; if (sub == 0 && u < {p.mu}) "
                          f"for (int v = 0; v < {p.mv}; ++v) part[{self.widx(p, 'u', 'v')}] = (T)0; }}")
                        continue
                    for v in range(p.mv):
                        E(f"T dws{p.t}_{c}_{v} = (T)0;")
        if self.NLY:
            E(f"__shared__ T ylds[{self.R * self.NLY}];")
        E(f"for (u64 tile = blockIdx.x; tile < {ntiles}; tile += gridDim.x) {{")
        E.level += 1
        E(f"const u64 row0 = tile * {R};")
        E("const u64 row = row0 + sub;")
        E("const bool rv = row < n;")
        E(f"const T* __restrict__ Yr = Y + (rv ? row : 0) * {self.D2};")
        E("const T* __restrict__ Wr = W" + ("" if self.shared else f" + row * {self.WN}") + ";")
        if not self.shared:
            E(f"T* __restrict__ Wgr = Wg + row * {self.WN};")
        self.emit_y_load(E, "Yr", "rv")
        for f in self.used_y:
            E(f"T dy{f} = (T)0;")
        if self.NLY:
            E(f"if (ul == 0) for (int q = 0; q < {self.NLY}; ++q) ylds[sub * {self.NLY} + q] = (T)0;")
        E("oeq_sync();")
        self.emit_x_stage(E)
        E("oeq_sync();")
        own = ("row", "rv")
        row_of = lambda r: (f"(row0 + {r})", f"(row0 + {r} < n)")

        def body(E, cconst=None):
            self.emit_x_regs(E)
            for i in self.used_in1:
                for m in range(self.in1[i].D):
                    E(f"T dx{i}_{m} = (T)0;")
            for oi in self.used_out:
                o = self.out[oi]
                E("{")
                E.level += 1
                self.emit_block_in(E, o, "g", "G", self.D3, own, row_of)

                def sink(E, p, v, expr):
                    if self.shared and p.looped:
                        # rows of the same wavefront hold separate sums for the same (u, v): fold them, then the
                        # first row's lane adds to the workgroup's partial row (its own words: no other lane touches them)
                        m = 32
                        while m >= self.P:
                            E(f"{expr} += oeq_shfl_xor({expr}, {m});")
                            m //= 2
                        E(f"if (sub == 0 && u < {p.mu}) part[{self.widx(p, 'u', v)}] += {expr};")
                    elif self.shared:
                        if self.NCH == 1:
                            E(f"  dws{p.t}_0_{v} += {expr};")
                        else:
                            for c in range(self.NCH):
                                E(f"  if (c == {c}) dws{p.t}_{c}_{v} += {expr};")
                    else:
                        E(f"  if ({self.act(p.a)}) Wgr[{self.widx(p, 'u', v)}] = {expr};")
                self.emit_backward_block(E, o, "Wr", sink)
                E.level -= 1
                E("}")
            for a in self.in1:
                if a.dim == 0:
                    continue
                E("{")
                E.level += 1
                if a.idx in self.used_in1:
                    self.emit_block_out(E, a, f"dx{a.idx}_", "Xg", self.D1, own, row_of)
                else:
                    if a.D > 1:
                        E("oeq_sync();")
                    self.emit_block_zero(E, a, "Xg", self.D1, own, row_of)
                E.level -= 1
                E("}")
        self.chunk_loop(E, body)
        # dY: reduce over the lanes of the row, lane 0 of each sub-row stores
        self.emit_dy_reduce(E)
        E("if (rv && ul == 0) {")
        E(f"    T* __restrict__ Ygr = Yg + row * {self.D2};")
        for f in range(self.D2):
            E(f"    Ygr[{f}] = " + (f"dy{f};" if f in self.used_y else
                                   f"{self.looped_dy_value(f)};" if f in self.looped_y else "(T)0;"))
        E("}")
        E.level -= 1
        E("}")
        if self.shared:
            for p in self.paths:
                if p.looped:
                    continue
                for c in range(self.NCH):
                    for v in range(p.mv):
                        E(f"{{ const int u = {c * self.P} + ul;")
                        # rows of the same wavefront (R > 1) hold separate partial sums: fold them
                        m = 32
                        while m >= self.P:
                            E(f"  dws{p.t}_{c}_{v} += oeq_shfl_xor(dws{p.t}_{c}_{v}, {m});")
                            m //= 2
                        E(f"  if (sub == 0 && u < {p.mu}) part[{self.widx(p, 'u', v)}] = dws{p.t}_{c}_{v}; }}")
        return E.text()

    # ------------------------------------------------ row indices shared inside a wavefront
    def _shfl_row(self, var: str):
        if self.R == 1:
            return lambda r: (f"{var}_u", f"({var}_u >= 0)")
        return lambda r: (f"oeq_shfl_i32({var}, ({r}) << {self.LOGP})", f"(oeq_shfl_i32({var}, ({r}) << {self.LOGP}) >= 0)")

    def render(self, prelude: str = None) -> str:
        env = jinja_env()
        if prelude is None:
            prelude = env.get_template("prelude.hip.jinja").render(T=self.T)
        tmpl = env.get_template({"tp": "tp_uvu.hip.jinja", "conv_atomic": "conv_atomic.hip.jinja",
                                 "conv_det": "conv_det.hip.jinja"}[self.kind])
        return tmpl.render(g=self, prelude=prelude)

    def describe(self) -> str:
        return (f"uvu[{self.kind}] T={self.T} P={self.P} R={self.R} chunks={self.NCH} paths={len(self.paths)} "
                f"nnz={sum(p.nnz for p in self.paths)} d1={self.D1} d2={self.D2} d3={self.D3} wn={self.WN} "
                f"lds={self.lds_elems * self.itemsize}B")

    # -------------------------------------------------------------- launch plan
    @property
    def dy_rows_per_block(self) -> int:
        return max(1, 256 // max(1, self.D2))

    def plan(self):
        """(forward steps, backward steps, workspace sizing) as plain dictionaries; the
        frontends turn them into ``runtime.Step`` records.  ``workspace`` is a function
        ``(nnz, node_count) -> bytes`` (0 when no workspace is needed)."""
        ROW, NODE, FIXED = 1, 2, 0
        w = 64
        if self.kind == "tp":
            fwd = [dict(kernel="forward", num_threads=w, grid_kind=ROW, work_per_block=self.R)]
            if self.shared:
                bwd = [dict(kernel="backward", num_threads=w, grid_kind=FIXED, num_blocks=self.dw_partials),
                       dict(kernel="backward_reduce", num_threads=256, grid_kind=FIXED,
                            num_blocks=(self.WN + 255) // 256)]
                ws = lambda nnz=0, nodes=0: self.dw_partials * self.WN * self.itemsize
            else:
                bwd = [dict(kernel="backward", num_threads=w, grid_kind=ROW, work_per_block=self.R)]
                ws = lambda nnz=0, nodes=0: 0
            return fwd, bwd, ws
        if self.kind == "conv_atomic":
            fwd = [dict(kernel="forward", num_threads=w, grid_kind=ROW, work_per_block=self.R)]
            bwd = [dict(kernel="backward", num_threads=w, grid_kind=ROW, work_per_block=self.R)]
            return fwd, bwd, (lambda nnz=0, nodes=0: 0)
        fwd = [dict(kernel="prep_forward", num_threads=256, grid_kind=ROW, work_per_block=256, prep=True),
               dict(kernel="forward", num_threads=w, grid_kind=NODE, work_per_block=self.R, grid_y=self.NCH)]
        bwd = [dict(kernel="prep_backward", num_threads=256, grid_kind=ROW, work_per_block=256, prep=True),
               dict(kernel="backward", num_threads=w, grid_kind=NODE, work_per_block=self.R, grid_y=self.NCH)]
        if self.NCH > 1:
            bwd.append(dict(kernel="backward_dy_reduce", num_threads=256, grid_kind=ROW,
                            work_per_block=self.dy_rows_per_block))

        def ws(nnz=0, nodes=0):
            b = 2 * (nodes + 1) * 8
            if self.NCH > 1:
                b += self.NCH * nnz * self.D2 * self.itemsize
            return b
        return fwd, bwd, ws
