"""Generator of gfx950 HIP source for dense ("uvw") tensor products with shared weights.

    Z[b, w, k] = sum_t sum_u  W_t[u, w] * T_t[b, u, k],    T_t[b, u, k] = c_t sum_ij C_ijk x[b, u, i] y[b, j]

is a genuine dense contraction over the multiplicity ``u`` and runs on the matrix cores:
``v_mfma_f32_16x16x4_f32`` / ``v_mfma_f64_16x16x4_f64`` (one 16x16 accumulator tile, K = 4 per
instruction), with the sparse Clebsch-Gordan part evaluated on the vector ALU directly into
MFMA operand registers (reference: the register-tiled CUDA-core matmul of
openequivariance/templates/wmm.cuh:1-88 called from loop_unroll_tp.cuh:74-78, :184, :209).

Tiling (lane = 16 * g + c, g = lane / 16, c = lane % 16; a batch tile is 16 rows):

* forward, one wavefront per (tile, output block):  A[i=c][k=g] = T[b=c, u] (VALU),  B[k=g][j=c] = W[u][w]
  from a pre-packed copy of W, accumulators = the 16 x mul_out tile of the output block; each lane
  ends up with contiguous runs of Z, so Z is stored with vector stores straight from registers.
* backward dX/dY, four wavefronts per tile (one 16-channel u-subtile each):
  dT^T[u, b] = sum_w W[u][w] dZ[b][w]:  A = W (pre-packed), B = the 16-row dZ tile, staged in LDS once per
  workgroup when it fits; then the CG transpose on the VALU accumulates dX (registers) and dY.
* backward dW, four or eight wavefronts per workgroup, persistent over batch tiles:
  dW[u, w] = sum_{b,k} T[b,u,k] dZ[b,w,k]:  A = T (VALU), B = dZ, accumulators = this wavefront's
  u-subtile of the paths of one pass; per-workgroup partial sums go to the workspace and a last kernel adds
  them in workgroup order (reproducible; no floating-point atomics).

X records, packed weights and (forward, dW) dZ are per-lane records of the ``mul x irrep`` layout, loaded
straight from global memory / L2.

Scope of this generator: shared weights.  A second operand with several copies per irrep (mul(in2) > 1)
is handled as one contraction over u per copy v, with the slice W[:, v, :] of the weights; the
benchmarks and MACE/NequIP-style models use a single copy.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Tuple

import numpy as np

from ..problem import TPProblem
from ..wigner import wigner_3j
from .common import Emitter, jinja_env, literal
from .uvu import Block, _blocks


def _ceil(a: int, b: int) -> int:
    return (a + b - 1) // b


@dataclass
class WPath:
    t: int
    a: Block
    b: Block
    o: Block
    coeff: float
    woff: int                       # offset of this path's weights in the external vector
    pairs: Dict[Tuple[int, int], List[Tuple[int, float]]] = field(default_factory=dict)
    wb: int = 0                     # offset (elements) of the forward-packed copy
    wa: int = 0                     # offset of the backward-packed copy
    v: int = 0                      # which copy of the second operand this path contracts with ...
    mv: int = 1                     # ... out of this many (the instruction's weights are [u][v][w])
    poff: int = 0                   # offset of this path's [u][w] slice in the dense dW partial rows

    @property
    def mu(self) -> int:
        return self.a.mul

    @property
    def mw(self) -> int:
        return self.o.mul

    @property
    def SU(self) -> int:            # K steps over u (forward): whole blocks of 16 channels, 4 steps each
        return 4 * _ceil(self.mu, 16)

    @property
    def SW(self) -> int:            # K steps over w (backward dX)
        return _ceil(self.mw, 4)

    @property
    def NTU(self) -> int:           # 16-wide tiles over u
        return _ceil(self.mu, 16)

    @property
    def NTW(self) -> int:           # 16-wide tiles over w
        return _ceil(self.mw, 16)

    def ordered_pairs(self):
        return sorted(self.pairs.items(), key=lambda kv: (kv[0][1], kv[0][0]))


class UVWGenerator:
    DW_WORKGROUPS = 256          # persistent dW workgroups: one per compute unit of an MI355X
    # Accumulator registers of one forward work item; an output block needing more is cut into ranges of its
    # w tiles.  (48 instead of 80, for a third wavefront per SIMD, measured slower on 64x0e+64x1o+64x2e: fp32
    # 0.329 -> 0.376 ms, fp64 0.566 -> 0.694 ms - the CG part of a tile is then computed once per range.)
    FWD_ACC_LIMIT = 80

    def __init__(self, problem: TPProblem):
        self.problem = problem
        self.kind = "uvw"
        self.T = {np.float32: "float", np.float64: "double"}[problem.irrep_dtype]
        self.itemsize = 4 if self.T == "float" else 8
        self.shared = bool(problem.shared_weights)
        if not self.shared and not getattr(self, "_allow_batched", False):
            raise NotImplementedError("this generator handles shared weights; see uvw_batched.py for per-row weights")
        # forward K loop: steps fetched per batch of loads, and unroll factor of the batch loop (measured on
        # MI355X: fp32 4 / 1, fp64 1 / 3; a loop written out on alternating register sets, so that nothing is
        # copied between sets, has 0.9 instead of 2.1 vector-ALU instructions per MFMA and measured 0.341
        # against 0.331 ms; larger groups for the cheap work items 0.361 - 0.422 against 0.359 ms)
        self.fwd_group, self.fwd_unroll = (4, 1) if self.T == "float" else (1, 3)
        # Tile shape: 16 x 16 x 4 in both types.  The fp32 forward on v_mfma_f32_32x32x2_f32 (32 batch rows per
        # tile, half the weight-operand loads per FLOP) passed the same parity tests and measured 0.371 ms (w
        # ranges of at most 96 accumulator registers, two wavefronts per SIMD) and 0.374 ms (whole output
        # blocks, 160 accumulators, one wavefront) against 0.318 ms: the CG vector-ALU work per FLOP is the
        # same in both shapes (one product per row and channel, used for all 64 w), a lane's X loads cover 8
        # instead of 16 channels of a row per group (twice the cache lines per load instruction: texture
        # addresser busy 50 % instead of 47 %, matrix core busy 51 % instead of 60 % of the kernel's cycles),
        # and the accumulators of a 32-row tile leave no room for the operands of the next group.
        # backward dW: fetch the operands of the next step while the current one runs (two register sets);
        # in fp64 the second set crosses the 512-register limit even per pass (1.31 against 1.22 ms)
        self.dw_prefetch = self.T == "float"
        self.in1, self.in2, self.out = _blocks(problem.irreps_in1), _blocks(problem.irreps_in2), _blocks(problem.irreps_out)
        self.D1, self.D2, self.D3 = problem.irreps_in1.dim, problem.irreps_in2.dim, problem.irreps_out.dim
        self.WN = problem.weight_numel
        self.paths: List[WPath] = []
        woff = 0
        for t, ins in enumerate(problem.instructions):
            if ins.connection_mode != "uvw":
                raise ValueError("UVWGenerator handles uvw instructions only")
            if not ins.has_weight:
                raise NotImplementedError("instructions without weights are not supported")
            a, b, o = self.in1[ins.i_in1], self.in2[ins.i_in2], self.out[ins.i_out]
            c = wigner_3j(a.l, b.l, o.l) * ins.path_weight
            # An instruction whose second operand has mv copies is mv contractions over u, one per copy v,
            # each with the slice W[:, v, :] of the instruction's weights and the v-th record of the Y block:
            # it is emitted as mv paths over single-copy blocks (reference: loop_unroll_tp.cuh:48-60 walks v)
            for v in range(b.mul):
                bv = Block(b.idx, 1, b.l, b.off + v * b.D)
                p = WPath(len(self.paths), a, bv, o, ins.path_weight, woff, v=v, mv=b.mul, poff=woff + v * a.mul * o.mul)
                for i, j, k in np.argwhere(np.abs(c) > 1e-14):
                    p.pairs.setdefault((int(i), int(j)), []).append((int(k), float(c[i, j, k])))
                self.paths.append(p)
            woff += a.mul * b.mul * o.mul
        if not self.paths:
            raise ValueError("Tensor product problem has no valid instructions!")
        self.used_in1 = sorted({p.a.idx for p in self.paths})
        self.used_out = sorted({p.o.idx for p in self.paths})
        self.used_y = sorted({p.b.off + j for p in self.paths for (_, j) in p.pairs})
        cost = lambda o: sum(p.o.D * p.NTW * p.SU for p in self.paths if p.o.idx == o.idx)
        # forward work items: (output block, range of its 16-wide w tiles), most expensive first.  A block
        # whose accumulator tile (D * tiles * 4 registers) exceeds FWD_ACC_LIMIT is cut into w ranges, each
        # a work item of its own: fewer accumulators per wavefront buy a third wavefront per SIMD, which
        # hides one wavefront's vector-ALU phases behind another's matrix-core phases
        limit = self.FWD_ACC_LIMIT
        self.fwd_order = []
        for o in sorted([o for o in self.out if o.dim > 0], key=lambda o: -cost(o)):
            nt_all = _ceil(o.mul, 16)
            parts = 1
            if o.idx in self.used_out:
                while 4 * o.D * _ceil(nt_all, parts) > limit and parts < nt_all:
                    parts += 1
            step = _ceil(nt_all, parts)
            for lo in range(0, nt_all, step):
                self.fwd_order.append((o, lo, min(nt_all, lo + step)))
        seg_cost = lambda it: cost(it[0]) * (it[2] - it[1]) / _ceil(it[0].mul, 16)
        self.fwd_order.sort(key=lambda it: -seg_cost(it))
        # Work items of a tile: one segment each.  (Packing the three segments of 64x0e+64x1o+64x2e into two
        # items of similar length, work 20 : 15 instead of 20 : 12 : 3, measured fp32 353 against 350 us and
        # fp64 670 against 604 us.)
        self.fwd_items = [[i] for i in range(len(self.fwd_order))]
        # dW kernel: output blocks split into two groups of similar MFMA work
        # (f64 accumulators are twice as wide: one group, four wavefronts, the whole register file)
        work = {o: sum(p.o.D * p.NTW * p.NTU for p in self.paths if p.o.idx == o) for o in self.used_out}
        self.dw_groups = 2 if (self.T == "float" and len(work) > 1) else 1
        self.dw_group, load = {}, [0, 0]
        for o in sorted(work, key=lambda k: -work[k]):
            gsel = 0 if (load[0] <= load[1] or self.dw_groups == 1) else 1
            self.dw_group[o] = gsel
            load[gsel] += work[o]
        # backward dX/dY: the 16-row dZ tile is staged in LDS when it fits (row stride padded against bank
        # conflicts of the B-operand reads: lanes c = 0..15 read 16 different rows at the same column)
        self.bwd_rs = self._pick_row_stride()
        self.bwd_lds = 16 * self.bwd_rs * self.itemsize <= 80 * 1024    # gfx950: 160 KB per CU
        # packed weight copies in the workspace
        pos = 0
        for p in self.paths:
            p.wb = pos
            pos += p.SU * 64 * p.NTW
        self.WB_SIZE = pos
        # backward copy: [u-subtile][group of VW steps][lane][VW], so that one 16-byte load per lane
        # is a contiguous 1 KB access of the wavefront
        self.VW = 16 // self.itemsize
        for p in self.paths:
            p.wa = pos
            pos += p.NTU * _ceil(p.SW, self.VW) * 64 * self.VW
        self.WA_END = pos
        self.PART_OFF = _ceil(pos, 64) * 64
        self.ws_elems = self.PART_OFF + self.DW_WORKGROUPS * self.WN

    # ------------------------------------------------------------------ helpers
    def forward_attr(self) -> str:
        """fp32: two wavefronts per SIMD (256 registers each) - the operands of the next group, of this path or
        the next, need the room; fp64 accumulators are twice as wide and take what a single wavefront gets."""
        return " __attribute__((amdgpu_waves_per_eu(2, 2)))" if self.T == "float" else ""

    def backward_attr(self) -> str:
        """Occupancy target of the dX/dY kernel: as many workgroups per CU (one wavefront per SIMD
        each) as the LDS tile allows; the register allocator then stays within that budget."""
        if not self.bwd_lds:
            return ""
        per_cu = max(1, min(4, (160 * 1024) // (16 * self.bwd_rs * self.itemsize + 4 * 16 * max(1, self.D2) * self.itemsize)))
        return f" __attribute__((amdgpu_waves_per_eu({per_cu}, {per_cu})))" if per_cu >= 3 else ""

    def _pick_row_stride(self) -> int:
        """Row stride (elements) of the dZ tile in LDS: the smallest padding for which the 32 lanes of
        one LDS pass (16 rows x 2 adjacent records) spread best over the 32 four-byte banks."""
        words = self.itemsize // 4
        best = None
        for pad in range(0, 33):
            rs = self.D3 + pad
            worst = 0
            for d in {o.D for o in self.out if o.dim}:
                hits = {}
                for c in range(16):
                    for g in range(2):
                        bank = ((c * rs + g * d) * words) % 32
                        hits[bank] = hits.get(bank, 0) + 1
                worst = max(worst, max(hits.values()))
            if best is None or worst < best[0]:
                best = (worst, rs)
            if worst == 1:
                break
        return best[1]

    def lit(self, v: float) -> str:
        return literal(v, self.T)

    def row(self, r: int) -> str:
        """Row of accumulator element r held by this lane (differs between the f32 and f64 MFMA)."""
        return f"(4 * g + {r})" if self.T == "float" else f"({4 * r} + g)"

    def paths_into(self, o: int) -> List[WPath]:
        return [p for p in self.paths if p.o.idx == o]

    def paths_from(self, a: int) -> List[WPath]:
        return [p for p in self.paths if p.a.idx == a]

    def oeq_index(self, p: WPath, u: str, w: str) -> str:
        """Position of W_t[u, v, w] (v = the path's copy of the second operand) in the external (oeq)
        weight vector: chunks of 32 enumerated (u-chunk, v-chunk, w-chunk), each stored
        [v_local][u_local][w_local] (weight_order.py)."""
        mu, mv, mw = p.mu, p.mv, p.mw
        vc, vl = divmod(p.v, 32)
        vlw = min(32, mv - 32 * vc)
        if mu <= 32 and mw <= 32:
            return f"{p.woff + 32 * vc * mu * mw + vl * mu * mw} + ({u}) * {mw} + ({w})"
        ul = "32" if mu % 32 == 0 else f"min(32, {mu} - (({u}) >> 5) * 32)"
        wl = "32" if mw % 32 == 0 else f"min(32, {mw} - (({w}) >> 5) * 32)"
        return (f"{p.woff} + (({u}) >> 5) * {32 * mv * mw} + {ul} * ({32 * vc * mw} + {vlw} * ((({w}) >> 5) * 32) + {vl} * {wl})"
                f" + (({u}) & 31) * {wl} + (({w}) & 31)")

    def emit_cg_forward(self, E: Emitter, p: WPath, x: str, y: str, out: str) -> None:
        """out{k} = sum_ij c_ijk {x}{i} * {y}{off+j}  (declares out0..)."""
        body, seen = [], []
        for (i, j), ks in p.ordered_pairs():
            body.append(f"{{ const T t_ = {x}{i} * {y}{p.b.off + j};")
            for k, val in ks:
                if k in seen:
                    body.append(f"  {out}{k} = oeq_fma({self.lit(val)}, t_, {out}{k});")
                else:
                    body.append(f"  {out}{k} = {self.lit(val)} * t_;")
                    seen.append(k)
            body.append("}")
        E("T " + ", ".join(f"{out}{k}" + ("" if k in seen else " = (T)0") for k in range(p.o.D)) + ";")
        E.extend(body)

    def emit_cg_matrix(self, E: Emitter, p: WPath, y: str, m: str) -> None:
        """{m}{i}_{k} = sum_j c_ijk {y}{off+j}: the CG tensor contracted with this row's second operand.
        It depends on the batch row only, so one evaluation serves every channel of the row."""
        terms = {}
        for (i, j), ks in p.ordered_pairs():
            for k, val in ks:
                terms.setdefault((i, k), []).append((j, val))
        for (i, k), lst in sorted(terms.items()):
            expr = " + ".join(f"{self.lit(val)} * {y}{p.b.off + j}" for j, val in lst)
            E(f"const T {m}{i}_{k} = {expr};")

    def emit_cg_apply(self, E: Emitter, p: WPath, x: str, m: str, out: str) -> None:
        """out{k} = sum_i {m}{i}_{k} * {x}{i}  (declares out0..)."""
        by_k = {}
        for (i, j), ks in p.ordered_pairs():
            for k, _ in ks:
                by_k.setdefault(k, set()).add(i)
        for k in range(p.o.D):
            if k not in by_k:
                E(f"T {out}{k} = (T)0;")
                continue
            idx = sorted(by_k[k])
            expr = f"{m}{idx[0]}_{k} * {x}{idx[0]}"
            for i in idx[1:]:
                expr = f"oeq_fma({m}{i}_{k}, {x}{i}, {expr})"
            E(f"T {out}{k} = {expr};")

    def emit_cg_backward(self, E: Emitter, p: WPath, dt: str, x: str, y: str, dx: str, dy: str) -> None:
        """dx_i += s_ij y_j, dy_j += s_ij x_i with s_ij = sum_k c_ijk dt_k."""
        for (i, j), ks in p.ordered_pairs():
            E("{")
            for n_, (k, val) in enumerate(ks):
                if n_ == 0:
                    E(f"  T s_ = {self.lit(val)} * {dt}{k};")
                else:
                    E(f"  s_ = oeq_fma({self.lit(val)}, {dt}{k}, s_);")
            E(f"  {dx}{i} = oeq_fma(s_, {y}{p.b.off + j}, {dx}{i});")
            E(f"  {dy}{p.b.off + j} = oeq_fma(s_, {x}{i}, {dy}{p.b.off + j});")
            E("}")

    # ================================================================== prep
    def prep_body(self) -> str:
        """Packs the external weight vector into the two MFMA operand layouts (zero padded)."""
        E = Emitter()
        E("const int q = blockIdx.x * 256 + threadIdx.x;")
        E("T* __restrict__ wsT = (T*)ws;")
        for p in self.paths:
            nb = p.SU * 64 * p.NTW
            E(f"if (q >= {p.wb} && q < {p.wb + nb}) {{   // forward copy of path {p.t}: [s][lane][nt]")
            E(f"    const int e = q - {p.wb};")
            E(f"    const int nt = e % {p.NTW}; const int ln = (e / {p.NTW}) & 63; const int s = e / {64 * p.NTW};")
            E(f"    const int u = 16 * (s >> 2) + 4 * (ln >> 4) + (s & 3); const int w = {p.NTW} * (ln & 15) + nt;   // K order of forward_body")
            E(f"    wsT[q] = (u < {p.mu} && w < {p.mw}) ? W[{self.oeq_index(p, 'u', 'w')}] : (T)0;")
            E("}")
            VW, SQ = self.VW, _ceil(p.SW, self.VW)
            na = p.NTU * SQ * 64 * VW
            E(f"if (q >= {p.wa} && q < {p.wa + na}) {{   // backward copy of path {p.t}: [mt][s / {VW}][lane][s % {VW}]")
            E(f"    const int e = q - {p.wa};")
            E(f"    const int ln = (e / {VW}) & 63; const int s = {VW} * ((e / {64 * VW}) % {SQ}) + e % {VW}; const int mt = e / {64 * VW * SQ};")
            E(f"    const int u = 16 * mt + (ln & 15); const int w = 4 * s + (ln >> 4);")
            E(f"    wsT[q] = (u < {p.mu} && w < {p.mw}) ? W[{self.oeq_index(p, 'u', 'w')}] : (T)0;")
            E("}")
        return E.text()

    @property
    def prep_blocks(self) -> int:
        return _ceil(self.WA_END, 256)

    # =============================================================== forward
    def forward_body(self) -> str:
        E = Emitter()
        NO = len(self.fwd_items)
        E("const int lane = threadIdx.x, c = lane & 15, g = lane >> 4;")
        if True:          # (kept as a block: the mapping below is the only one)
            # Work item = (batch tile, output block).  Workgroups are handed to the 8 XCDs round robin by
            # their linear id, and every XCD has an L2 of its own: the items of one tile get ids 8 apart,
            # i.e. consecutive turns of the same XCD, so that the X rows fetched for the first output
            # block are still in that L2 for the others.
            E("const u64 ntiles = gridDim.x, lin = blockIdx.x + (u64)blockIdx.y * gridDim.x;")
            # The last fifth of the tiles is laid out item-major instead (all their most expensive items, then
            # the next ...): the launch then ends on the cheap items, which shortens its ragged end
            # (measured: forward 356 -> 346 us in fp32, 616 -> 598 us in fp64; a third or a half: no better).
            head8 = "((ntiles - ntiles / 5) >> 3)"
            E(f"const u64 head = {head8} << 3, full = head * {NO};")
            E("u64 tile; int slot;")
            E(f"if (lin < full) {{ const u64 j = lin >> 3; slot = (int)(j % {NO}); tile = (j / {NO}) * 8 + (lin & 7); }}")
            E("else { const u64 rem = ntiles - head, l2 = lin - full; slot = (int)(l2 / rem); tile = head + l2 % rem; }")
        E("const u64 row0 = tile * 16;")
        E("if (row0 >= n) return;")
        E("const u64 rowA = min(row0 + (u64)c, n - 1);       // rows past the end repeat the last row, never stored")
        E("const T* __restrict__ wsT = (const T*)ws;")
        E(f"const T* __restrict__ Xr = X + rowA * {self.D1};")
        for f in self.used_y:
            E(f"const T y{f} = Y[rowA * {self.D2} + {f}];")
        # One work item = (batch tile, output block): blockIdx.y walks the output blocks from the most
        # to the least expensive, so the dispatcher fills the tail of the launch with the cheap ones
        # (whole tiles per wavefront leave a third of the machine idle while the last ones finish).
        return self._forward_items(E, lambda slot: f"slot == {slot}")

    def _forward_items(self, E: Emitter, select) -> str:
        for slot, item in enumerate(self.fwd_items):
            E(f"if ({select(slot)}) {{")
            E.level += 1
            for i in item:
                self._forward_segment(E, *self.fwd_order[i])
            E.level -= 1
            E("}")
        return E.text()

    def _forward_segment(self, E: Emitter, o: Block, nt_lo: int, nt_hi: int) -> None:
        if True:
            NT = _ceil(o.mul, 16)
            NTS = range(nt_lo, nt_hi)
            E(f"{{ // output block {o.idx}: {o.mul}x l={o.l}, w tiles {nt_lo} .. {nt_hi - 1} of {NT}")
            E.level += 1
            if o.idx not in self.used_out:
                for r in range(4):
                    E(f"{{ const u64 row = row0 + {self.row(r)}; if (row < n) for (int q = c; q < {o.dim}; q += 16) Z[row * {self.D3} + {o.off} + q] = (T)0; }}")
                E.level -= 1
                E("}")
                return
            for k in range(o.D):
                for nt in NTS:
                    E(f"V4 acc{k}_{nt} = {{0, 0, 0, 0}};")
            # The K loops of the segment's paths form ONE software pipeline of groups of GS steps: the X records
            # and weight slices of the next group are in flight while this group runs on the VALU and the matrix
            # core, and the last group of a path (peeled off its loop) has the first group of the NEXT path in
            # flight, so that only the first path of a work item waits for its operands with nothing to do.
            # What bounds this kernel is the L2 -> L1 stream of operands (every wavefront re-reads the packed
            # weights), so the bytes in flight per wavefront matter more than anything else here.
            GS = self.fwd_group
            paths = self.paths_into(o.idx)
            groups = {p.t: _ceil(p.SU, GS) for p in paths}

            def regs(p):
                return [f"n{p.t}x{j}_{i}" for j in range(GS) for i in range(p.a.D)] \
                    + [f"n{p.t}b{j}_{nt}" for j in range(GS) for nt in NTS]

            def load(E, p, gexp):
                NG = groups[p.t]
                for j in range(GS):
                    sexp = f"({gexp}) * {GS} + {j}"
                    need_clamp = (NG * GS != p.SU)
                    scl = f"min({sexp}, {p.SU - 1})" if need_clamp else sexp
                    # K index -> channel: step s of lane group g is u = 16 (s / 4) + 4 g + s % 4, so that the
                    # four steps of a group read four adjacent records of a row (one wide load per lane)
                    uexp = f"16 * (({sexp}) >> 2) + 4 * g + (({sexp}) & 3)"
                    ucl = uexp if (p.mu % 16 == 0 and not need_clamp) else f"min({uexp}, {p.mu - 1})"
                    E(f"{{ const T* __restrict__ xp = Xr + {p.a.off} + ({ucl}) * {p.a.D}; " + " ".join(f"n{p.t}x{j}_{i} = xp[{i}];" for i in range(p.a.D)))
                    E(f"  const T* __restrict__ bp = wsT + {p.wb} + (({scl}) * 64 + lane) * {NT}; " + " ".join(f"n{p.t}b{j}_{nt} = bp[{nt}];" for nt in NTS) + " }")

            def steps(E, p, sgexp):
                """The GS K steps of group ``sgexp`` of path p on the copies (c...) of its operand registers."""
                NG = groups[p.t]
                for j in range(GS):
                    E("{")
                    E.level += 1
                    E("const T " + ", ".join(f"x{i} = cn{p.t}x{j}_{i}" for i in range(p.a.D)) + ";")
                    self.emit_cg_apply(E, p, "x", "m", "t")
                    if p.mu % 16 != 0 or NG * GS != p.SU:
                        E(f"if (16 * ((({sgexp}) * {GS} + {j}) >> 2) + 4 * g + ((({sgexp}) * {GS} + {j}) & 3) >= {p.mu}) {{ " + " ".join(f"t{k} = (T)0;" for k in range(o.D)) + " }")
                    for k in range(o.D):
                        for nt in NTS:
                            E(f"acc{k}_{nt} = oeq_mfma(t{k}, cn{p.t}b{j}_{nt}, acc{k}_{nt});")
                    E.level -= 1
                    E("}")

            for p in paths:
                E("T " + ", ".join(regs(p)) + ";")
            load(E, paths[0], "0")
            for pi, p in enumerate(paths):
                NG = groups[p.t]
                nxt = paths[pi + 1] if pi + 1 < len(paths) else None
                E(f"{{ // path {p.t}: l = {p.a.l} x {p.b.l} -> {p.o.l}, coefficient {p.coeff:.9g}")
                E.level += 1
                # the CG tensor is contracted with the row's Y once per path; the small matrix is applied per channel
                self.emit_cg_matrix(E, p, "y", "m")
                E(f"#pragma unroll {self.fwd_unroll}")
                E(f"for (int sg = 0; sg < {NG}; ++sg) {{")
                E.level += 1
                E("const T " + ", ".join(f"c{r} = {r}" for r in regs(p)) + ";")
                E(f"if (sg + 1 < {NG}) {{")
                E.level += 1
                load(E, p, "sg + 1")
                E.level -= 1
                if nxt is not None:
                    E("} else {")
                    E.level += 1
                    load(E, nxt, "0")
                    E.level -= 1
                E("}")
                steps(E, p, "sg")
                E.level -= 1
                E("}")
                E.level -= 1
                E("}")
            # lane holds, for each of its 4 rows, w = NT*c + nt (nt < NT) and all k: a contiguous run
            for r in range(4):
                E(f"{{ const u64 row = row0 + {self.row(r)};")
                E(f"  if (row < n) {{ T* __restrict__ zp = Z + row * {self.D3} + {o.off} + {NT} * c * {o.D};")
                for nt in NTS:
                    guard = "" if o.mul % 16 == 0 else f"if ({NT} * c + {nt} < {o.mul}) "
                    E(f"    {guard}{{ " + " ".join(f"zp[{nt * o.D + k}] = acc{k}_{nt}[{r}];" for k in range(o.D)) + " }")
                E("  } }")
            E.level -= 1
            E("}")

    # ====================================================== backward: dX, dY
    def backward_body(self) -> str:
        E = Emitter()
        E("const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c = lane & 15, g = lane >> 4;")
        E("const u64 row0 = (u64)blockIdx.x * 16;")
        E("if (row0 >= n) return;")
        E("const u64 rowB = min(row0 + (u64)c, n - 1);")
        E("const bool bvalid = row0 + c < n;")
        E("const T* __restrict__ wsT = (const T*)ws;")
        E(f"const T* __restrict__ Xr = X + rowB * {self.D1};")
        E(f"const T* __restrict__ Gr = G + rowB * {self.D3};")
        E(f"__shared__ T dyl[4 * 16 * {max(1, self.D2)}];")
        if self.bwd_lds:
            # the dZ tile goes to LDS once per workgroup (coalesced, one HBM round trip), and every
            # wavefront reads its MFMA B operands from there
            RS = self.bwd_rs
            E(f"__shared__ T gl[16 * {RS}];")
            VW = self.VW
            if self.D3 % VW == 0:
                # 16-byte vectors, all requested before the first one is written to LDS
                NV, RV = 16 * self.D3 // VW, self.D3 // VW
                NQ = _ceil(NV, 256)
                E("if ((((unsigned long long)G) & 15ull) == 0) {")
                E.level += 1
                E(f"VT gv[{NQ}];")
                for q in range(NQ):
                    idx = f"(int)threadIdx.x + {256 * q}"
                    guard = "" if 256 * (q + 1) <= NV else f"if ({idx} < {NV}) "
                    E(f"{guard}{{ const int r_ = ({idx}) / {RV}, v_ = ({idx}) - r_ * {RV}; "
                      f"gv[{q}] = *(const VT*)(G + min(row0 + (u64)r_, n - 1) * {self.D3} + v_ * {VW}); }}")
                for q in range(NQ):
                    idx = f"(int)threadIdx.x + {256 * q}"
                    guard = "" if 256 * (q + 1) <= NV else f"if ({idx} < {NV}) "
                    E(f"{guard}{{ const int r_ = ({idx}) / {RV}, v_ = ({idx}) - r_ * {RV}; T* __restrict__ d_ = gl + r_ * {RS} + v_ * {VW}; "
                      + " ".join(f"d_[{i}] = gv[{q}][{i}];" for i in range(VW)) + " }")
                E.level -= 1
                E("} else")
            E(f"for (int q = threadIdx.x; q < 16 * {self.D3}; q += 256) {{")
            E(f"    const int r_ = q / {self.D3}, col_ = q - r_ * {self.D3};")
            E(f"    gl[r_ * {RS} + col_] = G[min(row0 + (u64)r_, n - 1) * {self.D3} + col_];")
            E("}")
        for f in self.used_y:
            E(f"const T y{f} = Y[rowB * {self.D2} + {f}];")
            E(f"T dy{f} = (T)0;")
        # X records and dX accumulators of this wavefront: u-subtiles mt = wave + 4q, rows r of the
        # accumulator tile.  X is read once for all paths that consume the block.  With the dZ tile in
        # LDS the work is ordered by in1 block, so only one block's X and dX are live at a time (plus the
        # next block's X, requested one block ahead); otherwise everything is loaded here.
        for ai in self.used_in1:
            a = self.in1[ai]
            for q in range(_ceil(_ceil(a.mul, 16), 4)):
                for r in range(4):
                    E("T " + ", ".join(f"x{ai}_{q}_{r}_{i}" for i in range(a.D)) + ";")
                    E("T " + ", ".join(f"dx{ai}_{q}_{r}_{i} = (T)0" for i in range(a.D)) + ";")

        def load_x(E, ai):
            a = self.in1[ai]
            for q in range(_ceil(_ceil(a.mul, 16), 4)):
                for r in range(4):
                    uexp = f"16 * (wave + {4 * q}) + {self.row(r)}"
                    E(f"{{ const T* __restrict__ xp = Xr + {a.off} + min({uexp}, {a.mul - 1}) * {a.D}; "
                      + " ".join(f"x{ai}_{q}_{r}_{i} = xp[{i}];" for i in range(a.D)) + " }")

        def store_dx(E, ai):
            a = self.in1[ai]
            for q in range(_ceil(_ceil(a.mul, 16), 4)):
                E(f"if (wave + {4 * q} < {_ceil(a.mul, 16)} && bvalid) {{")
                E(f"    const int mt = wave + {4 * q};")
                for r in range(4):
                    E(f"    {{ const int u = 16 * mt + {self.row(r)};")
                    guard = "" if a.mul % 16 == 0 else f"if (u < {a.mul}) "
                    E(f"      {guard}{{ T* __restrict__ xp = Xg + (row0 + c) * {self.D1} + {a.off} + u * {a.D}; "
                      + " ".join(f"xp[{i}] = dx{a.idx}_{q}_{r}_{i};" for i in range(a.D)) + " } }")
                E("}")
        by_in1 = self.bwd_lds
        if by_in1:
            load_x(E, self.used_in1[0])
        else:
            for ai in self.used_in1:
                load_x(E, ai)
        # Work list of this wavefront: (output block, path, u-subtile group).  The packed weight
        # fragments (MFMA A operand) of the next item are fetched into a second register set while
        # the current item runs, and the dZ records of the next output block are requested as soon
        # as the last matrix-core step of the current one is issued, so that neither L2 nor HBM
        # latency sits between two items.
        if by_in1:
            items = [(p.o.idx, p, q) for ai in self.used_in1 for p in self.paths_from(ai) for q in range(_ceil(p.NTU, 4))]
        else:
            items = [(oi, p, q) for oi in self.used_out for p in self.paths_into(oi) for q in range(_ceil(p.NTU, 4))]
        max_sw = max(_ceil(self.out[oi].mul, 4) for oi in self.used_out)
        NSETS = 1          # register sets of packed weight fragments (a second set, fetched one item ahead, measured no gain)
        E("T " + ", ".join(f"af{b_}_{s_}" for b_ in range(NSETS) for s_ in range(max_sw)) + ";")

        def load_a(E, j):
            oi, p, q = items[j]
            SW = _ceil(self.out[oi].mul, 4)
            mt = f"wave + {4 * q}" if p.NTU % 4 == 0 else f"min(wave + {4 * q}, {p.NTU - 1})"
            VW, SQ = self.VW, _ceil(SW, self.VW)
            E(f"{{ const T* __restrict__ ap = wsT + {p.wa} + (({mt}) * {SQ * 64} + lane) * {VW}; "
              + " ".join(f"af{j % NSETS}_{s_} = ap[{(s_ // VW) * 64 * VW + s_ % VW}];" for s_ in range(SW)) + " }")

        def load_gz(E, oi):
            o = self.out[oi]
            for s_ in range(_ceil(o.mul, 4)):
                wexp = f"{4 * s_} + g" if o.mul % 4 == 0 else f"min({4 * s_} + g, {o.mul - 1})"
                E(f"{{ const T* __restrict__ gp = Gr + {o.off} + ({wexp}) * {o.D}; "
                  + " ".join(f"gz{oi}_{s_}_{k} = gp[{k}];" for k in range(o.D)) + " }")
                if o.mul % 4 != 0:
                    E(f"if ({4 * s_} + g >= {o.mul}) {{ " + " ".join(f"gz{oi}_{s_}_{k} = (T)0;" for k in range(o.D)) + " }")

        if self.bwd_lds:
            E("oeq_block_sync();")
        else:
            for oi in self.used_out:
                o = self.out[oi]
                E("T " + ", ".join(f"gz{oi}_{s_}_{k}" for s_ in range(_ceil(o.mul, 4)) for k in range(o.D)) + ";")
            load_gz(E, items[0][0])
        load_a(E, 0)
        for j, (oi, p, q) in enumerate(items):
            o, a = self.out[oi], p.a
            SW = _ceil(o.mul, 4)
            last_of_block = (j + 1 == len(items)) or items[j + 1][0] != oi
            E(f"{{ // output block {oi}, path {p.t}, u-subtile wave + {4 * q}")
            E.level += 1
            # The two halves of an item sit in branches of their own (taken by every wavefront that
            # owns a u-subtile of this path): basic-block boundaries are what keeps the compiler from
            # sinking the vector-ALU halves of all items below the matrix-core work, which would keep
            # every accumulator alive and halve the occupancy.
            cond = f"wave + {4 * q} < {p.NTU}"
            if by_in1 and (j == 0 or items[j - 1][1].a.idx != a.idx):
                nxt = self.used_in1.index(a.idx) + 1
                if nxt < len(self.used_in1):
                    load_x(E, self.used_in1[nxt])
            if j + 1 < len(items) and NSETS == 2:
                load_a(E, j + 1)
            for k in range(o.D):
                E(f"V4 acc{k} = {{0, 0, 0, 0}};")
            E(f"if ({cond}) {{")
            E.level += 1
            if self.bwd_lds:
                E(f"const T* __restrict__ gb = gl + c * {self.bwd_rs} + {o.off} + g * {o.D};")
            for s_ in range(SW):
                if self.bwd_lds:
                    if o.mul % 4 == 0:
                        E("{ const T " + ", ".join(f"b{k} = gb[{4 * s_ * o.D + k}]" for k in range(o.D)) + ";")
                    else:
                        E(f"{{ const bool in_ = {4 * s_} + g < {o.mul}; const T* __restrict__ gq = in_ ? gb + {4 * s_ * o.D} : gl;")
                        E("  const T " + ", ".join(f"b{k} = in_ ? gq[{k}] : (T)0" for k in range(o.D)) + ";")
                    E("  " + " ".join(f"acc{k} = oeq_mfma(af{j % NSETS}_{s_}, b{k}, acc{k});" for k in range(o.D)) + " }")
                else:
                    E(" ".join(f"acc{k} = oeq_mfma(af{j % NSETS}_{s_}, gz{oi}_{s_}_{k}, acc{k});" for k in range(o.D)))
            E.level -= 1
            E("}")
            if j + 1 < len(items) and (NSETS == 1 or (last_of_block and not self.bwd_lds)):
                # the fragment registers (one set) and, at the end of a block, the dZ registers are free
                # from here on: request the next ones now, the vector-ALU part below covers the latency
                if NSETS == 1:
                    load_a(E, j + 1)
                if last_of_block and not self.bwd_lds:
                    load_gz(E, items[j + 1][0])
            E(f"if ({cond}) {{")
            E.level += 1
            for r in range(4):
                E(f"{{ // row {r} of the tile: channel u = 16 mt + row, batch row b = row0 + c")
                E("  const T " + ", ".join(f"dt{k} = acc{k}[{r}]" for k in range(o.D)) + ";")
                E.level += 1
                self.emit_cg_backward(E, p, "dt", f"x{a.idx}_{q}_{r}_", "y", f"dx{a.idx}_{q}_{r}_", "dy")
                E.level -= 1
                E("}")
            E.level -= 1
            E("}")
            E.level -= 1
            E("}")
            if by_in1 and (j + 1 == len(items) or items[j + 1][1].a.idx != a.idx):
                store_dx(E, a.idx)
        # ---- dX stores
        for a in self.in1:
            if a.dim == 0:
                continue
            if a.idx not in self.used_in1:
                E(f"if (wave == 0 && bvalid) for (int q = g; q < {a.dim}; q += 4) Xg[(row0 + c) * {self.D1} + {a.off} + q] = (T)0;")
            elif not by_in1:
                store_dx(E, a.idx)
        # ---- dY: sum over the 4 lane groups (channels), then over the 4 wavefronts, fixed order
        for f in self.used_y:
            E(f"dy{f} += oeq_shfl_xor(dy{f}, 16);")
            E(f"dy{f} += oeq_shfl_xor(dy{f}, 32);")
        E("if (g == 0) {")
        for f in range(self.D2):
            E(f"    dyl[(wave * 16 + c) * {self.D2} + {f}] = " + (f"dy{f};" if f in self.used_y else "(T)0;"))
        E("}")
        E("oeq_block_sync();")
        E(f"if (wave == 0 && g == 0 && bvalid) {{")
        E(f"    for (int f = 0; f < {self.D2}; ++f)")
        E(f"        Yg[(row0 + c) * {self.D2} + f] = ((dyl[c * {self.D2} + f] + dyl[(16 + c) * {self.D2} + f]) + dyl[(32 + c) * {self.D2} + f]) + dyl[(48 + c) * {self.D2} + f];")
        E("}")
        return E.text()

    # ============================================================ backward: dW
    # accumulator registers (32-bit) live in one pass of the dW kernel.  fp64: the 352 accumulators of the
    # 64-channel benchmark problem in one pass leave one wavefront per SIMD and no room for anything else;
    # two passes of 192 + 160 measured 0.70 -> 0.63 ms for that kernel, three or more passes lose again
    DW_ACC_BUDGET = {4: 352, 8: 192}

    def dw_passes(self):
        """(wavefront group, [(path, first w tile, end w tile), ...]) of the passes of the dW kernel.  The
        accumulators of all segments of a pass are live at once (4 registers per 16 x 16 tile, 8 in fp64);
        problems with many paths - every copy of a second operand with mul > 1 is a path of its own - are
        cut into passes of at most DW_ACC_BUDGET accumulator registers, each walking the batch again, and
        a single path that exceeds the budget is cut by ranges of its 16-wide w tiles, so that the register
        file is never oversubscribed (a kernel spilling hundreds of accumulators is slow, and its fp64
        results were not exact on the device)."""
        per_tile = 4 * (self.itemsize // 4)
        budget = self.DW_ACC_BUDGET[self.itemsize]
        passes = []
        for grp in range(self.dw_groups):
            segs = []
            for p in (p for p in self.paths if self.dw_group[p.o.idx] == grp):
                per_w = _ceil(p.NTU, 4) * per_tile                 # accumulator registers of one w tile
                if per_w > budget:
                    raise NotImplementedError(
                        f"uvw dW: {p.mu} channels of the first operand need {per_w} accumulator registers per "
                        f"16-wide tile of the output, more than the {budget} one pass may hold")
                step = min(p.NTW, budget // per_w)
                pieces = _ceil(p.NTW, step)
                step = _ceil(p.NTW, pieces)                        # pieces of about equal width
                segs += [(p, lo, min(p.NTW, lo + step)) for lo in range(0, p.NTW, step)]
            need = [_ceil(p.NTU, 4) * (hi - lo) * per_tile for p, lo, hi in segs]
            total = sum(need)
            count = max(1, _ceil(total, budget))
            target = total / count                   # passes of about equal accumulator count
            cur, used = [], 0
            for seg, nd in zip(segs, need):
                if cur and (used + nd > budget or used >= target):
                    passes.append((grp, cur))
                    cur, used = [], 0
                cur.append(seg)
                used += nd
            if cur:
                passes.append((grp, cur))
        return passes

    def backward_dw_body(self) -> str:
        E = Emitter()
        # eight wavefronts: wave & 3 selects the 16-channel u-subtile, wave >> 2 one of two groups of
        # output blocks (balanced by MFMA count), so that two wavefronts share each SIMD and cover
        # each other's load latency while the accumulators of one group fit half the register file.
        # Each group is a separate copy of the loop so that its accumulators are the only ones live.
        E("const int lane = threadIdx.x & 63, wave = (threadIdx.x >> 6) & 3, grp = threadIdx.x >> 8, c = lane & 15, g = lane >> 4;")
        E("const u64 ntiles = (n + 15) / 16;")
        E(f"T* __restrict__ part = (T*)ws + {self.PART_OFF} + (u64)blockIdx.x * {self.WN};")
        for grp, segs in self.dw_passes():
            # a pass: these segments' accumulators are the only ones live while the batch is walked once
            paths = [p for p, _, _ in segs]
            outs = sorted({p.o.idx for p in paths})
            ins = sorted({p.a.idx for p in paths})
            ys = sorted({p.b.off + j for p in paths for (_, j) in p.pairs})
            into = lambda oi, segs=segs: [sg for sg in segs if sg[0].o.idx == oi]
            # w tiles of an output block whose dZ records this pass reads
            tiles_of = {oi: sorted({nt for p, lo, hi in segs if p.o.idx == oi for nt in range(lo, hi)}) for oi in outs}
            E(f"if (grp == {grp}) {{")
            E.level += 1
            for p, lo, hi in segs:
                for q in range(_ceil(p.NTU, 4)):
                    for nt in range(lo, hi):
                        E(f"V4 acc{p.t}_{q}_{nt} = {{0, 0, 0, 0}};")
            if self.dw_prefetch:
                # One step = 4 batch rows (the K of one MFMA) of one tile.  The steps of all tiles of this
                # workgroup form one loop, software pipelined over two register sets when the registers
                # allow it: the operands of the next step are in flight while this one is computed (X and
                # dZ stream from HBM here, so the latency to cover is the long one).
                names = [f"y{f}" for f in ys]
                for ai in ins:
                    a_ = self.in1[ai]
                    names += [f"x{ai}_{q}_{i}" for q in range(_ceil(_ceil(a_.mul, 16), 4)) for i in range(a_.D)]
                for oi in outs:
                    o = self.out[oi]
                    names += [f"gz{oi}_{nt}_{k}" for nt in tiles_of[oi] for k in range(o.D)]

                def load(E, it, h, ys=ys, ins=ins, outs=outs, tiles_of=tiles_of):
                    E("{")
                    E.level += 1
                    E(f"const u64 b = (blockIdx.x + (u64)(({it}) >> 2) * gridDim.x) * 16 + 4 * (({it}) & 3) + g;   // batch row of this lane for both operands")
                    E("const bool bv = b < n;")
                    E("const u64 bc = bv ? b : n - 1;")
                    E(f"const T* __restrict__ Xr = X + bc * {self.D1};")
                    E(f"const T* __restrict__ Gr = G + bc * {self.D3};")
                    for f in ys:
                        E(f"S{h}y{f} = Y[bc * {self.D2} + {f}];")
                    E("if (!bv) { " + " ".join(f"S{h}y{f} = (T)0;" for f in ys) + " }     // rows past the end: T = 0 there")
                    for ai in ins:
                        a_ = self.in1[ai]
                        for q in range(_ceil(_ceil(a_.mul, 16), 4)):
                            uexp = f"16 * (wave + {4 * q}) + c"
                            ucl = uexp if a_.mul % 64 == 0 else f"min({uexp}, {a_.mul - 1})"
                            E(f"{{ const T* __restrict__ xp = Xr + {a_.off} + ({ucl}) * {a_.D}; "
                              + " ".join(f"S{h}x{ai}_{q}_{i} = xp[{i}];" for i in range(a_.D)) + " }")
                            if a_.mul % 64 != 0:
                                E(f"if ({uexp} >= {a_.mul}) {{ " + " ".join(f"S{h}x{ai}_{q}_{i} = (T)0;" for i in range(a_.D)) + " }")
                    for oi in outs:
                        o = self.out[oi]
                        for nt in tiles_of[oi]:
                            wexp = f"{16 * nt} + c"
                            wcl = wexp if o.mul % 16 == 0 else f"min({wexp}, {o.mul - 1})"
                            E(f"{{ const T* __restrict__ gp = Gr + {o.off} + ({wcl}) * {o.D}; "
                              + " ".join(f"S{h}gz{oi}_{nt}_{k} = gp[{k}];" for k in range(o.D)) + " }")
                    E.level -= 1
                    E("}")

                def compute(E, outs=outs, into=into):
                    for oi in outs:
                        o = self.out[oi]
                        for p, lo, hi in into(oi):
                            for q in range(_ceil(p.NTU, 4)):
                                E(f"if (wave + {4 * q} < {p.NTU}) {{  // path {p.t}, w tiles {lo} .. {hi - 1}")
                                E.level += 1
                                self.emit_cg_forward(E, p, f"x{p.a.idx}_{q}_", "y", "t")
                                for nt in range(lo, hi):
                                    for k in range(o.D):
                                        E(f"acc{p.t}_{q}_{nt} = oeq_mfma(t{k}, gz{oi}_{nt}_{k}, acc{p.t}_{q}_{nt});")
                                E.level -= 1
                                E("}")

                E("const int nsteps = blockIdx.x < ntiles ? 4 * (int)((ntiles - blockIdx.x + gridDim.x - 1) / gridDim.x) : 0;")
                nsets = 2
                for h in range(nsets):
                    E("T " + ", ".join(f"S{h}{nm} = (T)0" for nm in names) + ";")
                E("if (nsteps > 0) {")
                E.level += 1
                load(E, "0", 0)
                E.level -= 1
                E("}")
                if nsets == 1:
                    E("#pragma unroll 1")
                    E("for (int it = 0; it < nsteps; ++it) {")
                    E.level += 1
                    E("const T " + ", ".join(f"{nm} = S0{nm}" for nm in names) + ";")
                    compute(E)
                    E("if (it + 1 < nsteps) {")
                    E.level += 1
                    load(E, "it + 1", 0)
                    E.level -= 1
                    E("}")
                    E.level -= 1
                    E("}")
                else:
                    E("#pragma unroll 1")
                    E("for (int it = 0; it < nsteps; it += 2) {")     # nsteps is a multiple of 4
                    E.level += 1
                    for h in (0, 1):
                        E("{")
                        E.level += 1
                        E("const T " + ", ".join(f"{nm} = S{h}{nm}" for nm in names) + ";")
                        E(f"if (it + {h + 1} < nsteps) {{")
                        E.level += 1
                        load(E, f"it + {h + 1}", 1 - h)
                        E.level -= 1
                        E("}")
                        compute(E)
                        E.level -= 1
                        E("}")
                    E.level -= 1
                    E("}")
            else:
                E("for (u64 tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {")
                E.level += 1
                E("const u64 row0 = tile * 16;")
                E("#pragma unroll 1")
                E("for (int sp = 0; sp < 4; ++sp) {")
                E.level += 1
                E("const u64 b = row0 + 4 * sp + g;          // batch row of this lane for both operands")
                E("const bool bv = b < n;")
                E("const u64 bc = bv ? b : n - 1;")
                E(f"const T* __restrict__ Xr = X + bc * {self.D1};")
                E(f"const T* __restrict__ Gr = G + bc * {self.D3};")
                for f in ys:
                    E(f"const T y{f} = bv ? Y[bc * {self.D2} + {f}] : (T)0;     // zero rows past the end: T = 0 there")
                for ai in ins:
                    a_ = self.in1[ai]
                    for q in range(_ceil(_ceil(a_.mul, 16), 4)):
                        uexp = f"16 * (wave + {4 * q}) + c"
                        ucl = uexp if a_.mul % 64 == 0 else f"min({uexp}, {a_.mul - 1})"
                        E(f"const T* __restrict__ xp{ai}_{q} = Xr + {a_.off} + ({ucl}) * {a_.D};")
                        if a_.mul % 64 == 0:
                            E("const T " + ", ".join(f"x{ai}_{q}_{i} = xp{ai}_{q}[{i}]" for i in range(a_.D)) + ";")
                        else:
                            E("T " + ", ".join(f"x{ai}_{q}_{i} = xp{ai}_{q}[{i}]" for i in range(a_.D)) + ";")
                            E(f"if ({uexp} >= {a_.mul}) {{ " + " ".join(f"x{ai}_{q}_{i} = (T)0;" for i in range(a_.D)) + " }")
                for oi in outs:
                    o = self.out[oi]
                    E(f"{{ // output block {oi}: dZ records, w = 16 nt + c")
                    E.level += 1
                    for nt in tiles_of[oi]:
                        wexp = f"{16 * nt} + c"
                        wcl = wexp if o.mul % 16 == 0 else f"min({wexp}, {o.mul - 1})"
                        E(f"const T* __restrict__ gp{nt} = Gr + {o.off} + ({wcl}) * {o.D};")
                        E("const T " + ", ".join(f"gz{nt}_{k} = gp{nt}[{k}]" for k in range(o.D)) + ";")
                    for p, lo, hi in into(oi):
                        for q in range(_ceil(p.NTU, 4)):
                            E(f"if (wave + {4 * q} < {p.NTU}) {{  // path {p.t}, w tiles {lo} .. {hi - 1}")
                            E.level += 1
                            self.emit_cg_forward(E, p, f"x{p.a.idx}_{q}_", "y", "t")
                            for nt in range(lo, hi):
                                for k in range(o.D):
                                    E(f"acc{p.t}_{q}_{nt} = oeq_mfma(t{k}, gz{nt}_{k}, acc{p.t}_{q}_{nt});")
                            E.level -= 1
                            E("}")
                    E.level -= 1
                    E("}")
                E.level -= 1
                E("}")
                E.level -= 1
                E("}")
            # ---- partial sums of this workgroup, laid out [t][u][w]
            for p, lo, hi in segs:
                for q in range(_ceil(p.NTU, 4)):
                    E(f"if (wave + {4 * q} < {p.NTU}) {{")
                    for nt in range(lo, hi):
                        for r in range(4):
                            E(f"    {{ const int u = 16 * (wave + {4 * q}) + {self.row(r)}; const int w = {16 * nt} + c;")
                            E(f"      if (u < {p.mu} && w < {p.mw}) part[{p.poff} + u * {p.mw} + w] = acc{p.t}_{q}_{nt}[{r}]; }}")
                    E("}")
            E.level -= 1
            E("}")
        return E.text()

    def reduce_body(self) -> str:
        E = Emitter()
        E("const int q = blockIdx.x * 256 + threadIdx.x;")
        E(f"if (q >= {self.WN}) return;")
        E(f"const T* __restrict__ part = (const T*)ws + {self.PART_OFF};")
        E("T acc = (T)0;")
        E(f"for (int b = 0; b < {self.DW_WORKGROUPS}; ++b) acc += part[(u64)b * {self.WN} + q];")
        E("int dst = q;")
        for p in self.paths:
            E(f"if (q >= {p.poff} && q < {p.poff + p.mu * p.mw}) {{ const int e = q - {p.poff}; const int u = e / {p.mw}; const int w = e - u * {p.mw}; dst = {self.oeq_index(p, 'u', 'w')}; }}")
        E("Wg[dst] = acc;")
        return E.text()

    # ---------------------------------------------------------------- rendering
    def render(self, prelude: str = None) -> str:
        env = jinja_env()
        if prelude is None:
            prelude = env.get_template("prelude.hip.jinja").render(T=self.T)
        return env.get_template("tp_uvw.hip.jinja").render(g=self, prelude=prelude)

    def describe(self) -> str:
        return (f"uvw T={self.T} paths={len(self.paths)} d1={self.D1} d2={self.D2} d3={self.D3} wn={self.WN} "
                f"mfma=16x16x4 workspace={self.ws_elems * self.itemsize}B")

    def plan(self):
        FIXED, ROW = 0, 1
        fwd = [dict(kernel="prep_forward", num_threads=256, grid_kind=FIXED, num_blocks=self.prep_blocks),
               dict(kernel="forward", num_threads=64, grid_kind=ROW, work_per_block=16, grid_y=len(self.fwd_items))]
        bwd = [dict(kernel="prep_backward", num_threads=256, grid_kind=FIXED, num_blocks=self.prep_blocks),
               dict(kernel="backward", num_threads=256, grid_kind=ROW, work_per_block=16),
               dict(kernel="backward_dw", num_threads=256 * self.dw_groups, grid_kind=FIXED,
                    num_blocks=self.DW_WORKGROUPS),
               dict(kernel="backward_reduce", num_threads=256, grid_kind=FIXED, num_blocks=_ceil(self.WN, 256))]
        return fwd, bwd, (lambda nnz=0, nodes=0: self.ws_elems * self.itemsize)
