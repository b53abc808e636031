"""Bandwidth-oriented schedule for uvu kernels whose rows are 16-byte granular.

Same arithmetic and lane mapping as :class:`UVUGenerator`; what changes is how memory is
driven, because these kernels are bound by HBM and a wavefront only keeps the memory system
busy while it has many independent requests in flight:

* every global read of a work item is issued before anything waits: rows that have to be
  transposed (X, dZ) are copied global -> LDS by the LDS-DMA form of the vector load
  (``global_load_lds_dwordx4``: 16 bytes per lane, no registers held), the per-lane weights go
  to registers, then there is ONE wait;
* after that wait no load is issued until all stores of the item are out, so the in-order
  memory counter never forces a store drain;
* Z / dX leave through LDS as 16-byte vectors per lane (``global_store_dwordx4``), complete
  cache lines per instruction.

Eligibility (otherwise the generic schedule is used): per-row weights; row lengths, block
offsets and per-row block sizes are multiples of 16 bytes; multiplicities above 64 are
multiples of 64; tensors are 16-byte aligned (checked by the caller at launch time).
"""
from __future__ import annotations

from typing import List, Tuple

from ..problem import TPProblem
from .common import WAVE, Emitter
from .uvu import Block, Path, UVUGenerator


class UVUFastGenerator(UVUGenerator):

    @staticmethod
    def eligible(problem: TPProblem, kind: str) -> bool:
        try:
            g = UVUGenerator(problem, kind)
        except Exception:
            return False
        if g.shared or kind == "conv_det":
            return False
        vw = 16 // g.itemsize
        if g.D1 % vw or g.D3 % vw:
            return False
        blocks = [g.in1[i] for i in g.used_in1] + [b for b in g.out if b.dim] + [b for b in g.in1 if b.dim]
        for b in blocks:
            if b.off % vw:
                return False
            if g.NCH > 1:
                if b.mul % WAVE:
                    return False
            elif (b.mul * b.D) % vw:
                return False
        if g.NCH > 4:
            return False
        return True

    def __init__(self, problem: TPProblem, kind: str = "tp"):
        super().__init__(problem, kind)
        self.fast = True
        self.VW = 16 // self.itemsize
        self._cur_c = None
        # ---- LDS map (elements) -------------------------------------------------
        self.XB = 0
        x_sz = self.R * self.D1
        out_stage = [WAVE * self.out[i].D for i in self.used_out if self.out[i].D > 1]
        in_stage = [WAVE * b.D for b in self.in1 if b.D > 1 and b.dim]
        # forward: X rows | one output slot
        self.ZB = x_sz
        self.fwd_lds = x_sz + (max(out_stage) if out_stage else 0)
        # backward: X rows | all dZ slots of a chunk | one dX slot
        self.GB = x_sz
        self.gslot = {}
        pos = self.GB
        for i in self.used_out:
            o = self.out[i]
            if o.D > 1:
                self.gslot[i] = pos
                pos += self.R * self.dense(o) * o.D
        self.SB = pos
        self.bwd_lds = pos + (max(in_stage) if in_stage else 0)
        self.unroll_fwd = True
        self.unroll_bwd = self.NCH <= 2

    # number of channels of a block held per sub-row in a (dense) LDS slot
    def dense(self, blk: Block) -> int:
        return blk.mul if self.NCH == 1 else WAVE

    def describe(self) -> str:
        return super().describe() + f" fast(fwd_lds={self.fwd_lds * self.itemsize}B bwd_lds={self.bwd_lds * self.itemsize}B)"

    # ------------------------------------------------------------------ pieces
    def emit_lane_fast(self, E: Emitter, lds_elems: int) -> None:
        E("const int lane = threadIdx.x;")
        E(f"const int sub = lane >> {self.LOGP};")
        E(f"const int ul = lane & {self.P - 1};")
        E(f"__shared__ __attribute__((aligned(16))) T lds[{max(lds_elems, self.VW)}];")

    def emit_weights(self, E: Emitter, p: Path, wptr: str) -> None:
        """Weights were preloaded at the top of the item; alias them under the usual names."""
        for v in range(p.mv):
            E(f"const T w{p.t}_{v} = W{self._cur_c}_{p.t}_{v};")

    def emit_weight_preload(self, E: Emitter, c, wptr: str = "Wr") -> None:
        """c is an int (unrolled chunk) or the string 'c' (rolled loop)."""
        tag = c if isinstance(c, int) else "c"
        ue = f"({c * self.P} + ul)" if isinstance(c, int) else f"(c * {self.P} + ul)"
        for p in self.paths:
            act = "rv" if self.full(p.a) else f"(rv && {ue} < {p.a.mul})"
            for v in range(p.mv):
                E(f"const T W{tag}_{p.t}_{v} = {act} ? {wptr}[{self.widx(p, ue, v)}] : (T)0;")

    def emit_x_dma(self, E: Emitter, row_of) -> None:
        """Async copy of the R X rows into lds[XB + r*D1 + col]."""
        ppr = self.D1 // self.VW
        total = self.R * ppr
        iters = (total + WAVE - 1) // WAVE
        if self.kind == "tp":
            # rows row0 .. row0+R-1 are contiguous in memory
            E("{")
            E(f"    const u64 left = n - row0;")
            E(f"    const int avail = (int)(left < {self.R} ? left : {self.R}) * {ppr};")
            E(f"    const T* __restrict__ src = X + row0 * {self.D1};")
            for it in range(iters):
                E(f"    {{ const int q = lane + {it * 64}; if (q < avail) oeq_dma16(src + q * {self.VW}, lds + {self.XB + it * 64 * self.VW}); }}")
            E("}")
        else:
            for it in range(iters):
                E(f"{{ const int q = lane + {it * 64};")
                E(f"  const int r = q / {ppr};")
                E(f"  const int rr = r < {self.R} ? r : 0;")
                row, ok = row_of("rr")
                E(f"  const i64 grow = (i64){row};")
                E(f"  const bool ok = {ok};")
                E(f"  if (q < {total} && ok) oeq_dma16(X + (u64)grow * {self.D1} + (q - r * {ppr}) * {self.VW}, lds + {self.XB + it * 64 * self.VW}); }}")

    def emit_x_regs(self, E: Emitter) -> None:
        for i in self.used_in1:
            a = self.in1[i]
            for m in range(a.D):
                E(f"const T x{i}_{m} = {self.act(a)} ? lds[{self.XB} + sub * {self.D1} + {a.off} + u * {a.D} + {m}] : (T)0;")

    def emit_g_dma(self, E: Emitter, cexpr: str, row_of) -> None:
        """Async copy of chunk c of every dZ slot (l > 0) into its dense LDS slot."""
        for i in self.used_out:
            o = self.out[i]
            if o.D == 1:
                continue
            dn = self.dense(o)
            ppr = dn * o.D // self.VW
            total = self.R * ppr
            iters = (total + WAVE - 1) // WAVE
            coff = f" + {cexpr} * {WAVE * o.D}" if self.NCH > 1 else ""
            for it in range(iters):
                E(f"{{ const int q = lane + {it * 64};")
                if self.R == 1:
                    row, ok = row_of("0")
                    E(f"  if (q < {total} && {ok}) oeq_dma16(G + (u64){row} * {self.D3} + {o.off}{coff} + q * {self.VW}, lds + {self.gslot[i] + it * 64 * self.VW}); }}")
                else:
                    E(f"  const int r = q / {ppr};")
                    E(f"  const int rr = r < {self.R} ? r : 0;")
                    row, ok = row_of("rr")
                    E(f"  const i64 grow = (i64){row};")
                    E(f"  const bool ok = {ok};")
                    E(f"  if (q < {total} && ok) oeq_dma16(G + (u64)grow * {self.D3} + {o.off} + (q - r * {ppr}) * {self.VW}, lds + {self.gslot[i] + it * 64 * self.VW}); }}")

    def emit_g_regs(self, E: Emitter, o: Block) -> None:
        dn = self.dense(o)
        base = self.gslot[o.idx]
        for k in range(o.D):
            E(f"const T g{k} = {self.act(o)} ? lds[{base} + (sub * {dn} + ul) * {o.D} + {k}] : (T)0;")

    def emit_slot_out(self, E: Emitter, blk: Block, name: str, ptr: str, rowdim: int, row_of, base: int,
                      op: str = "store") -> None:
        """registers -> dense LDS slot -> global rows (16-byte vectors, or scalar atomics)."""
        dn = self.dense(blk)
        D = blk.D
        act = self.act(blk)
        E("oeq_sync();")
        E(f"if ({act}) {{ " + " ".join(f"lds[{base} + (sub * {dn} + ul) * {D} + {k}] = {name}{k};" for k in range(D)) + " }")
        E("oeq_sync();")
        coff = f" + c * {WAVE * D}" if self.NCH > 1 else ""
        if op == "store":
            ppr = dn * D // self.VW
            total = self.R * ppr
            iters = (total + WAVE - 1) // WAVE
            for it in range(iters):
                E(f"{{ const int q = lane + {it * 64};")
                if self.R == 1:
                    row, ok = row_of("0")
                    E(f"  if (q < {total} && {ok}) *(VT*)({ptr} + (u64){row} * {rowdim} + {blk.off}{coff} + q * {self.VW}) = *(const VT*)(lds + {base} + q * {self.VW}); }}")
                else:
                    E(f"  const int r = q / {ppr};")
                    E(f"  const int rr = r < {self.R} ? r : 0;")
                    row, ok = row_of("rr")
                    E(f"  const i64 grow = (i64){row};")
                    E(f"  const bool ok = {ok};")
                    E(f"  if (q < {total} && ok) *(VT*)({ptr} + (u64)grow * {rowdim} + {blk.off} + (q - r * {ppr}) * {self.VW}) = *(const VT*)(lds + {base} + q * {self.VW}); }}")
        else:
            L = dn * D
            total = self.R * L
            iters = (total + WAVE - 1) // WAVE
            for it in range(iters):
                E(f"{{ const int q = lane + {it * 64};")
                if self.R == 1:
                    row, ok = row_of("0")
                    E(f"  if (q < {total} && {ok}) oeq_atomic_add({ptr} + (u64){row} * {rowdim} + {blk.off}{coff} + q, lds[{base} + q]); }}")
                else:
                    E(f"  const int r = q / {L};")
                    E(f"  const int rr = r < {self.R} ? r : 0;")
                    row, ok = row_of("rr")
                    E(f"  const i64 grow = (i64){row};")
                    E(f"  const bool ok = {ok};")
                    E(f"  if (q < {total} && ok) oeq_atomic_add({ptr} + (u64)grow * {rowdim} + {blk.off} + (q - r * {L}), lds[{base} + q]); }}")

    def emit_block_out_fast(self, E, blk, name, ptr, rowdim, own_row, row_of, base, op="store"):
        if blk.D == 1:
            row, ok = own_row
            dst = f"{ptr}[(u64){row} * {rowdim} + {blk.off} + u]"
            stmt = f"oeq_atomic_add(&{dst}, {name}0);" if op == "atomic" else f"{dst} = {name}0;"
            E(f"if ({self.act(blk)} && {ok}) {{ {stmt} }}")
        else:
            self.emit_slot_out(E, blk, name, ptr, rowdim, row_of, base, op)

    def emit_zero_block_fast(self, E, blk, ptr, rowdim, own_row, row_of):
        """An output block nothing contributes to: plain zero stores (generic path)."""
        if blk.D > 1:
            E("oeq_sync();")
        save = self.ZB
        self.emit_block_zero(E, blk, ptr, rowdim, own_row, row_of)
        self.ZB = save

    # ------------------------------------------------------------------ rows
    def _rows(self):
        """(prologue emitter, own rows, row_of functions) for the operator family."""
        if self.kind == "tp":
            def prologue(E):
                E(f"const u64 row0 = (u64)blockIdx.x * {self.R};")
                E("const u64 row = row0 + sub;")
                E("const bool rv = row < n;")
                E(f"const T* __restrict__ Yr = Y + row * {self.D2};")
                E(f"const T* __restrict__ Wr = W + row * {self.WN};")
            own_x = own_z = ("row", "rv")
            xrow_of = zrow_of = (lambda r: (f"(row0 + {r})", f"(row0 + {r} < n)"))
            return prologue, own_x, own_z, xrow_of, zrow_of, "row"

        def prologue(E):
            self._edge_prologue(E)
        return prologue, ("xsrc", "rv"), ("zdst", "rv"), self._shfl_row("xsrc"), self._shfl_row("zdst"), "e"

    # =============================================================== forward
    def fast_forward_body(self) -> str:
        E = Emitter()
        atomic = (self.kind == "conv_atomic")
        self.emit_lane_fast(E, self.fwd_lds)
        prologue, own_x, own_z, xrow_of, zrow_of, _ = self._rows()
        prologue(E)
        self.emit_x_dma(E, xrow_of)
        for c in range(self.NCH):
            self.emit_weight_preload(E, c)
        self.emit_y_load(E, "Yr", "rv")
        E("oeq_wait_vm();")
        E("oeq_sync();")
        for c in range(self.NCH):
            self._cur_c = c
            E("{")
            E.level += 1
            E(f"const int c = {c};")
            E(f"const int u = {c * self.P} + ul;")
            self.emit_x_regs(E)
            for o in self.out:
                if o.dim == 0:
                    continue
                E("{")
                E.level += 1
                if o.idx in self.used_out:
                    self.emit_forward_block(E, o, "Wr")
                    self.emit_block_out_fast(E, o, "z", "Z", self.D3, own_z, zrow_of, self.ZB,
                                             op="atomic" if atomic else "store")
                elif not atomic:
                    self.emit_zero_block_fast(E, o, "Z", self.D3, own_z, zrow_of)
                E.level -= 1
                E("}")
            E.level -= 1
            E("}")
        return E.text()

    # ============================================================== backward
    def fast_backward_body(self) -> str:
        E = Emitter()
        atomic = (self.kind == "conv_atomic")
        self.emit_lane_fast(E, self.bwd_lds)
        prologue, own_x, own_z, xrow_of, zrow_of, rowvar = self._rows()
        prologue(E)
        E(f"T* __restrict__ Wgr = Wg + {rowvar} * {self.WN};")
        self.emit_x_dma(E, xrow_of)
        self.emit_y_load(E, "Yr", "rv")
        for f in self.used_y:
            E(f"T dy{f} = (T)0;")

        def chunk(E, c):
            tag = c if isinstance(c, int) else "c"
            self._cur_c = tag
            E("oeq_wait_lds();")                  # LDS reads of the previous chunk have completed,
            E("oeq_sync();")                      # its slots may be overwritten by the DMA
            self.emit_g_dma(E, str(c), zrow_of)
            self.emit_weight_preload(E, c)
            for i in self.used_out:               # l = 0 slots go straight to registers
                o = self.out[i]
                if o.D == 1:
                    row, ok = own_z
                    E(f"const T gs{i} = ({self.act(o)} && {ok}) ? G[(u64){row} * {self.D3} + {o.off} + u] : (T)0;")
            E("oeq_wait_vm();")
            E("oeq_sync();")
            self.emit_x_regs(E)
            for i in self.used_in1:
                for m in range(self.in1[i].D):
                    E(f"T dx{i}_{m} = (T)0;")
            for oi in self.used_out:
                o = self.out[oi]
                E("{")
                E.level += 1
                if o.D == 1:
                    E(f"const T g0 = gs{oi};")
                else:
                    self.emit_g_regs(E, o)

                def sink(E, p, v, expr):
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
                    self.emit_block_out_fast(E, a, f"dx{a.idx}_", "Xg", self.D1, own_x, xrow_of, self.SB,
                                             op="atomic" if atomic else "store")
                elif not atomic:
                    self.emit_zero_block_fast(E, a, "Xg", self.D1, own_x, xrow_of)
                E.level -= 1
                E("}")

        if self.unroll_bwd:
            for c in range(self.NCH):
                E("{")
                E.level += 1
                E(f"const int c = {c};")
                E(f"const int u = {c * self.P} + ul;")
                chunk(E, c)
                E.level -= 1
                E("}")
        else:
            E("#pragma unroll 1")
            E(f"for (int c = 0; c < {self.NCH}; ++c) {{")
            E.level += 1
            E(f"const int u = c * {self.P} + ul;")
            chunk(E, "c")
            E.level -= 1
            E("}")
        self.emit_dy_reduce(E)
        if self.kind == "tp":
            E("if (rv && ul == 0) {")
            E(f"    T* __restrict__ Ygr = Yg + row * {self.D2};")
        else:
            E("if (e < nnz && ul == 0) {")
            E(f"    T* __restrict__ Ygr = Yg + e * {self.D2};")
        for f in range(self.D2):
            E(f"    Ygr[{f}] = " + (f"dy{f};" if f in self.used_y else "(T)0;"))
        E("}")
        if self.kind != "tp":
            E("if (e < nnz && !rv) {")
            E(f"    for (int q = ul; q < {self.WN}; q += {self.P}) Wgr[q] = (T)0;")
            E("}")
        return E.text()

    # bodies used by the templates
    def tp_forward_body(self) -> str:
        return self.fast_forward_body()

    def tp_backward_body(self) -> str:
        return self.fast_backward_body()

    def conv_atomic_forward_body(self) -> str:
        return self.fast_forward_body()

    def conv_atomic_backward_body(self) -> str:
        return self.fast_backward_body()
