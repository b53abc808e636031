"""Register-direct schedule for uvu kernels: no LDS, no transposition.

In the ``mul x irrep`` layout element ``(u, m)`` sits at ``u * (2l+1) + m``, so with lane <-> channel
``u`` every lane owns a CONTIGUOUS record of ``2l+1`` words in X, Z, dZ and dX.  A lane therefore
reads and writes its records straight from/to global memory with per-lane vector accesses
(dword x1 / x3 / x4+x1 / x4+x3, dword aligned); consecutive lanes touch consecutive records, so a
wavefront still covers a contiguous span and every cache line it touches is fully used - the L1
merges the partial touches of the two instructions of a record.  Compared with staging through
LDS this removes all LDS traffic and all intra-wave synchronisation, frees the LDS limit on
occupancy, and lets the compiler issue every load of a work item up front (there is no fence in
the way), which is what keeps HBM busy.

It needs nothing from the problem's sizes (any multiplicity, any alignment), so it serves as
the general schedule for the batch product and the atomic convolution.

Stores are the exception where measurement favours a detour through LDS: a record store covers
only part of each cache line per instruction, and on MI355X streams of such partial-line writes
(Z is 73 % of the forward traffic) run about 20 % slower than full-line writes, and strided
atomics are several times slower than coalesced ones.  So the big outputs (Z; dX when it is
scattered with atomics) are transposed through a 2 KB LDS slot and leave as full 16-byte-per-lane
vector stores or as coalesced atomics; loads stay register-direct.
"""
from __future__ import annotations

from .. import tunables
from ..problem import TPProblem
from .common import WAVE, Emitter
from .uvu import Block, Path, UVUGenerator


class UVUDirectGenerator(UVUGenerator):
    def __init__(self, problem: TPProblem, kind: str = "tp", waves_per_eu: int = 0, vector_stores: bool = True):
        super().__init__(problem, kind)
        if (kind == "conv_det" and not getattr(self, "_allow_det", False)) or self.shared:
            raise NotImplementedError("direct schedule: batch product with per-row weights and atomic convolution")
        self.waves_per_eu = waves_per_eu
        # False: outputs are written with dword-aligned record stores only (for callers whose
        # output tensor is not 16-byte aligned)
        self.vector_stores = vector_stores
        # words per 16-byte vector store of the LDS-slot route (8-byte stores measured a tie on the
        # 128-channel MACE problem, 0.463 against 0.458 ms; 4-byte stores 0.77 ms)
        self.VW = max(1, 16 // self.itemsize)
        self.VTYPE = "VT"
        stage = [WAVE * b.D for b in list(self.out) + list(self.in1) if b.D > 1 and b.dim]
        self.lds_elems = max(stage) if stage else 0
        self.ZB = 0
        self.unroll_bwd_chunks = 1
        self._lazy = False            # set per kernel body by lazy_operands()
        # Batch product: every tensor is read or written exactly once.  The backward's loads and stores
        # carry the non-temporal hint (measured on the 128-channel MACE problem, warm and with flushed
        # caches alike: 0.63 -> 0.56 ms); on the forward the hint measured slower (stores: 0.46 -> 0.52 ms
        # with flushed caches), so it keeps plain accesses.  ``tunables.tp_nontemporal`` lists the accesses
        # that get the hint (fl, fs, bl, bs = forward / backward loads / stores).  Writing the backward's dX
        # through the LDS slot as full-line vector stores costs 37 registers on this problem and measured
        # slower (0.588 against 0.562 ms), so its dX keeps the record stores (dx_through_slot has the rule);
        # dealing a row to four wavefronts of one workgroup measured no gain either (forward 0.456 ms,
        # backward 0.59 ms).
        self._nt_modes = set(tunables.current.tp_nontemporal.split(",")) if kind == "tp" else set()
        self.nt_load = self.nt_store = False
        # one row per wavefront: the row index is wave-uniform and an out-of-range wavefront exits
        self.uniform_rows = (self.R == 1)
        self._cur_c = None

    def describe(self) -> str:
        return super().describe().replace(f"lds={0}B", "lds=0B") + " direct"

    # ------------------------------------------------------------------ pieces
    def emit_lane_direct(self, E: Emitter, lds: bool = False) -> None:
        E("const int lane = threadIdx.x;")
        E(f"const int sub = lane >> {self.LOGP};")
        E(f"const int ul = lane & {self.P - 1};")
        if lds and self.lds_elems:
            E(f"__shared__ __attribute__((aligned(16))) T lds[{self.lds_elems}];")

    # ---- stores through an LDS slot ---------------------------------------------
    def dense(self, blk: Block) -> int:
        """Channels of ``blk`` held per sub-row in the (gap-free) LDS slot."""
        return blk.mul if self.NCH == 1 else WAVE

    def vector_ok(self, blk: Block, rowdim: int) -> bool:
        """Rows of this block can be written as aligned 16-byte vectors."""
        vw = self.VW
        if not self.vector_stores or rowdim % vw or blk.off % vw:
            return False
        if self.NCH > 1:
            return blk.mul % WAVE == 0
        return (blk.mul * blk.D) % vw == 0

    def emit_slot_out(self, E: Emitter, blk: Block, names, ptr: str, rowdim: int, row_of, op: str) -> None:
        """registers -> LDS slot (transposed) -> global rows: 16-byte vectors per lane (op "store",
        needs vector_ok and 16-byte aligned tensors) or coalesced scalar atomics (op "atomic")."""
        dn, D, base = self.dense(blk), blk.D, self.ZB
        E("oeq_sync();")
        E(f"if ({self.act(blk)}) {{ " + " ".join(f"lds[{base} + (sub * {dn} + ul) * {D} + {k}] = {n};" for k, n in enumerate(names)) + " }")
        E("oeq_sync();")
        coff = f" + c * {WAVE * D}" if self.NCH > 1 else ""
        cnt = dn * D                       # elements per sub-row in the slot
        if op == "store":
            per_row, unit, total_it = cnt // self.VW, self.VW, None
        else:
            per_row, unit = cnt, 1
        total = self.R * per_row
        # a partly filled last chunk holds fewer valid channels than the slot has room for
        limit = f"{total}" if (self.NCH == 1 or self.full(blk)) else f"{self.chunk_count(blk)} * {D}"
        for it in range((total + WAVE - 1) // WAVE):
            E(f"{{ const int q = lane + {it * 64};")
            if self.R == 1:
                row, ok = row_of("0")
                guard = f"q < {limit}" + ("" if ok == "true" else f" && {ok}")
                tgt = f"{ptr} + (u64){row} * {rowdim} + {blk.off}{coff} + q * {unit}"
            else:
                E(f"  const int r = q / {per_row};")
                E(f"  const int rr = r < {self.R} ? r : 0;")
                row, ok = row_of("rr")
                E(f"  const u64 grow = (u64){row};")
                E(f"  const bool ok = {ok};")
                guard = f"q < {total} && ok"
                tgt = f"{ptr} + grow * {rowdim} + {blk.off} + (q - r * {per_row}) * {unit}"
            if op == "store" and self.nt_store:
                E(f"  if ({guard}) __builtin_nontemporal_store(*(const {self.VTYPE}*)(lds + {base} + q * {unit}), ({self.VTYPE}*)({tgt})); }}")
            elif op == "store":
                E(f"  if ({guard}) *({self.VTYPE}*)({tgt}) = *(const {self.VTYPE}*)(lds + {base} + q * {unit}); }}")
            else:
                E(f"  if ({guard}) oeq_atomic_add({tgt}, lds[{base} + q]); }}")

    def emit_block_store(self, E: Emitter, blk: Block, names, ptr: str, rowdim: int, own_row: str, row_of,
                         op: str, via_lds: bool) -> None:
        """One block of one chunk: registers -> memory, by the cheapest correct route."""
        if blk.D == 1 or not via_lds or (op == "store" and not self.vector_ok(blk, rowdim)):
            self.emit_record_store(E, names, f"{ptr} + (u64){own_row} * {rowdim} + {blk.off} + u * {blk.D}",
                                   self.act(blk), op)
        else:
            self.emit_slot_out(E, blk, names, ptr, rowdim, row_of, op)

    LAZY_OPERANDS = None      # None: by the rule of lazy_operands(); True / False force it

    def lazy_operands(self, direction: str) -> bool:
        """Batch product with many paths: request dZ and the weights one output block ahead of their use
        instead of all at the top of the row, and form the products x_i y_j that several paths share per
        output block instead of carrying each in a register (two in fp64) from its first use to its last.
        The carried products are what pushes the forward of the 68-path NequIP problem to 401 registers in
        fp32 and past 512 into scratch in fp64 (130 with this); it costs vector-ALU work where registers
        were not short.  Measured on MI355X over the reference's uvu set (batch 50 000, ms, eager / lazy):

            problem (channels, paths)     fp32 forward   fp32 backward  fp64 forward   fp64 backward
            mace-large   (128, 17)        0.452 / 0.486  0.559 / 0.572  0.962 / 0.961  1.345 / 1.369
            mace-medium  (128,  8)        0.169 / 0.186  0.229 / 0.216  0.351 / 0.365  0.731 / 0.486
            nequip-lips     (32, 30)      0.176 / 0.203  0.270 / 0.232  0.365 / 0.381  0.659 / 0.518
            nequip-aspirin  (64, 10)      0.089 / 0.096  0.116 / 0.120  0.177 / 0.187  0.276 / 0.254
            nequip-toluene  (64, 30)      0.344 / 0.374  0.469 / 0.442  0.731 / 0.748  1.132 / 1.025
            nequip-benzene  (64, 68)      1.006 / 1.060  1.408 / 1.195  5.432 / 2.080  6.051 / 2.905
            nequip-water    (32, 10)      0.039 / 0.040  0.058 / 0.061  0.089 / 0.096  0.153 / 0.130

        The rule below takes the lazy form where it wins by more than a few per cent: the forward in fp64
        from 40 paths on, the backward in fp64 or from 30 paths on."""
        if self.LAZY_OPERANDS is not None:
            return bool(self.LAZY_OPERANDS)
        if self.kind != "tp":
            return False
        fp64, n = self.T == "double", len(self.paths)
        if direction == "forward":
            return fp64 and n >= 40
        return fp64 or n >= 30

    def dx_through_slot(self, blk: Block) -> bool:
        """Batch product: dX of this block leaves through the LDS slot as full 16-byte-per-lane vectors instead of
        a lane's own record.  Measured on MI355X, backward in ms, records / slot: the single-path problems of
        the reference's roofline set with l1 = 3, 5, 5, 6, 7, 7 (records of 7 to 15 words) 0.483 / 0.445,
        1.006 / 0.660, 0.928 / 0.794, 1.261 / 1.123, 1.558 / 1.295, 1.592 / 1.212; l1 = 1 and 2 0.186 / 0.185 and
        0.357 / 0.330; against that the 17-path MACE problem (l1 <= 2) 0.562 / 0.588, its 24-path variant
        0.797 / 0.855, the 13-path 256-channel problem 0.320 / 0.329, the 11-path NequIP problem 0.079 / 0.078: long
        records and single paths take the slot, short records in many-path problems (where its registers are
        missed) keep the record stores."""
        if self.kind != "tp":
            return False
        return blk.D >= 7 or len(self.paths) == 1

    def uexpr(self, c) -> str:
        return f"({c * self.P} + ul)" if isinstance(c, int) else f"(c * {self.P} + ul)"

    def uclamp(self, blk: Block, c) -> str:
        """Channel index of this lane in chunk c, clamped into the block."""
        return self.uexpr(c) if self.full(blk) else f"min({self.uexpr(c)}, {blk.mul - 1})"

    def rows_always_stored(self) -> bool:
        """Batch product with several rows per wavefront: the lanes past the batch work on its last row once
        more and store it again (the same values to the same addresses) instead of storing nothing.  A store
        under ``if (row < n)`` splits the unrolled kernel into blocks, and the compiler then moves the
        arithmetic of what is stored later (all of dX) past the earlier ones, with every operand alive until
        then: the 30-path NequIP problem with 32 channels took 335 registers in fp32 and spilled in fp64
        (backward 1.35 ms against 0.39 ms of the forward)."""
        return self.kind == "tp"

    def act(self, blk: Block) -> str:
        rv = "true" if (self.uniform_rows or self.rows_always_stored()) else "rv"
        if self.full(blk):
            return rv
        return f"(u < {blk.mul})" if rv == "true" else f"(rv && u < {blk.mul})"

    def act_c(self, blk: Block, c) -> str:
        rv = "true" if (self.uniform_rows or self.rows_always_stored()) else "rv"
        if self.full(blk):
            return rv
        return f"({self.uexpr(c)} < {blk.mul})" if rv == "true" else f"(rv && {self.uexpr(c)} < {blk.mul})"

    def emit_record_load(self, E: Emitter, names, ptr: str, act: str, zero: bool = False) -> None:
        """Unconditional loads (the caller passes an address that is valid for every lane: idle
        lanes are clamped onto a valid row/channel).  Branch-free loads are what lets the compiler
        merge them into x3/x4 accesses and hoist them.  With ``zero`` idle lanes get 0 instead of
        the clamped lane's data (needed where the value feeds a cross-lane sum)."""
        rd = (lambda p, k: f"oeq_ldnt({p} + {k})") if self.nt_load else (lambda p, k: f"{p}[{k}]")
        if zero and act != "true":
            E("T " + ", ".join(names) + ";")
            E(f"{{ const T* __restrict__ p_ = {ptr}; " + " ".join(f"{n} = {rd('p_', k)};" for k, n in enumerate(names)) + " }")
            E(f"if (!({act})) {{ " + " ".join(f"{n} = (T)0;" for n in names) + " }")
        else:
            E(f"const T* __restrict__ p_{names[0]} = {ptr};")
            E("const T " + ", ".join(f"{n} = {rd('p_' + names[0], k)}" for k, n in enumerate(names)) + ";")

    def emit_record_store(self, E: Emitter, names, ptr: str, act: str, op: str = "store") -> None:
        if op == "atomic":
            E(f"if ({act}) {{ T* __restrict__ p_ = {ptr}; " + " ".join(f"oeq_atomic_add(p_ + {k}, {n});" for k, n in enumerate(names)) + " }")
        elif self.nt_store:
            E(f"if ({act}) {{ T* __restrict__ p_ = {ptr}; " + " ".join(f"oeq_stnt(p_ + {k}, {n});" for k, n in enumerate(names)) + " }")
        else:
            E(f"if ({act}) {{ T* __restrict__ p_ = {ptr}; " + " ".join(f"p_[{k}] = {n};" for k, n in enumerate(names)) + " }")

    def emit_y_load_direct(self, E: Emitter) -> None:
        for f in self.used_y:
            E(f"{'' if self._lazy else 'const '}T y{f} = Yr[{f}];")

    def emit_forget_products(self, E: Emitter) -> None:
        """Between two output blocks of a many-path problem: the products x_i y_j that several paths share
        are formed again per block instead of being carried, each in a register (two in fp64), from the
        first block that uses them to the last."""
        E(" ".join(f"OEQ_OPAQUE(y{f});" for f in self.used_y))

    def emit_weights(self, E: Emitter, p: Path, wptr: str) -> None:
        for v in range(p.mv):
            E(f"const T w{p.t}_{v} = W{self._cur_c}_{p.t}_{v};")

    def looped_weight(self, p: Path, wptr: str) -> str:
        """Unconditional load from the clamped channel, like every other load of this schedule."""
        idx = self.widx(p, self.uclamp(p.a, self._loop_c), "v")
        return f"oeq_ldnt({wptr} + {idx})" if self.nt_load else f"{wptr}[{idx}]"

    def emit_weight_preload(self, E: Emitter, c, wptr: str = "Wr", only=None) -> None:
        tag = c if isinstance(c, int) else "c"
        self._loop_c = c
        for p in self.paths:
            if p.looped or (only is not None and p.t not in only):
                continue
            for v in range(p.mv):
                idx = self.widx(p, self.uclamp(p.a, c), v)
                E(f"const T W{tag}_{p.t}_{v} = " + (f"oeq_ldnt({wptr} + {idx});" if self.nt_load else f"{wptr}[{idx}];"))

    def emit_x_preload(self, E: Emitter, c, xrow: str, only=None) -> None:
        tag = c if isinstance(c, int) else "c"
        for i in self.used_in1:
            if only is not None and i not in only:
                continue
            a = self.in1[i]
            self.emit_record_load(E, [f"X{tag}_{i}_{m}" for m in range(a.D)],
                                  f"X + (u64){xrow} * {self.D1} + {a.off} + {self.uclamp(a, c)} * {a.D}",
                                  self.act_c(a, c))

    def emit_x_alias(self, E: Emitter, tag, only=None) -> None:
        for i in self.used_in1:
            if only is not None and i not in only:
                continue
            for m in range(self.in1[i].D):
                E(f"const T x{i}_{m} = X{tag}_{i}_{m};")

    def _rows(self, E: Emitter, backward: bool = False):
        """Emit the row prologue; returns (x row, z row, per-row stream index)."""
        if self.kind == "tp":
            if self.uniform_rows:
                E("const u64 row = blockIdx.x;")          # wave-uniform; the grid has exactly n workgroups
                E("if (row >= n) return;")
                E("const bool rv = true; (void)rv;")
                rc = "row"
            else:
                E(f"const u64 row = (u64)blockIdx.x * {self.R} + sub;")
                E("const bool rv = row < n; (void)rv;")
                E("const u64 rowc = rv ? row : n - 1;")    # idle lanes work on the last row once more
                rc = "rowc"
            E(f"const T* __restrict__ Yr = Y + {rc} * {self.D2};")
            E(f"const T* __restrict__ Wr = W + {rc} * {self.WN};")
            if self.uniform_rows:
                self.xrow_of = self.zrow_of = (lambda r: ("row", "true"))
            else:
                base = f"(u64)blockIdx.x * {self.R}"
                self.xrow_of = self.zrow_of = (lambda r: (f"min({base} + {r}, n - 1)", "true"))
            return rc, rc, rc
        # convolution: an edge is idle when it is out of range or names a node that does not exist;
        # idle lanes read edge/node 0 (callers never launch with zero nodes) and store nothing
        if self.uniform_rows:
            E("const u64 e = blockIdx.x;")
            E("if (e >= nnz) return;")
            E("const u64 ec = e;")
            E("const i64 snd = cols[e], rcv = rows[e];")
        else:
            E(f"const u64 e = (u64)blockIdx.x * {self.R} + sub;")
            E("const u64 ec = e < nnz ? e : nnz - 1;")
            E("const i64 snd = cols[ec], rcv = rows[ec];")
        E("const bool ev = (snd >= 0 && snd < (i64)node_count && rcv >= 0 && rcv < (i64)node_count);")
        if self.uniform_rows:
            E("const bool rv = true; (void)rv;")
            E("if (!ev) {")                                 # whole wavefront: define dY / dW rows, then leave
            if backward:
                E(f"    for (int q = lane; q < {self.WN}; q += 64) Wg[e * {self.WN} + q] = (T)0;")
                E(f"    for (int q = lane; q < {self.D2}; q += 64) Yg[e * {self.D2} + q] = (T)0;")
            E("    return;")
            E("}")
            E("const u64 sndc = (u64)snd, rcvc = (u64)rcv;")
        else:
            E("const bool rv = ev && e < nnz;")
            E("const u64 sndc = rv ? (u64)snd : 0, rcvc = rv ? (u64)rcv : 0;")
        E(f"const T* __restrict__ Yr = Y + ec * {self.D2};")
        E(f"const T* __restrict__ Wr = W + ec * {self.WN};")
        if self.uniform_rows:
            self.xrow_of = (lambda r: ("sndc", "true"))
            self.zrow_of = (lambda r: ("rcvc", "true"))
        else:
            E("const int xsrc = rv ? (int)snd : -1;")
            E("const int zdst = rv ? (int)rcv : -1;")
            self.xrow_of = self._shfl_row("xsrc")
            self.zrow_of = self._shfl_row("zdst")
        return "sndc", "rcvc", "e"

    # =============================================================== forward
    def direct_forward_body(self) -> str:
        E = Emitter()
        atomic = (self.kind == "conv_atomic")
        self.nt_load, self.nt_store = "fl" in self._nt_modes, "fs" in self._nt_modes
        self.emit_lane_direct(E, lds=True)
        xrow, zrow, _ = self._rows(E)
        lazy = self._lazy = self.lazy_operands("forward")
        self.emit_y_load_direct(E)
        for c in range(self.NCH):
            self.emit_x_preload(E, c, xrow)
            if not lazy:
                self.emit_weight_preload(E, c)
        for c in range(self.NCH):
            self._cur_c = self._loop_c = c
            E("{")
            E.level += 1
            E(f"const int c = {c}; (void)c;")
            E(f"const int u = {c * self.P} + ul;")
            self.emit_x_alias(E, c)
            outs = [o for o in self.out if o.dim and o.idx in self.used_out]
            if lazy and outs:
                self.emit_weight_preload(E, c, only={p.t for p in self.paths_into(outs[0].idx)})
            for o in self.out:
                if o.dim == 0:
                    continue
                if lazy and o.idx in self.used_out:
                    # one output block's weights in flight ahead of the block being computed; the fence keeps
                    # the compiler from gathering the loads of all blocks at the top again
                    E("oeq_sched_fence();")
                    self.emit_forget_products(E)
                    nxt = outs[outs.index(o) + 1:]
                    if nxt:
                        self.emit_weight_preload(E, c, only={p.t for p in self.paths_into(nxt[0].idx)})
                E("{")
                E.level += 1
                if o.idx in self.used_out:
                    self.emit_forward_block(E, o, "Wr")
                    self.emit_block_store(E, o, [f"z{k}" for k in range(o.D)], "Z", self.D3, zrow, self.zrow_of,
                                          "atomic" if atomic else "store", via_lds=True)
                elif not atomic:
                    self.emit_record_store(E, ["(T)0"] * o.D, f"Z + (u64){zrow} * {self.D3} + {o.off} + u * {o.D}",
                                           self.act(o))
                E.level -= 1
                E("}")
            E.level -= 1
            E("}")
        return E.text()

    # ============================================================== backward
    def direct_backward_body(self) -> str:
        E = Emitter()
        atomic = (self.kind == "conv_atomic")
        self.nt_load, self.nt_store = "bl" in self._nt_modes, "bs" in self._nt_modes
        self.emit_lane_direct(E, lds=atomic or any(self.dx_through_slot(self.in1[i]) for i in self.used_in1))
        xrow, zrow, srow = self._rows(E, backward=True)
        E(f"T* __restrict__ Wgr = Wg + {srow} * {self.WN};")
        self._lazy = self.lazy_operands("backward")
        self.emit_y_load_direct(E)
        for f in self.used_y:
            E(f"T dy{f} = (T)0;")
        self.emit_looped_dy_begin(E)

        def chunk(E, c):
            tag = c if isinstance(c, int) else "c"
            self._cur_c = tag
            lazy = self._lazy

            def fetch(oi):
                o = self.out[oi]
                self.emit_record_load(E, [f"G{oi}_{k}" for k in range(o.D)],
                                      f"G + (u64){zrow} * {self.D3} + {o.off} + {self.uclamp(o, c)} * {o.D}",
                                      self.act(o), zero=True)
                if lazy:
                    self.emit_weight_preload(E, c, only={p.t for p in self.paths_into(oi)})
            self.emit_x_preload(E, c, xrow)
            if not lazy:
                self.emit_weight_preload(E, c)
            for oi in (self.used_out[:1] if lazy else self.used_out):
                fetch(oi)
            self.emit_x_alias(E, tag)
            for i in self.used_in1:
                for m in range(self.in1[i].D):
                    E(f"T dx{i}_{m} = (T)0;")
            for n_, oi in enumerate(self.used_out):
                o = self.out[oi]
                if lazy:
                    # dZ and weights of one output block in flight ahead of the block being worked on
                    E("oeq_sched_fence();")
                    self.emit_forget_products(E)
                    if n_ + 1 < len(self.used_out):
                        fetch(self.used_out[n_ + 1])
                E("{")
                E.level += 1
                for k in range(o.D):
                    E(f"const T g{k} = G{oi}_{k};")

                def sink(E, p, v, expr):
                    if self.nt_store:
                        E(f"  if ({self.act(p.a)}) oeq_stnt(Wgr + {self.widx(p, 'u', v)}, {expr});")
                    else:
                        E(f"  if ({self.act(p.a)}) Wgr[{self.widx(p, 'u', v)}] = {expr};")
                self.emit_backward_block(E, o, "Wr", sink)
                E.level -= 1
                E("}")
            for a in self.in1:
                if a.dim == 0:
                    continue
                if a.idx in self.used_in1:
                    self.emit_block_store(E, a, [f"dx{a.idx}_{m}" for m in range(a.D)], "Xg", self.D1, xrow,
                                          self.xrow_of, "atomic" if atomic else "store",
                                          via_lds=atomic or self.dx_through_slot(a))
                elif not atomic:
                    self.emit_record_store(E, ["(T)0"] * a.D, f"Xg + (u64){xrow} * {self.D1} + {a.off} + u * {a.D}",
                                           self.act(a))

        if self.NCH <= self.unroll_bwd_chunks:
            for c in range(self.NCH):
                E("{")
                E.level += 1
                E(f"const int c = {c}; (void)c;")
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
        # dY: sum over the lanes of the row in a fixed order (DPP row operations when a row fills the
        # wavefront - the total lands in lane 63 - else the xor butterfly, total in every lane)
        if self.P == 64:
            for f in self.used_y:
                E(f"dy{f} = oeq_wave_sum63(dy{f});")
            writer = "lane == 63"
        else:
            self.emit_dy_reduce(E)
            writer = "ul == 0"
        if self.kind == "tp":
            E(f"if ({writer}) {{")
            E(f"    T* __restrict__ Ygr = Yg + {'row' if self.uniform_rows else 'rowc'} * {self.D2};")
        else:
            E(f"if (e < nnz && {writer}) {{")
            E(f"    T* __restrict__ Ygr = Yg + e * {self.D2};")
        for f in range(self.D2):
            E(f"    Ygr[{f}] = " + (f"dy{f};" if f in self.used_y else
                                   f"{self.looped_dy_value(f)};" if f in self.looped_y else "(T)0;"))
        E("}")
        if self.kind != "tp":
            E("if (e < nnz && !rv) {")
            E(f"    for (int q = ul; q < {self.WN}; q += {self.P}) Wgr[q] = (T)0;")
            E("}")
        return E.text()

    def tp_forward_body(self) -> str:
        return self.direct_forward_body()

    def tp_backward_body(self) -> str:
        return self.direct_backward_body()

    def conv_atomic_forward_body(self) -> str:
        return self.direct_forward_body()

    def conv_atomic_backward_body(self) -> str:
        return self.direct_backward_body()
