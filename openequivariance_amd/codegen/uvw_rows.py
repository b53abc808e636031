"""uvw tensor products with shared weights and FEW weights.

    Z[b, w, k] = sum_t sum_u  W_t[u, w] * T_t[b, u, k],     T_t[b, u, k] = sum_ij c_ijk X[b, u, i] Y[b, j]

The matrix-core kernels of ``uvw.py`` tile u and w in 16s; a problem whose multiplicities are 1 or 6
on one side (the tetris polynomial layers of the reference's uvw benchmark,
benchmark/benchmark_configs.py:38-41) fills a sixteenth of such a tile, and its few hundred weights
make the work a stream over X, Y, Z.  Three vector-ALU kernels:

* forward and backward (dX, dY): a lane owns a batch row.  The weights are the same for every lane:
  a register holds 64 of them, one per lane, and each is read out as the scalar operand of a vector
  FMA; the whole contraction is unrolled at generation time.  A lane reads and writes contiguous
  records of its row (groups of at most ``CHUNK_WORDS`` words), which the compiler merges into
  multi-word accesses; consecutive lanes own consecutive rows, so a wavefront covers a contiguous
  span of each tensor.  The operands of the next group are requested before the current one is used.
* backward_dw: a lane owns weights.  Per tile of ``DW_ROWS`` rows the lanes first compute T of their
  rows into LDS, then dZ is staged a few rows at a time (the next batch travels to registers while
  this one is used), and every lane walks the rows for its weights:
  ``dW[e] += sum_k T[r, t(e) + k] dZ[r, g(e) + k]``, a loop of a few dozen instructions.  (The same sum
  with a row per lane, unrolled over the weights and summed across lanes with a transposing
  butterfly, is 15 000 instructions long, does not fit the instruction cache and ran at the speed of
  the matrix-core kernel it was to replace.)  Weights are dealt to (register, lane) positions by
  2 l3 + 1 so that a register's lanes share the trip count.  The wavefronts are persistent, write one
  partial row each, and backward_reduce sums the rows in a fixed order: deterministic.

What was measured on the way (MI355X, batch 50 000, fp32, first tetris layer): weights as scalar loads
at compile-time offsets are hoisted and spilled by the compiler (a lane read per weight does the same
job in one instruction); a conditional store in the middle of the unrolled code makes the compiler
move the arithmetic of everything stored later past it, with all its operands alive until then (512
registers and scratch): every store is unconditional, lanes past the batch repeat the last row;
Z written as a lane's own records (16 bytes of 64 different cache lines per instruction) takes 30 us for
74 MB whatever the arithmetic beside it, as whole-row runs through the LDS slot 17 us for the whole
kernel - provided the groups are cut so that all of them are whole numbers of vectors.
"""
from __future__ import annotations

import math

import numpy as np

from ..problem import TPProblem
from .common import Emitter, jinja_env
from .uvw import UVWGenerator, _ceil


class UVWRowsGenerator(UVWGenerator):
    CHUNK_WORDS = 32      # words of a row's record held in registers at a time (per operand)
    WAVES = 2048          # upper bound of the dW kernel's persistent wavefronts = partial dW rows
    MAX_WEIGHTS = 2048    # the contraction is unrolled: weights x (2 l3 + 1) vector FMAs ...
    MAX_FMAS = 6000       # ... which have to stay well within the 64 KB instruction cache

    @classmethod
    def suits(cls, problem: TPProblem) -> bool:
        """Few weights, and a matrix-core tiling that would be mostly padding: the instructions' [u][w]
        weight matrices fill less than half of the 16 x 16 tiles that cover them."""
        if not problem.shared_weights or problem.weight_numel > cls.MAX_WEIGHTS:
            return False
        real = padded = nt = fmas = 0
        for ins in problem.instructions:
            mu, mw = problem.irreps_in1[ins.i_in1].mul, problem.irreps_out[ins.i_out].mul
            mv, d3 = problem.irreps_in2[ins.i_in2].mul, problem.irreps_out[ins.i_out].ir.dim
            real += mu * mw
            padded += 16 * _ceil(mu, 16) * 16 * _ceil(mw, 16)
            nt += mu * mv * d3
            fmas += mu * mv * mw * d3
        if fmas > cls.MAX_FMAS:
            return False
        # the dW kernel keeps T of a tile's rows in LDS: at least 8 rows of it must fit its share
        itemsize = 4 if problem.irrep_dtype == np.float32 else 8
        return 2 * real < padded and 8 * (nt | 1) * itemsize <= cls.DW_T_BYTES

    def __init__(self, problem: TPProblem):
        super().__init__(problem)
        if not self.shared:
            raise ValueError("UVWRowsGenerator is for shared weights")
        if self.WN > self.MAX_WEIGHTS:
            raise ValueError(f"UVWRowsGenerator unrolls the contraction: at most {self.MAX_WEIGHTS} weights")
        self.kind = "uvw_rows"
        self.WNP = 64 * _ceil(self.WN, 64)
        # rows of a dW tile: as many (up to DW_ROWS) as keep T of the tile within its share of the LDS
        _, nt = self.t_offsets()
        self.dw_rows = self.DW_ROWS
        while self.dw_rows > 8 and self.dw_rows * (nt | 1) * self.itemsize > self.DW_T_BYTES:
            self.dw_rows //= 2
        if self.dw_rows * (nt | 1) * self.itemsize > self.DW_T_BYTES:
            raise ValueError("UVWRowsGenerator: T of 8 rows does not fit the LDS share of the dW kernel")
        self.ws_elems = self.WAVES * self.npos

    def describe(self) -> str:
        return (f"uvw shared weights, one row per lane T={self.T} paths={len(self.paths)} d1={self.D1} d2={self.D2} "
                f"d3={self.D3} wn={self.WN} (vector ALU, HBM bound) workspace={self.ws_elems * self.itemsize}B")

    # ------------------------------------------------------------------ pieces
    def groups(self, blocks):
        """A row cut into runs of whole channel records of at most CHUNK_WORDS words each: a list of groups, a
        group a list of (block, first channel, end channel), contiguous in memory.  A block's records are
        taken four (fp64: two) at a time as far as its multiplicity allows, so that the group is a whole number
        of 16-byte vectors and can leave through the LDS slot as whole-row runs; the records that are left
        over (fewer than four) form groups of their own, together with the left-overs of the next blocks."""
        vw = 16 // self.itemsize
        if sum(blk.dim for blk in blocks) <= self.CHUNK_WORDS:          # a short row is one group
            return [[(blk, 0, blk.mul) for blk in blocks if blk.dim]]
        out, cur, words, tails = [], [], 0, False

        def close():
            nonlocal cur, words, tails
            if cur:
                out.append(cur)
            cur, words, tails = [], 0, False

        def add(blk, lo, hi, tail):
            nonlocal words, tails
            cur.append((blk, lo, hi))
            words += (hi - lo) * blk.D
            tails = tails or tail
        for blk in blocks:
            if not blk.dim:
                continue
            step = vw // math.gcd(vw, blk.D)           # records per whole number of vectors
            full, pos = blk.mul // step * step, 0
            while pos < full:
                if tails:
                    close()
                room = max(0, self.CHUNK_WORDS - words) // (blk.D * step) * step
                if room == 0 and cur:
                    close()
                    continue
                take = min(full - pos, max(room, step))
                add(blk, pos, pos + take, False)
                pos += take
            if pos < blk.mul:
                if cur and (not tails or words + (blk.mul - pos) * blk.D > self.CHUNK_WORDS):
                    close()
                add(blk, pos, blk.mul, True)
        close()
        return out

    @staticmethod
    def span(group):
        """(first word, number of words) of a group within its row."""
        blk, lo, _ = group[0]
        start = blk.off + lo * blk.D
        return start, sum((hi - lo_) * b.D for b, lo_, hi in group)

    def windex(self, p, u: int, w: int) -> int:
        return int(eval(self.oeq_index(p, str(u), str(w)), {"min": min}))

    def paths_between(self, a_idx: int, o_idx: int):
        return [p for p in self.paths if p.a.idx == a_idx and p.o.idx == o_idx]

    def linked(self, xg, zg) -> bool:
        return any(self.paths_between(a.idx, o.idx) for a, _, _ in xg for o, _, _ in zg)

    def contraction(self, xg, zg):
        """(path, u, w) of the weights between two groups, in the order both kernels visit them."""
        for a, u0, u1 in xg:
            for o, w0, w1 in zg:
                for p in self.paths_between(a.idx, o.idx):
                    for u in range(u0, u1):
                        for w in range(w0, w1):
                            yield p, u, w

    def emit_rows(self, E: Emitter) -> None:
        E("const int lane = threadIdx.x;")

    def emit_weights(self, E: Emitter) -> None:
        """Weight e of the external order in lane e % 64 of register W(e / 64): one coalesced load each."""
        for q in range(self.WNP // 64):
            idx = f"{64 * q} + lane"
            E(f"const T W{q} = W[{idx}];" if 64 * (q + 1) <= self.WN else f"const T W{q} = W[min({idx}, {self.WN - 1})];")

    FENCE_WEIGHTS = 24    # the scheduler may not gather the lane reads of more weights than the SGPR file holds

    def emit_fence(self, E: Emitter, since: int) -> int:
        if since >= self.FENCE_WEIGHTS:
            E("oeq_sched_fence();")
            return 1
        return since + 1

    def weight(self, p, u: int, w: int) -> str:
        e = self.windex(p, u, w)
        return f"oeq_lane_value(W{e // 64}, {e % 64})"

    def emit_tile(self, E: Emitter, tile: str, zero_y: bool = False, rows: int = 64) -> None:
        """Lanes past the batch repeat its last row, stores included (the same values to the same addresses):
        no branch anywhere, so nothing of a row's arithmetic can be moved into a conditional block at the
        end of the kernel, which would keep every operand of the row alive until then."""
        E(f"const u64 tile0 = ({tile}) * {rows};")
        E("const u64 row_ = tile0 + lane;")
        E("const bool act = row_ < n" + (f" && lane < {rows};" if rows < 64 else ";"))
        E("const u64 row = act ? row_ : n - 1;")
        E(f"const T* __restrict__ Yr = Y + row * {self.D2};")
        for f in self.used_y:
            if zero_y:
                E(f"const T yr{f} = Yr[{f}];")
                E(f"const T y{f} = act ? yr{f} : (T)0;")
            else:
                E(f"const T y{f} = Yr[{f}];")

    def emit_group_load(self, E: Emitter, name: str, ptr: str, group) -> None:
        """{name}{word offset of the record}_{i} = the group's words of this lane's row."""
        start, words = self.span(group)
        E(f"const T* __restrict__ {name}p = {ptr} + {start};")
        decl = []
        for blk, lo, hi in group:
            for u in range(lo, hi):
                base = blk.off + u * blk.D
                decl += [f"{name}{base}_{i} = {name}p[{base + i - start}]" for i in range(blk.D)]
        E("const T " + ", ".join(decl) + ";")

    def slot_words(self) -> int:
        """LDS words of the slot that turns a wavefront's records (one row per lane) into whole-row runs."""
        vw = 16 // self.itemsize
        longest = max(self.span(g)[1] for blocks in (self.in1, self.out) for g in self.groups(blocks))
        return 64 * (max(self.CHUNK_WORDS, longest) + vw)      # (four records of l >= 4 exceed CHUNK_WORDS)

    def emit_group_store(self, E: Emitter, name: str, ptr: str, group, rowdim: int) -> None:
        """The group's words of all 64 rows -> memory.  A lane's own record store touches 16 bytes of 64
        different cache lines per instruction (measured: Z of the first tetris layer at 2 TB/s); through an
        LDS slot [row][words] the same data leaves as 16-byte vectors that cover whole 128-byte runs of a row.
        ``ptr`` is the tensor.  Slot rows past the batch hold the last row's values once more and are written
        onto it: a conditional store here would split the kernel into blocks, and the compiler then moves the
        arithmetic of values stored later (dY) past them, with every operand alive until then.  Groups that
        do not divide into vectors keep the record stores."""
        start, words = self.span(group)
        vw = 16 // self.itemsize
        vals = []
        for blk, lo, hi in group:
            for u in range(lo, hi):
                vals += [f"{name}{blk.off + u * blk.D}_{i}" for i in range(blk.D)]
        if words % vw:
            E(f"{{ T* __restrict__ q_ = {ptr} + row * {rowdim} + {start}; "
              + " ".join(f"q_[{j}] = {v};" for j, v in enumerate(vals)) + " }")
            return
        stride, per_row = words + vw, words // vw
        E("oeq_sync();")
        for j in range(0, words, vw):
            E(f"{{ VT v_; " + " ".join(f"v_[{h}] = {vals[j + h]};" for h in range(vw))
              + f" *(VT*)(slot + lane * {stride} + {j}) = v_; }}")
        E("oeq_sync();")
        for it in range(per_row):
            E(f"{{ const int q_ = {64 * it} + lane, r_ = q_ / {per_row}, c_ = q_ - r_ * {per_row};")
            E(f"  *(VTU*)({ptr} + (tile0 + r_ < n ? tile0 + r_ : n - 1) * {rowdim} + {start} + c_ * {vw}) = "
              f"*(const VT*)(slot + r_ * {stride} + c_ * {vw}); }}")

    # ----------------------------------------------------------------- forward
    def forward_body(self) -> str:
        """For a group of output records, walk the groups of input records that reach it; the next input group
        is requested before the current one is multiplied."""
        E = Emitter()
        self.emit_rows(E)
        E(f"__shared__ __attribute__((aligned(16))) T slot[{self.slot_words()}];")
        self.emit_weights(E)
        self.emit_tile(E, "(u64)blockIdx.x")
        E(f"const T* __restrict__ Xr = X + row * {self.D1};")
        E(f"T* __restrict__ Zr = Z + row * {self.D3};")
        xgs, zgs = self.groups(self.in1), self.groups(self.out)
        stages = [(zi, xi) for zi, zg in enumerate(zgs) for xi, xg in enumerate(xgs) if self.linked(xg, zg)]
        # a single input group stays in registers for the whole row; otherwise every stage requests the next
        # one's (a load issued after a group's stores cannot be waited for without waiting for those stores:
        # with one group nothing is loaded once the first output leaves)
        keep = len(xgs) == 1
        xname = (lambda s_: "x_") if keep else (lambda s_: f"x{s_}_")
        if stages:
            self.emit_group_load(E, xname(0), "Xr", xgs[stages[0][1]])
        done = set()
        for s_, (zi, xi) in enumerate(stages):
            zg, xg = zgs[zi], xgs[xi]
            E("oeq_sched_fence();")
            since = 0
            if s_ + 1 < len(stages) and not keep:
                self.emit_group_load(E, xname(s_ + 1), "Xr", xgs[stages[s_ + 1][1]])
            if zi not in done:
                done.add(zi)
                E("T " + ", ".join(f"z{o.off + w * o.D}_{k} = (T)0" for o, w0, w1 in zg for w in range(w0, w1)
                                   for k in range(o.D)) + ";")
            last = None
            for p, u, w in self.contraction(xg, zg):
                if (p.t, u) != last:
                    last = (p.t, u)
                    t = f"t{s_}_{p.t}_{u}_"
                    self.emit_cg_forward(E, p, f"{xname(s_)}{p.a.off + u * p.a.D}_", "y", t)
                z = f"z{p.o.off + w * p.o.D}_"
                since = self.emit_fence(E, since)
                E(f"{{ const T w_ = {self.weight(p, u, w)}; " + " ".join(
                    f"{z}{k} = oeq_fma(w_, {t}{k}, {z}{k});" for k in range(p.o.D)) + " }")
            if s_ + 1 == len(stages) or stages[s_ + 1][0] != zi:
                self.emit_group_store(E, "z", "Z", zg, self.D3)
        for zi, zg in enumerate(zgs):
            if zi not in done:                 # no instruction writes these records
                start, words = self.span(zg)
                E(f"{{ T* __restrict__ q_ = Zr + {start}; " + " ".join(f"q_[{i}] = (T)0;" for i in range(words)) + " }")
        return E.text()

    # ---------------------------------------------------------------- backward
    def backward_body(self) -> str:
        """dX, dY.  For a group of input records, walk the groups of dZ records it reaches (the next one
        requested ahead): dT = W dZ, then the CG transpose."""
        E = Emitter()
        self.emit_rows(E)
        E(f"__shared__ __attribute__((aligned(16))) T slot[{self.slot_words()}];")
        self.emit_weights(E)
        self.emit_tile(E, "(u64)blockIdx.x")
        for f in self.used_y:
            E(f"T dy{f} = (T)0;")
        E(f"const T* __restrict__ Xr = X + row * {self.D1};")
        E(f"const T* __restrict__ Gr = G + row * {self.D3};")
        E(f"T* __restrict__ Xgr = Xg + row * {self.D1};")
        xgs, zgs = self.groups(self.in1), self.groups(self.out)
        stages = [(xi, zi) for xi, xg in enumerate(xgs) for zi, zg in enumerate(zgs) if self.linked(xg, zg)]
        keep = len(zgs) == 1                   # a single dZ group stays in registers (see forward_body)
        gname = (lambda s_: "g_") if keep else (lambda s_: f"g{s_}_")
        if stages:
            self.emit_group_load(E, f"x{stages[0][0]}_", "Xr", xgs[stages[0][0]])
            self.emit_group_load(E, gname(0), "Gr", zgs[stages[0][1]])
        begun = set()
        for s_, (xi, zi) in enumerate(stages):
            xg, zg = xgs[xi], zgs[zi]
            E("oeq_sched_fence();")
            since = 0
            if s_ + 1 < len(stages):
                nxi, nzi = stages[s_ + 1]
                if nxi != xi:
                    self.emit_group_load(E, f"x{nxi}_", "Xr", xgs[nxi])
                if not keep:
                    self.emit_group_load(E, gname(s_ + 1), "Gr", zgs[nzi])
            if xi not in begun:
                begun.add(xi)
                E("T " + ", ".join(f"dx{a.off + u * a.D}_{i} = (T)0" for a, u0, u1 in xg for u in range(u0, u1)
                                   for i in range(a.D)) + ";")
            last, cgb = None, None
            for p, u, w in self.contraction(xg, zg):
                if (p.t, u) != last:
                    if last is not None:
                        self.emit_cg_backward(E, *cgb)
                    last = (p.t, u)
                    dt = f"dt{s_}_{p.t}_{u}_"
                    cgb = (p, dt, f"x{xi}_{p.a.off + u * p.a.D}_", "y", f"dx{p.a.off + u * p.a.D}_", "dy")
                    E("T " + ", ".join(f"{dt}{k} = (T)0" for k in range(p.o.D)) + ";")
                g = f"{gname(s_)}{p.o.off + w * p.o.D}_"
                since = self.emit_fence(E, since)
                E(f"{{ const T w_ = {self.weight(p, u, w)}; " + " ".join(
                    f"{dt}{k} = oeq_fma(w_, {g}{k}, {dt}{k});" for k in range(p.o.D)) + " }")
            if last is not None:
                self.emit_cg_backward(E, *cgb)
            if s_ + 1 == len(stages) or stages[s_ + 1][0] != xi:
                self.emit_group_store(E, "dx", "Xg", xg, self.D1)
        for xi, xg in enumerate(xgs):
            if xi not in begun:                # no instruction reads these records
                start, words = self.span(xg)
                E(f"{{ T* __restrict__ q_ = Xgr + {start}; " + " ".join(f"q_[{i}] = (T)0;" for i in range(words)) + " }")
        E(f"{{ T* __restrict__ yp = Yg + row * {self.D2}; " + " ".join(
            f"yp[{f}] = " + (f"dy{f};" if f in self.used_y else "(T)0;") for f in range(self.D2)) + " }")
        return E.text()

    # --------------------------------------------------------------------- dW
    def t_offsets(self):
        """Offset of T_t[u, :] in a row of the LDS copy of T, and the row's length."""
        off, acc = {}, 0
        for p in self.paths:
            for u in range(p.mu):
                off[(p.t, u)] = acc
                acc += p.o.D
        return off, acc

    def dw_positions(self):
        """Weights dealt to positions (register q = pos / 64, lane = pos % 64), registers filled with weights
        of one 2 l3 + 1 at a time: [(D, [(path, u, w) or None] * 64)] per register."""
        regs = []
        for D in sorted({p.o.D for p in self.paths}):
            ws = [(p, u, w) for p in self.paths if p.o.D == D for u in range(p.mu) for w in range(p.mw)]
            for i in range(0, len(ws), 64):
                chunk = ws[i:i + 64]
                regs.append((D, chunk + [None] * (64 - len(chunk))))
        return regs

    def dw_tables(self):
        """C initialisers: per position the offsets into a T row and a dZ row, and the external weight index
        (0xffff for the unused positions of a partly filled register)."""
        toff, _ = self.t_offsets()
        tb, gb, ext = [], [], []
        for D, lanes in self.dw_positions():
            for e in lanes:
                if e is None:
                    tb.append(0), gb.append(0), ext.append(0xffff)
                else:
                    p, u, w = e
                    tb.append(toff[(p.t, u)]), gb.append(p.o.off + w * p.o.D), ext.append(self.windex(p, u, w))
        assert sorted(x for x in ext if x != 0xffff) == list(range(self.WN))
        return (", ".join(map(str, tb)), ", ".join(map(str, gb)), ", ".join(map(str, ext)), len(ext))

    @property
    def npos(self) -> int:
        return 64 * len(self.dw_positions())

    def dw_lds(self):
        """(row stride of T, row stride of dZ, rows of dZ staged at a time): odd strides, and a batch of rows
        that keeps the workgroup within DW_LDS_BYTES so that four fit a compute unit."""
        _, nt = self.t_offsets()
        ts, gs = nt | 1, self.D3 | 1
        rb = self.dw_rows
        while rb > 1 and (self.dw_rows * ts + rb * gs) * self.itemsize > self.DW_LDS_BYTES:
            rb //= 2
        return ts, gs, rb

    DW_LDS_BYTES = 24 * 1024
    DW_UNROLL = 0         # rows of the dW loop unrolled together (0: by type, see backward_dw_body)
    DW_ROWS = 32          # rows of a dW tile (fewer when T of so many rows would not fit DW_T_BYTES)
    DW_T_BYTES = 16 * 1024

    def backward_dw_body(self) -> str:
        E = Emitter()
        ts, gs, rb = self.dw_lds()
        toff, nt = self.t_offsets()
        regs = self.dw_positions()
        R_ = self.dw_rows
        E("const int lane = threadIdx.x;")
        E(f"__shared__ T Tl[{R_ * ts}];")
        E(f"__shared__ T Gl[{rb * gs}];")
        for q in range(len(regs)):
            E(f"const int tb{q} = oeq_dw_t[{64 * q} + lane], gb{q} = oeq_dw_g[{64 * q} + lane];")
        E("T " + ", ".join(f"A{q} = (T)0" for q in range(len(regs))) + ";")
        E(f"const u64 tiles = (n + {R_ - 1}) / {R_};")
        E("for (u64 tile = blockIdx.x; tile < tiles; tile += gridDim.x) {")
        E.level += 1
        E(f"const u64 row0 = tile * {R_};")
        self.emit_tile(E, "tile", zero_y=True, rows=R_)
        # dZ: rb rows at a time, contiguous in memory; the next batch travels to registers while this one is used
        nit = _ceil(rb * self.D3, 64)
        dest = "i_" if gs == self.D3 else f"i_ + i_ / {self.D3}"
        E(f"T R[{nit}];")
        E("int limit;                     // words of the requested batch that lie within the tensor")

        def request(r0: str):
            E(f"{{ const T* __restrict__ gp = G + (row0 + {r0}) * {self.D3};")
            E(f"  const u64 left = n - (row0 + {r0});")
            E(f"  limit = (int)(left < {rb} ? left : {rb}) * {self.D3};")
            E("#pragma unroll")
            E(f"  for (int i = 0; i < {nit}; ++i) R[i] = gp[min(64 * i + lane, limit - 1)];")
            E("}")
        request("0")
        # T of this lane's row (zero past the batch, which also voids whatever dZ holds there)
        E(f"const T* __restrict__ Xr = X + row * {self.D1};")
        E("oeq_sync();")
        xgs = self.groups(self.in1)
        for xi, xg in enumerate(xgs):
            if not any(p.a.idx == a.idx for a, _, _ in xg for p in self.paths):
                continue
            E("{")
            E.level += 1
            self.emit_group_load(E, "x", "Xr", xg)
            for a, u0, u1 in xg:
                for p in self.paths:
                    if p.a.idx != a.idx:
                        continue
                    for u in range(u0, u1):
                        E("{")
                        self.emit_cg_forward(E, p, f"x{a.off + u * a.D}_", "y", "t")
                        E((f"if (lane < {R_}) {{ " if R_ < 64 else "{ ")
                          + " ".join(f"Tl[lane * {ts} + {toff[(p.t, u)] + k}] = t{k};" for k in range(p.o.D)) + " }")
                        E("}")
            E.level -= 1
            E("}")
        E(f"for (int r0 = 0; r0 < {R_} && row0 + r0 < n; r0 += {rb}) {{")
        E.level += 1
        E("oeq_sync();")
        E("#pragma unroll")
        E(f"for (int i = 0; i < {nit}; ++i) {{ const int i_ = 64 * i + lane; if (i_ < {rb * self.D3}) Gl[{dest}] = i_ < limit ? R[i] : (T)0; }}")
        E("oeq_sync();")
        E(f"if (r0 + {rb} < {R_} && row0 + r0 + {rb} < n) {{")
        E.level += 1
        request(f"r0 + {rb}")
        E.level -= 1
        E("}")
        # fp32: the whole batch unrolled, so that a row is an immediate offset of the LDS reads (35 -> 28 us on the
        # first tetris layer); fp64 has no registers for that (56 -> 82 us)
        E(f"#pragma unroll {self.DW_UNROLL or (rb if self.T == 'float' else 2)}")
        E(f"for (int r = 0; r < {rb}; ++r) {{")
        E(f"    const T* __restrict__ tr = Tl + (r0 + r) * {ts};")
        E(f"    const T* __restrict__ gr_ = Gl + r * {gs};")
        for q, (D, _) in enumerate(regs):
            E(f"    A{q} += " + " + ".join(f"tr[tb{q} + {k}] * gr_[gb{q} + {k}]" for k in range(D)) + ";")
        E("}")
        E.level -= 1
        E("}")
        E.level -= 1
        E("}")
        E(f"T* __restrict__ part = (T*)ws + (u64)blockIdx.x * {self.npos};")
        for q in range(len(regs)):
            E(f"part[{64 * q} + lane] = A{q};")
        return E.text()

    def reduce_body(self) -> str:
        """dW = sum over the wavefronts that ran.  A workgroup owns 16 positions; 64 threads share a position, each
        sums every 64th partial row in row order, and the 64 sums are added in a fixed order."""
        E = Emitter()
        E("const int l = threadIdx.x & 15, sub = threadIdx.x >> 4, pos = blockIdx.x * 16 + l;")
        E("__shared__ T sums[1024];")
        E(f"const u64 tiles = (n + {self.dw_rows - 1}) / {self.dw_rows};")
        E(f"const u64 rows = tiles < {self.WAVES} ? tiles : {self.WAVES};")
        E("const T* __restrict__ part = (const T*)ws;")
        E("T s = (T)0;")
        E("#pragma unroll 8")
        E(f"for (u64 r = sub; r < rows; r += 64) s += part[r * {self.npos} + pos];")
        E("sums[threadIdx.x] = s;")
        E("__syncthreads();")
        E("const int e = oeq_dw_e[pos];")
        E("if (sub == 0 && e != 0xffff) {")
        E("    T t = sums[l];")
        E("    for (int j = 1; j < 64; ++j) t += sums[16 * j + l];")
        E("    Wg[e] = t;")
        E("}")
        return E.text()

    def render(self, prelude: str = None) -> str:
        env = jinja_env()
        if prelude is None:
            prelude = env.get_template("prelude.hip.jinja").render(T=self.T)
        return env.get_template("tp_uvw_rows.hip.jinja").render(g=self, prelude=prelude)

    def plan(self):
        FIXED, ROW = 0, 1
        fwd = [dict(kernel="forward", num_threads=64, grid_kind=ROW, work_per_block=64)]
        bwd = [dict(kernel="backward", num_threads=64, grid_kind=ROW, work_per_block=64),
               dict(kernel="backward_dw", num_threads=64, grid_kind=ROW, work_per_block=self.dw_rows, num_blocks=self.WAVES),
               dict(kernel="backward_reduce", num_threads=1024, grid_kind=FIXED, num_blocks=self.npos // 16)]
        return fwd, bwd, (lambda nnz=0, nodes=0: self.ws_elems * self.itemsize)
