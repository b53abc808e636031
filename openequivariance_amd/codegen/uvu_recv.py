"""Deterministic fused convolution whose backward walks the edges in receiver order, in two passes.

The segmented backward of ``uvu_det.py`` owns one sender per wavefront and gathers a whole row of dZ
per edge: with d3 values per row that is E * d3 words of gathered traffic, the largest stream of the
kernel.  Here the edge list is walked in the order it is given (sorted by receiver):

* pass 1 (``backward``): a wavefront owns a tile of consecutive edges and one 64-channel chunk.  It
  keeps ``dZ[receiver]`` of the chunk in registers and reloads it only when the receiver changes
  (about once per in-degree edges), gathers ``X[sender]`` per edge (d1 words instead of d3), streams W
  and Y, writes dW[e] and dY[e], and writes the edge's contribution to dX[sender] into a spill row of
  its own in the workspace.  Nothing is accumulated across edges, so every tile is independent and the
  work is balanced whatever the degree distribution;
* pass 2 (``backward_dx``): a wavefront owns (sender, chunk) and sums the spill rows of the sender's
  edges in the order of the transpose permutation: fixed order, bit-reproducible.

Traffic next to the sender-order backward: the gather shrinks from E * d3 to E * d1 words, and
2 * E * d1 words of spill are added, so this order moves fewer bytes when d3 > 3 * d1 or so (the
gathers of dZ are partly served by caches, the spill is not).  The spill layout is this generator's
own: word w of lane u of chunk c of edge e at ``((e * chunks + c) * words + w) * P + u``, so that
every spill access of a wavefront is one contiguous run.

Workgroup ids map to (tile, chunk) so that each XCD (id modulo 8) sweeps a contiguous range of
tiles: the dZ row of a receiver whose edges span two tiles is then re-read from that XCD's L2.
"""
from __future__ import annotations

from ..problem import TPProblem
from .common import Emitter
from .uvu_det import UVUDetGenerator


class UVURecvGenerator(UVUDetGenerator):
    # Arithmetic form of pass 1 (see UVUGenerator.regroup_pairs).  With register loads, pass 1 holds a dZ row and an
    # edge's operands in registers and the regrouped form spills 27 instead of 13 words per lane on the 128-channel
    # MACE problem (2.63 against 2.08 ms); with the operands staged through LDS it needs fewer registers than the
    # pair-at-a-time form (175 against 218 there) and is faster on every shape measured (MACE 1.73 against 1.81 ms,
    # 256 channels with outputs of either parity 9.5 against 9.8 ms).
    regroup_pairs = False
    REGROUP_STAGED = True
    # Tile counts from 4096 to one tile per 16 edges and 2 / 4 / 8 spill rows in flight in pass 2 moved pass 1 by
    # less than 4 % (256 channels: 6.39 - 6.71 ms)
    MIN_TILE_ITERS = 8       # edge-loop iterations of the smallest tile
    MAX_TILES = 16384        # tiles per chunk of the largest launches (the tile then grows with the edge count)
    DX_UNROLL = 4            # spill rows in flight per lane group in pass 2
    # dZ words per lane above which pass 1 runs in several launches (0: never); with one row group per wavefront
    # RECV_SPLIT_WORDS_ONE_GROUP (30 paths, 102 words, 5000 nodes / 150 000 edges: at 32 channels - two row groups - 0.488
    # ms in one launch, 0.421 ms in two; at 64 channels 0.781 and 0.804 ms)
    RECV_SPLIT_WORDS = 100
    RECV_SPLIT_WORDS_ONE_GROUP = 128
    # the same for pass 1 with register loads.  fp64 (no stage): unsplit, the dZ row, an edge's operands and its results
    # need more than 512 registers (17 paths at 128 channels, 5000 nodes / 150 000 edges: 3.90 ms against 2.51 ms in
    # sender order); a launch per in1 block - 16 / 25 / 30 words held, 127 - 336 registers - takes 2.49 ms, and 30 paths
    # at 32 / 64 channels 1.00 / 1.73 ms against 1.32 / 1.98 ms
    RECV_SPLIT_WORDS_REGISTER_LOADS = {"float": 0, "double": 32}

    def __init__(self, problem: TPProblem, vector_stores: bool = True, idx_ctype: str = "i64", prefetch=None, staged=None,
                 backward_perm: bool = False, recv_split=None):
        # pass 1 is one launch: the per-edge dX rows cannot be split over launches of output-block groups.
        # ``backward_perm``: the edge list is in no order; pass 1 walks the receiver-grouped position list and pass
        # 2 the sender-grouped one, both built in the workspace by the grouping kernels.
        super().__init__(problem, vector_stores=vector_stores, idx_ctype=idx_ctype, allow_split=False,
                         backward_perm=backward_perm)
        assert self.H == 1
        self.lds_backward = False
        self.waves_per_eu = 0
        self.ordered_backward = False
        # words of dX one lane produces per edge (= spill words per lane)
        self.NW = sum(self.in1[i].D for i in self.used_in1)
        self.spill_row = self.NCH * self.NW * self.P              # words per edge
        # registers: dZ of the receiver + one or two sets of (X records, weights, Y)
        held = sum(self.out[i].D for i in self.used_out)
        per_edge = self.NW + sum(p.mv for p in self.paths) + len(self.used_y)
        # One register set measured faster than two on every shape tried (config 3: 0.182 vs 0.202 ms,
        # config 5: 7.93 vs 8.01 ms, the 128-channel MACE problem: 2.14 vs 5.05 ms, where two sets leave one
        # wavefront per SIMD); ``prefetch=True`` turns the second set on.
        self.prefetch_edges = bool(prefetch)
        # large per-edge footprints: hold the allocation to two wavefronts per SIMD (a handful of spilled
        # words) instead of one
        self.waves_hint = 2 if held + per_edge > 100 else 0
        # Pass 1 with the next edge's operands (X of the sender, W, Y) in flight to LDS by LDS-DMA, which holds
        # no registers: dZ of the receiver and one edge's operands together leave no room for a second register
        # set, so with register loads the loop runs one edge at a time with its load latency exposed.  Measured
        # backward, register loads against staged (both pair-at-a-time): MACE problem 2.07 -> 1.83 ms, 256 channels
        # with outputs of either parity 16.3 -> 9.9 ms, 256 channels 7.84 -> 7.74 ms, 32 channels 0.201 -> 0.179 ms.
        # The staged kernels are left to the occupancy their register count gives (138 - 175: two or three
        # wavefronts per SIMD).
        self.can_stage = self.T == "float" and self.P >= self.D2      # (the Y slab holds one word per lane of a row's group)
        self.staged_edges = self.can_stage and (True if staged is None else bool(staged))
        self.regroup_pairs = bool(self.REGROUP_STAGED and self.staged_edges)
        if self.staged_edges:
            self.waves_hint = 0
        # Pass 1 in several launches when the dZ row of a receiver is too long to hold beside an edge's operands
        # (312 words per lane with 68 paths: 512 registers and scratch): the output blocks are grouped so that no
        # in1 block is read by paths of two groups, hence every launch writes words of the per-edge dX rows that
        # no other launch writes, and its own rows of dW; dY goes through one partial row per (chunk, launch).
        self.spill_word, w = {}, 0
        for i in self.used_in1:
            for m in range(self.in1[i].D):
                self.spill_word[(i, m)] = w
                w += 1
        limit = ((self.RECV_SPLIT_WORDS if self.R > 1 else self.RECV_SPLIT_WORDS_ONE_GROUP) if self.staged_edges
                 else self.RECV_SPLIT_WORDS_REGISTER_LOADS[self.T]) \
            if recv_split is None else recv_split
        self.recv_groups = self._disjoint_groups(limit)
        self.HR = len(self.recv_groups)
        # pass 1 with register loads is worth choosing (fp64 only): every launch holds few
        # enough dZ words to leave room for an edge's operands and results
        self.register_loads_fit = (self.T == "double" and not self.staged_edges and
                                   max(sum(self.out[i].D for i in g_) for g_ in self.recv_groups)
                                   <= self.RECV_SPLIT_WORDS_REGISTER_LOADS["double"])
        self.dy_slots = self.NCH * self.HR
        if not backward_perm:
            self.dypart_off = "(2 * (node_count + 1) + node_count) * sizeof(i64)"
        self.spill_off = (f"((({self.dypart_off} + {self.dy_slots if self.dy_slots > 1 else 0}ull * nnz * {self.D2} * sizeof(T)) "
                          "+ 255ull) & ~255ull)")
        # the preparation's per-256-edge flags are not used here (pass 1 visits every edge and writes the
        # rows of edges naming no node itself): they go behind the spill
        self.flags_off = f"({self.spill_off} + nnz * {self.spill_row}ull * sizeof(T))"
        self.piece_base = f"((({self.flags_off} + 4ull * ((nnz + 255) / 256)) + 255ull) & ~255ull)"

    def describe(self) -> str:
        return super().describe() + f" receiver-order backward (spill {self.spill_row} words/edge)"

    # ------------------------------------------------------------------ plan
    def backward_steps(self):
        steps = [dict(kernel=name, num_threads=64, grid_kind=1, work_per_block=self.MIN_TILE_ITERS * self.R,
                      num_blocks=self.MAX_TILES, grid_y=self.NCH) for name, _ in self.backward_kernels()] \
            + [dict(kernel="backward_dx", num_threads=64, grid_kind=3, work_per_block=1, num_blocks=self.LONG, grid_y=self.NCH)]
        if self.dy_slots > 1:
            steps.append(dict(kernel="backward_dy_reduce", num_threads=256, grid_kind=1,
                              work_per_block=self.dy_rows_per_block))
        return steps

    def spill_bytes(self, nnz: int) -> int:
        return nnz * self.spill_row * self.itemsize

    def plan(self):
        fwd, bwd, _ = super().plan()

        def ws(nnz=0, nodes=0):
            return self.main_bytes(nnz, nodes) + self.piece_bytes(nnz, nodes)
        return fwd, bwd, ws

    def main_bytes(self, nnz: int, nodes: int) -> int:
        head = (2 * self.group_bytes(nnz, nodes) if self.backward_perm else 2 * (nodes + 1) * 8) + nodes * 8 \
            + self.dy_partial_bytes(nnz)
        return ((((head + 255) & ~255) + self.spill_bytes(nnz) + self.flag_bytes(nnz)) + 255) & ~255

    def _disjoint_groups(self, limit: int):
        """Groups of output blocks of at most ``limit`` words per channel (where the problem allows) such that no in1
        block is read by paths of two groups: the connected sets of (output block, in1 block) are packed in the
        order of their in1 blocks."""
        held = lambda outs: sum(self.out[i].D for i in outs)
        if not limit or held(self.used_out) <= limit:
            return [list(self.used_out)]
        sets = []                                        # (in1 blocks, output blocks) connected through paths
        for oi in self.used_out:
            ins, outs = {p.a.idx for p in self.paths_into(oi)}, {oi}
            for t in [t for t in sets if t[0] & ins]:
                sets.remove(t)
                ins |= t[0]
                outs |= t[1]
            sets.append((ins, outs))
        groups = []
        for ins, outs in sorted(sets, key=lambda t: min(t[0])):
            if groups and held(groups[-1]) + held(outs) <= limit:
                groups[-1] += sorted(outs)
            else:
                groups.append(sorted(outs))
        return [sorted(g_) for g_ in groups]

    def group_waves_hint(self) -> int:
        """``waves_hint`` for a launch of pass 1 (launches over groups are left to their register count)."""
        return self.waves_hint if self.HR == 1 else 0

    def backward_kernels(self):
        return [("backward" if h == 0 else f"backward_g{h}", h) for h in range(self.HR)]

    def backward_kernel_sources(self):
        def attr(h):
            with self._group(h, self.recv_groups):
                w = self.group_waves_hint()
            return f" __attribute__((amdgpu_waves_per_eu({w}, {w})))" if w else ""
        return [dict(name=name, threads=64, attr=attr(h), body=self._edges_body(h)) for name, h in self.backward_kernels()] \
            + [dict(name="backward_dx", threads=64, attr="", body=self._dx_body())]

    # ---------------------------------------------------------------- pass 1
    def _edges_body(self, h: int = 0) -> str:
        E = Emitter()
        R, P, NCH = self.R, self.P, self.NCH
        self.emit_lane_direct(E, lds=False)
        with self._group(h, self.recv_groups):
            return self._edges_body_staged(E, h) if self.staged_edges else self._edges_body_registers(E, h)

    def _edges_body_registers(self, E: Emitter, grp: int = 0) -> str:
        R, P, NCH = self.R, self.P, self.NCH
        self._emit_tile_header(E, grp)
        E("bool rv = false;")
        for oi in self.used_out:
            E("T " + ", ".join(f"G{oi}_{k} = (T)0" for k in range(self.out[oi].D)) + ";")
        E("i64 cur_rcv = -1;")
        if self.backward_perm:
            E("const i64* __restrict__ rlist = (const i64*)ws + 2 * (node_count + 1);     // edge ids grouped by receiver")
        names = []
        for i in self.used_in1:
            names += [f"x{i}_{m}" for m in range(self.in1[i].D)]
        names += [f"We_{p.t}_{v}" for p in self.paths for v in range(p.mv)]
        names += [f"y{f}" for f in self.used_y]

        def load_idx(E, it, q):
            E("{")
            E.level += 1
            if self.backward_perm:
                # the tile's positions of the receiver-grouped list name the edges
                E(f"const bool lv = {self.edge_pos(it)} < len;")
                E(f"const i64 e0 = rlist[lv ? beg + (u64){self.edge_pos(it)} : beg];")
                E("const bool ev = lv && e0 >= 0 && e0 < (i64)nnz;")
                E("const u64 e = ev ? (u64)e0 : nnz - 1;")
            else:
                E(f"const bool ev = {self.edge_pos(it)} < len;")
                E(f"const u64 e = ev ? beg + (u64){self.edge_pos(it)} : nnz - 1;      // idle lane groups re-read the last edge, masked below")
            E("const i64 snd = cols[e], rcv = rows[e];")
            E("const bool ok = ev && snd >= 0 && snd < (i64)node_count && rcv >= 0 && rcv < (i64)node_count;")
            E(f"I{q}e = e; I{q}ev = ev; I{q}rv = ok; I{q}n = ok ? (u64)snd : 0; I{q}r = ok ? rcv : -1;")
            E.level -= 1
            E("}")

        def load(E, h, q):
            E("{")
            E.level += 1
            E(f"const u64 e = I{q}e, sndc = I{q}n; const bool rv = I{q}rv;")
            E(f"const T* __restrict__ Yr = Y + e * {self.D2};")
            E(f"const T* __restrict__ Wr = W + e * {self.WN};")
            for f in self.used_y:
                E(f"S{h}y{f} = {self.ld('Yr', f)};")
            for p in self.paths:
                for v in range(p.mv):
                    E(f"S{h}We_{p.t}_{v} = {self.ld('Wr', self.widx(p, self.uclamp(p.a, 0), v))};")
            for i in self.used_in1:
                a = self.in1[i]
                E(f"{{ const T* __restrict__ p_ = X + sndc * {self.D1} + {a.off} + {self.uclamp(a, 0)} * {a.D}; "
                  + " ".join(f"S{h}x{i}_{m} = p_[{m}];" for m in range(a.D)) + " }")
                # dW and dY of an edge are proportional to x: zero it for idle lanes and invalid edges
                E(f"if (!({self.act(a)})) {{ " + " ".join(f"S{h}x{i}_{m} = (T)0;" for m in range(a.D)) + " }")
            E.level -= 1
            E("}")

        def pre(E, h):
            """dZ of the current edge's receiver, when it differs from the one held.  (Index set h is
            refilled for a later iteration before the arithmetic runs: what the arithmetic needs of it is
            copied here.)"""
            E(f"const bool cur_ev = I{h}ev;")
            if R == 1:
                # the receiver is the same for all lanes: a scalar branch, loads not predicated
                E(f"const int rcv_u = __builtin_amdgcn_readfirstlane((int)I{h}r);")
                E("if (rcv_u >= 0 && (i64)rcv_u != cur_rcv) {")
                E.level += 1
                E("cur_rcv = (i64)rcv_u;")
            else:
                E(f"if (I{h}r >= 0 && I{h}r != cur_rcv) {{")
                E.level += 1
                E(f"cur_rcv = I{h}r;")
            for oi in self.used_out:
                o = self.out[oi]
                E(f"{{ const T* __restrict__ p_ = G + (u64)cur_rcv * {self.D3} + {o.off} + {self.uclamp(o, 0)} * {o.D}; "
                  + " ".join(f"G{oi}_{k} = p_[{k}];" for k in range(o.D)) + " }")
                if not self.full(o):
                    E(f"if (!(u < {o.mul})) {{ " + " ".join(f"G{oi}_{k} = (T)0;" for k in range(o.D)) + " }")
            E.level -= 1
            E("}")

        def compute(E, h):
            E("const u64 e = cur_e; rv = cur_rv;")
            E(f"T* __restrict__ Wgr = Wg + e * {self.WN};")
            for f in self.used_y:
                E(f"T dy{f} = (T)0;")
            for i in self.used_in1:
                E("T " + ", ".join(f"dx{i}_{m} = (T)0" for m in range(self.in1[i].D)) + ";")
            for oi in self.used_out:
                o = self.out[oi]
                E("{")
                E.level += 1
                for k in range(o.D):
                    E(f"const T g{k} = G{oi}_{k};")

                def sink(E, p, v, expr):
                    # (an edge that names no node has x = 0, hence dW = dY = 0: its rows are written like any other)
                    ok = "cur_ev" if self.full(p.a) else f"(cur_ev && u < {p.a.mul})"
                    E(f"  if ({ok}) {self.st('Wgr', self.widx(p, 'u', v), expr)}")
                self.emit_backward_block(E, o, "Wr", sink)
                E.level -= 1
                E("}")
            self.emit_dy_sum(E)
            writer = "ul == 0" if P < 64 else "lane == 63"
            E(f"if (cur_ev && {writer}) {{")
            if self.dy_slots > 1:
                E(f"    T* __restrict__ Ygr = (T*)((char*)ws + DYPART_OFF) + ((u64)(c * {self.HR} + {grp}) * nnz + e) * {self.D2};")
            else:
                E(f"    T* __restrict__ Ygr = Yg + e * {self.D2};")
            for f in range(self.D2):
                E(f"    Ygr[{f}] = " + (f"dy{f};" if f in self.used_y else "(T)0;"))
            E("}")
            # this edge's contribution to dX[sender]: every slot of an existing edge is written (zeros for an
            # edge that names no node: the dZ held belongs to another edge then)
            E("if (cur_ev) {")
            E(f"    T* __restrict__ sp = spill + ((e * {NCH} + c) * {self.NW}) * {P} + ul;")
            for i in self.used_in1:
                for m in range(self.in1[i].D):
                    E(f"    oeq_stnt(sp + {self.spill_word[(i, m)] * P}, rv ? dx{i}_{m} : (T)0);")
            E("}")
        self.emit_pingpong_loop(E, names, load_idx, load, compute, prefetch_first=self.prefetch_edges, pre=pre,
                                index_decl="u64 I0e = 0, I1e = 0, I0n = 0, I1n = 0; i64 I0r = -1, I1r = -1; "
                                           "bool I0rv = false, I1rv = false, I0ev = false, I1ev = false;")
        return E.text()

    def _emit_tile_header(self, E: Emitter, grp: int) -> None:
        """(tile, chunk) of the workgroup, the tile's range of list positions, and - over a position list built on
        the fly - the zero rows of the edges that are in no group."""
        R, P, NCH = self.R, self.P, self.NCH
        E("// (tile, chunk) of this workgroup: ids are dealt to the 8 XCDs round robin, each XCD gets a contiguous run of items")
        E(f"const u64 tiles = gridDim.x, items = tiles * {NCH};")
        E("const u64 bid = blockIdx.x + (u64)blockIdx.y * gridDim.x;")
        E("const u64 xcd = bid & 7, turn = bid >> 3;")
        E("const u64 item = xcd * (items >> 3) + min(xcd, items & 7) + turn;")
        E(f"const int c = (int)(item % {NCH}); (void)c;")
        E(f"const u64 tile = item / {NCH};")
        E(f"const int u = c * {P} + ul;")
        E(f"const u64 per = ((nnz + tiles - 1) / tiles + {R - 1}) / {R} * {R};       // edges per tile")
        if self.backward_perm:
            # positions of the receiver-grouped list: it holds the edges with a valid receiver, nothing behind them
            E("i64 listed_ = ((const i64*)ws)[node_count]; if (listed_ < 0) listed_ = 0; if (listed_ > (i64)nnz) listed_ = (i64)nnz;")
            E("const u64 last = (u64)listed_;")
        else:
            E("const u64 last = nnz;")
        E("const u64 beg = min(tile * per, last);")
        E("const int len = (int)(min(beg + per, last) - beg);")
        E(f"const int maxlen = (len + {R - 1}) / {R};")
        E(f"T* __restrict__ spill = (T*)((char*)ws + {self.spill_off});")
        self._cur_c = "e"
        if self.backward_perm:
            # Edges naming no receiver are in no group: nobody visits them.  The grouping kernels leave one flag per
            # 256 edges; the first workgroup of every chunk ORs them and, only if one is set, walks the edge list
            # and zeroes the rows of such edges: dW, dY (or this chunk's dY partial) and the dX row pass 2 will read.
            E("if (tile == 0) {")
            E.level += 1
            E("const int* __restrict__ bad_ = (const int*)((const char*)ws + FLAGS_OFF);")
            E("int any_ = 0;")
            E("for (u64 q = lane; q < (nnz + 255) / 256; q += 64) any_ |= bad_[q];")
            for m in (32, 16, 8, 4, 2, 1):
                E(f"any_ |= oeq_shfl_xor_i32(any_, {m});")
            E("if (any_) {")
            E.level += 1
            E("for (u64 e = lane; e < nnz; e += 64) {")
            E.level += 1
            E("const i64 r_ = rows[e];")
            E("if (r_ >= 0 && r_ < (i64)node_count) continue;")
            if grp == 0:
                E(f"if (c == 0) for (int q = 0; q < {self.WN}; ++q) Wg[e * {self.WN} + q] = (T)0;")
            if self.dy_slots > 1:
                E(f"{{ T* __restrict__ p_ = (T*)((char*)ws + DYPART_OFF) + ((u64)(c * {self.HR} + {grp}) * nnz + e) * {self.D2}; "
                  f"for (int q = 0; q < {self.D2}; ++q) p_[q] = (T)0; }}")
            else:
                E(f"if (c == 0) for (int q = 0; q < {self.D2}; ++q) Yg[e * {self.D2} + q] = (T)0;")
            if grp == 0:        # (the whole row: the later launches do not visit these edges either)
                E(f"{{ T* __restrict__ p_ = spill + ((e * {NCH} + c) * {self.NW}) * {P}; for (int q = 0; q < {self.NW * P}; ++q) p_[q] = (T)0; }}")
            E.level -= 1
            E("}")
            E.level -= 1
            E("}")
            E.level -= 1
            E("}")

    def _edges_body_staged(self, E: Emitter, grp: int = 0) -> str:
        """Pass 1 through the LDS stage of the forward (same operands: X records of the sender, path weights, Y):
        the edge loop of emit_staged_loop over the tile's consecutive edges, dZ of the receiver held in registers
        and reloaded when the receiver changes, the edge's dW / dY / dX rows kept in registers and stored at the top
        of the next iteration."""
        R, P, NCH = self.R, self.P, self.NCH
        nt = 2 if self.nontemporal else 0
        self._emit_tile_header(E, grp)
        E("bool rv = false;")
        for oi in self.used_out:
            E("T " + ", ".join(f"G{oi}_{k} = (T)0" for k in range(self.out[oi].D)) + ";")
        E("i64 cur_rcv = -1, rawR = -1, rcv0 = -1;")
        slabs, words = self._forward_slabs()
        y_off = words - 64
        E(f"__shared__ __attribute__((aligned(16))) T stage[{words}];")
        res = [f"pw_{p.t}_{v}" for p in self.paths for v in range(p.mv)] + [f"pdy{f}" for f in self.used_y] \
            + [f"pdx{i}_{m}" for i in self.used_in1 for m in range(self.in1[i].D)]
        E("T " + ", ".join(f"{n} = (T)0" for n in res) + "; u64 pe = 0; bool pv = false, pev = false;")

        def dma(E, e, n):
            E("{")
            E.level += 1
            E(f"const u64 e = {e}, sndc = {n};")
            E("rawR = rows[e];")
            E(f"const T* __restrict__ Wr = W + e * {self.WN};")
            E(f"OEQ_DMA(4, {nt}, Y + e * {self.D2} + min(ul, {self.D2 - 1}), stage + {y_off});")
            for kind, key, k0, w, so in slabs:
                if kind == "W":
                    p, v = key
                    E(f"OEQ_DMA(4, {nt}, Wr + {self.widx(p, self.uclamp(p.a, 0), v)}, stage + {so});")
            for kind, key, k0, w, so in slabs:
                if kind == "X":
                    a = self.in1[key]
                    E(f"OEQ_DMA({4 * w}, 0, X + sndc * {self.D1} + {a.off} + {self.uclamp(a, 0)} * {a.D} + {k0}, stage + {so});")
            E.level -= 1
            E("}")

        def readback(E):
            # the receiver of this iteration's edge was requested with its operands (rawR is overwritten by the
            # requests of this iteration, below)
            E("rcv0 = rawR;")
            E(f"const bool cur_ev = {self.edge_pos('it')} < len;")
            E("rv = cur_rv && rcv0 >= 0 && rcv0 < (i64)node_count;")
            for f in self.used_y:
                E(f"const T y{f} = stage[{y_off} + sub * {P} + {f}];")
            for kind, key, k0, w, so in slabs:
                if kind == "W":
                    p, v = key
                    E(f"const T We_{p.t}_{v} = stage[{so} + lane];")
            for i in self.used_in1:
                a = self.in1[i]
                parts = []
                for kind, key, k0, w, so in slabs:
                    if kind == "X" and key == i:
                        parts += [f"stage[{so} + lane * {self.dma_stride(w)} + {r}]" for r in range(w)]
                # dW and dY of an edge are proportional to x: zero it for idle lanes and invalid edges
                E(f"const bool a{i}_ = {self.act(a)};")
                E("const T " + ", ".join(f"xr{i}_{m} = {parts[m]}" for m in range(a.D)) + ";")
                E("const T " + ", ".join(f"x{i}_{m} = a{i}_ ? xr{i}_{m} : (T)0" for m in range(a.D)) + ";")

        def flush(E):
            """Per-edge results of the edge computed last: dW row, dY row (or partial), dX row."""
            E("{")
            E.level += 1
            E("const u64 e = pe;")
            E(f"T* __restrict__ Wgr = Wg + e * {self.WN};")
            for p in self.paths:
                ok = "pev" if self.full(p.a) else f"(pev && u < {p.a.mul})"
                for v in range(p.mv):
                    E(f"if ({ok}) {self.st('Wgr', self.widx(p, 'u', v), f'pw_{p.t}_{v}')}")
            writer = "ul == 0" if P < 64 else "lane == 63"
            E(f"if (pev && {writer}) {{")
            if self.dy_slots > 1:
                E(f"    T* __restrict__ Ygr = (T*)((char*)ws + DYPART_OFF) + ((u64)(c * {self.HR} + {grp}) * nnz + e) * {self.D2};")
            else:
                E(f"    T* __restrict__ Ygr = Yg + e * {self.D2};")
            for f in range(self.D2):
                E(f"    Ygr[{f}] = " + (f"pdy{f};" if f in self.used_y else "(T)0;"))
            E("}")
            E("if (pev) {")
            E(f"    T* __restrict__ sp = spill + ((e * {NCH} + c) * {self.NW}) * {P} + ul;")
            for i in self.used_in1:
                for m in range(self.in1[i].D):
                    E(f"    oeq_stnt(sp + {self.spill_word[(i, m)] * P}, pv ? pdx{i}_{m} : (T)0);")
            E("}")
            E.level -= 1
            E("}")

        def pre(E):
            """dZ of this edge's receiver, when it differs from the one held."""
            if R == 1:
                # the receiver is the same for all lanes: a scalar branch, loads not predicated
                E("const int rcv_u = __builtin_amdgcn_readfirstlane(rv ? (int)rcv0 : -1);")
                E("if (rcv_u >= 0 && (i64)rcv_u != cur_rcv) {")
                E.level += 1
                E("cur_rcv = (i64)rcv_u;")
            else:
                E("if (rv && rcv0 != cur_rcv) {")
                E.level += 1
                E("cur_rcv = rcv0;")
            for oi in self.used_out:
                o = self.out[oi]
                E(f"{{ const T* __restrict__ p_ = G + (u64)cur_rcv * {self.D3} + {o.off} + {self.uclamp(o, 0)} * {o.D}; "
                  + " ".join(f"G{oi}_{k} = p_[{k}];" for k in range(o.D)) + " }")
                if not self.full(o):
                    E(f"if (!(u < {o.mul})) {{ " + " ".join(f"G{oi}_{k} = (T)0;" for k in range(o.D)) + " }")
            E.level -= 1
            E("}")

        def compute(E, h):
            E("const u64 e = cur_e;")
            for f in self.used_y:
                E(f"T dy{f} = (T)0;")
            for i in self.used_in1:
                E("T " + ", ".join(f"dx{i}_{m} = (T)0" for m in range(self.in1[i].D)) + ";")
            for oi in self.used_out:
                o = self.out[oi]
                E("{")
                E.level += 1
                for k in range(o.D):
                    E(f"const T g{k} = G{oi}_{k};")

                def sink(E, p, v, expr):
                    E(f"  pw_{p.t}_{v} = {expr};")
                self.emit_backward_block(E, o, "Wr", sink)
                E.level -= 1
                E("}")
            self.emit_dy_sum(E)
            E(" ".join(f"pdy{f} = dy{f};" for f in self.used_y))
            E(" ".join(f"pdx{i}_{m} = dx{i}_{m};" for i in self.used_in1 for m in range(self.in1[i].D)))
            E("pe = e; pv = rv; pev = cur_ev;")
        plist = None
        if self.backward_perm:
            E("const i64* __restrict__ rlist = (const i64*)ws + 2 * (node_count + 1);     // edge ids grouped by receiver")
            plist = "rlist"
        self.emit_staged_loop(E, self.edge_pos, plist, "cols", dma, readback, compute, flush, pre=pre)
        return E.text()

    # ---------------------------------------------------------------- pass 2
    def _dx_body(self) -> str:
        E = Emitter()
        P, NCH, U = self.P, self.NCH, self.DX_UNROLL
        self.emit_lane_direct(E, lds=False)
        if self.backward_perm:
            E(f"const i64* __restrict__ elist = {self.bwd_list};     // edge ids grouped by sender")
        else:
            E("const IDX* __restrict__ elist = tperm;     // edge ids in (sender, receiver) order")

        def key(E, pos):
            E(f"{{ const i64 e0_ = (i64)elist[{pos}]; if (e0_ >= 0 && e0_ < (i64)nnz) kv_ = (i64)cols[e0_]; }}")
        self._node_setup(E, self.bwd_ptr_off, key=key)
        E(f"const T* __restrict__ spill = (const T*)((const char*)ws + {self.spill_off});")
        E("T " + ", ".join(f"acc{w} = (T)0" for w in range(self.NW)) + ";")
        E(f"for (int it = 0; it < maxlen; it += {U}) {{")
        E.level += 1
        for k in range(U):
            E(f"const bool ev{k} = {self.edge_pos(f'it + {k}')} < len;")
            E(f"const i64 raw{k} = elist[ev{k} ? (u64)(beg + {self.edge_pos(f'it + {k}')}) : (u64)(nnz - 1)];")
        for k in range(U):
            E(f"const bool ok{k} = ev{k} && raw{k} >= 0 && raw{k} < (i64)nnz;")
            E(f"const T* __restrict__ sp{k} = spill + (((u64)(ok{k} ? raw{k} : 0) * {NCH} + c) * {self.NW}) * {P} + ul;")
            E("const T " + ", ".join(f"v{k}_{w} = oeq_ldnt(sp{k} + {w * P})" for w in range(self.NW)) + ";")
        for k in range(U):
            E(" ".join(f"acc{w} += ok{k} ? v{k}_{w} : (T)0;" for w in range(self.NW)))
        E.level -= 1
        E("}")
        E("const bool rv = nv; (void)rv;")
        names, w = {}, 0
        for i in self.used_in1:
            names[i] = [f"acc{w + m}" for m in range(self.in1[i].D)]
            w += self.in1[i].D
        self.emit_node_output(E, self.in1, self.used_in1, lambda a: names[a.idx], "Xg", self.D1, via_lds=False,
                              zero_unused=True, add_existing=False)
        return E.text()
