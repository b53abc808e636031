"""Deterministic fused convolution with register-direct loads.

Edges are sorted by receiver.  One wavefront owns (a tile of R nodes, one 64-channel chunk) and
walks the node's edge list in order, so every sum has a fixed order and nothing is atomic:

* forward: the node is the receiver; per incoming edge the lane reads its X records of the
  sender, its weights and Y, and accumulates Z[node] in registers; Z is written once per node;
* backward: the node is the sender; the edge list is the (sender, receiver)-sorted order given by
  ``transpose_perm``; per outgoing edge the lane reads its dZ records of the receiver, weights
  and Y, writes dW[e] (coalesced) and dY[e] (per-chunk partial when the multiplicity spans several
  chunks), and accumulates dX[node] in registers.

The edge loop is software-pipelined: operands of the next edge are requested while the current one is
computed, either into a second register set (emit_pingpong_loop) or, for fp32 problems whose
multiplicity fits one chunk, through LDS by LDS-DMA (emit_staged_loop), which needs one register set
and so keeps more wavefronts resident.

The backward launches its nodes longest first (order_backward), and when one edge's operands would not
leave room for two wavefronts per SIMD it runs as one launch per group of output blocks (out_groups).

All loads are unconditional from clamped, range-checked indices (see uvu_direct.py); an edge
that is out of range for its lane, or names a node that does not exist, contributes zero.  The
CSR pointers come from the prep kernels of the template (workspace).  The backward reads sender
and receiver of the permuted edge itself, so the graph need not be symmetric (the reference's
kernel reads both at the unpermuted position: templates/loop_unroll_conv_det.cuh:151-198).
"""
from __future__ import annotations

import contextlib

from .. import tunables
from ..problem import TPProblem
from .common import Emitter, WAVE
from .uvu_direct import UVUDirectGenerator


class UVUDetGenerator(UVUDirectGenerator):
    _allow_det = True
    SPLIT_WORDS = 80
    # words per group when the backward is split (fp64, 5000 nodes / 150 000 edges, 64 -> 24 words per group: 17 paths
    # at 128 channels 3.12 -> 2.52 ms, 68 paths 9.38 -> 7.56 ms, 30 paths 2.11 -> 1.98 and 1.27 -> 1.33 ms)
    SPLIT_TARGET = {"float": 64, "double": 24}
    FWD_SPLIT_WORDS = {"float": 100, "double": 32}
    FWD_COHERENT = True
    # int64 words of one on-the-fly grouping of the edges in the workspace: group pointers and fill cursors
    # (node_count + 1 each), the position list (nnz), the counters (node_count + 1) and the ticket of the
    # counting kernel
    GROUP_WORDS = "(3 * (node_count + 1) + nnz + 1)"

    @staticmethod
    def group_bytes(nnz: int, nodes: int) -> int:
        return (3 * (nodes + 1) + nnz + 1) * 8

    def __init__(self, problem: TPProblem, prefetch_backward=None, vector_stores: bool = True,
                 forward_perm: bool = False, backward_perm: bool = False, idx_ctype: str = "i64",
                 allow_split: bool = True, lds=None, long_node=None, fwd_split=None):
        super().__init__(problem, "conv_det", vector_stores=vector_stores)
        self.idx_ctype = idx_ctype
        # True: the forward walks the receiver-grouped edge order listed in the workspace (built on
        # the fly from an unsorted edge list) instead of the edge list itself
        self.forward_perm = forward_perm
        # True: the backward likewise walks a sender-grouped order built in the workspace
        # (pointers | cursors | position list | node order | dY partials) instead of the caller's transpose
        # permutation (receiver pointers | sender pointers | node order | dY partials)
        self.backward_perm = backward_perm
        # the backward launches the nodes in descending order of their edge count (order_backward writes
        # the node list behind the pointers): with two launch rounds of wavefronts the long nodes then
        # run first and the short ones fill the tail
        self.ordered_backward = True
        extra = " + node_count"
        if backward_perm:
            # behind the forward's grouping (pointers | cursors | position list | counters | ticket), so that
            # both stay valid side by side and a graph prepared once serves forward and backward calls alike
            base = self.GROUP_WORDS
            self.bwd_ptr_off = base
            self.bwd_list = f"((const i64*)ws + {base} + 2 * (node_count + 1))"
            self.bwd_order = f"((const i64*)ws + 2 * {base})"
            self.dypart_off = f"(2 * {base}{extra}) * sizeof(i64)"
        else:
            self.bwd_ptr_off = "(node_count + 1)"
            self.bwd_list = "tperm"
            self.bwd_order = "((const i64*)ws + 2 * (node_count + 1))"
            self.dypart_off = f"(2 * (node_count + 1){extra}) * sizeof(i64)"
        # Backward: registers per edge = dZ records + weights + Y ("words").  Above SPLIT_WORDS the
        # kernel would not fit two wavefronts per SIMD even without prefetch, so the output blocks of a
        # chunk are split into H groups, one backward launch per group (each launch reads only its blocks of
        # dZ and W; launch 0 writes dX, the later ones add to it; dY goes through per-(chunk, group) partials).
        def words_of(outs):
            ps = [p for p in self.paths if p.o.idx in outs]
            return (sum(self.out[i].D for i in outs) + sum(p.mv for p in ps)
                    + len({p.b.off + v * p.b.D + j for p in ps for v in range(p.mv) for (_, j) in p.pairs}))
        words = words_of(self.used_out)
        H = 1
        split = tunables.current.det_split                      # 0: never; a number: threshold for A/B runs
        limit = split if split else self.SPLIT_WORDS
        if words > limit and split != 0 and allow_split:
            H = min(len(self.used_out), -(-words // self.SPLIT_TARGET[self.T]))
        self.out_groups = [[] for _ in range(H)]
        for oi in sorted(self.used_out, key=lambda i: -(self.out[i].D + len(self.paths_into(i)))):
            min(self.out_groups, key=words_of).append(oi)
        self.out_groups = [sorted(g_) for g_ in self.out_groups]
        self.H = H
        self.dy_slots = self.NCH * H               # dY partial rows per edge (summed by backward_dy_reduce)
        # behind the dY partials: one int per 256 edges, set by the preparation when one of those edges names
        # a node that does not exist (see emit_invalid_edge_rows)
        part = f" + {self.dy_slots}ull * nnz * {self.D2} * sizeof(T)" if self.dy_slots > 1 else ""
        self.flags_off = f"((({self.dypart_off}{part}) + 7ull) & ~7ull)"
        words = max(words_of(g_) for g_ in self.out_groups)
        # fetch the next edge's operands while the current edge is being computed; pays when the
        # per-edge register footprint is small enough to keep several wavefronts per SIMD
        if prefetch_backward is None:
            prefetch_backward = tunables.current.det_prefetch
        # (fp64: every word is two registers, and the second set does not fit what two wavefronts per SIMD leave
        # each: with it the 32-channel NequIP backward spilled 636 bytes per lane and took 1.26 instead of 0.43 ms,
        # the 128-channel MACE backward 19.4 instead of 6.3 ms)
        self.prefetch_backward = ((words <= 80 and self.T == "float") if prefetch_backward is None
                                  else prefetch_backward)
        # W / Y / dW / dY are touched once: the streaming hint keeps them from evicting the gathered rows
        # (256 channels, without the hint: forward 2.58 -> 2.73 ms, backward 7.68 -> 8.91 ms)
        self.nontemporal = True
        # backward operands of the next edge travel global -> LDS without passing through registers
        # (LDS-DMA), which leaves room for a third wavefront per SIMD; see emit_staged_loop
        def stage_words_of(outs):
            return WAVE * (sum(self.dma_stride(w) for i in outs for _, w in self.dma_pieces(self.out[i].D))
                           + sum(p.mv for p in self.paths if p.o.idx in outs) + 1)
        self.stage_words = max(stage_words_of(g_) for g_ in self.out_groups)      # of the largest group
        lds = tunables.current.det_lds if lds is None else lds
        stage_waves = (160 * 1024) // (4 * self.stage_words * 4)        # wavefronts per SIMD the stage leaves room for
        # one chunk per node: also at two wavefronts per SIMD (the register pipeline then has one); chunked
        # problems only when three fit (config 5, two: 1 % slower than the register pipeline)
        small = self.NCH == 1 and H == 1
        fits = self.T == "float" and self.P >= self.D2 and (stage_waves >= 3 or (small and stage_waves >= 2))
        self.lds_backward = fits and lds is not False
        if self.lds_backward:
            self.waves_per_eu = min(3, stage_waves)
        elif self.prefetch_backward:
            # two register sets: hold the allocation to what two wavefronts per SIMD leave each (256 registers)
            self.waves_per_eu = 2
        # the forward likewise when the multiplicity fits one chunk: few wavefronts per node, so the
        # registers saved buy a fifth wavefront per SIMD (with several chunks per node it measured 1 % slower)
        fwd_words = self._forward_slabs()[1]
        # (with several chunks it pays where an edge brings many operands: 26 - 27 words per lane, forward 0.650 ->
        # 0.640 ms on the 128-channel MACE problem and 3.65 -> 3.49 ms on 256 channels with outputs of either
        # parity; with 22 words, 256 channels and 13 paths, 2.583 -> 2.596 ms; not over a position list built on the
        # fly - the unsorted MACE forward went 0.741 -> 0.775 ms)
        fwd_operands = sum(self.in1[i].D for i in self.used_in1) + sum(p.mv for p in self.paths)
        self.lds_forward = (self.T == "float" and self.P >= self.D2 and lds is not False
                            and (self.NCH == 1 or (fwd_operands >= 26 and not forward_perm) or lds is True)
                            and 16 * (fwd_words + self.lds_elems) * 4 <= 160 * 1024)
        # Forward: the sums of every output block of a node stay in registers across its edge list.  Beyond
        # FWD_SPLIT_WORDS words per lane the loop spilled them (5000 nodes, 150 000 edges, fp32 / fp64: 30 paths and 102
        # words 0.68 / 3.33 ms, 68 paths and 312 words 19.6 / 44.6 ms), so the output blocks are dealt into groups, one
        # forward launch per group: each launch reads X, Y and its own weights and writes its blocks of Z (the same
        # problems then 0.35 / 0.75 and 1.14 / 2.71 ms; 71 words in one launch: 0.38 / 0.95 ms, in two 0.41 / 0.99).
        # With the groups cut along the in1 blocks (coherent_groups) a launch gathers only its own X blocks and finer
        # groups pay in fp64, where one launch needs 366 registers: 71 words in groups of at most 32, 0.94 -> 0.88 ms; 102
        # words 0.51 -> 0.42 ms; 312 words 2.29 -> 2.02 ms; 256 channels with outputs of either parity 1.84 -> 1.45 ms
        # (fp32, groups of 64 instead of 100: 71 words 0.375 -> 0.388 ms, 312 words 1.04 -> 0.95 ms).
        z_regs = lambda outs: sum(self.out[i].D for i in outs)
        HF = 1
        fsplit = self.FWD_SPLIT_WORDS[self.T] if fwd_split is None else fwd_split
        if fsplit and z_regs(self.used_out) > fsplit:
            HF = min(len(self.used_out), -(-z_regs(self.used_out) // fsplit))
        self.fwd_groups = self.coherent_groups(HF, z_regs) if self.FWD_COHERENT else self.dealt_groups(HF, z_regs)
        self.uniform_rows = False          # validity is per lane (edge lists differ between sub-rows)
        self.chunk_in_grid = True
        # the regrouped backward arithmetic (see UVUGenerator.regroup_pairs) where registers are to spare: measured
        # on one GPU in one process, 32 channels (LDS-staged loop) 0.165 against 0.170 ms with it, 256 channels
        # (two register sets, 256 registers) 7.78 against 7.61 ms
        self.regroup_pairs = self.lds_backward
        # A node whose edge list is longer than LONG times the mean (at least PIECE_MIN_EDGES) is not walked
        # by its own wavefront: the edge list is cut at multiples of that length, and every piece of a long
        # node is walked by one of the wavefronts launched behind the nodes (two per tile of the list: the
        # piece of the long node that ends in the tile and of the one that begins in it).  A piece leaves its
        # sums in a partial row of the workspace; the wavefront that finishes last (a counter per long node)
        # adds the pieces in list order and writes the node's row, so the result does not depend on timing
        # (reference: the edge list dealt to the warps in equal shares and a fix-up kernel for the seams,
        # templates/loop_unroll_conv_det.cuh:33-133).  0: every node is walked by one wavefront.
        self.LONG = max(0, int(tunables.current.long_node)) if long_node is None else int(long_node)
        # byte offset (C expression) of the piece area in the workspace: counters, then partial rows
        self.piece_base = f"((({self.flags_off} + 4ull * ((nnz + 255) / 256)) + 255ull) & ~255ull)"

    def dealt_groups(self, n: int, words_of):
        """The output blocks in n groups of about equal ``words_of``, largest block first."""
        groups = [[] for _ in range(n)]
        for oi in sorted(self.used_out, key=lambda i: -words_of([i])):
            min(groups, key=words_of).append(oi)
        return [sorted(g_) for g_ in groups if g_] or [[]]

    def coherent_groups(self, n: int, words_of):
        """The output blocks in n groups of about equal ``words_of``, cut from the list ordered by the in1 block
        their paths read: a launch gathers only the X blocks its paths use, so groups that share them gather
        less."""
        first_in = lambda oi: min((p.a.idx for p in self.paths_into(oi)), default=0)
        order = sorted(self.used_out, key=lambda oi: (first_in(oi), oi))
        total = words_of(order)
        groups, acc = [[]], 0
        for oi in order:
            w = words_of([oi])
            if groups[-1] and len(groups) < n and acc + w / 2 > total * len(groups) / n:
                groups.append([])
            groups[-1].append(oi)
            acc += w
        return [sorted(g_) for g_ in groups if g_] or [[]]

    @contextlib.contextmanager
    def _group(self, h: int, groups=None):
        """Restricts the generator to the paths into the output blocks of group h (of the backward launches, or
        of ``groups``)."""
        saved = (self.paths, self.used_out, self.used_in1, self.used_y)
        outs = (self.out_groups if groups is None else groups)[h]
        self.paths = [p for p in saved[0] if p.o.idx in outs]
        self.used_out = list(outs)
        self.used_in1 = sorted({p.a.idx for p in self.paths})
        self.used_y = sorted({p.b.off + v * p.b.D + j for p in self.paths for v in range(p.mv) for (_, j) in p.pairs})
        try:
            yield
        finally:
            self.paths, self.used_out, self.used_in1, self.used_y = saved

    def backward_kernels(self):
        """(kernel name, group) of the backward launches, in launch order."""
        return [("backward" if h == 0 else f"backward_g{h}", h) for h in range(self.H)]

    def forward_kernels(self):
        """(kernel name, group) of the forward launches, in launch order."""
        return [("forward" if h == 0 else f"forward_g{h}", h) for h in range(len(self.fwd_groups))]

    def forward_kernel_sources(self):
        """The forward's compute kernels as the templates emit them: name and body."""
        return [dict(name=name, body=self.conv_det_forward_body(h)) for name, h in self.forward_kernels()]

    def forward_steps(self, step: dict):
        """One launch like ``step`` per group of output blocks."""
        return [dict(step, kernel=name) for name, _ in self.forward_kernels()]

    def backward_kernel_sources(self):
        """The backward's compute kernels as the templates emit them: name, workgroup size, attributes, body."""
        return [dict(name=name, threads=64, attr=self.backward_attr(), body=self.conv_det_backward_body(h))
                for name, h in self.backward_kernels()]

    def act(self, blk):
        return "rv" if self.full(blk) else f"(rv && u < {blk.mul})"

    def act_c(self, blk, c):
        return self.act(blk)

    def uexpr(self, c) -> str:
        return "u"

    # ------------------------------------------------------------------ common
    PIECE_MIN_EDGES = 32          # OEQ_PIECE_MIN_EDGES of the C ABI
    PIECE_GROUP = 32              # pieces added by one wavefront at the first level of a long node's sum

    def piece_tiles(self, nnz: int, nodes: int) -> int:
        """Tiles of the edge list (host mirror of oeq_piece_tiles in the kernels and of the launch grid)."""
        if not self.LONG or nnz == 0 or nodes == 0:
            return 0
        t = max(self.PIECE_MIN_EDGES, self.LONG * (-(-nnz // nodes)))
        return -(-nnz // t)

    @property
    def piece_row_words(self) -> int:
        return max(self.D1, self.D3)

    def piece_bytes(self, nnz: int, nodes: int) -> int:
        """Counters (four ints per tile and chunk: group and node level of both slots) and partial rows (two
        per tile) of the piece area."""
        tiles = self.piece_tiles(nnz, nodes)
        if tiles == 0:
            return 0
        return 256 + ((16 * self.NCH * tiles + 255) & ~255) + 2 * tiles * self.piece_row_words * self.itemsize

    def emit_piece_helpers(self) -> str:
        """Device functions shared by the kernels of one code object (rendered once by the templates)."""
        return "\n".join([
            "// edges per piece of a long node's list, and tiles of that length in the whole list",
            "static __device__ __forceinline__ u64 oeq_piece_edges(u64 nnz, u64 node_count) {",
            f"    const u64 t_ = {self.LONG}ull * (node_count ? (nnz + node_count - 1) / node_count : 0);",
            f"    return t_ < {self.PIECE_MIN_EDGES}ull ? {self.PIECE_MIN_EDGES}ull : t_;",
            "}",
            "static __device__ __forceinline__ u64 oeq_piece_tiles(u64 nnz, u64 node_count) {",
            "    const u64 t_ = oeq_piece_edges(nnz, node_count);",
            f"    return {'(nnz + t_ - 1) / t_' if self.LONG else '0'};",
            "}"])

    def _node_setup(self, E: Emitter, ptr_off: str, order: str = None, key=None) -> None:
        """One node per wavefront, or - for the wavefronts launched behind the nodes - one piece of a long
        node's edge list.  With multiplicity <= 32 the wavefront's R = 64/P lane groups walk interleaved
        sub-lists of the edges (edge beg + it*R + sub) and their partial sums are combined in a fixed order
        at the end, which shortens the serial edge loop R-fold.  ``key(E, pos)`` emits statements that
        set ``kv_`` (i64) to the node owning list position ``pos`` (anything out of range: not a node);
        without it every node is walked whole."""
        R = self.R
        self.pieces = bool(self.LONG and key)
        # The launch is ordered chunk by chunk (blockIdx.y): the wavefronts in flight then gather from one
        # chunk's share of X / dZ, a fraction of the tensor that the 256 MB Infinity Cache can hold.  Giving
        # the chunks of a node consecutive workgroup ids instead measured slower (256 channels: forward
        # 2.58 -> 2.75 ms, backward 7.49 -> 9.72 ms).
        E("const int c = blockIdx.y; (void)c;")
        E("const u64 bx_ = blockIdx.x;")
        E(f"const int u = c * {self.P} + ul;")
        E(f"const i64* __restrict__ ptr = (const i64*)ws + {ptr_off};")
        E("u64 node = node_count; i64 beg = 0, end = 0;")
        if self.pieces:
            E("// pieces are in use when the launch has wavefronts behind the nodes (the entry point that must not")
            E("// allocate launches none: every node is then walked whole)")
            E("const bool pieces_on = gridDim.x > node_count, piece = bx_ >= node_count;")
            E("const u64 TL = oeq_piece_edges(nnz, node_count), tiles_ = oeq_piece_tiles(nnz, node_count);")
            E("u64 slot = 0, qh = 0; int npieces = 0;")
            E("if (!piece) {")
            E.level += 1
        if order:
            E(f"const i64 nd_ = bx_ < node_count ? {order}[bx_] : -1;")
            E("if (nd_ >= 0 && (u64)nd_ < node_count) node = (u64)nd_;")
        else:
            E("if (bx_ < node_count) node = bx_;")
        E("if (node < node_count && nnz > 0) { beg = ptr[node]; end = ptr[node + 1]; }")
        E("if (beg < 0) beg = 0;")
        E("if (end > (i64)nnz) end = (i64)nnz;")
        E("if (end < beg) end = beg;")
        if self.pieces:
            E("if (pieces_on && (u64)(end - beg) > TL) { node = node_count; end = beg; }     // a long node: walked in pieces, see below")
            E.level -= 1
            E("} else {")
            E.level += 1
            E("const u64 w_ = bx_ - node_count, q_ = w_ >> 1; const bool head_ = (w_ & 1) != 0;")
            E("const u64 a0_ = q_ * TL, a1_ = min(a0_ + TL, nnz);")
            E("if (a0_ < nnz) {")
            E.level += 1
            E("i64 kv_ = -1;")
            key(E, "(head_ ? a1_ - 1 : a0_)")
            E("if (kv_ >= 0 && kv_ < (i64)node_count) {")
            E.level += 1
            E("i64 b_ = ptr[kv_], e_ = ptr[kv_ + 1];")
            E("if (b_ < 0) b_ = 0;")
            E("if (e_ > (i64)nnz) e_ = (i64)nnz;")
            E("if (e_ < b_) e_ = b_;")
            E("// the tile's head piece belongs to the long node that begins in it, the other to the one that began before it")
            E("if ((u64)(e_ - b_) > TL && (head_ ? (u64)b_ >= a0_ : (u64)b_ < a0_)) {")
            E("    node = (u64)kv_; beg = head_ ? b_ : (i64)a0_; end = min(e_, (i64)a1_); slot = w_;")
            E("    qh = (u64)b_ / TL; npieces = (int)((u64)(e_ - 1) / TL - qh) + 1;")
            E("}")
            E.level -= 1
            E("}")
            E.level -= 1
            E("}")
            E.level -= 1
            E("}")
        # every lane of the wavefront holds the same node and range: keep them in scalar registers
        E("node = oeq_uniform_u64(node); beg = (i64)oeq_uniform_u64((u64)beg); end = (i64)oeq_uniform_u64((u64)end);")
        if self.pieces:
            E("qh = oeq_uniform_u64(qh); npieces = __builtin_amdgcn_readfirstlane(npieces);")
        E("const bool nv = node < node_count;")
        E("const int len = (int)(end - beg);")
        E(f"const int maxlen = (len + {R - 1}) / {R};")
        self.noderow_of = (lambda r: ("node", "nv"))

    def emit_node_output(self, E: Emitter, blocks, used, regs_of, ptr: str, rowdim: int, via_lds: bool,
                         zero_unused: bool, add_existing: bool, elsewhere=()) -> None:
        """The sums a wavefront holds for its node (registers ``regs_of(block)`` of the blocks in ``used``) ->
        row ``node`` of ``ptr``; blocks nothing contributes to are zero-filled (``zero_unused``); with
        ``add_existing`` the row already holds the sums of an earlier launch and is added to; blocks in
        ``elsewhere`` are written by another launch and left alone.  A piece
        stores its sums in its partial row instead; the piece of a node that finishes last adds all pieces
        in list order and writes the node's row."""
        for blk in blocks:
            if blk.idx in used and blk.dim:
                self.emit_sub_sum(E, regs_of(blk))

        def store(E, base: str, row: str, existing: bool, zero: bool, agent: bool = False):
            for blk in blocks:
                if blk.dim == 0:
                    continue
                E("{")
                E.level += 1
                dst = f"{base} + {row} * {rowdim} + {blk.off} + u * {blk.D}"
                if agent:                   # a partial row, read by a wavefront that may sit on another XCD
                    if blk.idx in used:
                        E(f"if ({self.store_act(blk)}) {{ T* __restrict__ p_ = {dst}; "
                          + " ".join(f"oeq_st_agent(p_ + {m}, {n});" for m, n in enumerate(regs_of(blk))) + " }")
                elif blk.idx in used and self.R == 1 and via_lds:
                    self.emit_block_store(E, blk, regs_of(blk), base, rowdim, row, (lambda r: (row, "nv")), "store",
                                          via_lds=True)
                elif blk.idx in used:
                    if existing:            # the launches of the earlier groups have written this row: add to it
                        E(f"if ({self.store_act(blk)}) {{ const T* __restrict__ q_ = {dst}; "
                          + " ".join(f"{n} += q_[{m}];" for m, n in enumerate(regs_of(blk))) + " }")
                    self.emit_record_store(E, regs_of(blk), dst, self.store_act(blk))
                elif zero and blk.idx not in elsewhere:
                    self.emit_record_store(E, ["(T)0"] * blk.D, dst, self.store_act(blk))
                E.level -= 1
                E("}")
        if not self.pieces:
            store(E, ptr, "node", add_existing, zero_unused)
            return
        G = self.PIECE_GROUP
        E("if (!piece) {")
        E.level += 1
        store(E, ptr, "node", add_existing, zero_unused)
        E.level -= 1
        E("} else if (nv) {")
        E.level += 1
        E("// counters: one per slot for the groups of pieces, one per slot for the whole node")
        E(f"int* __restrict__ tk_ = (int*)((char*)ws + {self.piece_base}) + (u64)c * 4 * tiles_;")
        E(f"T* __restrict__ prow_ = (T*)((char*)ws + {self.piece_base} + ((16ull * {self.NCH} * tiles_ + 255ull) & ~255ull) + 256ull);")
        store(E, "prow_", "slot", False, False, agent=True)
        E(f"// Piece k of the node sits in slot 2 qh + 1 (k = 0) or 2 (qh + k).  The pieces are added in two levels, each")
        E(f"// by whoever finishes last: groups of {G} consecutive pieces in list order (the sum replaces the group's first")
        E(f"// piece), then the groups in order.  Which wavefront adds does not change what is added in which order.")
        E("// The partial rows are written and read at agent scope; a ticket is drawn when the row's stores have completed")
        E("// (release / acquire fences here would write back and invalidate this XCD's whole L2 once per piece: with 256")
        E("// nodes of 586 edges among 150 000 the forward took 0.32 ms with them and 0.22 ms without any pieces).")
        E(f"const int k_own_ = slot == 2 * qh + 1 ? 0 : (int)(slot / 2 - qh);")
        E(f"int first_ = (k_own_ / {G}) * {G}, cnt_ = min({G}, npieces - first_), stride_ = 1, level_ = 0;")
        E("oeq_wait_vm();")
        E("int old_ = 0;")
        E("if (lane == 0) old_ = oeq_ticket_add(tk_ + (first_ == 0 ? 2 * qh + 1 : 2 * (qh + (u64)first_)));")
        E("old_ = __builtin_amdgcn_readfirstlane(old_);")
        E("bool go_ = old_ == cnt_ - 1;")
        E("while (go_) {")
        E.level += 1
        for blk in blocks:
            if blk.idx in used and blk.dim:
                E(" ".join(f"{n} = (T)0;" for n in regs_of(blk)))
        E("for (int i_ = 0; i_ < cnt_; ++i_) {")
        E.level += 1
        E("const int kk_ = first_ + i_ * stride_;")
        E("const u64 srow_ = kk_ == 0 ? 2 * qh + 1 : 2 * (qh + (u64)kk_);")
        for blk in blocks:
            if blk.idx in used and blk.dim:
                E(f"{{ const T* __restrict__ q_ = prow_ + srow_ * {rowdim} + {blk.off} + {self.uclamp(blk, 0)} * {blk.D}; "
                  + " ".join(f"{n} += oeq_ld_agent(q_ + {m});" for m, n in enumerate(regs_of(blk))) + " }")
        E.level -= 1
        E("}")
        E("const u64 grow_ = first_ == 0 ? 2 * qh + 1 : 2 * (qh + (u64)first_);       // slot of the group's first piece")
        E(f"if (level_ == 1 || npieces <= {G}) {{")
        E.level += 1
        store(E, ptr, "node", add_existing, zero_unused)
        E("if (lane == 0) tk_[level_ == 1 ? 2 * tiles_ + 2 * qh + 1 : grow_] = 0;")
        E("go_ = false;")
        E.level -= 1
        E("} else {")
        E.level += 1
        store(E, "prow_", "grow_", False, False, agent=True)
        E("if (lane == 0) tk_[grow_] = 0;")
        E("oeq_wait_vm();")
        E("old_ = 0;")
        E("if (lane == 0) old_ = oeq_ticket_add(tk_ + 2 * tiles_ + 2 * qh + 1);")
        E("old_ = __builtin_amdgcn_readfirstlane(old_);")
        E(f"first_ = 0; cnt_ = (npieces + {G - 1}) / {G}; stride_ = {G}; level_ = 1;")
        E("go_ = old_ == cnt_ - 1;")
        E.level -= 1
        E("}")
        E.level -= 1
        E("}")
        E.level -= 1
        E("}")

    def ld(self, ptr: str, idx) -> str:
        return f"oeq_ldnt({ptr} + {idx})" if self.nontemporal else f"{ptr}[{idx}]"

    def st(self, ptr: str, idx, val: str) -> str:
        return f"oeq_stnt({ptr} + {idx}, {val});" if self.nontemporal else f"{ptr}[{idx}] = {val};"

    def edge_pos(self, it: str) -> str:
        return f"(({it}) * {self.R} + sub)" if self.R > 1 else f"({it})"

    def emit_sub_sum(self, E: Emitter, names) -> None:
        """Add the partial sums of the R lane groups (fixed order); every lane ends with the total."""
        m = 32
        while m >= self.P:
            for n in names:
                E(f"{n} += oeq_shfl_xor({n}, {m});")
            m //= 2

    def store_act(self, blk) -> str:
        base = "nv" if self.R == 1 else "(nv && sub == 0)"
        return base if self.full(blk) else f"({base} && u < {blk.mul})"

    ORDER_THREADS = 1024
    ORDER_BINS = 256

    def order_step(self) -> dict:
        return dict(kernel="order_backward", num_threads=self.ORDER_THREADS, grid_kind=0, num_blocks=1, prep=True)

    def order_bytes(self, nodes: int) -> int:
        return nodes * 8 if self.ordered_backward else 0

    def backward_steps(self):
        """Launches of the segmented backward behind the pointer / position-list preparation."""
        steps = [self.order_step()] if self.ordered_backward else []
        steps += [dict(kernel=name, num_threads=64, grid_kind=3, work_per_block=1, num_blocks=self.LONG, grid_y=self.NCH)
                  for name, _ in self.backward_kernels()]
        if self.dy_slots > 1:
            steps.append(dict(kernel="backward_dy_reduce", num_threads=256, grid_kind=1,
                              work_per_block=self.dy_rows_per_block))
        return steps

    def dy_partial_bytes(self, nnz: int) -> int:
        return self.dy_slots * nnz * self.D2 * self.itemsize if self.dy_slots > 1 else 0

    @staticmethod
    def flag_bytes(nnz: int) -> int:
        """Alignment slack + one int per 256 edges (flags of edges naming no node)."""
        return 8 + 4 * ((nnz + 255) // 256)

    def emit_invalid_edge_rows(self, E: Emitter, grp: int) -> None:
        """Edges whose sender or receiver is out of range contribute nothing and are never visited by a
        sender's wavefront (or are visited and skipped), so nobody would write their dW / dY rows.  The
        preparation kernels leave one flag per 256 edges; the first workgroup of every (chunk, group)
        launch row ORs them and, only if some edge is flagged, walks the edge list and writes zeros into
        the rows of those edges: dW and dY (or this launch's dY partial slot)."""
        E("if (bx_ == 0) {")
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
        E("const i64 s_ = cols[e], r_ = rows[e];")
        E("if (s_ >= 0 && s_ < (i64)node_count && r_ >= 0 && r_ < (i64)node_count) continue;")
        if grp == 0:
            E(f"if (c == 0) for (int q = 0; q < {self.WN}; ++q) Wg[e * {self.WN} + q] = (T)0;")
        if self.dy_slots > 1:
            E(f"{{ T* __restrict__ p_ = (T*)((char*)ws + DYPART_OFF) + ((u64)(c * {self.H} + {grp}) * nnz + e) * {self.D2}; "
              f"for (int q = 0; q < {self.D2}; ++q) p_[q] = (T)0; }}")
        elif grp == 0:
            E(f"if (c == 0) for (int q = 0; q < {self.D2}; ++q) Yg[e * {self.D2} + q] = (T)0;")
        E.level -= 1
        E("}")
        E.level -= 1
        E("}")
        E.level -= 1
        E("}")

    def plan(self):
        fwd, bwd, _ = super().plan()
        for s in fwd:
            if s["kernel"] == "forward":
                s.update(work_per_block=1, grid_kind=3, num_blocks=self.LONG)
        fwd = [t for s in fwd for t in (self.forward_steps(s) if s["kernel"] == "forward" else [s])]
        bwd = [s for s in bwd if s["kernel"] == "prep_backward"] + self.backward_steps()

        def ws(nnz=0, nodes=0):
            return self.main_bytes(nnz, nodes) + self.piece_bytes(nnz, nodes)
        return fwd, bwd, ws

    def main_bytes(self, nnz: int, nodes: int) -> int:
        """Workspace in front of the piece area (``piece_base``): both pointer arrays, the node order, the dY
        partial rows and the flags of edges naming no node, rounded up to 256 bytes."""
        b = 2 * (nodes + 1) * 8 + self.order_bytes(nodes) + self.dy_partial_bytes(nnz) + self.flag_bytes(nnz)
        return (b + 255) & ~255

    def forward_workspace_model(self):
        """(fixed, per node, per edge) bytes the forward steps use when no node is cut into pieces."""
        return 8, 8, 0

    # ================================================================= forward
    def conv_det_forward_body(self, h: int = 0) -> str:
        with self._group(h, self.fwd_groups):
            return self._forward_body(h)

    def _forward_body(self, h: int) -> str:
        E = Emitter()
        self.emit_lane_direct(E, lds=True)
        if self.forward_perm:
            E("const i64* __restrict__ eperm = (const i64*)ws + 2 * (node_count + 1);")

        def key(E, pos):
            if self.forward_perm:
                E(f"{{ const i64 e0_ = eperm[{pos}]; if (e0_ >= 0 && e0_ < (i64)nnz) kv_ = (i64)rows[e0_]; }}")
            else:
                E(f"kv_ = (i64)rows[{pos}];")
        self._node_setup(E, "0", key=key)
        self._cur_c = "e"
        for oi in self.used_out:
            E("T " + ", ".join(f"z{oi}_{k} = (T)0" for k in range(self.out[oi].D)) + ";")
        # operands of one edge; the loop computes on one set while the loads of the following edge are
        # in flight (software pipelining hides the gather latency, which dominates when a node has few
        # edges and few wavefronts are resident)
        names = []
        for i in self.used_in1:
            names += [f"x{i}_{m}" for m in range(self.in1[i].D)]
        names += [f"We_{p.t}_{v}" for p in self.paths for v in range(p.mv)]
        names += [f"y{f}" for f in self.used_y]
        def load_idx(E, it, q):
            """Edge position, sender (clamped) and validity of iteration ``it`` into index set q."""
            E("{")
            E.level += 1
            E(f"const bool ev = {self.edge_pos(it)} < len;")
            if self.forward_perm:
                E(f"const u64 j = ev ? (u64)(beg + {self.edge_pos(it)}) : (u64)(nnz - 1);")
                E("const i64 e0 = eperm[j];")
                E("const bool ok_e = ev && e0 >= 0 && e0 < (i64)nnz;")
                E("const u64 e = ok_e ? (u64)e0 : 0;")
                E("const i64 snd = cols[e];")
                E("const bool rv = ok_e && snd >= 0 && snd < (i64)node_count;")
            else:
                E(f"const u64 e = ev ? (u64)(beg + {self.edge_pos(it)}) : (u64)(nnz - 1);   // idle lanes re-read the last edge, masked below")
                E("const i64 snd = cols[e];")
                E("const bool rv = ev && snd >= 0 && snd < (i64)node_count;")
            E(f"I{q}e = e; I{q}rv = rv; I{q}n = rv ? (u64)snd : 0;")
            E.level -= 1
            E("}")

        def load(E, h, q):
            """Operands of the edge described by index set q into register set h."""
            E("{")
            E.level += 1
            E(f"const u64 e = I{q}e, sndc = I{q}n; const bool rv = I{q}rv;")
            E(f"const T* __restrict__ Yr = Y + e * {self.D2};")
            E(f"const T* __restrict__ Wr = W + e * {self.WN};")
            for f in self.used_y:
                E(f"S{h}y{f} = {self.ld('Yr', f)};")
            for i in self.used_in1:
                a = self.in1[i]
                E(f"{{ const T* __restrict__ p_ = X + sndc * {self.D1} + {a.off} + {self.uclamp(a, 0)} * {a.D}; "
                  + " ".join(f"S{h}x{i}_{m} = p_[{m}];" for m in range(a.D)) + " }")
                # everything an edge adds is proportional to x: zero it for idle lanes
                E(f"if (!({self.act(a)})) {{ " + " ".join(f"S{h}x{i}_{m} = (T)0;" for m in range(a.D)) + " }")
            for p in self.paths:
                for v in range(p.mv):
                    E(f"S{h}We_{p.t}_{v} = {self.ld('Wr', self.widx(p, self.uclamp(p.a, 0), v))};")
            E.level -= 1
            E("}")

        def compute(E, h):
            for oi in self.used_out:
                self.emit_forward_block(E, self.out[oi], "Wr", zname=f"z{oi}_", declare=False)
        if self.lds_forward:
            self._emit_staged_forward(E, compute)
        else:
            self.emit_pingpong_loop(E, names, load_idx, load, compute)
        E("const bool rv = nv;")
        self.emit_node_output(E, self.out, self.used_out, lambda o: [f"z{o.idx}_{k}" for k in range(o.D)], "Z", self.D3,
                              via_lds=True, zero_unused=(h == 0), add_existing=False,
                              elsewhere={oi for g_ in self.fwd_groups for oi in g_} - set(self.used_out))
        return E.text()

    def uclamp(self, blk, c) -> str:
        return "u" if self.full(blk) else f"min(u, {blk.mul - 1})"

    def emit_pingpong_loop(self, E: Emitter, names, load_idx, load, compute, prefetch_first: bool = True,
                           pre=None, index_decl: str = None) -> None:
        """The edge loop as a three-stage software pipeline.  Stage 1 (two iterations ahead) resolves
        the indices of an edge - a chain of dependent loads: position list, edge id, neighbour row - into
        one of two index sets; stage 2 (one iteration ahead) requests the edge's operands into one of two
        register sets; stage 3 computes.  With the index chain inside stage 2 an iteration lasted three
        memory round trips, whatever the amount of arithmetic.  The loop body is emitted twice (one copy
        per register set), so nothing is copied from "next" to "current".  ``load_idx(E, it, q)`` fills
        index set q for iteration ``it``, ``load(E, h, q)`` register set h from index set q, and
        ``compute(E, h)`` sees the operand names without prefix and the edge as ``cur_e`` / ``cur_rv``.
        ``prefetch_first=False`` (large register footprints) keeps one register set and requests the next
        edge's operands after the arithmetic; its indices are still resolved an iteration early.
        ``pre(E, h)``, when given, is emitted in front of the prefetch requests of every iteration (loads it
        issues are then older than the prefetch and can be waited for without draining it); it sees the
        current edge as index set h.  ``index_decl`` replaces the declaration of the two index sets."""
        nsets = 2 if prefetch_first else 1
        for h in range(nsets):
            E("T " + ", ".join(f"S{h}{n} = (T)0" for n in names) + ";")
        E(index_decl or "u64 I0e = 0, I1e = 0, I0n = 0, I1n = 0; bool I0rv = false, I1rv = false;")
        E("if (maxlen > 0) {")
        E.level += 1
        load_idx(E, "0", 0)
        load(E, 0, 0)
        E.level -= 1
        E("}")
        E("if (maxlen > 1) {")
        E.level += 1
        load_idx(E, "1", 1)
        E.level -= 1
        E("}")
        E("for (int it = 0; it < maxlen; it += 2) {")
        E.level += 1
        for h in (0, 1):
            if h == 1:
                E("if (it + 1 >= maxlen) break;")
            E("{")
            E.level += 1
            hs = h if prefetch_first else 0
            E("const T " + ", ".join(f"{n} = S{hs}{n}" for n in names) + ";")
            E(f"const u64 cur_e = I{h}e; const bool cur_rv = I{h}rv; (void)cur_e; (void)cur_rv;")
            if pre:
                pre(E, h)
            if prefetch_first:
                E(f"if (it + {h + 1} < maxlen) {{")
                E.level += 1
                load(E, 1 - h, 1 - h)
                E.level -= 1
                E("}")
                E(f"if (it + {h + 2} < maxlen) {{")
                E.level += 1
                load_idx(E, f"it + {h + 2}", h)
                E.level -= 1
                E("}")
                compute(E, h)
            else:
                compute(E, h)
                E(f"if (it + {h + 1} < maxlen) {{")
                E.level += 1
                load(E, 0, 1 - h)
                E.level -= 1
                E("}")
                E(f"if (it + {h + 2} < maxlen) {{")
                E.level += 1
                load_idx(E, f"it + {h + 2}", h)
                E.level -= 1
                E("}")
            E.level -= 1
            E("}")
        E.level -= 1
        E("}")

    # ------------------------------------------------------- LDS-staged operands
    @staticmethod
    def dma_pieces(D: int):
        """Split a record of D words into LDS-DMA transfers (the hardware moves 1, 3 or 4 words per lane):
        list of (first word, words), as few as possible."""
        best = {0: []}
        for n in range(1, D + 1):
            best[n] = min(([*best[n - w], (n - w, w)] for w in (4, 3, 1) if n - w >= 0), key=len)
        return best[D]

    @staticmethod
    def dma_stride(words: int) -> int:
        """Words between the LDS destinations of consecutive lanes: a 3-word transfer lands at a 4-word
        lane stride (measured on gfx950), 1- and 4-word transfers are packed."""
        return 4 if words == 3 else words

    def emit_staged_loop(self, E: Emitter, pos_of, pos_list, nbr_list: str, dma, readback, compute, flush=None, pre=None) -> None:
        """The edge loop with the operands of the next edge in flight to LDS while the current edge is
        computed.  An LDS-DMA load holds no registers while it is outstanding, so this pipeline needs one
        register set where emit_pingpong_loop needs two.  Four stages, none of which consumes a load
        issued in the same iteration (the vector-memory counter retires in order, so waiting for a load
        in the middle of an iteration would drain everything requested before it): the edge id of
        iteration it+3 (``pos_list``[``pos_of``(it+3)], or the position itself without a list), the neighbour
        row of it+2 (``nbr_list``[edge id]),
        the operands of it+1 into the stage (``dma``), and the arithmetic of ``it``.  The values the first
        two return are range-checked at the top of the following iteration.  Per iteration: read the
        staged operands into registers, wait until every lane has them (the stage is then free), check
        last iteration's indices, store last iteration's per-edge results (``flush``), issue the three
        requests, compute.  The compiler does not order LDS reads after an outstanding LDS-DMA write by
        itself, hence the explicit wait at the top; it waits for every earlier vector-memory access, which
        is why the per-edge stores are issued in front of the requests and not from inside the
        arithmetic, where they would be the youngest accesses at the next wait.  ``pre``, when given, is emitted
        between the stores and the requests: register loads it issues (consumed by the arithmetic of this
        iteration) are older than the requests and can be waited for without draining them."""
        def pos(it):
            return f"(({pos_of(it)}) < len ? (u64)(beg + {pos_of(it)}) : (u64)(nnz - 1))"

        def fetch(it):
            return f"{pos_list}[{pos(it)}]" if pos_list else f"(i64){pos(it)}"

        def edge_ok(raw, it):
            return f"(({pos_of(it)}) < len && {raw} >= 0 && {raw} < (i64)nnz)"

        def nbr_ok(raw):
            return f"({raw} >= 0 && {raw} < (i64)node_count)"
        E("u64 e0 = 0, e1 = 0, e2 = 0, n1 = 0; bool v0 = false, v1 = false, v2 = false; i64 rawE = 0, rawN = 0;")
        # prologue: dependent loads, paid once per node
        E("if (maxlen > 0) {")
        E.level += 1
        E(f"const i64 t_ = {fetch('0')}; v0 = {edge_ok('t_', '0')}; e0 = v0 ? (u64)t_ : 0;")
        E(f"const i64 r_ = {nbr_list}[e0]; v0 = v0 && {nbr_ok('r_')}; n1 = v0 ? (u64)r_ : 0;")
        dma(E, "e0", "n1")
        E.level -= 1
        E("}")
        E("if (maxlen > 1) {")
        E.level += 1
        E(f"const i64 t_ = {fetch('1')}; v1 = {edge_ok('t_', '1')}; e1 = v1 ? (u64)t_ : 0;")
        E(f"rawN = {nbr_list}[e1];")
        E.level -= 1
        E("}")
        E(f"if (maxlen > 2) rawE = {fetch('2')};")
        E("for (int it = 0; it < maxlen; ++it) {")
        E.level += 1
        E("const u64 cur_e = e0; const bool cur_rv = v0; (void)cur_e; (void)cur_rv;")
        E("oeq_wait_vm();")
        E("oeq_sync();")
        readback(E)
        E("oeq_wait_lds();")
        E("oeq_sync();")
        if flush:
            E("if (it > 0) {")
            E.level += 1
            flush(E)
            E.level -= 1
            E("}")
        if pre:
            pre(E)
        # indices requested during the previous iteration
        E(f"v1 = v1 && {nbr_ok('rawN')}; n1 = v1 ? (u64)rawN : 0;")
        E(f"v2 = {edge_ok('rawE', 'it + 2')}; e2 = v2 ? (u64)rawE : 0;")
        E("if (it + 1 < maxlen) {")
        E.level += 1
        dma(E, "e1", "n1")
        E.level -= 1
        E("}")
        E(f"if (it + 2 < maxlen) rawN = {nbr_list}[e2];")
        E(f"if (it + 3 < maxlen) rawE = {fetch('it + 3')};")
        compute(E, 0)
        E("e0 = e1; v0 = v1; e1 = e2; v1 = v2;")
        E.level -= 1
        E("}")
        if flush:
            E("if (maxlen > 0) {")
            E.level += 1
            flush(E)
            E.level -= 1
            E("}")

    # ================================================================ backward
    def conv_det_backward_body(self, grp: int = 0) -> str:
        with self._group(grp):
            return self._backward_body(grp)

    def _backward_body(self, grp: int) -> str:
        E = Emitter()
        self.emit_lane_direct(E, lds=False)
        list_t = "IDX" if self.bwd_list == "tperm" else "i64"
        E(f"const {list_t}* __restrict__ elist = {self.bwd_list};     // edge ids in (sender, ...) order")

        def key(E, pos):
            E(f"{{ const i64 e0_ = (i64)elist[{pos}]; if (e0_ >= 0 && e0_ < (i64)nnz) kv_ = (i64)cols[e0_]; }}")
        self._node_setup(E, self.bwd_ptr_off, self.bwd_order if self.ordered_backward else None, key=key)
        self.emit_invalid_edge_rows(E, grp)
        self._cur_c = "e"
        # this node's own X chunk (fixed over the edge loop)
        E("bool rv = nv;")
        E("const u64 nodec = nv ? node : 0;")
        for i in self.used_in1:
            a = self.in1[i]
            self.emit_record_load(E, [f"x{i}_{m}" for m in range(a.D)],
                                  f"X + nodec * {self.D1} + {a.off} + {self.uclamp(a, 0)} * {a.D}", self.act(a), zero=True)
            E("T " + ", ".join(f"dx{i}_{m} = (T)0" for m in range(a.D)) + ";")
        names = [f"G{oi}_{k}" for oi in self.used_out for k in range(self.out[oi].D)]
        names += [f"We_{p.t}_{v}" for p in self.paths for v in range(p.mv)]
        names += [f"y{f}" for f in self.used_y]
        def load_idx(E, it, q):
            """Edge id, receiver (clamped) and validity of iteration ``it`` into index set q: a chain of two
            dependent loads (position list, then the edge's receiver), kept off the data loads' critical path."""
            E("{")
            E.level += 1
            E(f"const bool ev = {self.edge_pos(it)} < len;")
            E(f"const u64 j = ev ? (u64)(beg + {self.edge_pos(it)}) : (u64)(nnz - 1);")
            E("const i64 e0 = elist[j];")
            E("const bool ok_e = ev && e0 >= 0 && e0 < (i64)nnz;")
            E("const u64 e = ok_e ? (u64)e0 : 0;")
            E("const i64 rcv = rows[e];")
            E("const bool rv = ok_e && rcv >= 0 && rcv < (i64)node_count;")
            E(f"I{q}e = e; I{q}rv = rv; I{q}n = rv ? (u64)rcv : 0;")
            E.level -= 1
            E("}")

        def load(E, h, q):
            E("{")
            E.level += 1
            E(f"const u64 e = I{q}e, rcvc = I{q}n; const bool rv = I{q}rv;")
            E(f"const T* __restrict__ Yr = Y + e * {self.D2};")
            E(f"const T* __restrict__ Wr = W + e * {self.WN};")
            for f in self.used_y:
                E(f"S{h}y{f} = {self.ld('Yr', f)};")
            for p in self.paths:
                for v in range(p.mv):
                    E(f"S{h}We_{p.t}_{v} = {self.ld('Wr', self.widx(p, self.uclamp(p.a, 0), v))};")
            for oi in self.used_out:
                o = self.out[oi]
                E(f"{{ const T* __restrict__ p_ = G + rcvc * {self.D3} + {o.off} + {self.uclamp(o, 0)} * {o.D}; "
                  + " ".join(f"S{h}G{oi}_{k} = p_[{k}];" for k in range(o.D)) + " }")
                # every gradient of an edge is proportional to dZ: zero it for idle lanes
                E(f"if (!({self.act(o)})) {{ " + " ".join(f"S{h}G{oi}_{k} = (T)0;" for k in range(o.D)) + " }")
            E.level -= 1
            E("}")

        def compute(E, h):
            E("const u64 e = cur_e; rv = cur_rv;")
            E(f"T* __restrict__ Wgr = Wg + e * {self.WN};")
            for f in self.used_y:
                E(f"T dy{f} = (T)0;")
            for oi in self.used_out:
                o = self.out[oi]
                E("{")
                E.level += 1
                for k in range(o.D):
                    E(f"const T g{k} = G{oi}_{k};")

                def sink(E, p, v, expr):
                    if self.lds_backward:          # stored at the top of the next iteration (flush)
                        E(f"  pw_{p.t}_{v} = {expr};")
                    else:
                        E(f"  if ({self.act(p.a)}) {self.st('Wgr', self.widx(p, 'u', v), expr)}")
                self.emit_backward_block(E, o, "Wr", sink)
                E.level -= 1
                E("}")
            self.emit_dy_sum(E)
            if self.lds_backward:
                E(" ".join(f"pdy{f} = dy{f};" for f in self.used_y) + " pe = e; pv = rv;")
                return
            writer = "ul == 0" if self.P < 64 else "lane == 63"
            E(f"if (rv && {writer}) {{")
            if self.dy_slots > 1:
                E(f"    T* __restrict__ Ygr = (T*)((char*)ws + DYPART_OFF) + ((u64)(c * {self.H} + {grp}) * nnz + e) * {self.D2};")
            else:
                E(f"    T* __restrict__ Ygr = Yg + e * {self.D2};")
            for f in range(self.D2):
                E(f"    Ygr[{f}] = " + (f"dy{f};" if f in self.used_y else "(T)0;"))
            E("}")
        if self.lds_backward:
            self._emit_staged_backward(E, compute, grp)
        else:
            self.emit_pingpong_loop(E, names, load_idx, load, compute, prefetch_first=self.prefetch_backward)
        E("rv = nv;")
        self.emit_node_output(E, self.in1, self.used_in1, lambda a: [f"dx{a.idx}_{m}" for m in range(a.D)], "Xg", self.D1,
                              via_lds=False, zero_unused=(grp == 0), add_existing=(grp > 0))
        return E.text()

    def _forward_slabs(self):
        """(slabs, words) of the forward stage: X records of the sender, path weights, Y."""
        slabs, off = [], 0
        for i in self.used_in1:
            for k0, w in self.dma_pieces(self.in1[i].D):
                slabs.append(("X", i, k0, w, off))
                off += WAVE * self.dma_stride(w)
        for p in self.paths:
            for v in range(p.mv):
                slabs.append(("W", (p, v), 0, 1, off))
                off += WAVE
        return slabs, off + WAVE

    def _emit_staged_forward(self, E: Emitter, compute) -> None:
        nt = 2 if self.nontemporal else 0
        slabs, words = self._forward_slabs()
        y_off = words - WAVE
        E(f"__shared__ __attribute__((aligned(16))) T stage[{words}];")

        def dma(E, e, n):
            E("{")
            E.level += 1
            E(f"const u64 e = {e}, sndc = {n};")
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
            E("const bool rv = cur_rv;")
            for f in self.used_y:
                E(f"const T y{f} = stage[{y_off} + sub * {self.P} + {f}];")
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
                # everything an edge adds is proportional to x: zero it for idle lanes
                # (read unconditionally, then masked: a conditional expression would put a branch around every LDS read)
                E(f"const bool a{i}_ = {self.act(a)};")
                E("const T " + ", ".join(f"xr{i}_{m} = {parts[m]}" for m in range(a.D)) + ";")
                E("const T " + ", ".join(f"x{i}_{m} = a{i}_ ? xr{i}_{m} : (T)0" for m in range(a.D)) + ";")
        self.emit_staged_loop(E, self.edge_pos, "eperm" if self.forward_perm else None, "cols", dma, readback, compute)

    def _emit_staged_backward(self, E: Emitter, compute, grp: int = 0) -> None:
        """Stage layout (words): per transfer a [64 lanes x lane stride] slab in lane order - the dZ records
        of every output block, one word per path weight, and one slab whose lane (sub, f) holds Y[e_sub][f]."""
        nt = 2 if self.nontemporal else 0          # cache policy bit "nt" for the streamed operands
        slabs, off = [], 0                         # (kind, key, first word, words, slab offset)
        for oi in self.used_out:
            for k0, w in self.dma_pieces(self.out[oi].D):
                slabs.append(("G", oi, k0, w, off))
                off += WAVE * self.dma_stride(w)
        for p in self.paths:
            for v in range(p.mv):
                slabs.append(("W", (p, v), 0, 1, off))
                off += WAVE
        y_off = off
        off += WAVE
        assert off <= self.stage_words
        E(f"__shared__ __attribute__((aligned(16))) T stage[{off}];")

        def dma(E, e, n):
            E("{")
            E.level += 1
            E(f"const u64 e = {e}, rcvc = {n};")
            E(f"const T* __restrict__ Wr = W + e * {self.WN};")
            E(f"OEQ_DMA(4, {nt}, Y + e * {self.D2} + min(ul, {self.D2 - 1}), stage + {y_off});")
            for kind, key, k0, w, so in slabs:
                if kind == "W":
                    p, v = key
                    E(f"OEQ_DMA(4, {nt}, Wr + {self.widx(p, self.uclamp(p.a, 0), v)}, stage + {so});")
            for kind, key, k0, w, so in slabs:
                if kind == "G":
                    o = self.out[key]
                    E(f"OEQ_DMA({4 * w}, 0, G + rcvc * {self.D3} + {o.off} + {self.uclamp(o, 0)} * {o.D} + {k0}, stage + {so});")
            E.level -= 1
            E("}")

        def readback(E):
            E("rv = cur_rv;")
            for f in self.used_y:
                E(f"const T y{f} = stage[{y_off} + sub * {self.P} + {f}];")
            for kind, key, k0, w, so in slabs:
                if kind == "W":
                    p, v = key
                    E(f"const T We_{p.t}_{v} = stage[{so} + lane];")
            for oi in self.used_out:
                o = self.out[oi]
                parts = []
                for kind, key, k0, w, so in slabs:
                    if kind == "G" and key == oi:
                        parts += [f"stage[{so} + lane * {self.dma_stride(w)} + {r}]" for r in range(w)]
                # every gradient of an edge is proportional to dZ: zero it for idle lanes
                # (read unconditionally, then masked: a conditional expression would put a branch around every LDS read)
                E(f"const bool a{oi}_ = {self.act(o)};")
                E("const T " + ", ".join(f"Gr{oi}_{k} = {parts[k]}" for k in range(o.D)) + ";")
                E("const T " + ", ".join(f"G{oi}_{k} = a{oi}_ ? Gr{oi}_{k} : (T)0" for k in range(o.D)) + ";")
        def flush(E):
            """Per-edge results of the edge computed last (dW row, dY row)."""
            E("{")
            E.level += 1
            E("const u64 e = pe; const bool rv = pv;")
            E(f"T* __restrict__ Wgr = Wg + e * {self.WN};")
            for p in self.paths:
                for v in range(p.mv):
                    E(f"if ({self.act(p.a)}) {self.st('Wgr', self.widx(p, 'u', v), f'pw_{p.t}_{v}')}")
            writer = "ul == 0" if self.P < 64 else "lane == 63"
            E(f"if (rv && {writer}) {{")
            if self.dy_slots > 1:
                E(f"    T* __restrict__ Ygr = (T*)((char*)ws + DYPART_OFF) + ((u64)(c * {self.H} + {grp}) * nnz + e) * {self.D2};")
            else:
                E(f"    T* __restrict__ Ygr = Yg + e * {self.D2};")
            for f in range(self.D2):
                E(f"    Ygr[{f}] = " + (f"pdy{f};" if f in self.used_y else "(T)0;"))
            E("}")
            E.level -= 1
            E("}")
        E("T " + ", ".join([f"pw_{p.t}_{v} = (T)0" for p in self.paths for v in range(p.mv)]
                           + [f"pdy{f} = (T)0" for f in self.used_y]) + "; u64 pe = 0; bool pv = false;")
        self.emit_staged_loop(E, self.edge_pos, "elist", "rows", dma, readback, compute, flush)

    def emit_dy_sum(self, E: Emitter) -> None:
        """Sum dy* over the lanes of a row in a fixed order.  A full wavefront per row uses the
        DPP row operations (total lands in lane 63); smaller groups use the xor butterfly."""
        if self.P == 64:
            for f in self.used_y:
                E(f"dy{f} = oeq_wave_sum63(dy{f});")
        else:
            self.emit_dy_reduce(E)
