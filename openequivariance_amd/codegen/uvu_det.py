"""Deterministic fused convolution with register-direct loads.

Edges are sorted by receiver.  One wavefront owns (a tile of R nodes, one 64-channel chunk) and
walks the node's edge list in order, so every sum has a fixed order and nothing is atomic:

* forward: the node is the receiver; per incoming edge the lane reads its X records of the
  sender, its weights and Y, and accumulates Z[node] in registers; Z is written once per node;
* backward: the node is the sender; the edge list is the (sender, receiver)-sorted order given by
  ``transpose_perm``; per outgoing edge the lane reads its dZ records of the receiver, weights
  and Y, writes dW[e] (coalesced) and dY[e] (per-chunk partial when the multiplicity spans several
  chunks), and accumulates dX[node] in registers.

All loads are unconditional from clamped, range-checked indices (see uvu_direct.py); an edge
that is out of range for its lane, or names a node that does not exist, contributes zero.  The
CSR pointers come from the prep kernels of the template (workspace).  The backward reads sender
and receiver of the permuted edge itself, so the graph need not be symmetric (the reference's
kernel reads both at the unpermuted position: templates/loop_unroll_conv_det.cuh:151-198).
"""
from __future__ import annotations

from ..problem import TPProblem
from .common import Emitter
from .uvu_direct import UVUDirectGenerator


class UVUDetGenerator(UVUDirectGenerator):
    _allow_det = True

    def __init__(self, problem: TPProblem):
        super().__init__(problem, "conv_det")
        self.uniform_rows = False          # validity is per lane (edge lists differ between sub-rows)
        self.chunk_in_grid = True

    def act(self, blk):
        return "rv" if self.full(blk) else f"(rv && u < {blk.mul})"

    def act_c(self, blk, c):
        return self.act(blk)

    def uexpr(self, c) -> str:
        return "u"

    # ------------------------------------------------------------------ common
    def _node_setup(self, E: Emitter, ptr_off: str) -> None:
        R = self.R
        E("const int c = blockIdx.y; (void)c;")
        E(f"const int u = c * {self.P} + ul;")
        if R == 1:
            E("const u64 node = blockIdx.x;")
        else:
            E(f"const u64 node = (u64)blockIdx.x * {R} + sub;")
        E("const bool nv = node < node_count;")
        E(f"const i64* __restrict__ ptr = (const i64*)ws + {ptr_off};")
        E("i64 beg = 0, end = 0;")
        E("if (nv && nnz > 0) { beg = ptr[node]; end = ptr[node + 1]; }")
        E("if (beg < 0) beg = 0;")
        E("if (end > (i64)nnz) end = (i64)nnz;")
        E("if (end < beg) end = beg;")
        E("const int len = (int)(end - beg);")
        E("int maxlen = len;")
        m = 32
        while m >= self.P:
            E(f"maxlen = max(maxlen, oeq_shfl_xor_i32(maxlen, {m}));")
            m //= 2
        if R == 1:
            E("maxlen = __builtin_amdgcn_readfirstlane(maxlen);")
        base = "node" if R == 1 else f"((u64)blockIdx.x * {R} + {{r}})"
        if R == 1:
            self.noderow_of = (lambda r: ("node", "nv"))
        else:
            self.noderow_of = (lambda r: (f"((u64)blockIdx.x * {R} + {r})", f"((u64)blockIdx.x * {R} + {r} < node_count)"))

    # ================================================================= forward
    def conv_det_forward_body(self) -> str:
        E = Emitter()
        self.emit_lane_direct(E, lds=True)
        self._node_setup(E, "0")
        self._cur_c = "e"
        for oi in self.used_out:
            E("T " + ", ".join(f"z{oi}_{k} = (T)0" for k in range(self.out[oi].D)) + ";")
        E("for (int it = 0; it < maxlen; ++it) {")
        E.level += 1
        E("const bool ev = it < len;")
        E("const u64 e = ev ? (u64)(beg + it) : (u64)(nnz - 1);     // idle lanes re-read the last edge, masked below")
        E("const i64 snd = cols[e];")
        E("const bool rv = ev && snd >= 0 && snd < (i64)node_count;")
        E("const u64 sndc = rv ? (u64)snd : 0;")
        E(f"const T* __restrict__ Yr = Y + e * {self.D2};")
        E(f"const T* __restrict__ Wr = W + e * {self.WN};")
        self.emit_y_load_direct(E)
        # X records of the sender (zero for idle lanes: everything they add is proportional to x)
        for i in self.used_in1:
            a = self.in1[i]
            self.emit_record_load(E, [f"x{i}_{m}" for m in range(a.D)],
                                  f"X + sndc * {self.D1} + {a.off} + {self.uclamp(a, 0)} * {a.D}", self.act(a), zero=True)
        for p in self.paths:
            for v in range(p.mv):
                E(f"const T We_{p.t}_{v} = Wr[{self.widx(p, self.uclamp(p.a, 0), v)}];")
        for oi in self.used_out:
            self.emit_forward_block(E, self.out[oi], "Wr", zname=f"z{oi}_", declare=False)
        E.level -= 1
        E("}")
        E("const bool rv = nv;")
        for o in self.out:
            if o.dim == 0:
                continue
            E("{")
            E.level += 1
            if o.idx in self.used_out:
                self.emit_block_store(E, o, [f"z{o.idx}_{k}" for k in range(o.D)], "Z", self.D3, "node",
                                      self.noderow_of, "store", via_lds=True)
            else:
                self.emit_record_store(E, ["(T)0"] * o.D, f"Z + node * {self.D3} + {o.off} + u * {o.D}", self.act(o))
            E.level -= 1
            E("}")
        return E.text()

    def uclamp(self, blk, c) -> str:
        return "u" if self.full(blk) else f"min(u, {blk.mul - 1})"

    # ================================================================ backward
    def conv_det_backward_body(self) -> str:
        E = Emitter()
        self.emit_lane_direct(E, lds=False)
        self._node_setup(E, "(node_count + 1)")
        self._cur_c = "e"
        # this node's own X chunk (fixed over the edge loop)
        E("bool rv = nv;")
        E("const u64 nodec = nv ? node : 0;")
        for i in self.used_in1:
            a = self.in1[i]
            self.emit_record_load(E, [f"x{i}_{m}" for m in range(a.D)],
                                  f"X + nodec * {self.D1} + {a.off} + {self.uclamp(a, 0)} * {a.D}", self.act(a), zero=True)
            E("T " + ", ".join(f"dx{i}_{m} = (T)0" for m in range(a.D)) + ";")
        E("for (int it = 0; it < maxlen; ++it) {")
        E.level += 1
        E("const bool ev = it < len;")
        E("const u64 j = ev ? (u64)(beg + it) : (u64)(nnz - 1);")
        E("const i64 e0 = tperm[j];")
        E("const bool ok_e = ev && e0 >= 0 && e0 < (i64)nnz;")
        E("const u64 e = ok_e ? (u64)e0 : 0;")
        E("const i64 rcv = rows[e];")
        E("rv = ok_e && rcv >= 0 && rcv < (i64)node_count;")
        E("const u64 rcvc = rv ? (u64)rcv : 0;")
        E(f"const T* __restrict__ Yr = Y + e * {self.D2};")
        E(f"const T* __restrict__ Wr = W + e * {self.WN};")
        E(f"T* __restrict__ Wgr = Wg + e * {self.WN};")
        self.emit_y_load_direct(E)
        for f in self.used_y:
            E(f"T dy{f} = (T)0;")
        for p in self.paths:
            for v in range(p.mv):
                E(f"const T We_{p.t}_{v} = Wr[{self.widx(p, self.uclamp(p.a, 0), v)}];")
        for oi in self.used_out:
            o = self.out[oi]
            self.emit_record_load(E, [f"G{oi}_{k}" for k in range(o.D)],
                                  f"G + rcvc * {self.D3} + {o.off} + {self.uclamp(o, 0)} * {o.D}", self.act(o), zero=True)
        for oi in self.used_out:
            o = self.out[oi]
            E("{")
            E.level += 1
            for k in range(o.D):
                E(f"const T g{k} = G{oi}_{k};")

            def sink(E, p, v, expr):
                E(f"  if ({self.act(p.a)}) Wgr[{self.widx(p, 'u', v)}] = {expr};")
            self.emit_backward_block(E, o, "Wr", sink)
            E.level -= 1
            E("}")
        self.emit_dy_sum(E)
        writer = "ul == 0" if self.P < 64 else "lane == 63"
        E(f"if (rv && {writer}) {{")
        if self.NCH > 1:
            E(f"    T* __restrict__ Ygr = (T*)((char*)ws + DYPART_OFF) + ((u64)c * nnz + e) * {self.D2};")
        else:
            E(f"    T* __restrict__ Ygr = Yg + e * {self.D2};")
        for f in range(self.D2):
            E(f"    Ygr[{f}] = " + (f"dy{f};" if f in self.used_y else "(T)0;"))
        E("}")
        E.level -= 1
        E("}")
        E("rv = nv;")
        for a in self.in1:
            if a.dim == 0:
                continue
            dst = f"Xg + node * {self.D1} + {a.off} + u * {a.D}"
            if a.idx in self.used_in1:
                self.emit_record_store(E, [f"dx{a.idx}_{m}" for m in range(a.D)], dst, self.act(a))
            else:
                self.emit_record_store(E, ["(T)0"] * a.D, dst, self.act(a))
        return E.text()

    def emit_dy_sum(self, E: Emitter) -> None:
        """Sum dy* over the lanes of a row in a fixed order.  A full wavefront per row uses the
        DPP row operations (total lands in lane 63); smaller groups use the xor butterfly."""
        if self.P == 64:
            for f in self.used_y:
                E(f"dy{f} = oeq_wave_sum63(dy{f});")
        else:
            self.emit_dy_reduce(E)
