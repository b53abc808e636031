"""Fused convolution over an unsorted edge list (``deterministic=False``) without float atomics
in the forward pass.

fp32 atomics on MI355X retire at a few hundred G lane-operations per second, and the forward
scatters d3 values per edge, so an atomic forward is several times slower than its memory traffic.
Instead every forward call first groups the edges by receiver with a counting sort (integer
atomics: two per edge), then runs the segmented forward of the deterministic variant over that
order: one wavefront per (node, 64-channel chunk), Z written once per node.  The order of the
edges inside a node's group depends on the order in which the integer atomics land, so the
floating-point sums may differ in the last bits between runs, like the atomic kernel they replace
(reference: templates/loop_unroll_conv_atomic.cuh:25-141 scatters with atomicAdd).

The backward scatters only d1 values per edge (dX), dW and dY being per-edge outputs.  While d1 is
very small it keeps the register-direct kernel with coalesced atomics; from ATOMIC_BACKWARD_MAX_D1
values per edge on, the backward groups the edges by sender in the same way and runs the
deterministic variant's backward over that order (the atomics retire slower than the row gathers of
the segmented backward, and the grouping is reused from the workspace while the graph stays the same).

Workspace: (node_count + 1) group pointers, (node_count + 1) fill cursors and nnz edge positions,
all int64, for the forward; behind them the same three arrays of the grouped backward (by sender), its
node order and its per-chunk dY partial sums.  The two groupings do not overlap, so a workspace
prepared by one forward and one backward call serves later calls on the same graph unchanged.
"""
from __future__ import annotations

from .. import tunables
from ..problem import TPProblem
from .common import jinja_env
from .uvu_det import UVUDetGenerator
from .uvu_direct import UVUDirectGenerator
from .uvu_recv import UVURecvGenerator


class UVUSortedGenerator:
    kind = "conv_atomic"
    SCAN_THREADS = 1024

    # dX values per edge from which the grouped backward is the starting choice.  Measured with the grouping
    # rebuilt on every call: 288 per edge - atomic 202 us, grouped 200 us, a tie; 2304 per edge - atomic
    # 9.1 ms, grouped 7.7 ms.  With the grouping reused from the workspace (a model calls one graph many
    # times): 288 per edge - atomic 204 us, grouped 161 us; 1152 per edge - atomic 2.90 ms, grouped 2.22 ms.
    # Below a couple of cache lines per edge the atomics are few and the starting choice stays atomic; the
    # torch operator measures both on first use either way.
    ATOMIC_BACKWARD_MAX_D1 = 128

    # dZ row / X row from which the grouped backward runs in receiver order (same measurements as the rule of the
    # deterministic operator, conv.RECV_ORDER_MIN_RATIO; here the receiver grouping costs a second counting sort)
    RECV_ORDER_MIN_RATIO = 5.5

    def __init__(self, problem: TPProblem, vector_stores: bool = True, grouped_backward=None, idx_ctype: str = "i64",
                 recv_backward=None):
        self.problem = problem
        self.fwd = UVUDetGenerator(problem, forward_perm=True, vector_stores=vector_stores, idx_ctype=idx_ctype)
        if grouped_backward is None:
            forced = tunables.current.conv_backward               # "grouped" / "atomic": A/B runs
            grouped_backward = (forced == "grouped") if forced else self.fwd.D1 >= self.ATOMIC_BACKWARD_MAX_D1
        self.grouped_backward = grouped_backward
        self.recv_backward = False
        if grouped_backward:
            self.bwd = UVUDetGenerator(problem, backward_perm=True, vector_stores=vector_stores, idx_ctype=idx_ctype)
            if recv_backward is not False and (recv_backward or self.fwd.D3 >= self.RECV_ORDER_MIN_RATIO * self.fwd.D1):
                # long dZ rows: the two-pass backward in receiver order (pass 1 over the receiver grouping, which the
                # backward then builds as well; pass 2 over the sender grouping), where pass 1 can stage its operands
                # (fp32).  In fp64 pass 1 with register loads, one launch per in1 block, runs over the position list as
                # well, but the second counting sort costs what it gains: the MACE problem, 10 000 nodes / 300 000 edges,
                # backward 5.16 ms in sender order, 5.32 ms in receiver order; it is taken on request only
                recv = UVURecvGenerator(problem, vector_stores=vector_stores, idx_ctype=idx_ctype, backward_perm=True)
                if recv_backward is True or recv.staged_edges:
                    self.bwd, self.recv_backward = recv, True
        else:
            self.bwd = UVUDirectGenerator(problem, "conv_atomic", vector_stores=vector_stores)
            self.bwd.idx_ctype = idx_ctype
        self.T = self.fwd.T
        self.D1, self.D2, self.D3, self.WN = self.fwd.D1, self.fwd.D2, self.fwd.D3, self.fwd.WN
        self.NCH = self.fwd.NCH
        # one piece area (counters and partial rows of long nodes) behind everything else, shared by both directions
        if grouped_backward:
            self.fwd.piece_base = self.bwd.piece_base
        else:
            self.fwd.piece_base = f"((({self.fwd.GROUP_WORDS}) * sizeof(i64) + 255ull) & ~255ull)"

    def describe(self) -> str:
        return ("sorted forward: " + self.fwd.describe()
                + (" | grouped backward: " if self.grouped_backward else " | atomic backward: ") + self.bwd.describe())

    def render(self, prelude: str = None) -> str:
        env = jinja_env()
        if prelude is None:
            prelude = env.get_template("prelude.hip.jinja").render(T=self.T)
        return env.get_template("conv_sorted.hip.jinja").render(g=self, prelude=prelude)

    def plan(self):
        ROW, NODE, FIXED = 1, 2, 0
        f = self.fwd
        S = self.SCAN_THREADS

        def grouping(sfx):
            return [dict(kernel="group_clear" + sfx, num_threads=256, grid_kind=NODE, work_per_block=256,
                         prep=True, counter_clear=True),
                    dict(kernel="group_count" + sfx, num_threads=S, grid_kind=ROW, work_per_block=S, prep=True),
                    dict(kernel="group_fill" + sfx, num_threads=256, grid_kind=ROW, work_per_block=256, prep=True)]
        fwd = grouping("") + f.forward_steps(dict(kernel="forward", num_threads=64, grid_kind=3, work_per_block=1,
                                                  num_blocks=f.LONG, grid_y=f.NCH))
        G = f.group_bytes
        if not self.grouped_backward:
            _, bwd, _ = self.bwd.plan()

            def ws(nnz=0, nodes=0):
                return ((G(nnz, nodes) + 255) & ~255) + f.piece_bytes(nnz, nodes)
            return fwd, bwd, ws
        b = self.bwd
        bwd = (grouping("_recv") if self.recv_backward else []) + grouping("_backward") + b.backward_steps()

        def ws(nnz=0, nodes=0):
            if self.recv_backward:
                return b.main_bytes(nnz, nodes) + b.piece_bytes(nnz, nodes)
            main = 2 * G(nnz, nodes) + b.order_bytes(nodes) + b.dy_partial_bytes(nnz) + b.flag_bytes(nnz)
            return ((main + 255) & ~255) + b.piece_bytes(nnz, nodes)
        return fwd, bwd, ws

    def forward_workspace_model(self):
        """(fixed, per node, per edge) bytes the forward steps use when no node is cut into pieces."""
        return 32, 24, 8
