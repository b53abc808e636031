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

The backward keeps the register-direct kernel with coalesced atomics: it scatters only d1 values
per edge (dX) while dW and dY are per-edge outputs.

Workspace: (node_count + 1) group pointers, (node_count + 1) fill cursors and nnz edge positions,
all int64, rebuilt on every forward call.
"""
from __future__ import annotations

from ..problem import TPProblem
from .common import jinja_env
from .uvu_det import UVUDetGenerator
from .uvu_direct import UVUDirectGenerator


class UVUSortedGenerator:
    kind = "conv_atomic"
    SCAN_THREADS = 1024

    def __init__(self, problem: TPProblem, vector_stores: bool = True):
        self.problem = problem
        self.fwd = UVUDetGenerator(problem, forward_perm=True, vector_stores=vector_stores)
        self.bwd = UVUDirectGenerator(problem, "conv_atomic", vector_stores=vector_stores)
        self.T = self.fwd.T
        self.D1, self.D2, self.D3, self.WN = self.fwd.D1, self.fwd.D2, self.fwd.D3, self.fwd.WN
        self.NCH = self.fwd.NCH

    def describe(self) -> str:
        return "sorted forward: " + self.fwd.describe() + " | atomic backward: " + self.bwd.describe()

    def render(self, prelude: str = None) -> str:
        env = jinja_env()
        if prelude is None:
            prelude = env.get_template("prelude.hip.jinja").render(T=self.T)
        return env.get_template("conv_sorted.hip.jinja").render(g=self, prelude=prelude)

    def plan(self):
        ROW, NODE, FIXED = 1, 2, 0
        f = self.fwd
        fwd = [dict(kernel="group_clear", num_threads=256, grid_kind=NODE, work_per_block=256),
               dict(kernel="group_count", num_threads=256, grid_kind=ROW, work_per_block=256),
               dict(kernel="group_scan", num_threads=self.SCAN_THREADS, grid_kind=FIXED, num_blocks=1),
               dict(kernel="group_fill", num_threads=256, grid_kind=ROW, work_per_block=256),
               dict(kernel="forward", num_threads=64, grid_kind=NODE, work_per_block=1, grid_y=f.NCH)]
        _, bwd, _ = self.bwd.plan()

        def ws(nnz=0, nodes=0):
            return (2 * (nodes + 1) + nnz) * 8
        return fwd, bwd, ws
