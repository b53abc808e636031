"""The benchmark workloads: problems, seeded synthetic inputs and algorithmic work.

Each workload names the problem, generates its inputs on the host with
``numpy.random.default_rng(seed)`` (seed 12345 + configuration index, the default seed of the
reference's suites: openequivariance/benchmark/TestBenchmarkSuite.py:36), moves them to the
GPU and exposes ``forward()`` / ``backward()`` closures that call the C-ABI entry points on
preallocated outputs.  The byte model is the reference's own for the batch product
(openequivariance/benchmark/perf_metrics_utils.py:11-44) and the compulsory traffic for the
fused convolution (every tensor touched once).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, Optional

import numpy as np

from .conv import TensorProductConv
from .problem import ChannelwiseTPP, FullyConnectedTPProblem, TPProblem
from .sh import random_unit_vectors, spherical_harmonics
from .tensor_product import TensorProduct

MACE = ("128x0e+128x1o+128x2e", "1x0e+1x1o+1x2e+1x3o", "128x0e+128x1o+128x2e+128x3o")
# the same inputs with every triangle-allowed output kept, also the unnatural parities 1e, 2o, 3e
MACE_ALL = ("128x0e+128x1o+128x2e", "1x0e+1x1o+1x2e+1x3o", "128x0e+128x1o+128x1e+128x2e+128x2o+128x3o+128x3e")
NEQUIP = ("32x0e+32x1o+32x2e", "1x0e+1x1o+1x2e", "32x0e+32x1o+32x2e")
NEQUIP_ALL = ("32x0e+32x1o+32x2e", "1x0e+1x1o+1x2e", "32x0e+32x1o+32x1e+32x2e+32x2o")
LARGE_ALL = ("256x0e+256x1o+256x2e", "1x0e+1x1o+1x2e+1x3o", "256x0e+256x1o+256x1e+256x2e+256x2o")
LARGE = ("256x0e+256x1o+256x2e", "1x0e+1x1o+1x2e+1x3o", "256x0e+256x1o+256x2e")
DENSE = ("64x0e+64x1o+64x2e", "1x0e+1x1o+1x2e", "64x0e+64x1o+64x2e")
# reference: benchmark/benchmark_configs.py:45-48 (the larger of its two per-row-weights problems)
# reference: benchmark/benchmark_configs.py:38-41 (the other two problems of its uvw benchmark; shared weights)
TETRIS_POLY = {"1": ("1x0e+1x1o+1x2e+1x3o", "1x0e+1x1o+1x2e+1x3o", "64x0e+24x1e+24x1o+16x2e+16x2o"),
               "2": ("64x0e+24x1e+24x1o+16x2e+16x2o", "1x0e+1x1o+1x2e+1x3o", "1x0o+6x0e")}
DIFFDOCK_L2 = ("10x1o+10x1e+48x0e+48x0o", "1x0e+1x1o+1x2e", "10x1o+10x1e+48x0e+48x0o")
DIFFDOCK_L1 = ("10x1o+10x1e+48x0e+48x0o", "1x0e+1x1o", "10x1o+10x1e+48x0e+48x0o")


def _normal(rng, shape, dtype, scale=1.0, chunk=1 << 24):
    """N(0, scale^2) samples drawn in chunks directly in the target precision."""
    out = np.empty(shape, dtype=dtype)
    flat = out.reshape(-1)
    for s in range(0, flat.size, chunk):
        e = min(flat.size, s + chunk)
        flat[s:e] = rng.standard_normal(e - s, dtype=np.float32 if dtype == np.float32 else np.float64)
    if scale != 1.0:
        out *= dtype(scale)
    return out


@dataclass
class Case:
    op: object
    tensors: Dict[str, object]
    forward: Callable[[], None]
    backward: Callable[[], None]
    host: Dict[str, np.ndarray] = field(default_factory=dict)
    # convolutions: ``forward`` / ``backward`` prepare the graph (CSR pointers, position lists, node order) on
    # every call, as the operators do by default; these reuse the preparation left in the workspace, the
    # regime of an operator built with graph_cache=True whose layers call one graph many times
    forward_prepared: Optional[Callable[[], None]] = None
    backward_prepared: Optional[Callable[[], None]] = None
    # the operator a user calls: forward through the torch custom op, backward through autograd
    torch_step: Optional[Callable[[], None]] = None


@dataclass
class Workload:
    name: str
    description: str
    kind: str                    # "tp" | "conv"
    irreps: tuple
    units: int                   # rows / edges per step
    unit: str
    bound: str                   # "hbm" | "mfma"
    dtype: str
    seed: int
    config: dict
    nodes: int = 0
    deterministic: bool = False
    sh_lmax: Optional[int] = None
    mode: str = "uvu"
    w_scale: float = 1.0
    alg_bytes: Dict[str, int] = field(default_factory=dict)
    alg_flops: Dict[str, int] = field(default_factory=dict)
    min_traffic: Dict[str, int] = field(default_factory=dict)
    # True: X, W and G are drawn on the GPU with torch's generator (the large workload's weights
    # are 10.6 GB; drawing them on the host takes minutes); the graph and Y still come from numpy
    device_inputs: bool = False
    # probe graphs: receivers drawn from the first ``receiver_pool`` nodes only (0: from all), so that the dZ
    # rows the backward gathers fit a cache of a known size
    receiver_pool: int = 0
    # uvw problems: one weight vector for the batch (True) or one per row (False)
    shared: bool = True

    @property
    def data_note(self) -> str:
        if self.device_inputs and self.kind == "tp":
            return "synthetic (X, Y and dZ seeded on the host, the per-row weights drawn on the GPU)"
        return ("synthetic (graph and Y seeded on the host, X / W / dZ drawn on the GPU)" if self.device_inputs
                else "synthetic")

    def read_write_split(self, direction: str):
        """(bytes read, bytes written) of the algorithmic traffic of one launch."""
        prob = self.problem()
        s = 4 if self.dtype == "f32" else 8
        d1, d2, d3, wn = prob.irreps_in1.dim, prob.irreps_in2.dim, prob.irreps_out.dim, prob.weight_numel
        if self.kind == "tp":
            n = self.units
            w = wn if prob.shared_weights else wn * n
            written = n * d3 * s if direction == "forward" else (n * (d1 + d2) + w) * s
        else:
            E, N = self.units, self.nodes
            written = N * d3 * s if direction == "forward" else (E * (d2 + wn) + N * d1) * s
        return self.alg_bytes[direction] - written, written

    # ------------------------------------------------------------------ problem
    def problem(self) -> TPProblem:
        dt = np.float32 if self.dtype == "f32" else np.float64
        if self.mode == "uvw":
            return FullyConnectedTPProblem(*self.irreps, shared_weights=self.shared, internal_weights=False,
                                           irrep_dtype=dt, weight_dtype=dt)
        if self.irreps == ("1x2e", "1x3e", "1x2e"):
            return TPProblem(*self.irreps, [(0, 0, 0, "uvu", True)], shared_weights=False, internal_weights=False)
        return ChannelwiseTPP(*self.irreps, irrep_dtype=dt, weight_dtype=dt)

    # ------------------------------------------------------------------- inputs
    def graph(self, rng):
        """rows (receivers), cols (senders)[, transpose_perm] for the convolution workloads."""
        N, E = self.nodes, self.units
        if self.name.startswith("large"):
            deg = rng.poisson(40, N)
            rows = np.repeat(np.arange(N, dtype=np.int64), deg)
            cols = rng.integers(0, N, rows.size).astype(np.int64)
        else:
            rows = rng.integers(0, self.receiver_pool or N, E).astype(np.int64)
            cols = rng.integers(0, N, E).astype(np.int64)
            clash = rows == cols
            cols[clash] = (cols[clash] + 1 + rng.integers(0, N - 1, int(clash.sum()))) % N
        tperm = None
        if self.deterministic:
            order = np.lexsort((cols, rows))
            rows, cols = rows[order], cols[order]
            tperm = np.lexsort((np.arange(rows.size), rows, cols)).astype(np.int64)
        return rows, cols, tperm

    def host_inputs(self, n_rows: Optional[int] = None):
        """Seeded host arrays; ``n_rows`` truncates the batch for the CPU sample (TP only)."""
        prob = self.problem()
        dt = np.float32 if self.dtype == "f32" else np.float64
        rng = np.random.default_rng(self.seed)
        d1, d2, d3, wn = prob.irreps_in1.dim, prob.irreps_in2.dim, prob.irreps_out.dim, prob.weight_numel
        h = {}
        if self.kind == "tp":
            n = self.units if n_rows is None else n_rows
            h["X"] = _normal(rng, (n, d1), dt)
            if self.sh_lmax is not None:
                h["Y"] = spherical_harmonics(self.sh_lmax, random_unit_vectors(n, rng)).astype(dt)
            else:
                h["Y"] = rng.uniform(size=(n, d2)).astype(dt)
            wshape = (wn,) if prob.shared_weights else (n, wn)
            if not self.device_inputs:
                h["W"] = _normal(rng, wshape, dt, self.w_scale)
            h["G"] = _normal(rng, (n, d3), dt)
        else:
            rows, cols, tperm = self.graph(rng)
            E = rows.size
            h["rows"], h["cols"] = rows, cols
            if tperm is not None:
                h["tperm"] = tperm
            if not self.device_inputs:
                h["X"] = _normal(rng, (self.nodes, d1), dt)
            h["Y"] = spherical_harmonics(self.sh_lmax, random_unit_vectors(E, rng)).astype(dt)
            if not self.device_inputs:
                h["W"] = _normal(rng, (E, wn), dt)
                h["G"] = _normal(rng, (self.nodes, d3), dt)
        return prob, h

    # -------------------------------------------------------------------- build
    def build(self, device) -> Case:
        import torch
        prob, h = self.host_inputs()
        t = {k: torch.from_numpy(v).to(device) for k, v in h.items()}
        if self.device_inputs and self.kind == "tp":
            # per-row weights: the one large tensor is drawn on the GPU, the CPU baseline gets its first rows
            gen = torch.Generator(device=device)
            gen.manual_seed(self.seed)
            t["W"] = torch.randn(h["X"].shape[0], prob.weight_numel, device=device, generator=gen,
                                 dtype=torch.float32 if self.dtype == "f32" else torch.float64) * self.w_scale
            h["W"] = t["W"][:8192].cpu().numpy()
        elif self.device_inputs:
            gen = torch.Generator(device=device)
            gen.manual_seed(self.seed)
            tdt = torch.float32 if self.dtype == "f32" else torch.float64
            E = h["rows"].size
            t["X"] = torch.randn(self.nodes, prob.irreps_in1.dim, device=device, dtype=tdt, generator=gen)
            t["W"] = torch.randn(E, prob.weight_numel, device=device, dtype=tdt, generator=gen)
            t["G"] = torch.randn(self.nodes, prob.irreps_out.dim, device=device, dtype=tdt, generator=gen)
            # the host copies the CPU baseline needs: node tensors whole, per-edge ones for a sample
            h["X"], h["G"] = t["X"].cpu().numpy(), t["G"].cpu().numpy()
            h["W"] = t["W"][:8192].cpu().numpy()
        stream = torch.cuda.current_stream().cuda_stream
        if self.kind == "tp":
            op = TensorProduct(prob, torch_op=True)
            n = h["X"].shape[0]
            t["Z"] = torch.empty((n, prob.irreps_out.dim), dtype=t["X"].dtype, device=device)
            t["Xg"], t["Yg"], t["Wg"] = (torch.empty_like(t[k]) for k in ("X", "Y", "W"))
            p = {k: v.data_ptr() for k, v in t.items()}

            def fwd():
                op.forward_raw(n, p["X"], p["Y"], p["Z"], p["W"], stream)

            def bwd():
                op.backward_raw(n, p["X"], p["Xg"], p["Y"], p["Yg"], p["W"], p["Wg"], p["G"], stream)
            self.units = n
            leaves = [t[k].detach().requires_grad_(True) for k in ("X", "Y", "W")]
            torch_step = self._torch_step(op.forward, leaves, (), t["G"])
        else:
            op = TensorProductConv(prob, torch_op=True, deterministic=self.deterministic)
            E, N = h["rows"].size, self.nodes
            self.units = E
            self._fill_conv_bytes(prob, E, N)
            t["Z"] = torch.zeros((N, prob.irreps_out.dim), dtype=t["X"].dtype, device=device)
            t["Xg"] = torch.zeros_like(t["X"])
            t["Yg"], t["Wg"] = torch.empty_like(t["Y"]), torch.empty_like(t["W"])
            p = {k: v.data_ptr() for k, v in t.items()}
            tp_ptr = p.get("tperm", 0)
            ws = op.workspace_ptr(E, N)
            det = self.deterministic

            def fwd(prepared=False, zero=True):
                if not op.forward_overwrites:
                    t["Z"].zero_()              # atomic kernels accumulate: part of the operator's work
                op.exec_conv_rawptrs(p["X"], p["Y"], p["W"], p["Z"], p["rows"], p["cols"], E, N, ws, tp_ptr, stream,
                                     prepared=prepared, counters_zero=zero)

            def bwd(prepared=False, zero=True):
                if not op.backward_overwrites:
                    t["Xg"].zero_()             # likewise for the backward that scatters dX with atomics
                op.backward_rawptrs(p["X"], p["Xg"], p["Y"], p["Yg"], p["W"], p["Wg"], p["G"], p["rows"], p["cols"],
                                    E, N, ws, tp_ptr, stream, prepared=prepared, counters_zero=zero)
            # the first calls clear the grouping counters of the (uninitialised) workspace; every call leaves
            # them zeroed, so the timed ones skip that step, as the torch operator does on its own workspace
            fwd(zero=False)
            bwd(zero=False)
            leaves = [t[k].detach().requires_grad_(True) for k in ("X", "Y", "W")]
            index = tuple(t[k] for k in ("rows", "cols", "tperm") if k in t)
            return Case(op, t, fwd, bwd, h, lambda: fwd(True), lambda: bwd(True),
                        self._torch_step(op.forward, leaves, index, t["G"]))
        return Case(op, t, fwd, bwd, h, torch_step=torch_step)

    @staticmethod
    def _torch_step(forward, leaves, index, G):
        """One forward + backward through the torch operator: returns (run forward, run backward of its result)."""
        state = {}

        def run_forward():
            for a in leaves:
                a.grad = None
            state["z"] = forward(*leaves, *index)

        def run_backward():
            state.pop("z").backward(G)
        return run_forward, run_backward

    def _fill_conv_bytes(self, prob, E, N):
        s = 4 if self.dtype == "f32" else 8
        d1, d2, d3, wn = prob.irreps_in1.dim, prob.irreps_in2.dim, prob.irreps_out.dim, prob.weight_numel
        self.alg_bytes = {"forward": E * (d2 + wn) * s + N * (d1 + d3) * s + E * 16,
                          "backward": 2 * E * (d2 + wn) * s + N * (2 * d1 + d3) * s + E * 24}
        # What a schedule must move when no gathered row is found in a cache: the forward reads X[sender] per
        # edge; the backward either gathers dZ[receiver] per edge (sender order) or gathers X[sender] and
        # writes and re-reads a dX row per edge (receiver order), whichever is less.
        self.min_traffic = {"forward": self.alg_bytes["forward"] + E * d1 * s,
                            "backward": self.alg_bytes["backward"] + E * min(d3, 3 * d1) * s}
        self.config["edges"] = int(E)


def _tp_bytes(prob, n, s):
    d1, d2, d3, wn = prob.irreps_in1.dim, prob.irreps_in2.dim, prob.irreps_out.dim, prob.weight_numel
    w = wn if prob.shared_weights else wn * n
    return {"forward": (n * (d1 + d2 + d3) + w) * s, "backward": (n * (2 * d1 + 2 * d2 + d3) + 2 * w) * s}


def get(name: str) -> Workload:
    if name == "mace_uvu":
        w = Workload(name, "MACE-style per-edge uvu TP, 128x0e+128x1o+128x2e (x) SH(lmax 3) -> l3<=3, 17 paths, "
                     "batch 50000, fp32, forward+backward", "tp", MACE, 50000, "edges/s", "hbm", "f32", 12346,
                     {"batch": 50000, "paths": 17}, sh_lmax=3)
        w.alg_bytes = _tp_bytes(w.problem(), w.units, 4)
        return w
    if name == "mace_uvu_all_parities":
        w = Workload(name, "per-edge uvu TP, 128x0e+128x1o+128x2e (x) SH(lmax 3) -> every triangle-allowed l3<=3 of either "
                     "parity, 24 paths, batch 50000, fp32, forward+backward", "tp", MACE_ALL, 50000, "edges/s", "hbm",
                     "f32", 12346, {"batch": 50000, "paths": 24}, sh_lmax=3)
        w.alg_bytes = _tp_bytes(w.problem(), w.units, 4)
        return w
    if name == "readme_uvu":
        w = Workload(name, "single-path uvu TP 1x2e (x) 1x3e -> 1x2e, batch 1000, fp32", "tp",
                     ("1x2e", "1x3e", "1x2e"), 1000, "rows/s", "hbm", "f32", 12345, {"batch": 1000, "paths": 1})
        w.alg_bytes = _tp_bytes(w.problem(), w.units, 4)
        return w
    if name.startswith("nequip_conv_det_receivers"):
        # the deterministic NequIP convolution on a graph whose receivers are all among the first k nodes: a dZ
        # working set of k x 4480 bytes for the backward's gathers (probe of what cache-resident dZ would buy)
        k = int(name[len("nequip_conv_det_receivers"):])
        w = get("nequip_conv_det")
        w.name, w.receiver_pool = name, k
        w.description += f", receivers among the first {k} nodes only"
        return w
    if name in ("nequip_conv_atomic", "nequip_conv_det"):
        det = name.endswith("det")
        return Workload(name, "NequIP-style fused uvu conv, 32x0e+32x1o+32x2e (x) SH(lmax 2), 11 paths, 5000 nodes, "
                        "150000 edges, fp32, forward+backward, " + ("deterministic (receiver-sorted)" if det else "atomic (unsorted)"),
                        "conv", NEQUIP, 150000, "edges/s", "hbm", "f32", 12347,
                        {"nodes": 5000, "paths": 11, "deterministic": det}, nodes=5000, deterministic=det, sh_lmax=2)
    if name in ("large_conv_det", "large_conv_atomic"):
        det = name.endswith("det")
        return Workload(name, "large fused uvu conv, 256x0e+256x1o+256x2e (x) SH(lmax 3) -> l3<=2, 13 paths, 20000 nodes, "
                        "Poisson(40) in-degree (~800000 edges), fp32, forward+backward, "
                        + ("deterministic" if det else "atomic"),
                        "conv", LARGE, 800000, "edges/s", "hbm", "f32", 12349,
                        {"nodes": 20000, "paths": 13, "deterministic": det}, nodes=20000, deterministic=det, sh_lmax=3,
                        device_inputs=True)
    if name in ("mace_conv_det", "mace_conv_atomic", "mace_conv_det_f64", "mace_conv_atomic_f64"):
        # (the reference's convolution benchmark runs this problem in fp32 and in fp64, test/benchmark.py:179-188)
        dt = "f64" if name.endswith("_f64") else "f32"
        det = "_det" in name
        return Workload(name, "MACE-style fused uvu conv (the problem of the tensor-product benchmark as a convolution), "
                        f"128x0e+128x1o+128x2e (x) SH(lmax 3) -> l3<=3, 17 paths, 10000 nodes, 300000 edges, fp{dt[1:]}, "
                        "forward+backward, " + ("deterministic (receiver-sorted)" if det else "unsorted"),
                        "conv", MACE, 300000, "edges/s", "hbm", dt, 12350,
                        {"nodes": 10000, "paths": 17, "deterministic": det}, nodes=10000, deterministic=det, sh_lmax=3)
    if name in ("benzene_conv_det", "benzene_conv_det_f64"):
        # the largest problem of the reference's list (test/benchmark.py:44-55, nequip-revmd17-benzene): 68 paths, 312
        # output words per channel, forward and backward in several launches over groups of output blocks
        from .benchmark.benchmark_configs import nequip_conv
        irreps = tuple(s_.replace(" ", "") for s_ in [c for c in nequip_conv if c[3] == "nequip-revmd17-benzene"][0][:3])
        dt = "f64" if name.endswith("_f64") else "f32"
        return Workload(name, "NequIP-style fused uvu conv with irreps of either parity up to l = 3 (nequip-revmd17-benzene of "
                        f"the reference's problem list), 64 channels, 68 paths, 5000 nodes, 150000 edges, fp{dt[1:]}, "
                        "forward+backward, deterministic (receiver-sorted)",
                        "conv", irreps, 150000, "edges/s", "hbm", dt, 12353,
                        {"nodes": 5000, "paths": 68, "deterministic": True}, nodes=5000, deterministic=True, sh_lmax=3)
    if name == "nequip_conv_det_all_parities":
        return Workload(name, "fused uvu conv, 32x0e+32x1o+32x2e (x) SH(lmax 2) -> every triangle-allowed l3<=2 of either "
                        "parity, 15 paths, 5000 nodes, 150000 edges, fp32, forward+backward, deterministic (receiver-sorted)",
                        "conv", NEQUIP_ALL, 150000, "edges/s", "hbm", "f32", 12347,
                        {"nodes": 5000, "paths": 15, "deterministic": True}, nodes=5000, deterministic=True, sh_lmax=2)
    if name == "large_conv_det_all_parities":
        return Workload(name, "large fused uvu conv, 256x0e+256x1o+256x2e (x) SH(lmax 3) -> every triangle-allowed l3<=2 of "
                        "either parity, 18 paths, 20000 nodes, Poisson(40) in-degree (~800000 edges), fp32, "
                        "forward+backward, deterministic",
                        "conv", LARGE_ALL, 800000, "edges/s", "hbm", "f32", 12349,
                        {"nodes": 20000, "paths": 18, "deterministic": True}, nodes=20000, deterministic=True, sh_lmax=3,
                        device_inputs=True)
    if name in ("dense_uvw_f32", "dense_uvw_f64"):
        dt = "f32" if name.endswith("f32") else "f64"
        w = Workload(name, "dense uvw TP with shared weights, 64x0e+64x1o+64x2e (x) SH(lmax 2) -> 64x0e+64x1o+64x2e, "
                     f"11 paths, batch 100000, {dt}, forward+backward", "tp", DENSE, 100000, "rows/s", "mfma", dt,
                     12348, {"batch": 100000, "paths": 11}, sh_lmax=2, mode="uvw", w_scale=0.125)
        prob = w.problem()
        dense = sum(2 * int(np.prod(t.path_shape)) * prob.irreps_out[t.i_out].ir.dim for t in prob.instructions)
        w.alg_flops = {"forward": dense * w.units, "backward": 2 * dense * w.units}
        w.alg_bytes = _tp_bytes(prob, w.units, 4 if dt == "f32" else 8)
        return w
    if name in ("diffdock_uvw_f32", "diffdock_uvw_f64", "diffdock1_uvw_f32", "diffdock1_uvw_f64"):
        dt = "f32" if name.endswith("f32") else "f64"
        L = 1 if name.startswith("diffdock1") else 2
        irreps = DIFFDOCK_L1 if L == 1 else DIFFDOCK_L2
        w = Workload(name, f"uvw TP with a weight vector per row (DiffDock-L={L} of the reference's uvw benchmark), "
                     f"{irreps[0]} (x) SH(lmax {L}) -> {irreps[2]}, batch 50000, {dt}, forward+backward", "tp", irreps,
                     50000, "rows/s", "hbm", dt, 12351, {"batch": 50000}, sh_lmax=L, mode="uvw", w_scale=0.2, shared=False,
                     device_inputs=True)
        prob = w.problem()
        w.config["paths"] = len(prob.instructions)
        w.description = w.description.replace(", batch 50000", f", {len(prob.instructions)} instructions, "
                                              f"{prob.weight_numel} weights per row, batch 50000")
        w.alg_bytes = _tp_bytes(prob, w.units, 4 if dt == "f32" else 8)
        return w
    if name.startswith("tetris_poly") and name[11:] in ("1_uvw_f32", "1_uvw_f64", "2_uvw_f32", "2_uvw_f64"):
        which, dt = name[11], name[-3:]
        irreps = TETRIS_POLY[which]
        w = Workload(name, f"uvw TP with shared weights, tetris-poly-{which} of the reference's uvw benchmark, "
                     f"{irreps[0]} (x) SH(lmax 3) -> {irreps[2]}, batch 50000, {dt}, forward+backward", "tp", irreps,
                     50000, "rows/s", "hbm", dt, 12352, {"batch": 50000}, sh_lmax=3, mode="uvw", w_scale=0.2)
        w.config["paths"] = len(w.problem().instructions)
        w.alg_bytes = _tp_bytes(w.problem(), w.units, 4 if dt == "f32" else 8)
        return w
    raise KeyError(f"unknown workload {name!r}")


ALL = ("readme_uvu", "mace_uvu", "mace_uvu_all_parities", "nequip_conv_atomic", "nequip_conv_det", "nequip_conv_det_all_parities",
       "large_conv_det", "large_conv_atomic", "large_conv_det_all_parities", "mace_conv_det", "mace_conv_atomic",
       "mace_conv_det_f64", "mace_conv_atomic_f64", "benzene_conv_det", "benzene_conv_det_f64", "dense_uvw_f32", "dense_uvw_f64", "diffdock_uvw_f32", "diffdock_uvw_f64", "diffdock1_uvw_f32", "diffdock1_uvw_f64",
       "tetris_poly1_uvw_f32", "tetris_poly1_uvw_f64", "tetris_poly2_uvw_f32", "tetris_poly2_uvw_f64")
