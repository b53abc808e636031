"""``TensorProductConv``: fused gather - tensor product - scatter over graph edges.

Host-side mirror of the reference's ``oeq.TensorProductConv`` / ``LoopUnrollConv``
(reference: openequivariance/implementations/convolution/LoopUnrollConv.py:7-90,
ConvolutionBase.py:72-100 and :560-709): same constructor
``(problem, torch_op=False, deterministic=False)``, same ``forward`` signatures
(five arguments, plus ``transpose_perm`` when deterministic), first and second
derivatives through torch custom ops, raw-pointer entry points.

``rows`` are receivers (where Z rows are accumulated), ``cols`` are senders
(where X rows are gathered), both int64.  The deterministic variant requires
the edge list sorted by receiver and ``transpose_perm[j]`` = position in that
list of the j-th edge in (sender, receiver) order; it makes no symmetry
assumption about the graph.
"""
from __future__ import annotations

import typing

import numpy as np
import torch

from . import runtime as rt
from . import tunables
from .autograd_glue import double_backward_terms
from .codegen.uvu_det import UVUDetGenerator
from .codegen.uvu_direct import UVUDirectGenerator
from .codegen.uvu_recv import UVURecvGenerator
from .codegen.uvu_sorted import UVUSortedGenerator
from .problem import TPProblem
from .tensor_product import _contiguous, _make_steps, _on_device, validate_problem
from .weight_order import WeightReorder
from .wigner import wigner_3j


def flops_data_per_tp(config: TPProblem, direction: str):
    """(flops, bytes, nnz) per edge by the reference's model
    (reference: convolution/ConvolutionBase.py:11-43)."""
    s = np.dtype(config.irrep_dtype).itemsize
    L1, L2, L3 = config.irreps_in1, config.irreps_in2, config.irreps_out
    if direction == "forward":
        ops_per_nz, words = 3, L1.dim + L2.dim + L3.dim + config.weight_numel
    elif direction == "backward":
        ops_per_nz, words = 9, 2 * L1.dim + 2 * L2.dim + L3.dim + 2 * config.weight_numel
    else:
        raise ValueError(direction)
    ops = nnz = 0
    for ins in config.instructions:
        c = wigner_3j(L1[ins.i_in1].ir.l, L2[ins.i_in2].ir.l, L3[ins.i_out].ir.l)
        k = int(np.count_nonzero(np.abs(c) > 1e-14))
        nnz += k
        ops += ops_per_nz * k * L1[ins.i_in1].mul * L2[ins.i_in2].mul
        if ins.connection_mode == "uvu":
            ops += L3[ins.i_out].mul * L3[ins.i_out].ir.dim
        else:
            ops += L1[ins.i_in1].mul * L2[ins.i_in2].mul * L3[ins.i_out].ir.dim * L3[ins.i_out].mul
    return ops, words * s, nnz


class CoordGraph:
    """Receiver-sorted COO graph with its transpose permutation
    (reference: convolution/ConvolutionBase.py:45-70, vectorised)."""

    def __init__(self, coords, rows, cols, name="graph"):
        rows, cols = np.asarray(rows), np.asarray(cols)
        assert len(rows) == len(cols)
        self.nnz = len(rows)
        self.node_count = coords.shape[0] if hasattr(coords, "shape") else int(coords)
        self.coords, self.name = coords, name
        order = np.lexsort((cols, rows))
        self.rows, self.cols = rows[order], cols[order]
        self.order = order
        self.transpose_perm = np.lexsort((np.arange(self.nnz), self.rows, self.cols)).astype(self.rows.dtype)


def sort_by_receiver(rows: "torch.Tensor", cols: "torch.Tensor", node_count: typing.Optional[int] = None):
    """Graph preparation for ``deterministic=True`` on the tensors' own device (no torch_geometric):
    returns ``(rows_sorted, cols_sorted, receiver_perm, transpose_perm)`` where ``receiver_perm``
    sorts the edges by (receiver, sender) - apply it to the per-edge tensors Y and W - and
    ``transpose_perm`` lists the sorted edges in (sender, receiver) order, the last argument of
    ``TensorProductConv.forward``.  Same result as ``CoordGraph`` (reference:
    convolution/ConvolutionBase.py:45-70) and as the ``sort_by`` recipe of the reference's README
    (README.md:110-118); both sorts are stable, so the permutations are unique."""
    assert rows.dtype == torch.int64 and cols.dtype == torch.int64 and rows.shape == cols.shape and rows.dim() == 1
    if rows.numel() == 0:
        return rows, cols, rows.clone(), rows.clone()
    n = int(node_count) if node_count is not None else int(torch.maximum(rows.max(), cols.max()).item()) + 1
    receiver_perm = torch.argsort(rows * n + cols, stable=True)
    rows_s, cols_s = rows[receiver_perm], cols[receiver_perm]
    transpose_perm = torch.argsort(cols_s * n + rows_s, stable=True)
    return rows_s, cols_s, receiver_perm, transpose_perm


# d3 / d1 from which the deterministic backward walks the edges in receiver order (see select_conv_generator)
RECV_ORDER_MIN_RATIO = 5.5


def select_conv_generator(config: TPProblem, deterministic: bool, vector_stores: bool = True, idx_dtype=np.int64):
    """Kernel generator of the fused convolution: one node per wavefront with fixed summation order
    when deterministic; otherwise a forward that groups the edges by receiver on the fly and a
    backward with coalesced atomics."""
    idx_ctype = "i64" if np.dtype(idx_dtype) == np.dtype(np.int64) else "int"
    if deterministic:
        order = tunables.current.det_backward
        if order is None:
            # Static rule, by the shape of the problem only (a clock would make the choice - and with it every
            # bit of the result - differ between processes).  The sender order gathers a dZ row per edge (d3
            # words, reads); the receiver order gathers an X row and writes and re-reads a dX row (3 d1 words,
            # half of them writes), and pays off when pass 1 can stage its operands through LDS.  Measured
            # backward, sender against receiver order, each as the first operator of a fresh process and in
            # steady state: d3 / d1 = 3.9 (32 channels) 0.162 / 0.175 ms, 4.8 (256 channels) 7.53 / 7.68 ms, 5.7
            # (32 channels, outputs of either parity) 0.223 / 0.208 ms, 7.1 (256 channels, either parity) 10.94 /
            # 9.43 ms, 7.9 (the 128-channel MACE problem) 2.14 / 1.71 ms.  Without the stage (fp64, or fewer
            # channels than Y components) pass 1 runs one edge at a time: 16.3 against 10.96 ms at 7.1; those
            # problems keep the sender order, except in fp64 where pass 1 can run as one launch per group of
            # output blocks with few dZ words held (the MACE problem in fp64, 10 000 nodes / 300 000 edges: 5.04
            # / 4.77 ms; 30 paths at 32 channels 1.32 / 1.00 ms).
            order = "send"
            if config.irreps_out.dim >= RECV_ORDER_MIN_RATIO * config.irreps_in1.dim:
                g = UVURecvGenerator(config, vector_stores=vector_stores, idx_ctype=idx_ctype)
                if g.staged_edges or g.register_loads_fit:
                    return g
        if order == "recv":
            return UVURecvGenerator(config, vector_stores=vector_stores, idx_ctype=idx_ctype)
        return UVUDetGenerator(config, vector_stores=vector_stores, idx_ctype=idx_ctype)
    if tunables.current.conv_forward == "atomic":     # A/B measurements only
        g = UVUDirectGenerator(config, "conv_atomic", vector_stores=vector_stores)
        g.idx_ctype = idx_ctype
        return g
    return UVUSortedGenerator(config, vector_stores=vector_stores, idx_ctype=idx_ctype)


class _StreamWorkspace:
    """Device scratch of one operator on one stream, and which graph its preparation areas
    (CSR pointers, position lists, node order) currently describe."""

    def __init__(self):
        self.buffer, self.size = None, 0
        self.retired = []            # outgrown buffers that a captured HIP graph may still name
        self.captured = False        # a HIP graph capture has used this workspace
        self.fwd_key = self.bwd_key = None
        self.refs = {}               # index tensors of the cached keys, kept alive so that their addresses stay theirs
        # (nnz, node_count) of the last completed call of each direction, while nothing else has written the
        # workspace since: the counters of the on-the-fly grouping are then known to be zero where a call
        # with the same sizes keeps them, and the step that clears them is skipped
        self.zero_fwd = self.zero_bwd = None


class TensorProductConv:
    """Drop-in for ``oeq.TensorProductConv``."""
    next_conv_id = 0

    def __init__(self, config: TPProblem, torch_op: bool = False, deterministic: bool = False,
                 idx_dtype=np.int64, graph_cache: typing.Optional[bool] = None):
        """``graph_cache=True`` (default: ``tunables.graph_cache``, off) lets the torch operators skip the
        graph preparation when a call names the same index tensors as the previous one (same addresses,
        same in-place version counters, same sizes).  The key cannot see writes that bypass torch's version
        counter - memory wrapped with from_blob / DLPack, kernels of other libraries writing into a
        preallocated neighbour list, a HIP graph replay rewriting a static index buffer - so it is for
        callers who know that their index tensors change only through torch."""
        assert isinstance(config, TPProblem)
        self.config = config
        self.L1, self.L2, self.L3 = config.irreps_in1, config.irreps_in2, config.irreps_out
        self.torch_op, self.deterministic = torch_op, deterministic
        if np.dtype(idx_dtype) not in (np.dtype(np.int64), np.dtype(np.int32)):
            raise NotImplementedError("index tensors must be int64 or int32")
        # reference: LoopUnrollConv.py:53,78 (idx_type_map = {np.int32: "int", np.int64: "long"})
        self.idx_dtype = np.dtype(idx_dtype).type
        self._torch_idx = torch.int64 if self.idx_dtype == np.int64 else torch.int32
        self._torch_dtype = {np.float32: torch.float32, np.float64: torch.float64}[config.irrep_dtype]
        self._dims = (self.L1.dim, self.L2.dim, self.L3.dim, config.weight_numel)
        self.conv_id = TensorProductConv.next_conv_id
        TensorProductConv.next_conv_id += 1

        mode = validate_problem(config)
        for (mul, ir) in self.L2:
            assert mul == 1, "TensorProductConv requires multiplicity 1 for every irrep of the second operand"
        if mode != "uvu":
            raise NotImplementedError("TensorProductConv supports uvu problems")

        self.generator = select_conv_generator(config, deterministic, idx_dtype=self.idx_dtype)
        # True: the forward writes every row of Z itself; False: it accumulates into a zeroed Z
        self.forward_overwrites = not isinstance(self.generator, UVUDirectGenerator) or deterministic
        # likewise for dX in the backward (the per-edge backward accumulates with atomics)
        self.backward_overwrites = deterministic or getattr(self.generator, "grouped_backward", False)
        # the deterministic backward walks the caller's transpose permutation
        self.backward_needs_tperm = deterministic
        self.jit_kernel = self.generator.render()
        self._ws_fns = []
        self._ws_last = (None, 0)          # (sizes, bytes) of the last workspace query
        self.internal = self._build(self.generator, self.jit_kernel)
        self._workspaces: typing.Dict[tuple, _StreamWorkspace] = {}      # (device, stream) -> scratch
        # Unsorted edge lists: whether the backward scatters dX with float atomics or groups the edges by
        # sender first depends on the row length AND on the graph (atomics per edge against the gathers of
        # the segmented kernel); the generator's rule of thumb is only the starting point.  The torch
        # operator times both on the first backward call of each size class and keeps the faster one
        # (``tunables.conv_backward`` = atomic | grouped or ``tunables.autotune`` = False switch the measurement off).  The
        # deterministic operator never chooses by timing: which kernel runs must not depend on a stopwatch
        # if results are to repeat bit for bit from one process to the next.
        self._bwd_variants = {}
        self._bwd_choice: typing.Dict[tuple, str] = {}
        if isinstance(self.generator, UVUSortedGenerator):
            self._bwd_default = "grouped" if self.generator.grouped_backward else "atomic"
            self._bwd_variants[self._bwd_default] = (self.internal, self.backward_overwrites)
        self.autotune = (bool(self._bwd_variants) and tunables.current.autotune
                         and tunables.current.conv_backward is None)
        self.graph_cache = tunables.current.graph_cache if graph_cache is None else bool(graph_cache)
        self._internal_unaligned = None
        self._reorder = WeightReorder(config)
        self.reorder_weights_e3nn_to_oeq = self._reorder.e3nn_to_oeq
        self.reorder_weights_oeq_to_e3nn = self._reorder.oeq_to_e3nn
        if torch_op:
            self._setup_torch_module()

    def _build(self, generator, source=None) -> "rt.ConvImpl":
        """Compile one kernel set of this operator.  Every set shares the operator's workspace, which is
        sized for the largest of them."""
        fwd, bwd, ws = generator.plan()
        self._ws_fns.append(ws)
        need_ws = rt.STEP_NEEDS_WORKSPACE if ws(1, 1) > 0 else 0
        need_tp = rt.STEP_NEEDS_TPERM if self.backward_needs_tperm else 0
        code = rt.compile_source(source if source is not None else generator.render())
        impl = rt.ConvImpl(code, _make_steps(fwd, need_ws), _make_steps(bwd, need_ws | need_tp))
        model = getattr(generator, "forward_workspace_model", None)
        impl.set_forward_workspace(*(model() if model else (0, 0, 0)))
        return impl

    def _ws_bytes(self, nnz: int, node_count: int) -> int:
        key = (nnz, node_count, len(self._ws_fns))
        if key != self._ws_last[0]:
            self._ws_last = (key, max(f(nnz, node_count) for f in self._ws_fns))
        return self._ws_last[1]

    def _backward_variant(self, name: str):
        """(kernel set, whether its backward overwrites dX) of a backward variant of the unsorted operator,
        compiled on first need."""
        if name not in self._bwd_variants:
            g = UVUSortedGenerator(self.config, grouped_backward=(name == "grouped"),
                                   idx_ctype="i64" if self.idx_dtype == np.int64 else "int")
            self._bwd_variants[name] = (self._build(g), name == "grouped")
            for rec in self._workspaces.values():            # the workspace may have to grow: sizes are re-checked per call
                rec.bwd_key = None
        return self._bwd_variants[name]

    @staticmethod
    def name():
        return "LoopUnrollConv"

    # ------------------------------------------------------------------ helpers
    def _workspace_record(self, nnz: int, node_count: int, stream: typing.Optional[int] = None) -> _StreamWorkspace:
        """The operator's scratch for ``stream`` (torch's current one by default), grown on demand.  Every
        stream gets its own, so two streams using one operator do not share CSR pointers or position
        lists.  A buffer that has been outgrown is freed unless a HIP graph capture has used it: a captured
        graph has the address baked in, so such buffers stay alive as long as the operator (the reference
        allocates its workspace once at a fixed size: ConvolutionBase.py:93-100)."""
        dev = torch.cuda.current_device()
        sid = (dev, self._stream(dev) if stream is None else int(stream))
        rec = self._workspaces.get(sid)
        if rec is None:
            rec = self._workspaces[sid] = _StreamWorkspace()
        need = self._ws_bytes(nnz, node_count)
        if need > rec.size:
            if rec.captured and rec.buffer is not None:
                rec.retired.append(rec.buffer)
            rec.size = int(need * 1.25) + 256
            rec.buffer = torch.empty(rec.size, dtype=torch.uint8, device=f"cuda:{dev}")
            rec.fwd_key = rec.bwd_key = rec.zero_fwd = rec.zero_bwd = None
            rec.refs.clear()
        return rec

    def workspace_ptr(self, nnz: int, node_count: int, stream: typing.Optional[int] = None) -> int:
        """Device scratch for a call with this many edges and nodes on ``stream`` (0 when the
        kernels use none).  Calling it invalidates nothing, but whoever launches with it outside the
        operator's own entry points is responsible for the ``prepared`` flag."""
        if self._ws_bytes(nnz, node_count) == 0:
            return 0
        return self._workspace_record(nnz, node_count, stream).buffer.data_ptr()

    @staticmethod
    def _stream(device_index: typing.Optional[int] = None) -> int:
        """torch's current stream on the device as a raw handle (the binding call is many times cheaper than
        building a torch.cuda.Stream object per launch)."""
        return torch._C._cuda_getCurrentRawStream(torch.cuda.current_device() if device_index is None else device_index)

    def _check(self, x, y, w, rows, cols, tperm=None, g=None):
        """Shapes, dtypes and devices, before anything is launched: the kernels dereference every
        pointer they are handed, so a host tensor or a tensor of another GPU must never reach them."""
        E, N = rows.shape[0], x.shape[0]
        d1, d2, d3, wn = self._dims
        if N >= 2 ** 31:
            raise ValueError("node count must be below 2^31")
        if x.ndim != 2 or x.shape[1] != d1:
            raise ValueError(f"L1_in must have shape [nodes, {d1}], got {tuple(x.shape)}")
        if y.shape != (E, d2):
            raise ValueError(f"L2_in must have shape [{E}, {d2}], got {tuple(y.shape)}")
        if w.shape != (E, wn):
            raise ValueError(f"weights must have shape [{E}, {wn}], got {tuple(w.shape)}")
        if g is not None and g.shape != (N, d3):
            raise ValueError(f"L3_grad must have shape [{N}, {d3}], got {tuple(g.shape)}")
        if self.deterministic and tperm is None:
            raise ValueError("the deterministic convolution needs transpose_perm")
        dev, tdt, idt = x.device, self._torch_dtype, self._torch_idx
        for name, t in (("rows", rows), ("cols", cols), ("transpose_perm", tperm)):
            if t is None:
                continue
            if t.dtype != idt or t.shape != (E,):
                raise TypeError(f"{name} must be an {idt} tensor of shape [{E}]")
            if t.device != dev or not t.is_cuda:
                self._device_error(name, t, x)
        for name, t in (("L1_in", x), ("L2_in", y), ("weights", w), ("L3_grad", g)):
            if t is None:
                continue
            if t.dtype != tdt:
                raise TypeError(f"tensors must be {tdt}")
            if t.device != dev or not t.is_cuda:
                self._device_error(name, t, x)

    @staticmethod
    def _device_error(name, t, x):
        if not t.is_cuda:
            raise ValueError(f"{name} is on {t.device}: every tensor, index tensors included, must be on the GPU "
                             "(there is no CPU implementation)")
        raise ValueError(f"{name} is on {t.device}, L1_in on {x.device}: all tensors must share one device")

    def _pick(self, *ptrs):
        """The forward kernels write Z with 16-byte vector stores; a misaligned tensor (rare: a view
        with an odd storage offset) gets a variant without them, compiled on first need."""
        if any(int(p) % 16 for p in ptrs):
            if self._internal_unaligned is None:
                g = select_conv_generator(self.config, self.deterministic, vector_stores=False, idx_dtype=self.idx_dtype)
                self._internal_unaligned = self._build(g)
            return self._internal_unaligned
        return self.internal

    # ---------------------------------------------------------- raw entry points
    def exec_conv_rawptrs(self, L1_in, L2_in, weights, L3_out, rows, cols, nnz, node_count, workspace=0,
                          transpose_perm=0, stream=None, prepared=False, counters_zero=False):
        """reference: extension/convolution.hpp:121-147.  Without ``workspace`` the operator's own scratch
        for the stream is used.  ``prepared=True`` promises that the workspace still holds the forward
        preparation of exactly this graph (left by an earlier forward call): the preparation kernels are
        then skipped.  ``counters_zero=True`` promises that the counters the operator keeps in the workspace
        are zero (a zero-filled workspace, or one last written by a completed call of this operator with the
        same sizes): the step that clears them is skipped."""
        nnz, node_count = int(nnz), int(node_count)
        if nnz > 0 and not (rows and cols):
            raise ValueError("rows / cols must be device pointers")
        impl = self._pick(L1_in, L2_in, weights, L3_out)
        if not workspace:
            rec = self._workspace_record(nnz, node_count, stream)
            rec.fwd_key = rec.zero_fwd = rec.zero_bwd = None    # the caller's graph is unknown to the cache
            workspace = rec.buffer.data_ptr() if self._ws_bytes(nnz, node_count) else 0
        impl.exec_conv_rawptrs(L1_in, L2_in, weights, L3_out, rows, cols, nnz, node_count,
                               workspace, transpose_perm, self._stream() if stream is None else stream, prepared,
                               counters_zero)

    def backward_rawptrs(self, L1_in, L1_grad, L2_in, L2_grad, weights, weights_grad, L3_grad, rows, cols, nnz,
                         node_count, workspace=0, transpose_perm=0, stream=None, prepared=False, impl=None,
                         counters_zero=False):
        """reference: extension/convolution.hpp:149-173; ``workspace`` and ``prepared`` as in
        exec_conv_rawptrs (the backward keeps its own preparation in the workspace).  ``impl`` selects
        another kernel set of this operator (see _backward_variant) instead of the default one."""
        nnz, node_count = int(nnz), int(node_count)
        if nnz > 0 and not (rows and cols):
            raise ValueError("rows / cols must be device pointers")
        if self.backward_needs_tperm and nnz > 0 and not transpose_perm:
            raise ValueError("the deterministic backward needs transpose_perm (a device pointer), got 0")
        if impl is None:
            impl = self._pick(L1_in, L1_grad, L2_in, L2_grad, weights, weights_grad, L3_grad)
        if not workspace:
            rec = self._workspace_record(nnz, node_count, stream)
            rec.bwd_key = rec.zero_fwd = rec.zero_bwd = None
            workspace = rec.buffer.data_ptr() if self._ws_bytes(nnz, node_count) else 0
        impl.backward_rawptrs(L1_in, L1_grad, L2_in, L2_grad, weights, weights_grad, L3_grad, rows, cols,
                              nnz, node_count, workspace, transpose_perm,
                              self._stream() if stream is None else stream, prepared, counters_zero)

    def _time_backward_variants(self, run, names=("atomic", "grouped"), repeats: int = 3) -> str:
        """Fastest of the backward variants on the caller's own tensors: one untimed call each (compilation,
        graph preparation), then the best of ``repeats`` timed calls between HIP events."""
        best = {}
        for name in names:
            run(name)
            times = []
            for _ in range(repeats):
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                run(name)
                b.record()
                b.synchronize()
                times.append(a.elapsed_time(b))
            best[name] = min(times)
        self.last_tuning = best
        return min(best, key=best.get)

    def _cached_call(self, which: str, rows, cols, tperm, E: int, N: int, launch, tag: str = "",
                     stream: typing.Optional[int] = None) -> None:
        """Run ``launch(workspace pointer, prepared, counters_zero)`` for the torch operators.  The graph preparation a
        call leaves in the stream's workspace is reused by the next call of the same direction when it
        names the same graph: same index tensors (address and in-place version counter), same sizes.  The
        tensors are kept referenced while their key is cached, so the addresses cannot be handed to other
        tensors meanwhile.  Under HIP graph capture, and on a workspace that a capture has used, the
        preparation always runs: a replay may rewrite the workspace behind the cache's back."""
        if self._ws_bytes(E, N) == 0:
            launch(0, False, False)
            return
        rec = self._workspace_record(E, N, stream)
        if torch.cuda.is_current_stream_capturing():
            rec.captured = True
        key = None
        if self.graph_cache and not rec.captured:
            key = (tag, E, N) + tuple((t.data_ptr(), t._version) for t in (rows, cols, tperm) if t is not None)
        attr, zattr, other = which + "_key", "zero_" + which, "zero_" + ("bwd" if which == "fwd" else "fwd")
        prepared = key is not None and getattr(rec, attr) == key
        # every call leaves the grouping counters it used zeroed; a call with other sizes keeps them elsewhere
        # (the kernel sets of the backward variants differ in whether they group at all, hence the tag)
        counters_zero = not rec.captured and getattr(rec, zattr) == (E, N, tag)
        if (getattr(rec, other) or (None,))[:2] != (E, N):
            setattr(rec, other, None)
        setattr(rec, attr, None)
        setattr(rec, zattr, None)
        launch(rec.buffer.data_ptr(), prepared, counters_zero)
        setattr(rec, attr, key)
        setattr(rec, zattr, None if rec.captured else (E, N, tag))
        rec.refs[which] = (rows, cols, tperm) if key is not None else None

    # ------------------------------------------------------------------ torch ops
    def _setup_torch_module(self) -> None:
        """reference: ConvolutionBase.py:560-709."""
        L3_dim = self.L3.dim
        det = self.deterministic
        cid = self.conv_id

        def fwd_impl(L1_in, L2_in, weights, rows, cols, tperm):
            x, y, w, rows, cols, tperm = _contiguous(L1_in, L2_in, weights, rows, cols, tperm)
            self._check(x, y, w, rows, cols, tperm)
            E, N = rows.shape[0], x.shape[0]
            # the atomic kernels accumulate into Z; the deterministic ones write every row
            out = (torch.empty if self.forward_overwrites else torch.zeros)((N, L3_dim), dtype=x.dtype, device=x.device)
            with _on_device(x.device):
                stream = self._stream(x.device.index)
                self._cached_call("fwd", rows, cols, tperm, E, N, lambda ws, prepared, zero: self.exec_conv_rawptrs(
                    x.data_ptr(), y.data_ptr(), w.data_ptr(), out.data_ptr(), rows.data_ptr(), cols.data_ptr(), E, N,
                    ws, tperm.data_ptr() if tperm is not None else 0, stream=stream, prepared=prepared,
                    counters_zero=zero), stream=stream)
            return out

        def bwd_run(x, y, w, g, rows, cols, tperm, E, N, variant=None):
            """One backward pass into fresh outputs with the default kernel set or a named variant."""
            impl, overwrites = (None, self.backward_overwrites) if variant is None else self._backward_variant(variant)
            if variant is not None and any(int(t.data_ptr()) % 16 for t in (x, y, w, g)):
                impl, overwrites, variant = None, self.backward_overwrites, None     # misaligned views: the default set only
            xg = (torch.empty_like if overwrites else torch.zeros_like)(x)
            yg, wg = torch.empty_like(y), torch.empty_like(w)
            stream = self._stream(x.device.index)
            self._cached_call("bwd", rows, cols, tperm, E, N, lambda ws, prepared, zero: self.backward_rawptrs(
                x.data_ptr(), xg.data_ptr(), y.data_ptr(), yg.data_ptr(), w.data_ptr(), wg.data_ptr(), g.data_ptr(),
                rows.data_ptr(), cols.data_ptr(), E, N, ws, tperm.data_ptr() if tperm is not None else 0,
                stream=stream, prepared=prepared, impl=impl, counters_zero=zero), tag=variant or "", stream=stream)
            return [xg, yg, wg]

        def bwd_impl(L1_in, L2_in, weights, L3_grad, rows, cols, tperm):
            x, y, w, g, rows, cols, tperm = _contiguous(L1_in, L2_in, weights, L3_grad, rows, cols, tperm)
            self._check(x, y, w, rows, cols, tperm, g)
            E, N = rows.shape[0], x.shape[0]
            with _on_device(x.device):
                if not self.autotune or E == 0:
                    return bwd_run(x, y, w, g, rows, cols, tperm, E, N)
                size_class = (E.bit_length(), N.bit_length())
                if size_class not in self._bwd_choice:
                    if torch.cuda.is_current_stream_capturing():       # no clocks inside a capture: rule of thumb
                        return bwd_run(x, y, w, g, rows, cols, tperm, E, N)
                    self._bwd_choice[size_class] = self._time_backward_variants(
                        lambda name: bwd_run(x, y, w, g, rows, cols, tperm, E, N, name))
                return bwd_run(x, y, w, g, rows, cols, tperm, E, N, self._bwd_choice[size_class])

        # the two variants differ only in the trailing transpose_perm argument, which torch's operator
        # schemas need spelled out
        if not det:
            @torch.library.custom_op(f"openequivariance_amd::conv_forward{cid}", mutates_args=(), device_types="cuda")
            def forward(L1_in: torch.Tensor, L2_in: torch.Tensor, weights: torch.Tensor, rows: torch.Tensor,
                        cols: torch.Tensor) -> torch.Tensor:
                return fwd_impl(L1_in, L2_in, weights, rows, cols, None)

            @torch.library.custom_op(f"openequivariance_amd::conv_backward{cid}", mutates_args=(), device_types="cuda")
            def backward_helper(L1_in: torch.Tensor, L2_in: torch.Tensor, weights: torch.Tensor, L3_grad: torch.Tensor,
                                rows: torch.Tensor, cols: torch.Tensor) -> typing.List[torch.Tensor]:
                return bwd_impl(L1_in, L2_in, weights, L3_grad, rows, cols, None)
        else:
            @torch.library.custom_op(f"openequivariance_amd::conv_forward{cid}", mutates_args=(), device_types="cuda")
            def forward(L1_in: torch.Tensor, L2_in: torch.Tensor, weights: torch.Tensor, rows: torch.Tensor,
                        cols: torch.Tensor, transpose_perm: torch.Tensor) -> torch.Tensor:
                return fwd_impl(L1_in, L2_in, weights, rows, cols, transpose_perm)

            @torch.library.custom_op(f"openequivariance_amd::conv_backward{cid}", mutates_args=(), device_types="cuda")
            def backward_helper(L1_in: torch.Tensor, L2_in: torch.Tensor, weights: torch.Tensor, L3_grad: torch.Tensor,
                                rows: torch.Tensor, cols: torch.Tensor,
                                transpose_perm: torch.Tensor) -> typing.List[torch.Tensor]:
                return bwd_impl(L1_in, L2_in, weights, L3_grad, rows, cols, transpose_perm)

        @forward.register_fake
        def _(L1_in, L2_in, weights, *index):
            return L1_in.new_empty(L1_in.shape[0], L3_dim)

        @backward_helper.register_fake
        def _(L1_in, L2_in, weights, L3_grad, *index):
            return [L1_in.new_empty(*L1_in.shape), L2_in.new_empty(*L2_in.shape), weights.new_empty(*weights.shape)]

        def setup_context(ctx, inputs, output):
            ctx.L1_in, ctx.L2_in, ctx.weights, *ctx.index = inputs

        def backward(ctx, grad_output):
            r = backward_helper(ctx.L1_in, ctx.L2_in, ctx.weights, grad_output, *ctx.index)
            return (r[0], r[1], r[2]) + (None,) * len(ctx.index)

        forward.register_autograd(backward, setup_context=setup_context)

        def setup_context_double_backward(ctx, inputs, output):
            ctx.L1_in, ctx.L2_in, ctx.weights, ctx.L3_grad, *ctx.index = inputs

        def double_backward(ctx, grad_output):
            terms = double_backward_terms(forward, backward_helper, ctx.L1_in, ctx.L2_in, ctx.weights, ctx.L3_grad,
                                          grad_output[0], grad_output[1], grad_output[2], tuple(ctx.index))
            return terms + (None,) * len(ctx.index)

        backward_helper.register_autograd(double_backward, setup_context=setup_context_double_backward)
        self.forward = forward
        self.backward_helper = backward_helper

    def __call__(self, *args):
        return self.forward(*args)

    # -------------------------------------------- correctness / timing (harness)
    def _reference(self, reference_implementation):
        if reference_implementation is None:
            raise NotImplementedError("pass reference_implementation=...: no CPU reference ships with this package "
                                      "(the reference's default, e3nn, is an optional third-party dependency)")
        return reference_implementation(self.config)

    def test_correctness_forward(self, graph, thresh, prng_seed, reference_implementation=None,
                                 check_reproducible=True, torch_op=False):
        """Output against a reference implementation on seeded buffers, and (five repeats) whether
        the output repeats bit for bit (reference: ConvolutionBase.py:172-249)."""
        from .benchmark.correctness_utils import check_similiarity
        from .benchmark.random_buffer_utils import get_random_buffers_forward_conv
        in1, in2, weights, out = get_random_buffers_forward_conv(self.config, graph.node_count, graph.nnz, prng_seed)
        ref_out, test_out = out.copy(), out.copy()
        self._reference(reference_implementation).forward_cpu(L1_in=in1.copy(), L2_in=in2.copy(), weights=weights.copy(),
                                                              L3_out=ref_out, graph=graph)
        self.forward_cpu(L1_in=in1.copy(), L2_in=in2.copy(), weights=weights.copy(), L3_out=test_out, graph=graph)
        result = {"thresh": thresh, "output": check_similiarity("output", test_out, ref_out, thresh)}
        if check_reproducible:
            same = True
            for _ in range(5):
                again = out.copy()
                self.forward_cpu(L1_in=in1.copy(), L2_in=in2.copy(), weights=weights.copy(), L3_out=again, graph=graph)
                same = same and bool(np.all(again == test_out))
            result["output"]["num_reproducibility_trials"] = 5
            result["output"]["bitwise_reproducible"] = same
        return result

    def test_correctness_backward(self, graph, thresh, prng_seed, reference_implementation=None):
        """reference: ConvolutionBase.py:445-494."""
        from .benchmark.correctness_utils import check_similiarity
        from .benchmark.random_buffer_utils import get_random_buffers_backward_conv
        in1, in2, out_grad, weights, wg, g1, g2 = get_random_buffers_backward_conv(self.config, graph.node_count,
                                                                                   graph.nnz, prng_seed)
        grads = []
        for impl in (self._reference(reference_implementation), self):
            bufs = dict(weights_grad=wg.copy(), L1_grad=g1.copy(), L2_grad=g2.copy())
            impl.backward_cpu(L1_in=in1.copy(), L2_in=in2.copy(), L3_grad=out_grad.copy(), weights=weights.copy(),
                              graph=graph, **bufs)
            grads.append(bufs)
        result = {"thresh": thresh}
        for name, key in (("weight_grad", "weights_grad"), ("in1_grad", "L1_grad"), ("in2_grad", "L2_grad")):
            result[name] = check_similiarity(name, grads[1][key], grads[0][key], thresh)
        return result

    def test_correctness_double_backward(self, graph, thresh, prng_seed, reference_implementation=None):
        """Second derivatives through the torch op against a differentiable reference
        (reference: ConvolutionBase.py:496-557)."""
        from .benchmark.correctness_utils import check_similiarity
        from .benchmark.random_buffer_utils import get_random_buffers_backward_conv
        assert self.torch_op
        in1, in2, out_grad, weights, _, _, _ = get_random_buffers_backward_conv(self.config, graph.node_count,
                                                                                graph.nnz, prng_seed)
        scale = float(np.random.default_rng(seed=prng_seed * 2).standard_normal(1)[0])
        got = []
        for tp in (self, reference_implementation(self.config, torch_op=True) if reference_implementation
                   else self._reference(None)):
            dev = getattr(tp, "device", "cuda")
            a, b, w, g = (torch.tensor(t, device=dev, requires_grad=True) for t in (in1, in2, weights, out_grad))
            args = [a, b, w, torch.tensor(graph.rows, device=dev), torch.tensor(graph.cols, device=dev)]
            if tp.deterministic:
                args.append(torch.tensor(graph.transpose_perm, device=dev))
            out = tp.forward(*args)
            out.backward(g, create_graph=True, retain_graph=True, inputs=[a, b, w])
            dummy = torch.norm(a.grad) + torch.norm(b.grad) + torch.norm(w.grad)
            dummy.backward(torch.tensor(scale, device=dev, dtype=dummy.dtype), retain_graph=True, inputs=[g, a, b, w])
            got.append([t.grad.detach().cpu().numpy() for t in (g, a, b, w)])
        return {name: check_similiarity(name, got[0][i], got[1][i], thresh)
                for i, name in enumerate(("output_grad", "in1_grad", "in2_grad", "weights_grad"))}

    def _timed(self, num_warmup, num_iter, run, reset=lambda: None, stream=0):
        times = np.zeros(num_iter, dtype=np.float32)
        timer = rt.GPUTimer(stream)
        for _ in range(num_warmup):
            run()
        for i in range(num_iter):
            reset()
            timer.clear_L2_cache()
            timer.start()
            run()
            times[i] = timer.stop_clock_get_elapsed()
        return times

    def benchmark_forward(self, num_warmup, num_iter, graph, prng_seed=12345):
        """reference: ConvolutionBase.py:251-318."""
        from .benchmark.random_buffer_utils import get_random_buffers_forward_conv
        assert graph.rows.dtype == self.idx_dtype and graph.cols.dtype == self.idx_dtype
        in1, in2, weights, out = get_random_buffers_forward_conv(self.config, graph.node_count, graph.nnz, prng_seed)
        idx = [graph.rows, graph.cols] + ([graph.transpose_perm] if self.deterministic else [])
        if self.torch_op:
            t = [torch.tensor(a, device="cuda") for a in (in1, in2, weights, *idx)]
            times = self._timed(num_warmup, num_iter, lambda: self.forward(*t), stream=self._stream())
        else:
            bufs = [rt.DeviceBuffer(a) for a in (in1, in2, weights, out, graph.rows, graph.cols)]
            tp = rt.DeviceBuffer(graph.transpose_perm) if self.deterministic else None
            nbytes = self._ws_bytes(graph.nnz, graph.node_count)
            ws = rt.DeviceBuffer(nbytes) if nbytes else None
            ptrs = [b.data_ptr() for b in bufs]
            zero = (lambda: None) if self.forward_overwrites else (lambda: bufs[3].zero())
            times = self._timed(num_warmup, num_iter, lambda: self.internal.exec_conv_rawptrs(
                *ptrs, graph.nnz, graph.node_count, ws.data_ptr() if ws else 0, tp.data_ptr() if tp else 0, 0), zero)
        ops, data, _ = flops_data_per_tp(self.config, "forward")
        return self.calculate_bench_stats("forward", ops + self.config.irreps_out.dim, data, times, graph, num_warmup,
                                          num_iter, prng_seed)

    def benchmark_backward(self, num_warmup, num_iter, graph, prng_seed=12345):
        """reference: ConvolutionBase.py:321-411."""
        from .benchmark.random_buffer_utils import get_random_buffers_backward_conv
        assert graph.rows.dtype == self.idx_dtype and graph.cols.dtype == self.idx_dtype
        in1, in2, out_grad, weights, wg, g1, g2 = get_random_buffers_backward_conv(self.config, graph.node_count,
                                                                                   graph.nnz, prng_seed)
        if self.torch_op:
            x, y, w = (torch.tensor(a, device="cuda", requires_grad=True) for a in (in1, in2, weights))
            idx = [torch.tensor(a, device="cuda") for a in
                   [graph.rows, graph.cols] + ([graph.transpose_perm] if self.deterministic else [])]
            out, g = self.forward(x, y, w, *idx), torch.tensor(out_grad, device="cuda")
            times = self._timed(num_warmup, num_iter, lambda: out.backward(g, retain_graph=True, inputs=[x, y, w]),
                                lambda: [t.grad.zero_() for t in (x, y, w)], stream=self._stream())
        else:
            bufs = [rt.DeviceBuffer(a) for a in (in1, g1, in2, g2, weights, wg, out_grad, graph.rows, graph.cols)]
            tp = rt.DeviceBuffer(graph.transpose_perm) if self.deterministic else None
            nbytes = self._ws_bytes(graph.nnz, graph.node_count)
            ws = rt.DeviceBuffer(nbytes) if nbytes else None
            ptrs = [b.data_ptr() for b in bufs]
            zero = (lambda: None) if self.backward_overwrites else (lambda: bufs[1].zero())
            times = self._timed(num_warmup, num_iter, lambda: self.internal.backward_rawptrs(
                *ptrs, graph.nnz, graph.node_count, ws.data_ptr() if ws else 0, tp.data_ptr() if tp else 0, 0), zero)
        ops, data, _ = flops_data_per_tp(self.config, "backward")
        return self.calculate_bench_stats("backward", ops + self.config.irreps_out.dim, data, times, graph, num_warmup,
                                          num_iter, prng_seed)

    def calculate_bench_stats(self, direction, ops_per_tp, data_per_tp, time_millis, graph, num_warmup, num_iter,
                              prng_seed):
        """Result record of the reference's convolution benchmarks (ConvolutionBase.py:413-443):
        per-edge work model times the edge count over each measured time."""
        t = np.asarray(time_millis, dtype=np.float64)
        return {"direction": direction, "flops_per_tp": ops_per_tp, "data_per_tp": data_per_tp,
                "time_millis": [float(v) for v in t],
                "throughputs_gflops": [float(v) for v in graph.nnz * ops_per_tp / (t * 1e6)],
                "bandwidth_gbps": [float(v) for v in graph.nnz * data_per_tp / (t * 1e6)],
                "L1": str(self.config.irreps_in1), "L2": str(self.config.irreps_in2), "L3": str(self.config.irreps_out),
                "graph_node_count": graph.node_count, "graph_adj_nnz": graph.nnz,
                "num_warmup": num_warmup, "num_iter": num_iter, "prng_seed": prng_seed}

    # ---------------------------------------------------- numpy entry points (tests)
    def forward_cpu(self, L1_in, L2_in, weights, L3_out, graph) -> None:
        """Host arrays; ``graph`` has rows / cols / node_count / nnz (and transpose_perm when
        deterministic) (reference: ConvolutionBase.py:106-137)."""
        assert graph.rows.dtype == self.idx_dtype
        x, y, w = rt.DeviceBuffer(L1_in), rt.DeviceBuffer(L2_in), rt.DeviceBuffer(weights)
        L3_out[...] = 0
        z = rt.DeviceBuffer(L3_out)
        r, c = rt.DeviceBuffer(graph.rows), rt.DeviceBuffer(graph.cols)
        tp = rt.DeviceBuffer(graph.transpose_perm) if self.deterministic else None
        nbytes = self._ws_bytes(graph.nnz, graph.node_count)
        ws = rt.DeviceBuffer(nbytes) if nbytes else None
        self.internal.exec_conv_rawptrs(x.data_ptr(), y.data_ptr(), w.data_ptr(), z.data_ptr(), r.data_ptr(),
                                        c.data_ptr(), graph.nnz, graph.node_count, ws.data_ptr() if ws else 0,
                                        tp.data_ptr() if tp else 0, 0)
        rt.stream_synchronize(0)
        L3_out[...] = z.copy_to_host()

    def backward_cpu(self, L1_in, L1_grad, L2_in, L2_grad, L3_grad, weights, weights_grad, graph) -> None:
        """reference: ConvolutionBase.py:139-170."""
        assert graph.rows.dtype == self.idx_dtype
        x, y, w, g = (rt.DeviceBuffer(a) for a in (L1_in, L2_in, weights, L3_grad))
        L1_grad[...] = 0
        xg, yg, wg = rt.DeviceBuffer(L1_grad), rt.DeviceBuffer(L2_grad), rt.DeviceBuffer(weights_grad)
        r, c = rt.DeviceBuffer(graph.rows), rt.DeviceBuffer(graph.cols)
        tp = rt.DeviceBuffer(graph.transpose_perm) if self.deterministic else None
        nbytes = self._ws_bytes(graph.nnz, graph.node_count)
        ws = rt.DeviceBuffer(nbytes) if nbytes else None
        self.internal.backward_rawptrs(x.data_ptr(), xg.data_ptr(), y.data_ptr(), yg.data_ptr(), w.data_ptr(),
                                       wg.data_ptr(), g.data_ptr(), r.data_ptr(), c.data_ptr(), graph.nnz,
                                       graph.node_count, ws.data_ptr() if ws else 0, tp.data_ptr() if tp else 0, 0)
        rt.stream_synchronize(0)
        L1_grad[...] = xg.copy_to_host()
        L2_grad[...] = yg.copy_to_host()
        weights_grad[...] = wg.copy_to_host()


LoopUnrollConv = TensorProductConv


class LoopUnrollConvDeterministic(TensorProductConv):
    """reference: convolution/LoopUnrollConv.py:93-101"""

    def __init__(self, config, idx_dtype=np.int64, torch_op=False):
        super().__init__(config, torch_op=torch_op, deterministic=True, idx_dtype=idx_dtype)

    @staticmethod
    def name():
        return "LoopUnrollConvDeterministic"


class LoopUnrollConvAtomic(TensorProductConv):
    """The variant for unsorted edge lists (reference: convolution/LoopUnrollConv.py:103-111)."""

    def __init__(self, config, idx_dtype=np.int64, torch_op=False):
        super().__init__(config, torch_op=torch_op, deterministic=False, idx_dtype=idx_dtype)

    @staticmethod
    def name():
        return "LoopUnrollConvAtomic"


class LoopUnrollConvScatterSum:
    """Unfused baseline: the batch tensor product on gathered node features followed by a scatter
    sum over the receivers (reference: convolution/LoopUnrollConv.py:113-160).  It materialises the
    per-edge output, which the fused kernels avoid; the harness times it beside them."""
    deterministic = False

    def __init__(self, config, idx_dtype=np.int64, torch_op=True):
        from .tensor_product import TensorProduct
        assert torch_op, "the unfused baseline exists as a torch operator only"
        self.config, self.torch_op, self.idx_dtype = config, True, np.int64
        self.L1, self.L2, self.L3 = config.irreps_in1, config.irreps_in2, config.irreps_out
        self.reference_tp = TensorProduct(config, torch_op=True)

    @staticmethod
    def name():
        return "LoopUnrollConvScatterSum"

    def forward(self, L1_in, L2_in, weights, rows, cols):
        per_edge = self.reference_tp(L1_in[cols], L2_in, weights)
        out = per_edge.new_zeros(L1_in.shape[0], self.L3.dim)
        return out.index_add_(0, rows, per_edge)

    __call__ = forward

    def forward_cpu(self, L1_in, L2_in, weights, L3_out, graph):
        per_edge = np.zeros((graph.nnz, self.L3.dim), dtype=L3_out.dtype)
        self.reference_tp.forward_cpu(np.ascontiguousarray(L1_in[graph.cols]), L2_in, per_edge, weights)
        L3_out[...] = 0
        np.add.at(L3_out, graph.rows, per_edge)

    def backward_cpu(self, L1_in, L1_grad, L2_in, L2_grad, L3_grad, weights, weights_grad, graph):
        gathered_grad = np.zeros((graph.nnz, self.L1.dim), dtype=L1_grad.dtype)
        self.reference_tp.backward_cpu(np.ascontiguousarray(L1_in[graph.cols]), gathered_grad, L2_in, L2_grad,
                                       np.ascontiguousarray(L3_grad[graph.rows]), weights, weights_grad)
        L1_grad[...] = 0
        np.add.at(L1_grad, graph.cols, gathered_grad)

    # the timing / comparison methods of the fused operator work on any object with these entry points
    _reference = TensorProductConv._reference
    _timed = TensorProductConv._timed
    _stream = staticmethod(TensorProductConv._stream)
    test_correctness_forward = TensorProductConv.test_correctness_forward
    test_correctness_backward = TensorProductConv.test_correctness_backward
    benchmark_forward = TensorProductConv.benchmark_forward
    benchmark_backward = TensorProductConv.benchmark_backward
    calculate_bench_stats = TensorProductConv.calculate_bench_stats
