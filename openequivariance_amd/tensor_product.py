"""``TensorProduct``: the batch Clebsch-Gordan tensor product operator.

Host-side mirror of the reference's ``oeq.TensorProduct`` / ``LoopUnrollTP``
(reference: openequivariance/implementations/LoopUnrollTP.py:12-105,
TensorProductBase.py:11-298): same constructor, same callable
``tp(X, Y, W) -> Z``, same torch custom-op wiring with first and second
derivatives, same raw-pointer and numpy entry points and the same weight
reordering helpers.  Underneath, the kernels are generated for gfx950, compiled
with hipRTC and launched through the C-ABI runtime on torch's current stream.
"""
from __future__ import annotations

import typing

import numpy as np
import torch

from . import runtime as rt
from .autograd_glue import double_backward_terms
from .codegen.uvu import UVUGenerator
from .codegen.uvu_direct import UVUDirectGenerator
from .codegen.uvw_batched import UVWBatchedGenerator
from .problem import TPProblem
from .weight_order import WeightReorder
from .wigner import wigner_3j


def _make_steps(descs, flags: int = 0):
    """Plan dictionaries of a generator -> ``runtime.Step`` records.  ``flags`` (STEP_NEEDS_*) apply to
    every step of the plan; a step's own ``prep=True`` marks it as graph preparation, ``counter_clear=True``
    as one that only zeroes counters which the operator's other steps leave zeroed again."""
    return [rt.Step.make(d["kernel"], d["num_threads"], d.get("smem", 0), d.get("grid_kind", rt.GRID_PER_ROW),
                         d.get("work_per_block", 1), d.get("num_blocks", 0), d.get("grid_y", 1),
                         flags | (rt.STEP_GRAPH_PREP if d.get("prep") else 0)
                         | (rt.STEP_COUNTER_CLEAR if d.get("counter_clear") else 0)) for d in descs]


class _NoSwitch:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def _contiguous(*tensors):
    return tuple(t if t is None or t.is_contiguous() else t.contiguous() for t in tensors)


def _on_device(device):
    """Context that makes ``device`` current: nothing at all when it already is (the usual case; entering
    torch.cuda.device costs several microseconds per call)."""
    return _NO_SWITCH if device.index == torch.cuda.current_device() else torch.cuda.device(device)


def select_generator(config: TPProblem):
    """The kernel generator of a batch tensor product: MFMA kernels for uvw with shared weights (vector-ALU
    kernels with a row per lane when the weights are few and the multiplicities small),
    streaming vector-ALU kernels for uvw with per-row weights, the persistent two-stage dW
    reduction for uvu with shared weights, register-direct streaming kernels otherwise."""
    mode = validate_problem(config)
    if mode == "uvw" and config.shared_weights:
        from .codegen.uvw import UVWGenerator
        from .codegen.uvw_rows import UVWRowsGenerator
        # a few hundred weights on multiplicities far below a 16 x 16 tile: one row per lane on the vector ALU
        return UVWRowsGenerator(config) if UVWRowsGenerator.suits(config) else UVWGenerator(config)
    if mode == "uvw":
        from .codegen.uvw_batched import UVWBatchedGenerator
        return UVWBatchedGenerator(config)
    if config.shared_weights:
        return UVUGenerator(config, "tp")
    return UVUDirectGenerator(config, "tp")


def validate_problem(config: TPProblem) -> str:
    """Checks shared by every operator (reference: LoopUnrollTP.py:23-30).  Returns the mode."""
    if len(config.instructions) == 0:
        raise ValueError("Tensor product problem has no valid intructions!")
    mode = config.instructions[0].connection_mode
    for inst in config.instructions:
        assert inst.connection_mode == mode, "all instructions must share one connection mode"
    assert mode in ("uvu", "uvw"), f"connection mode {mode!r} is not supported (uvu and uvw are)"
    assert config.irrep_dtype == config.weight_dtype, "irrep_dtype and weight_dtype must be equal"
    return mode


class TensorProductBase:
    next_tp_id = 0   # unique suffix of the torch op names (reference: TensorProductBase.py:12)

    @staticmethod
    def load_cg_tensor(l1, l2, l3):
        return wigner_3j(l1, l2, l3)

    def __init__(self, config: TPProblem, torch_op: bool = False):
        assert isinstance(config, TPProblem)
        assert isinstance(torch_op, bool)
        self.config, self.torch_op = config, torch_op
        self.L1, self.L2, self.L3 = config.irreps_in1, config.irreps_in2, config.irreps_out
        self.irrep_dtype, self.weight_dtype = config.irrep_dtype, config.weight_dtype
        self.tp_id = TensorProductBase.next_tp_id
        TensorProductBase.next_tp_id += 1

    def __call__(self, L1_in, L2_in, weights):
        return self.forward(L1_in, L2_in, weights)


class TensorProduct(TensorProductBase):
    """Drop-in for ``oeq.TensorProduct(problem, torch_op=True)``."""

    def __init__(self, problem: TPProblem, torch_op: bool = True):
        super().__init__(problem, torch_op=torch_op)
        config = self.config
        mode = validate_problem(config)
        self.is_uvw = (mode == "uvw")
        self.generator = select_generator(config)
        self.jit_kernel = self.generator.render()
        code = rt.compile_source(self.jit_kernel)
        fwd, bwd, ws = self.generator.plan()
        self.workspace_bytes = ws()
        self._step_flags = rt.STEP_NEEDS_WORKSPACE if self.workspace_bytes else 0
        self.internal = rt.TPImpl(code, _make_steps(fwd, self._step_flags), _make_steps(bwd, self._step_flags))
        self._torch_dtype = {np.float32: torch.float32, np.float64: torch.float64}[self.irrep_dtype]
        self._dims = (self.L1.dim, self.L2.dim, self.L3.dim, config.weight_numel)
        self._workspaces = {}                 # (device, stream) -> scratch tensor (fixed size, never regrown)
        self._internal_unaligned = None       # kernels without 16-byte vector stores, compiled on first need

        self._reorder = WeightReorder(config)
        self.reorder_weights_e3nn_to_oeq = self._reorder.e3nn_to_oeq
        self.reorder_weights_oeq_to_e3nn = self._reorder.oeq_to_e3nn

        if self.torch_op:
            self._setup_torch_custom_op()

    @staticmethod
    def name():
        return "LoopUnrollTP"

    # ----------------------------------------------------------- raw entry points
    def _workspace_ptr(self, stream=None) -> int:
        """Scratch of this operator for ``stream`` (packed weights, dW partial sums): one buffer per
        stream, so that two streams using one operator do not overwrite each other's partial sums."""
        if self.workspace_bytes == 0:
            return 0
        dev = torch.cuda.current_device()
        key = (dev, self._stream(dev) if stream is None else int(stream))
        buf = self._workspaces.get(key)
        if buf is None:
            buf = self._workspaces[key] = torch.empty(self.workspace_bytes, dtype=torch.uint8, device=f"cuda:{dev}")
        return buf.data_ptr()

    @staticmethod
    def _stream(device_index: typing.Optional[int] = None) -> int:
        """torch's current stream on the device as a raw handle."""
        return torch._C._cuda_getCurrentRawStream(torch.cuda.current_device() if device_index is None else device_index)

    def _pick(self, *ptrs):
        aligned = all(int(p) % 16 == 0 for p in ptrs)
        if not aligned and isinstance(self.generator, UVUDirectGenerator):
            # rare: a caller-supplied tensor that is not 16-byte aligned -> kernels without vector stores
            if self._internal_unaligned is None:
                g = UVUDirectGenerator(self.config, "tp", vector_stores=False)
                fwd, bwd, _ = g.plan()
                self._internal_unaligned = rt.TPImpl(rt.compile_source(g.render()), _make_steps(fwd, self._step_flags),
                                                     _make_steps(bwd, self._step_flags))
            return self._internal_unaligned
        if isinstance(self.generator, UVWBatchedGenerator) and self.generator.pairs and any(int(p) % 8 for p in ptrs):
            # the same for the per-row-weights uvw kernels, which move fp32 weights two words at a time
            if self._internal_unaligned is None:
                g = UVWBatchedGenerator(self.config, pairs=False)
                fwd, bwd, _ = g.plan()
                self._internal_unaligned = rt.TPImpl(rt.compile_source(g.render()), _make_steps(fwd, self._step_flags),
                                                     _make_steps(bwd, self._step_flags))
            return self._internal_unaligned
        return self.internal

    def forward_raw(self, batch, L1_in, L2_in, L3_out, weights, stream=None) -> None:
        """Device pointers as integers (reference: TensorProductBase.py:41-49)."""
        impl = self._pick(L1_in, L2_in, L3_out, weights)
        impl.exec_tensor_product(int(batch), L1_in, L2_in, L3_out, weights, self._workspace_ptr(stream),
                                 self._stream() if stream is None else stream)

    def backward_raw(self, batch_size, L1_in, L1_grad, L2_in, L2_grad, weights, weights_grad, L3_grad,
                     stream=None) -> None:
        """reference: TensorProductBase.py:51-61."""
        impl = self._pick(L1_in, L1_grad, L2_in, L2_grad, weights, weights_grad, L3_grad)
        impl.backward(int(batch_size), L1_in, L1_grad, L2_in, L2_grad, weights, weights_grad, L3_grad,
                      self._workspace_ptr(stream), self._stream() if stream is None else stream)

    # ------------------------------------------------- numpy entry points (tests)
    def forward_cpu(self, L1_in, L2_in, L3_out, weights) -> None:
        """Host arrays in, result written into ``L3_out``; ``weights`` in e3nn order
        (reference: TensorProductBase.py:63-84)."""
        w = np.zeros_like(weights)
        self.reorder_weights_e3nn_to_oeq(weights, w, not self.config.shared_weights)
        bufs = [rt.DeviceBuffer(a) for a in (L1_in, L2_in, L3_out, w)]
        ws = rt.DeviceBuffer(self.workspace_bytes) if self.workspace_bytes else None
        self.internal.exec_tensor_product(L1_in.shape[0], bufs[0].data_ptr(), bufs[1].data_ptr(), bufs[2].data_ptr(),
                                          bufs[3].data_ptr(), ws.data_ptr() if ws else 0, 0)
        rt.stream_synchronize(0)
        L3_out[...] = bufs[2].copy_to_host()

    def backward_cpu(self, L1_in, L1_grad, L2_in, L2_grad, L3_grad, weights, weights_grad) -> None:
        """reference: TensorProductBase.py:86-112; weights and weights_grad in e3nn order."""
        w = np.zeros_like(weights)
        self.reorder_weights_e3nn_to_oeq(weights, w, not self.config.shared_weights)
        x, y, g = rt.DeviceBuffer(L1_in), rt.DeviceBuffer(L2_in), rt.DeviceBuffer(L3_grad)
        xg, yg = rt.DeviceBuffer(L1_grad), rt.DeviceBuffer(L2_grad)
        wd, wg = rt.DeviceBuffer(w), rt.DeviceBuffer(weights_grad)
        ws = rt.DeviceBuffer(self.workspace_bytes) if self.workspace_bytes else None
        self.internal.backward(L1_in.shape[0], x.data_ptr(), xg.data_ptr(), y.data_ptr(), yg.data_ptr(),
                               wd.data_ptr(), wg.data_ptr(), g.data_ptr(), ws.data_ptr() if ws else 0, 0)
        rt.stream_synchronize(0)
        L1_grad[...] = xg.copy_to_host()
        L2_grad[...] = yg.copy_to_host()
        wg_oeq = wg.copy_to_host().copy()
        self.reorder_weights_oeq_to_e3nn(wg_oeq, weights_grad, not self.config.shared_weights)

    # ------------------------------------------------------------------ torch op
    def _setup_torch_custom_op(self) -> None:
        """reference: TensorProductBase.py:234-298 (forward, backward, double backward)."""
        L3_dim = self.L3.dim
        shared = self.config.shared_weights

        @torch.library.custom_op(f"openequivariance_amd::tp_forward{self.tp_id}", mutates_args=(), device_types="cuda")
        def forward(L1_in: torch.Tensor, L2_in: torch.Tensor, weights: torch.Tensor) -> torch.Tensor:
            x, y, w = _contiguous(L1_in, L2_in, weights)
            self._check_inputs(x, y, w)
            out = torch.empty((x.shape[0], L3_dim), dtype=x.dtype, device=x.device)
            with _on_device(x.device):
                self.forward_raw(x.shape[0], x.data_ptr(), y.data_ptr(), out.data_ptr(), w.data_ptr(),
                                 self._stream(x.device.index))
            return out

        @forward.register_fake
        def _(L1_in, L2_in, weights):
            return L1_in.new_empty(L1_in.shape[0], L3_dim)

        self.forward = forward

        @torch.library.custom_op(f"openequivariance_amd::tp_grad_helper{self.tp_id}", mutates_args=(), device_types="cuda")
        def backward_helper(L1_in: torch.Tensor, L2_in: torch.Tensor, weights: torch.Tensor,
                            L3_grad: torch.Tensor) -> typing.List[torch.Tensor]:
            x, y, w, g = _contiguous(L1_in, L2_in, weights, L3_grad)
            self._check_inputs(x, y, w, g)
            xg, yg, wg = torch.empty_like(x), torch.empty_like(y), torch.empty_like(w)
            with _on_device(x.device):
                self.backward_raw(x.shape[0], x.data_ptr(), xg.data_ptr(), y.data_ptr(), yg.data_ptr(),
                                  w.data_ptr(), wg.data_ptr(), g.data_ptr(), self._stream(x.device.index))
            return [xg, yg, wg]

        @backward_helper.register_fake
        def _(L1_in, L2_in, weights, L3_grad):
            return [L1_in.new_empty(*L1_in.shape), L2_in.new_empty(*L2_in.shape), weights.new_empty(*weights.shape)]

        self.backward_helper = backward_helper

        def setup_context(ctx, inputs, output):
            ctx.L1_in, ctx.L2_in, ctx.weights = inputs

        def backward(ctx, grad_output):
            r = backward_helper(ctx.L1_in, ctx.L2_in, ctx.weights, grad_output)
            return r[0], r[1], r[2]

        forward.register_autograd(backward, setup_context=setup_context)

        def setup_context_double_backward(ctx, inputs, output):
            ctx.L1_in, ctx.L2_in, ctx.weights, ctx.L3_grad = inputs

        def double_backward(ctx, grad_output):
            return double_backward_terms(forward, backward_helper, ctx.L1_in, ctx.L2_in, ctx.weights, ctx.L3_grad,
                                         grad_output[0], grad_output[1], grad_output[2])

        backward_helper.register_autograd(double_backward, setup_context=setup_context_double_backward)

    def _check_inputs(self, x, y, w, g=None) -> None:
        """Shapes, dtypes and devices, before anything is launched (the kernels dereference every
        pointer they are handed)."""
        B = x.shape[0]
        d1, d2, d3, wn = self._dims
        if x.ndim != 2 or x.shape[1] != d1:
            raise ValueError(f"L1_in must have shape [batch, {d1}], got {tuple(x.shape)}")
        if y.shape != (B, d2):
            raise ValueError(f"L2_in must have shape [{B}, {d2}], got {tuple(y.shape)}")
        want = (wn,) if self.config.shared_weights else (B, wn)
        if w.shape != want:
            raise ValueError(f"weights must have shape {want}, got {tuple(w.shape)}")
        if g is not None and g.shape != (B, d3):
            raise ValueError(f"L3_grad must have shape [{B}, {d3}], got {tuple(g.shape)}")
        dev, tdt = x.device, self._torch_dtype
        for name, t in (("L1_in", x), ("L2_in", y), ("weights", w), ("L3_grad", g)):
            if t is None:
                continue
            if t.dtype != tdt:
                raise TypeError(f"tensors must be {tdt}")
            if not t.is_cuda:
                raise ValueError(f"{name} is on {t.device}: all tensors must be on the GPU (there is no CPU implementation)")
            if t.device != dev:
                raise ValueError(f"{name} is on {t.device}, L1_in on {x.device}: all tensors must share one device")

    # ------------------------------------------------------------------ timing
    def benchmark_forward(self, num_warmup: int, num_iter: int, L1_in, L2_in, L3_buffer, weights) -> np.ndarray:
        """Milliseconds of ``num_iter`` forward passes, caches flushed before each (reference:
        TensorProductBase.py:115-151).  With ``torch_op`` the torch operator is timed (allocation
        and dispatch included), otherwise the C-ABI call on preallocated buffers."""
        times = np.zeros(num_iter, dtype=np.float32)
        if self.torch_op:
            x, y, w = (torch.tensor(a, device="cuda") for a in (L1_in, L2_in, weights))
            timer = rt.GPUTimer(self._stream())
            run = lambda: self.forward(x, y, w)
        else:
            bufs = [rt.DeviceBuffer(a) for a in (L1_in, L2_in, L3_buffer, weights)]
            n, ptrs = L1_in.shape[0], [b.data_ptr() for b in bufs]
            ws = rt.DeviceBuffer(self.workspace_bytes) if self.workspace_bytes else None
            timer = rt.GPUTimer(0)
            run = lambda: self.internal.exec_tensor_product(n, *ptrs, ws.data_ptr() if ws else 0, 0)
        for _ in range(num_warmup):
            run()
        for i in range(num_iter):
            timer.clear_L2_cache()
            timer.start()
            run()
            times[i] = timer.stop_clock_get_elapsed()
        return times

    def benchmark_backward(self, num_warmup: int, num_iter: int, L1_in, L2_in, L3_buffer, weights, L1_grad, L2_grad,
                           weights_grad) -> np.ndarray:
        """reference: TensorProductBase.py:153-218; ``L3_buffer`` is the output gradient."""
        times = np.zeros(num_iter, dtype=np.float32)
        if self.torch_op:
            x, y, w = (torch.tensor(a, device="cuda", requires_grad=True) for a in (L1_in, L2_in, weights))
            out, g = self.forward(x, y, w), torch.tensor(L3_buffer, device="cuda")
            timer = rt.GPUTimer(self._stream())
            run = lambda: out.backward(gradient=g, retain_graph=True, inputs=[x, y, w])
            reset = lambda: [t.grad.zero_() for t in (x, y, w)]
        else:
            bufs = [rt.DeviceBuffer(a) for a in (L1_in, L1_grad, L2_in, L2_grad, weights, weights_grad, L3_buffer)]
            n, ptrs = L1_in.shape[0], [b.data_ptr() for b in bufs]
            ws = rt.DeviceBuffer(self.workspace_bytes) if self.workspace_bytes else None
            timer = rt.GPUTimer(0)
            run = lambda: self.internal.backward(n, *ptrs, ws.data_ptr() if ws else 0, 0)
            reset = lambda: None
        for _ in range(num_warmup):
            run()
        for i in range(num_iter):
            reset()
            timer.clear_L2_cache()
            timer.start()
            run()
            times[i] = timer.stop_clock_get_elapsed()
        if self.torch_op:
            L1_grad[:], L2_grad[:], weights_grad[:] = (t.grad.numpy(force=True) for t in (x, y, w))
        return times

    # ------------------------------------------------------ work / traffic models
    def calculate_flops_forward(self, batch_size: int) -> dict:
        """FLOP model of the reference (LoopUnrollTP.py:77-91)."""
        tpp = self.config
        if self.is_uvw:
            dense = sum(2 * np.prod(ins.path_shape) * tpp.irreps_out[ins.i_out].ir.dim for ins in tpp.instructions)
            return {"dense_contraction": int(dense) * batch_size, "total": int(dense) * batch_size}
        cg = lin = 0
        for ins in tpp.instructions:
            l1, l2, l3 = tpp.irreps_in1[ins.i_in1].ir.l, tpp.irreps_in2[ins.i_in2].ir.l, tpp.irreps_out[ins.i_out].ir.l
            nnz = int(np.count_nonzero(np.abs(wigner_3j(l1, l2, l3)) > 1e-14))
            cg += nnz * ins.path_shape[0] * ins.path_shape[1]
            lin += (2 * l3 + 1) * int(np.prod(ins.path_shape))
        out = {"CG_decomposition": 3 * cg * batch_size, "linear_combination": lin * batch_size, "outer_products": 0}
        out["total"] = sum(out.values())
        return out

    def calculate_flops_backward(self, batch_size: int) -> dict:
        """reference: LoopUnrollTP.py:93-105."""
        tpp = self.config
        if self.is_uvw:
            dense = sum(4 * np.prod(ins.path_shape) * tpp.irreps_out[ins.i_out].ir.dim for ins in tpp.instructions)
            return {"dense_contraction": int(dense) * batch_size, "total": int(dense) * batch_size}
        cg = 0
        for ins in tpp.instructions:
            l1, l2, l3 = tpp.irreps_in1[ins.i_in1].ir.l, tpp.irreps_in2[ins.i_in2].ir.l, tpp.irreps_out[ins.i_out].ir.l
            nnz = int(np.count_nonzero(np.abs(wigner_3j(l1, l2, l3)) > 1e-14))
            cg += nnz * ins.path_shape[0] * ins.path_shape[1]
        return {"backward": 9 * cg * batch_size, "total": 9 * cg * batch_size}

    def calculate_memory_streamed_forward(self, batch_size: int) -> dict:
        """Minimum bytes moved (reference: benchmark/perf_metrics_utils.py:11-25)."""
        s = np.dtype(self.irrep_dtype).itemsize
        wn = self.config.weight_numel
        w = wn if self.config.shared_weights else wn * batch_size
        d = {"input": (self.L1.dim + self.L2.dim) * batch_size * s, "weights": w * s, "output": self.L3.dim * batch_size * s}
        d["total"] = sum(d.values())
        return d

    def calculate_memory_streamed_backward(self, batch_size: int) -> dict:
        """reference: benchmark/perf_metrics_utils.py:27-44."""
        s = np.dtype(self.irrep_dtype).itemsize
        wn = self.config.weight_numel
        w = wn if self.config.shared_weights else wn * batch_size
        d = {"input": (self.L1.dim + self.L2.dim + self.L3.dim) * batch_size * s + w * s,
             "output": (self.L1.dim + self.L2.dim) * batch_size * s + w * s}
        d["total"] = sum(d.values())
        return d


LoopUnrollTP = TensorProduct
