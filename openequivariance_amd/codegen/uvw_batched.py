"""uvw tensor products with per-row weights (``shared_weights=False``), e.g. the DiffDock layers
of the reference's benchmark set (openequivariance/benchmark/benchmark_configs.py:44-48).

    Z[b, w, k] = sum_t sum_u  W[b, t, u, w] * T_t[b, u, k]

With a separate weight matrix per row there is no operand reuse across the batch: the op is a
batched matrix-vector product that streams ``weight_numel`` words per row and is bound by HBM,
so it runs on the vector ALU, one wavefront per row (reference: loop_unroll_tp.cuh:56-78 streams
the same weights through shared memory into a CUDA-core matmul):

* forward: lanes <-> channel u compute T_t[u, :] and park it in LDS; then lanes <-> output
  channel w walk u, reading one coalesced weight row per step and T by LDS broadcast;
* backward: lanes <-> u; each lane streams its own weight row W[b,t,u,:] (contiguous per lane),
  reads dZ by LDS broadcast, forms dT (-> dX, dY through the CG transpose) and writes its dW row.

The external (oeq) weight order is addressed in place by index arithmetic.
"""
from __future__ import annotations

from ..problem import TPProblem
from .common import Emitter, jinja_env
from .uvw import UVWGenerator, _ceil


class UVWBatchedGenerator(UVWGenerator):
    _allow_batched = True

    def __init__(self, problem: TPProblem):
        super().__init__(problem)
        if self.shared:
            raise ValueError("UVWBatchedGenerator is for per-row weights")
        self.kind = "uvw_batched"
        self.t_lds = max(p.mu * p.o.D for p in self.paths)
        self.ws_elems = 0

    def describe(self) -> str:
        return (f"uvw per-row weights T={self.T} paths={len(self.paths)} d1={self.D1} d2={self.D2} d3={self.D3} "
                f"wn={self.WN} (vector ALU, HBM bound)")

    # ----------------------------------------------------------------- forward
    def forward_body(self) -> str:
        E = Emitter()
        E("const int lane = threadIdx.x;")
        E("const u64 row = blockIdx.x;")
        E("if (row >= n) return;")
        E(f"__shared__ T tl[{max(1, self.t_lds)}];")
        E(f"const T* __restrict__ Xr = X + row * {self.D1};")
        E(f"const T* __restrict__ Wr = W + row * {self.WN};")
        for f in self.used_y:
            E(f"const T y{f} = Y[row * {self.D2} + {f}];")
        for o in self.out:
            if o.dim == 0:
                continue
            for wc in range(_ceil(o.mul, 64)):
                E(f"{{ // output block {o.idx}, channels {64 * wc} .. ")
                E.level += 1
                E(f"const int w = {64 * wc} + lane;")
                E(f"const int wcl = min(w, {o.mul - 1});")
                E("T " + ", ".join(f"z{k} = (T)0" for k in range(o.D)) + ";")
                for p in self.paths_into(o.idx):
                    E(f"// path {p.t}")
                    E("oeq_sync();")
                    for uc in range(_ceil(p.mu, 64)):
                        E(f"{{ const int u = {64 * uc} + lane;")
                        E(f"  if (u < {p.mu}) {{")
                        E(f"    const T* __restrict__ xp = Xr + {p.a.off} + u * {p.a.D};")
                        E("    const T " + ", ".join(f"x{i} = xp[{i}]" for i in range(p.a.D)) + ";")
                        E.level += 2
                        self.emit_cg_forward(E, p, "x", "y", "t")
                        E.level -= 2
                        E("    " + " ".join(f"tl[u * {o.D} + {k}] = t{k};" for k in range(o.D)))
                        E("  } }")
                    E("oeq_sync();")
                    E("#pragma unroll 4")
                    E(f"for (int u = 0; u < {p.mu}; ++u) {{")
                    E(f"    const T wv = Wr[{self.oeq_index(p, 'u', 'wcl')}];")
                    for k in range(o.D):
                        E(f"    z{k} = oeq_fma(wv, tl[u * {o.D} + {k}], z{k});")
                    E("}")
                E(f"if (w < {o.mul}) {{ T* __restrict__ zp = Z + row * {self.D3} + {o.off} + w * {o.D}; "
                  + " ".join(f"zp[{k}] = z{k};" for k in range(o.D)) + " }")
                E.level -= 1
                E("}")
        return E.text()

    # ---------------------------------------------------------------- backward
    def backward_body(self) -> str:
        E = Emitter()
        E("const int lane = threadIdx.x;")
        E("const u64 row = blockIdx.x;")
        E("if (row >= n) return;")
        E(f"__shared__ T gl[{max(1, self.D3)}];")
        E(f"const T* __restrict__ Xr = X + row * {self.D1};")
        E(f"const T* __restrict__ Wr = W + row * {self.WN};")
        E(f"T* __restrict__ Wgr = Wg + row * {self.WN};")
        E(f"for (int q = lane; q < {self.D3}; q += 64) gl[q] = G[row * {self.D3} + q];")
        E("oeq_sync();")
        for f in self.used_y:
            E(f"const T y{f} = Y[row * {self.D2} + {f}];")
            E(f"T dy{f} = (T)0;")
        for a in self.in1:
            if a.dim == 0:
                continue
            for uc in range(_ceil(a.mul, 64)):
                E(f"{{ // input block {a.idx}, channels {64 * uc} ..")
                E.level += 1
                E(f"const int u = {64 * uc} + lane;")
                E(f"const bool act = u < {a.mul};")
                E(f"const int ucl = min(u, {a.mul - 1});")
                E(f"const T* __restrict__ xp = Xr + {a.off} + ucl * {a.D};")
                E("const T " + ", ".join(f"x{i} = xp[{i}]" for i in range(a.D)) + ";")
                E("T " + ", ".join(f"dx{i} = (T)0" for i in range(a.D)) + ";")
                for p in self.paths_from(a.idx):
                    o = p.o
                    E(f"{{ // path {p.t}")
                    E.level += 1
                    self.emit_cg_forward(E, p, "x", "y", "t")
                    E("T " + ", ".join(f"dt{k} = (T)0" for k in range(o.D)) + ";")
                    E("#pragma unroll 4")
                    E(f"for (int w = 0; w < {p.mw}; ++w) {{")
                    E(f"    const int wi = {self.oeq_index(p, 'ucl', 'w')};")
                    E("    const T wv = Wr[wi];")
                    E("    const T " + ", ".join(f"g{k} = gl[{o.off} + w * {o.D} + {k}]" for k in range(o.D)) + ";")
                    for k in range(o.D):
                        E(f"    dt{k} = oeq_fma(wv, g{k}, dt{k});")
                    E("    if (act) Wgr[wi] = " + " + ".join(f"t{k} * g{k}" for k in range(o.D)) + ";")
                    E("}")
                    E("if (!act) { " + " ".join(f"dt{k} = (T)0;" for k in range(o.D)) + " }")
                    self.emit_cg_backward(E, p, "dt", "x", "y", "dx", "dy")
                    E.level -= 1
                    E("}")
                if self.paths_from(a.idx):
                    E(f"if (act) {{ T* __restrict__ dp = Xg + row * {self.D1} + {a.off} + u * {a.D}; "
                      + " ".join(f"dp[{i}] = dx{i};" for i in range(a.D)) + " }")
                else:
                    E(f"if (act) {{ T* __restrict__ dp = Xg + row * {self.D1} + {a.off} + u * {a.D}; "
                      + " ".join(f"dp[{i}] = (T)0;" for i in range(a.D)) + " }")
                E.level -= 1
                E("}")
        for f in self.used_y:
            E(f"dy{f} = oeq_wave_sum63(dy{f});")
        E("if (lane == 63) {")
        for f in range(self.D2):
            E(f"    Yg[row * {self.D2} + {f}] = " + (f"dy{f};" if f in self.used_y else "(T)0;"))
        E("}")
        return E.text()

    def render(self, prelude: str = None) -> str:
        env = jinja_env()
        if prelude is None:
            prelude = env.get_template("prelude.hip.jinja").render(T=self.T)
        return env.get_template("tp_uvw_batched.hip.jinja").render(g=self, prelude=prelude)

    def plan(self):
        fwd = [dict(kernel="forward", num_threads=64, grid_kind=1, work_per_block=1)]
        bwd = [dict(kernel="backward", num_threads=64, grid_kind=1, work_per_block=1)]
        return fwd, bwd, (lambda nnz=0, nodes=0: 0)
