"""uvw tensor products with per-row weights (``shared_weights=False``), e.g. the DiffDock layers
of the reference's benchmark set (openequivariance/benchmark/benchmark_configs.py:44-48).

    Z[b, w, k] = sum_t sum_u  W[b, t, u, w] * T_t[b, u, k]

With a separate weight matrix per row there is no operand reuse across the batch: the op is a
batched matrix-vector product that streams ``weight_numel`` words per row and is bound by HBM,
so it runs on the vector ALU, one wavefront per row (reference: loop_unroll_tp.cuh:56-78 streams
the same weights through shared memory into a CUDA-core matmul).  Both kernels read and write the
weights in the order they lie in memory - the external order keeps each 32 x 32 chunk [u][w] of a
path contiguous - so that a wavefront's access is one 256- or 512-byte run:

* forward: lanes <-> channel u compute T_t[u, :] of every path into a group of output blocks and
  park it in LDS; then lanes <-> (output channel w, a slice of u) walk the chunks with the loads a
  fixed number of steps ahead of the multiplies, branch-free, T read from LDS; the slices are
  summed with lane exchanges at the end of an output block;
* backward: a chunk goes global -> registers (two chunks ahead) -> LDS, padded to an odd row length;
  lanes <-> (u, a slice of w) then read their row of it, form dT (-> dX, dY through the CG
  transpose) against dZ in LDS and put dW = T (x) dZ back into the same LDS words, which leave in
  memory order again.

The external (oeq) weight order is addressed in place by index arithmetic.
"""
from __future__ import annotations

from ..problem import TPProblem
from .common import Emitter, jinja_env
from .uvw import UVWGenerator, _ceil


class UVWBatchedGenerator(UVWGenerator):
    _allow_batched = True

    def __init__(self, problem: TPProblem, pairs: bool = True):
        """``pairs``: fp32 weights move two words per lane where a chunk's offset and width are even (an 8-byte
        access sustains more of the HBM rate than a 4-byte one); needs W and dW at 8-byte aligned addresses."""
        super().__init__(problem)
        self.pairs = bool(pairs) and self.T == "float" and self.WN % 2 == 0
        if self.shared:
            raise ValueError("UVWBatchedGenerator is for per-row weights")
        self.kind = "uvw_batched"
        self.t_lds = max([sum(p.mu * o.D for o in ph for p in self.paths_into(o.idx)) for ph in self.forward_phases()] + [0])
        self.ws_elems = 0

    def describe(self) -> str:
        return (f"uvw per-row weights T={self.T} paths={len(self.paths)} d1={self.D1} d2={self.D2} d3={self.D3} "
                f"wn={self.WN} (vector ALU, HBM bound)")

    def ld2(self, ptr: str) -> str:
        return f"oeq_ldnt2({ptr})" if self.NONTEMPORAL else f"*(const V2*)({ptr})"

    def st2(self, ptr: str, val: str) -> str:
        return f"oeq_stnt2({ptr}, {val});" if self.NONTEMPORAL else f"*(V2*)({ptr}) = {val};"

    def ld(self, ptr: str) -> str:
        return f"oeq_ldnt({ptr})" if self.NONTEMPORAL else f"*({ptr})"

    def st(self, ptr: str, val: str) -> str:
        return f"oeq_stnt({ptr}, {val});" if self.NONTEMPORAL else f"*({ptr}) = {val};"

    # ------------------------------------------------------------ weight order
    @staticmethod
    def chunks(mul: int):
        """(chunk number, width) of the 32-wide pieces of a multiplicity, as the external weight
        order cuts it (weight_order.py)."""
        return [(c, min(32, mul - 32 * c)) for c in range(_ceil(mul, 32))]

    def chunk_base(self, p, uc: int, wc: int) -> int:
        """Offset of the [u_local][w_local] slice (contiguous, ul * wl words) that holds chunk
        (uc, wc) of path ``p``'s copy of the second operand."""
        mu, mv, mw = p.mu, p.mv, p.mw
        vc, vl = divmod(p.v, 32)
        vlw = min(32, mv - 32 * vc)
        ul, wl = min(32, mu - 32 * uc), min(32, mw - 32 * wc)
        base = p.woff + uc * 32 * mv * mw + ul * (32 * vc * mw + vlw * (32 * wc) + vl * wl)
        assert base == eval(self.oeq_index(p, str(32 * uc), str(32 * wc)), {"min": min})
        return base

    @staticmethod
    def _split(width: int):
        """Lanes <-> (position in a chunk of ``width`` <= 32, slice): the power of two the positions
        are padded to, its log2, and the number of slices."""
        lp = 1
        while lp < width:
            lp *= 2
        return lp, lp.bit_length() - 1, 64 // lp

    # ----------------------------------------------------------------- forward
    FORWARD_AHEAD = 16    # weight loads in flight ahead of the one being multiplied
    T_LDS_WORDS = 4096    # T of the paths into the output blocks of one phase stays below this many words

    def forward_phases(self):
        """Output blocks grouped so that T of every path into a group fits the LDS budget together: a phase
        computes all its T first and then streams its weights as one pipeline."""
        phases, words = [[]], 0
        for o in self.out:
            if o.dim == 0:
                continue
            w = sum(p.mu * o.D for p in self.paths_into(o.idx))
            if phases[-1] and words + w > self.T_LDS_WORDS:
                phases.append([])
                words = 0
            phases[-1].append(o)
            words += w
        return [ph for ph in phases if ph]

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
        for phase in self.forward_phases():
            # lanes <-> (V adjacent channels, a slice of u) within a chunk of output channels.  Lanes past the
            # chunk's width repeat its last columns: what they add up is never stored and never meets the other
            # lanes (the reduction over the slices keeps wq).  One step = one access of every lane: row
            # us + ns * j of a [ul][wl] slice; the last step of a slice whose rows do not divide re-reads the
            # last row with T = 0.
            toff, acc, groups, steps, lanes = {}, 0, [], [], []
            for o in phase:
                wcs = self.chunks(o.mul)
                into = self.paths_into(o.idx)
                width = {wc: 2 if self.pairs and wl % 2 == 0 and all(
                             self.chunk_base(p, uc, wc) % 2 == 0 for p in into for uc, _ in self.chunks(p.mu)) else 1
                         for wc, wl in wcs}
                for wc, wl in wcs:
                    lp, lg, _ = self._split(wl // width[wc])
                    lanes.append(f"const int wq{o.idx}_{wc} = min(lane & {lp - 1}, {wl // width[wc] - 1}), "
                                 f"us{o.idx}_{wc} = lane >> {lg};")
                for p in into:
                    toff[p.t] = acc
                    acc += p.mu * o.D
                per = max(1, 40 // (o.D * max(width.values())))
                for g0 in range(0, len(wcs), per):
                    grp = wcs[g0:g0 + per]
                    groups.append(dict(o=o, grp=grp, width=width, first=len(steps)))
                    for p in into:
                        for wc, wl in grp:
                            V = width[wc]
                            _, _, ns = self._split(wl // V)
                            for uc, ul in self.chunks(p.mu):
                                full, tail = divmod(ul, ns)
                                for j in range(full + (1 if tail else 0)):
                                    r = f"us{o.idx}_{wc} + {ns * j}"
                                    steps.append(dict(V=V, z=f"z{o.idx}_{wc}", wq=f"wq{o.idx}_{wc}", wl=wl, D=o.D,
                                                      base=self.chunk_base(p, uc, wc), t=toff[p.t] + 32 * uc * o.D,
                                                      row=r if j < full else f"min({r}, {ul - 1})",
                                                      ok=None if j < full else f"us{o.idx}_{wc} < {tail}"))
                    groups[-1]["last"] = len(steps)
            assert acc <= max(1, self.t_lds)

            def load(i):
                if i < len(steps):
                    st = steps[i]
                    addr = f"Wr + {st['base']} + {st['V']} * {st['wq']} + ({st['row']}) * {st['wl']}"
                    if st["V"] == 2:
                        E(f"const V2 wv{i} = {self.ld2(addr)};")
                    else:
                        E(f"const T wv{i}[1] = {{{self.ld(addr)}}};")

            def multiply(i):
                st = steps[i]
                for k in range(st["D"]):
                    t_ = f"tl[{st['t'] + k} + ({st['row']}) * {st['D']}]"
                    if st["ok"]:
                        t_ = f"({st['ok']}) ? {t_} : (T)0"
                    E(f"{{ const T t_ = {t_}; " + " ".join(
                        f"{st['z']}_{h}_{k} = oeq_fma(wv{i}[{h}], t_, {st['z']}_{h}_{k});" for h in range(st["V"])) + " }")

            E(f"{{ // output blocks {[o.idx for o in phase]}: T of every path into them, then their weights as one stream")
            E.level += 1
            for ln in lanes:
                E(ln)
            for i in range(self.FORWARD_AHEAD):
                load(i)
            paths = [p for o in phase for p in self.paths_into(o.idx)]
            for p in paths:
                for uc in range(_ceil(p.mu, 64)):
                    E(f"const T* __restrict__ xp{p.t}_{uc} = Xr + {p.a.off} + min({64 * uc} + lane, {p.mu - 1}) * {p.a.D};")
                    E("const T " + ", ".join(f"x{p.t}_{uc}_{i} = xp{p.t}_{uc}[{i}]" for i in range(p.a.D)) + ";")
            E("oeq_sync();")
            for p in paths:
                for uc in range(_ceil(p.mu, 64)):
                    E(f"{{ const int u = {64 * uc} + lane;   // path {p.t}")
                    E.level += 1
                    self.emit_cg_forward(E, p, f"x{p.t}_{uc}_", "y", "t")
                    E(f"if (u < {p.mu}) {{ " + " ".join(f"tl[{toff[p.t]} + u * {p.o.D} + {k}] = t{k};" for k in range(p.o.D)) + " }")
                    E.level -= 1
                    E("}")
            E("oeq_sync();")
            for gr in groups:
                o, width = gr["o"], gr["width"]
                E(f"// output block {o.idx}, channels {32 * gr['grp'][0][0]} ..")
                for wc, wl in gr["grp"]:
                    E("T " + ", ".join(f"z{o.idx}_{wc}_{h}_{k} = (T)0" for h in range(width[wc]) for k in range(o.D)) + ";")
                for i in range(gr["first"], gr["last"]):
                    load(i + self.FORWARD_AHEAD)
                    multiply(i)
                for wc, wl in gr["grp"]:
                    V = width[wc]
                    cols = wl // V
                    lp, lg, ns = self._split(cols)
                    z = f"z{o.idx}_{wc}"
                    s = lp
                    while s < 64:
                        E(" ".join(f"{z}_{h}_{k} += oeq_shfl_xor({z}_{h}_{k}, {s});" for h in range(V) for k in range(o.D)))
                        s *= 2
                    E(f"if (lane < {cols}) {{ T* __restrict__ zp = Z + row * {self.D3} + {o.off} + ({32 * wc} + {V} * lane) * {o.D}; "
                      + " ".join(f"zp[{h * o.D + k}] = {z}_{h}_{k};" for h in range(V) for k in range(o.D)) + " }")
            E.level -= 1
            E("}")
        return E.text()

    # ---------------------------------------------------------------- backward
    PREFETCH = 2          # weight chunks whose loads are in flight ahead of the one being worked on

    COMPUTE_UNROLL = 4    # steps of a chunk's row loop in flight; all 16 at once would take 100 more registers
    NONTEMPORAL = True    # the weights and their gradient are touched once
    def backward_body(self) -> str:
        E = Emitter()
        E("const int lane = threadIdx.x;")
        E("const u64 row = blockIdx.x;")
        E("if (row >= n) return;")
        E(f"__shared__ T gl[{max(1, self.D3)}];")
        E(f"__shared__ T tile[{32 * 33}];")
        E(f"const T* __restrict__ Xr = X + row * {self.D1};")
        E(f"const T* __restrict__ Wr = W + row * {self.WN};")
        E(f"T* __restrict__ Wgr = Wg + row * {self.WN};")
        # every [ul][wl] weight chunk of the row, in the order it is worked on
        jobs = []
        for a in self.in1:
            if a.dim == 0:
                continue
            for uc, ul in self.chunks(a.mul):
                for p in self.paths_from(a.idx):
                    for wc, wl in self.chunks(p.mw):
                        jobs.append((a.idx, uc, p.t, ul * wl, self.chunk_base(p, uc, wc)))

        def width(job):
            return 2 if self.pairs and job[3] % 2 == 0 and job[4] % 2 == 0 else 1

        def regs(job):
            return width(job) * _ceil(job[3], 64 * width(job))
        nbuf = self.PREFETCH + 1
        for b in range(min(nbuf, len(jobs))):
            E(f"T r{b}_[{max(regs(job) for job in jobs[b::nbuf])}];")

        def request(n):
            if n < len(jobs):
                _, _, _, words, base = jobs[n]
                V = width(jobs[n])
                E(f"// chunk {n}: {words} words at {base}")
                for i in range(_ceil(words, 64 * V)):
                    guard = "" if 64 * V * (i + 1) <= words else f"if ({64 * V * i} + {V} * lane < {words}) "
                    if V == 2:
                        E(f"{guard}{{ const V2 v_ = {self.ld2(f'Wr + {base + 128 * i} + 2 * lane')}; "
                          f"r{n % nbuf}_[{2 * i}] = v_[0]; r{n % nbuf}_[{2 * i + 1}] = v_[1]; }}")
                    else:
                        E(f"{guard}r{n % nbuf}_[{i}] = {self.ld(f'Wr + {base + 64 * i} + lane')};")

        for n in range(self.PREFETCH):
            request(n)
        E(f"for (int q = lane; q < {self.D3}; q += 64) gl[q] = G[row * {self.D3} + q];")
        E("oeq_sync();")
        for f in self.used_y:
            E(f"const T y{f} = Y[row * {self.D2} + {f}];")
            E(f"T dy{f} = (T)0;")
        n = 0
        for a in self.in1:
            if a.dim == 0:
                continue
            for uc, ul in self.chunks(a.mul):
                lp, lg, ns = self._split(ul)
                E(f"{{ // input block {a.idx}, channels {32 * uc} ..")
                E.level += 1
                E(f"const int uq = lane & {lp - 1}, ws = lane >> {lg};")
                E(f"const bool act = uq < {ul};")
                E(f"const int ur = min(uq, {ul - 1});")
                E(f"const T* __restrict__ xp = Xr + {a.off} + ({32 * uc} + ur) * {a.D};")
                E("const T " + ", ".join(f"x{i} = xp[{i}]" for i in range(a.D)) + ";")
                E("T " + ", ".join(f"dx{i} = (T)0" for i in range(a.D)) + ";")
                for p in self.paths_from(a.idx):
                    o = p.o
                    E(f"{{ // path {p.t}")
                    E.level += 1
                    self.emit_cg_forward(E, p, "x", "y", "t")
                    E("T " + ", ".join(f"dt{k} = (T)0" for k in range(o.D)) + ";")
                    for wc, wl in self.chunks(p.mw):
                        S = wl | 1
                        assert jobs[n][:3] == (a.idx, uc, p.t) and jobs[n][4] == self.chunk_base(p, uc, wc)
                        base, words = jobs[n][4], ul * wl

                        def pos(c):
                            return f"{c}" if S == wl else (f"{c} + (({c}) >> {wl.bit_length() - 1})" if wl & (wl - 1) == 0
                                                           else f"{c} + ({c}) / {wl}")
                        E(f"{{ // weights [{ul}][{wl}] at {base}: through LDS, one row per lane afterwards")
                        E.level += 1
                        V = width(jobs[n])
                        for i in range(_ceil(words, 64 * V)):
                            guard = "" if 64 * V * (i + 1) <= words else f"if ({64 * V * i} + {V} * lane < {words}) "
                            E(f"{guard}{{ " + " ".join(f"tile[{pos(f'{64 * V * i + h} + {V} * lane')}] = r{n % nbuf}_[{V * i + h}];"
                                                        for h in range(V)) + " }")
                        E("oeq_sync();")
                        request(n + self.PREFETCH)
                        full, tail = divmod(wl, ns)

                        def step(wq):
                            E(f"  const T wv = tile[ur * {S} + {wq}];")
                            E("  const T " + ", ".join(f"g{k} = gl[{o.off + 32 * wc * o.D + k} + ({wq}) * {o.D}]"
                                                       for k in range(o.D)) + ";")
                            for k in range(o.D):
                                E(f"  dt{k} = oeq_fma(wv, g{k}, dt{k});")
                            E(("  if (act) " if lp != ul else "  ") + f"tile[ur * {S} + {wq}] = "
                              + " + ".join(f"t{k} * g{k}" for k in range(o.D)) + ";")
                        if full:
                            E(f"#pragma unroll {self.COMPUTE_UNROLL}")
                            E(f"for (int j = 0; j < {full}; ++j) {{")
                            step(f"ws + {ns} * j")
                            E("}")
                        if tail:
                            E(f"if (ws < {tail}) {{")
                            step(f"ws + {ns * full}")
                            E("}")
                        E("oeq_sync();")
                        for i in range(_ceil(words, 64 * V)):
                            guard = "" if 64 * V * (i + 1) <= words else f"if ({64 * V * i} + {V} * lane < {words}) "
                            if V == 2:
                                E(f"{guard}{{ V2 v_; " + " ".join(f"v_[{h}] = tile[{pos(f'{128 * i + h} + 2 * lane')}];" for h in range(2))
                                  + " " + self.st2(f"Wgr + {base + 128 * i} + 2 * lane", "v_") + " }")
                            else:
                                E(guard + self.st(f"Wgr + {base + 64 * i} + lane", f"tile[{pos(f'{64 * i} + lane')}]"))
                        E("oeq_sync();")
                        E.level -= 1
                        E("}")
                        n += 1
                    s = lp
                    while s < 64:
                        E(" ".join(f"dt{k} += oeq_shfl_xor(dt{k}, {s});" for k in range(o.D)))
                        s *= 2
                    E("if (!act || ws != 0) { " + " ".join(f"dt{k} = (T)0;" for k in range(o.D)) + " }")
                    self.emit_cg_backward(E, p, "dt", "x", "y", "dx", "dy")
                    E.level -= 1
                    E("}")
                E(f"if (act && ws == 0) {{ T* __restrict__ dp = Xg + row * {self.D1} + {a.off} + ({32 * uc} + uq) * {a.D}; "
                  + " ".join(f"dp[{i}] = dx{i};" for i in range(a.D)) + " }")
                E.level -= 1
                E("}")
        assert n == len(jobs)
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
