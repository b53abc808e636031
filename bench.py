"""Headline benchmark: MACE-style uvu tensor product, forward + backward, on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload mace_uvu|nequip_conv_atomic|...]

A step is one forward and one backward pass of the hot path over one batch of synthetic,
seeded inputs that already live in HBM.  Prints ONE JSON line.  Besides the whole-job
throughput (edges/s) it reports, for the dominant kernel, the achieved algorithmic bandwidth
measured with HIP events around every launch of the timed region, and a CPU baseline (the
e3nn-equivalent torch implementation on the host cores, on a bounded sample).  Without
``--workload`` the headline fields are those of ``mace_uvu`` and the key ``workloads`` holds the
same measurements for every other benchmark configuration (fused convolutions, dense uvw, the
single-path example), each timed with the same protocol in the same process.
"""
from __future__ import annotations

import argparse
import json
import os
import pathlib
import sys
import time

ROOT = pathlib.Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_FP32_PEAK_TFLOPS = 157.3
MFMA_FP64_PEAK_TFLOPS = 78.6


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default=None,
                    help="time this workload only (default: mace_uvu as the headline and every other benchmark "
                         "configuration under the key 'workloads')")
    ap.add_argument("--headline-only", action="store_true", help="mace_uvu only, without the other configurations")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-cold", action="store_true", help="skip the flushed-cache timing leg")
    ap.add_argument("--cpu-sample", type=int, default=0, help="edges in the CPU sample (0 = automatic)")
    return ap.parse_args()


class Events:
    """HIP event pairs on torch's current stream (the stream every kernel is launched on)."""

    def __init__(self):
        import torch
        self.torch = torch
        self.pairs = {}

    def wrap(self, name, fn):
        a = self.torch.cuda.Event(enable_timing=True)
        b = self.torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        self.pairs.setdefault(name, []).append((a, b))

    def times_ms(self, name):
        return [a.elapsed_time(b) for a, b in self.pairs.get(name, [])]

    def mean_ms(self, name):
        v = self.times_ms(name)
        return sum(v) / len(v) if v else float("nan")

    def median_min_ms(self, name):
        v = sorted(self.times_ms(name))
        if not v:
            return float("nan"), float("nan")
        mid = len(v) // 2
        med = v[mid] if len(v) % 2 else 0.5 * (v[mid - 1] + v[mid])
        return med, v[0]


def load_traffic(key):
    """Measured HBM bytes per launch from committed counter summaries (None when absent)."""
    p = ROOT / "profiles" / "traffic.json"
    if p.exists():
        try:
            return json.loads(p.read_text()).get(key)
        except Exception:
            return None
    return None


def cpu_baseline(wl, case, sample, seconds=10.0):
    """e3nn-equivalent torch implementation on the host cores, forward+backward, in the precision of the workload, on a
    bounded sample of the same seeded inputs (the op is independent per row/edge, so the rate of
    the sample is the rate of the workload).  This is the only place where the oracle package is
    used by the benchmark: as the thing timed beside the GPU, never as the product."""
    from oracle import spec, torch_cpu
    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
    h = case.host
    if wl.mode == "uvw":
        oprob = spec.fully_connected(*wl.irreps, shared_weights=wl.shared)
    elif wl.name == "readme_uvu":
        oprob = spec.Problem(*wl.irreps, [(0, 0, 0, "uvu", True)], shared_weights=False)
    else:
        oprob = spec.channelwise(*wl.irreps)
    if wl.kind == "tp":
        n = sample or min(wl.units, {"mace_uvu": 1000, "readme_uvu": 1000}.get(wl.name, 2000))
        W = h["W"] if h["W"].ndim == 1 else h["W"][:n]
        args_ = (h["X"][:n], h["Y"][:n], W, h["G"][:n])
        sec = torch_cpu.time_forward_backward(oprob, *args_, threads=cores, repeats=1)
        reps = max(1, min(20, int(seconds / max(sec, 1e-3))))
        sec = torch_cpu.time_forward_backward(oprob, *args_, threads=cores, repeats=reps)
        what = f"first {n} rows of the same seeded batch, {reps} repeats"
    else:
        n = min(sample or min(wl.units, 5000), h["W"].shape[0])
        rows, cols = h["rows"][:n], h["cols"][:n]
        args_ = (h["X"], h["Y"][:n], h["W"][:n], h["G"])
        sec = torch_cpu.time_forward_backward(oprob, *args_, threads=cores, repeats=1, rows=rows, cols=cols)
        reps = max(1, min(20, int(seconds / max(sec, 1e-3))))
        sec = torch_cpu.time_forward_backward(oprob, *args_, threads=cores, repeats=reps, rows=rows, cols=cols)
        what = f"first {n} edges of the same seeded graph (all nodes), {reps} repeats"
    return {"value": round(n / sec, 1), "unit": wl.unit, "cores": cores, "kind": "port",
            "sample": what + f"; torch CPU einsum + autograd, {'fp32' if wl.dtype == 'f32' else 'fp64'} "
                      "(e3nn itself is not installable offline)"}


COPY_SRC = r"""
// Plain streaming copy: reads n 16-byte vectors and writes n 16-byte vectors, nothing else.
extern "C" __global__ __launch_bounds__(256) void oeq_copy_calibration(const float4* __restrict__ in, float4* __restrict__ out, unsigned long long n) {
    for (unsigned long long i = (unsigned long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (unsigned long long)gridDim.x * 256)
        out[i] = in[i];
}
"""

STREAM_SRC = r"""
// Streaming probe with a fixed read:write mix: every thread reads NR vectors (one from each of NR
// input streams) and writes NW (one to each of NW output streams), nothing else.  VEC = floats per
// access (2 or 4), NT = 1 for non-temporal accesses; the grid is what the host launches (one element
// per thread when oversubscribed, a grid-stride loop over few workgroups when persistent).
typedef float vN __attribute__((ext_vector_type(VEC)));
static __device__ __forceinline__ vN ld(const vN* p) { return NT ? __builtin_nontemporal_load(p) : *p; }
static __device__ __forceinline__ void st(vN* p, vN v) { if (NT) __builtin_nontemporal_store(v, p); else *p = v; }
extern "C" __global__ __launch_bounds__(256) void oeq_stream_probe(const vN* __restrict__ in, vN* __restrict__ out, unsigned long long n) {
    vN keep = (vN)(0.f);
    for (unsigned long long i = (unsigned long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (unsigned long long)gridDim.x * 256) {
        vN acc = (vN)(1.f);
#pragma unroll
        for (int r = 0; r < NR; ++r) acc += ld(in + r * n + i);
#pragma unroll
        for (int w = 0; w < NW; ++w) st(out + w * n + i, acc);
        keep += acc;
    }
    if (NW == 0 && keep.x == 12345.678f) out[0] = keep;       // keeps the loads alive; never true for zero inputs
}
"""

# (label, non-temporal, floats per access, workgroups: 0 = one element per thread, k = k per compute unit)
PROBE_VARIANTS = [(f"{'nt' if nt else 'plain'}/{4 * vec}B/{'1 elem per thread' if k == 0 else f'{k} workgroups per CU'}", nt, vec, k)
                  for nt in (1, 0) for vec in (4, 2) for k in (0, 4, 8, 16)]


def stream_probe(nr, nw, total_bytes=3 << 30, reps=5, variants=None):
    """Best GB/s over a sweep of plain streaming kernels that read ``nr`` and write ``nw`` vectors per
    thread (3 GiB per launch, so that the 256 MiB Infinity Cache does not help; best of ``reps``
    launches per variant): what the memory system sustains for this read:write mix, the practical
    ceiling of a kernel with it.  The sweep covers temporal / non-temporal accesses, 8- and 16-byte
    accesses, and oversubscribed / persistent grids; returns (best GB/s, label of the best variant,
    {label: GB/s})."""
    import ctypes as C
    import torch
    from openequivariance_amd import runtime as rt
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    stream = torch.cuda.current_stream().cuda_stream
    n16 = total_bytes // 16 // (nr + nw)
    src = torch.zeros(max(nr, 1) * n16 * 4, dtype=torch.float32, device="cuda")
    dst = torch.empty(max(nw, 1) * n16 * 4, dtype=torch.float32, device="cuda")
    table = {}
    for label, nt, vec, k in (variants or PROBE_VARIANTS):
        n = n16 * (4 // vec)
        grid = (n + 255) // 256 if k == 0 else cus * k
        if grid >= 2 ** 31:
            continue
        opts = tuple(rt.DEFAULT_OPTIONS) + (f"-DNR={nr}", f"-DNW={nw}", f"-DVEC={vec}", f"-DNT={nt}")
        mod = rt.Module(rt.compile_source(STREAM_SRC, options=opts))
        args = [C.c_void_p(src.data_ptr()), C.c_void_p(dst.data_ptr()), C.c_uint64(n)]
        best = float("inf")
        for r in range(reps + 2):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            mod.launch("oeq_stream_probe", grid, 256, args, stream=stream)
            b.record()
            b.synchronize()
            if r >= 2:
                best = min(best, a.elapsed_time(b))
        table[label] = round((nr + nw) * n16 * 16 / (best * 1e-3) / 1e9, 1)
    top = max(table, key=table.get)
    return table[top], top, table


def torch_stream_reference(total_bytes=3 << 30, reps=5):
    """The same kind of measurement with torch's own elementwise kernels, as an outside reference:
    copy_ (1 read : 1 write), add (2 : 1), sum (read only), fill_ (write only)."""
    import torch
    out = {}

    def best_ms(fn):
        best = float("inf")
        for r in range(reps + 2):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            fn()
            b.record()
            b.synchronize()
            if r >= 2:
                best = min(best, a.elapsed_time(b))
        return best
    n = total_bytes // 4 // 3
    x, y, z = (torch.zeros(n, dtype=torch.float32, device="cuda") for _ in range(3))
    out["torch copy_ (1:1)"] = round(2 * n * 4 / (best_ms(lambda: y.copy_(x)) * 1e-3) / 1e9, 1)
    out["torch add (2:1)"] = round(3 * n * 4 / (best_ms(lambda: torch.add(x, y, out=z)) * 1e-3) / 1e9, 1)
    out["torch sum (1:0)"] = round(n * 4 / (best_ms(lambda: x.sum()) * 1e-3) / 1e9, 1)
    out["torch fill_ (0:1)"] = round(n * 4 / (best_ms(lambda: x.fill_(1.0)) * 1e-3) / 1e9, 1)
    return out


def mix_of(read_bytes, write_bytes):
    """Small-integer read:write mix closest to the given byte counts (each side at most 4)."""
    best = None
    for nr in range(0, 5):
        for nw in range(0, 5):
            if nr + nw == 0:
                continue
            err = abs(nr / (nr + nw) - read_bytes / (read_bytes + write_bytes))
            if best is None or err < best[0] - 1e-12:
                best = (err, nr, nw)
    return best[1], best[2]


def copy_calibration(steps):
    """A copy kernel of known size (1 GiB read + 1 GiB written per launch), used to scale the
    FETCH_SIZE / WRITE_SIZE counters of rocprofv3: run it under the same --pmc as the workload."""
    import ctypes as C
    import torch
    from openequivariance_amd import runtime as rt
    nbytes = 1 << 30
    src = torch.ones(nbytes // 4, dtype=torch.float32, device="cuda")
    dst = torch.empty_like(src)
    mod = rt.Module(rt.compile_source(COPY_SRC))
    stream = torch.cuda.current_stream().cuda_stream
    for _ in range(steps):
        mod.launch("oeq_copy_calibration", 256 * 16, 256,
                   [C.c_void_p(src.data_ptr()), C.c_void_p(dst.data_ptr()), C.c_uint64(nbytes // 16)], stream=stream)
    torch.cuda.synchronize()
    assert torch.equal(src[:1024], dst[:1024])
    print(json.dumps({"workload": "copy_calibration", "bytes_read_per_launch": nbytes,
                      "bytes_written_per_launch": nbytes, "launches": steps}))


ROW_SHAPE_SRC = r"""
// Copy kernel in the shape of the uvu batch product: one workgroup of WPR wavefronts per row reads RD
// and writes WR pieces of 1 KB of that row (the pieces dealt to the wavefronts in contiguous ranges),
// all loads issued before the first store.  NT = 1: non-temporal accesses.
typedef float v4 __attribute__((ext_vector_type(4)));
extern "C" __global__ __launch_bounds__(64 * WPR) void oeq_row_shape_probe(const v4* __restrict__ in, v4* __restrict__ out) {
    const unsigned row = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const v4* ip = in + (unsigned long long)row * (RD * 64) + lane;
    v4* op = out + (unsigned long long)row * (WR * 64) + lane;
    constexpr int NR = (RD + WPR - 1) / WPR, NW = (WR + WPR - 1) / WPR;
    v4 r[NR], acc = (v4)(0.f);
#pragma unroll
    for (int i = 0; i < NR; ++i) { const int pc = wave * NR + i; r[i] = pc < RD ? (NT ? __builtin_nontemporal_load(ip + pc * 64) : ip[pc * 64]) : (v4)(0.f); }
#pragma unroll
    for (int i = 0; i < NR; ++i) acc += r[i];
#pragma unroll
    for (int i = 0; i < NW; ++i) {
        const int pc = wave * NW + i;
        if (pc < WR) { const v4 v = acc + (float)i; if (NT) __builtin_nontemporal_store(v, op + pc * 64); else op[pc * 64] = v; }
    }
}
"""


def row_shape_probe(read_kb, write_kb, rows=50000, reps=5):
    """GB/s of copy kernels that move ``read_kb`` in and ``write_kb`` out per row with 1, 2 or 4 wavefronts
    per row, temporal and non-temporal: what the memory system sustains for the row-per-workgroup shape of
    the uvu batch kernels (forward 13 : 36 KB, backward 49 : 13 KB per row of the 128-channel MACE problem)."""
    import ctypes as C
    import torch
    from openequivariance_amd import runtime as rt
    stream = torch.cuda.current_stream().cuda_stream
    src = torch.zeros(rows * read_kb * 256, dtype=torch.float32, device="cuda")
    dst = torch.empty(rows * write_kb * 256, dtype=torch.float32, device="cuda")
    table = {}
    for wpr in (1, 2, 4):
        for nt in (0, 1):
            opts = tuple(rt.DEFAULT_OPTIONS) + (f"-DWPR={wpr}", f"-DNT={nt}", f"-DRD={read_kb}", f"-DWR={write_kb}")
            mod = rt.Module(rt.compile_source(ROW_SHAPE_SRC, options=opts))
            args = [C.c_void_p(src.data_ptr()), C.c_void_p(dst.data_ptr())]
            best = float("inf")
            for r in range(reps + 2):
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                mod.launch("oeq_row_shape_probe", rows, 64 * wpr, args, stream=stream)
                b.record()
                b.synchronize()
                if r >= 2:
                    best = min(best, a.elapsed_time(b))
            table[f"{wpr} wavefront{'s' if wpr > 1 else ''} per row, {'non-temporal' if nt else 'plain'}"] = \
                {"GB/s": round(rows * (read_kb + write_kb) * 1024 / (best * 1e-3) / 1e9, 1), "us": round(best * 1e3, 1)}
    return table


def stream_calibration():
    """Sustained rate of plain streaming kernels for several read:write mixes: the whole sweep per
    mix, its best variant, and torch's own elementwise kernels beside it."""
    out = {"workload": "stream_calibration", "unit": "GB/s", "peak": HBM_PEAK_GBS, "mixes": {}}
    for nr, nw in ((1, 0), (4, 1), (3, 1), (2, 1), (1, 1), (1, 3), (0, 1)):
        best, label, table = stream_probe(nr, nw)
        out["mixes"][f"read{nr}_write{nw}"] = {"best": best, "best_variant": label, "sweep": table}
    out["torch"] = torch_stream_reference()
    out["row_shape"] = {"uvu forward, 13 KB in / 36 KB out per row": row_shape_probe(13, 36),
                        "uvu backward, 49 KB in / 13 KB out per row": row_shape_probe(49, 13)}
    print(json.dumps(out))



# ---------------------------------------------------------------------------------------------------
# Probe: would a banded, channel-sliced sender-order backward of the large convolution move fewer bytes
# across the fabric?  Stand-in kernels with the real access shapes of config 5 (13 paths, 256 channels,
# dZ rows of 11 008 words, W rows of 3 328) and sum arithmetic.
MUL = 256
# (in1 block, out words D, Z column start, W column start)
PATHS = [(0, 1, 0, 0), (1, 1, 256, 256), (2, 1, 512, 512),
         (0, 3, 768, 768), (1, 3, 1536, 1024), (1, 3, 2304, 1280), (2, 3, 3072, 1536), (2, 3, 3840, 1792),
         (0, 5, 4608, 2048), (1, 5, 5888, 2304), (1, 5, 7168, 2560), (2, 5, 8448, 2816), (2, 5, 9728, 3072)]
IN1 = [(0, 1), (256, 3), (1024, 5)]      # offset, D
D1, D3, WN, D2 = 2304, 11008, 3328, 16


def band_probe_source(S, group, name, nt=1, dyw=1, noG=0, noW=0, noX=0):
    """Wavefront = (band k of receivers -> XCD k mod 8, slice j of S channels, tile of senders); lane group
    sub (64 / S groups) walks a contiguous run of senders of band k in (band, sender, receiver) order, keeps
    the sender's dX partial in registers, gathers the dZ slice of each edge's receiver (from the band: a
    working set of N / K receivers x S channels x 43 words per XCD), streams the W slice in and the dW slice
    out.  noG = 1 gathers from 8 rows only (every gather hits cache), 2 drops the gathers; noW drops the W
    loads (1), the dW stores (2) or both (3); noX the X loads; dyw = 0 the dY partial stores."""
    paths = [p for p in PATHS if group is None or p[0] in group]
    blocks = sorted({p[0] for p in paths})
    R = 64 // S
    L = []
    A = L.append
    A("typedef long long i64; typedef unsigned long long u64;")
    A("static __device__ __forceinline__ float ldnt(const float* p) { return %s; }" % ("__builtin_nontemporal_load(p)" if nt else "*p"))
    A("static __device__ __forceinline__ void stnt(float* p, float v) { %s; }" % ("__builtin_nontemporal_store(v, p)" if nt else "*p = v"))
    A(f'extern "C" __global__ __launch_bounds__(64) void {name}(const float* __restrict__ X, float* __restrict__ Xp, const float* __restrict__ W, float* __restrict__ Wg,')
    A("    const float* __restrict__ G, const float* __restrict__ Y, float* __restrict__ Yp, const i64* __restrict__ blist, const i64* __restrict__ bptr,")
    A("    const i64* __restrict__ rows, const i64* __restrict__ cols, u64 nnz, u64 N, int K, int SPG, int NSL, int tiles)")
    A("{")
    A(f"  const int lane = threadIdx.x, sub = lane / {S}, ul = lane % {S};")
    A("  const u64 bid = blockIdx.x; const int xcd = (int)(bid & 7); const u64 turn = bid >> 3;")
    A("  const int phases = K / 8;")
    A("  const u64 per_xcd = (u64)NSL * phases * tiles; if (turn >= per_xcd) return;")
    A("  const int j = (int)(turn / ((u64)phases * tiles)); const u64 rem = turn % ((u64)phases * tiles);")
    A("  const int phase = (int)(rem / tiles); const u64 tile = rem % tiles; const int k = phase * 8 + xcd;")
    A(f"  u64 sa = (tile * {R} + sub) * (u64)SPG; if (sa > N) sa = N; u64 sb = sa + SPG; if (sb > N) sb = N;")
    A("  const i64 pa = bptr[(u64)k * (N + 1) + sa], pb = bptr[(u64)k * (N + 1) + sb];")
    A("  const int len = (int)(pb - pa); int maxlen = len;")
    for m in (32, 16, 8, 4, 2, 1):
        if m >= S:
            A(f"  maxlen = max(maxlen, __shfl_xor(maxlen, {m}, 64));")
    A(f"  const int u = j * {S} + ul;")
    names = []
    for t, (b, D, zo, wo) in enumerate(paths):
        names += [f"g{t}_{d}" for d in range(D)] + [f"w{t}"]
    for b in blocks:
        names += [f"x{b}_{d}" for d in range(IN1[b][1])]
    names += ["yv"]
    A("  float " + ", ".join(f"N{n} = 0.f" for n in names) + ";")
    for b in blocks:
        A("  float " + ", ".join(f"dx{b}_{d} = 0.f" for d in range(IN1[b][1])) + ";")
    A("  u64 Ie0 = 0, Ie1 = 0, Ir0 = 0, Ir1 = 0, Is0 = 0, Is1 = 0; bool Iv0 = false, Iv1 = false; i64 cur_s = -1;")

    def idx(it, q):
        A(f"  {{ const bool ev = ({it}) < len; const u64 pos = ev ? (u64)(pa + ({it})) : (u64)(nnz - 1); const u64 e = (u64)blist[pos];")
        A(f"    Ie{q} = e; Iv{q} = ev; Ir{q} = " + ("(u64)(rows[e] & 7)" if noG == 1 else "(u64)rows[e]") + f";  Is{q} = (u64)cols[e]; }}")

    def load(q):
        A(f"  {{ const u64 e = Ie{q}, r = Ir{q}, s = Is{q};")
        A(f"    const float* __restrict__ Wr = W + e * {WN}; const float* __restrict__ Gr = G + r * {D3}; const float* __restrict__ Xr = X + s * {D1};")
        A(f"    Nyv = ldnt(Y + e * {D2} + (ul & 15));")
        for t, (b, D, zo, wo) in enumerate(paths):
            if noW & 1:
                A(f"    Nw{t} = Nyv;")
            else:
                A(f"    Nw{t} = ldnt(Wr + {wo} + u);")
        for t, (b, D, zo, wo) in enumerate(paths):
            if noG == 2:
                A("    " + " ".join(f"Ng{t}_{d} = Nyv;" for d in range(D)))
            else:
                A(f"    {{ const float* __restrict__ p_ = Gr + {zo} + u * {D}; " + " ".join(f"Ng{t}_{d} = p_[{d}];" for d in range(D)) + " }")
        for b in blocks:
            off, D = IN1[b]
            if noX:
                A("    " + " ".join(f"Nx{b}_{d} = Nyv;" for d in range(D)))
            else:
                A(f"    {{ const float* __restrict__ p_ = Xr + {off} + u * {D}; " + " ".join(f"Nx{b}_{d} = p_[{d}];" for d in range(D)) + " }")
        A("  }")

    def flush():
        A("    if (cur_s >= 0) {")
        A(f"      float* __restrict__ q_ = Xp + ((u64)k * N + (u64)cur_s) * {D1};")
        for b in blocks:
            off, D = IN1[b]
            for d in range(D):
                A(f"      q_[{off} + u * {D} + {d}] = dx{b}_{d}; dx{b}_{d} = 0.f;")
        A("    }")
    A("  if (maxlen > 0) {")
    idx("0", 0)
    load(0)
    A("  }")
    A("  if (maxlen > 1) {")
    idx("1", 1)
    A("  }")
    A("  for (int it = 0; it < maxlen; it += 2) {")
    for h in (0, 1):
        if h == 1:
            A("    if (it + 1 >= maxlen) break;")
        A("    {")
        A("    const float " + ", ".join(f"{n} = N{n}" for n in names) + ";")
        A(f"    const u64 e = Ie{h}; const bool ev = Iv{h}; const i64 s = ev ? (i64)Is{h} : cur_s;")
        A(f"    if (it + {h + 1} < maxlen) {{")
        load(1 - h)
        A("    }")
        A(f"    if (it + {h + 2} < maxlen) {{")
        idx(f"it + {h + 2}", h)
        A("    }")
        A("    if (s != cur_s) {")
        flush()
        A("      cur_s = s; }")
        A("    float dy = 0.f;")
        for t, (b, D, zo, wo) in enumerate(paths):
            bd = IN1[b][1]
            A(f"    {{ float sg = " + " + ".join(f"g{t}_{d}" for d in range(D)) + f"; float dw = sg * x{b}_0 * yv; ")
            if noW & 2:
                A(f"      if (ev && dw == 1.2345f) stnt(Wg + e * {WN} + {wo} + u, dw);")
            else:
                A(f"      if (ev) stnt(Wg + e * {WN} + {wo} + u, dw);")
            A("      " + " ".join(f"dx{b}_{d} = __builtin_fmaf(sg * w{t}, yv, dx{b}_{d});" for d in range(bd)) + f" dy += sg * w{t}; }}")
        if dyw:
            for m in (8, 4, 2, 1):
                A(f"    dy += __shfl_xor(dy, {m}, 64);")
            A(f"    if (ev && ul < 16) Yp[((u64)(j * 3 + {0 if group is None else group[0]}) * nnz + e) * 16 + ul] = dy;")
        A("    }")
    A("  }")
    A("  if (true) {")
    flush()
    A("  }")
    A("}")
    return "\n".join(L)




def conv_band_probe():
    """Times the stand-in for slices of 16 / 32 / 64 channels and 8 / 16 / 32 receiver bands, and - to see what
    bounds the loop - with parts of the traffic switched off.  The sender-order backward it would replace
    takes 7.5 ms on the same graph."""
    import ctypes as C
    import torch
    from openequivariance_amd import runtime as rt
    torch.manual_seed(0)
    dev = torch.device("cuda:0")
    N, deg = 20000, 40
    rows = torch.repeat_interleave(torch.arange(N), torch.poisson(torch.full((N,), float(deg))).long())
    E = rows.numel()
    cols = torch.randint(0, N, (E,))
    rows, cols = rows.to(dev), cols.to(dev)
    W = torch.empty(E * WN, device=dev).normal_()
    Wg = torch.empty(E * WN, device=dev)
    G = torch.empty(N * D3, device=dev).normal_()
    X = torch.empty(N * D1, device=dev).normal_()
    Y = torch.empty(E * D2, device=dev).normal_()
    stream = torch.cuda.current_stream().cuda_stream
    modes = dict(full={}, gathers_always_hit=dict(noG=1), no_W_no_dW=dict(noW=3), no_gathers=dict(noG=2),
                 only_W_loads=dict(noG=2, noX=1, dyw=0, noW=2), only_dW_stores=dict(noG=2, noX=1, dyw=0, noW=1),
                 only_W_and_dW=dict(noG=2, noX=1, dyw=0))
    variants = [(S, K, "full") for S in (16, 32, 64) for K in (8, 16, 32)] + [(64, 16, m) for m in modes if m != "full"] \
        + [(16, 32, "no_W_no_dW")]
    out = {"workload": "conv_band_probe", "edges": E, "nodes": N, "unit": "ms per backward-equivalent",
           "sender_order_backward_ms": 7.5, "variants": []}
    compiled = {}
    for S, K, mode in variants:
        R, NSL, SPG = 64 // S, MUL // S, 8
        band = rows // ((N + K - 1) // K)
        blist = torch.argsort((band * N + cols) * N + rows)
        kk = (band * N + cols)[blist]
        q = torch.arange(K, device=dev).repeat_interleave(N + 1) * N + torch.arange(N + 1, device=dev).repeat(K)
        bptr = torch.searchsorted(kk, q).contiguous()
        Xp = torch.empty(K * N * D1, device=dev)
        Yp = torch.empty(NSL * 3 * E * 16, device=dev)
        tiles = (N + R * SPG - 1) // (R * SPG)
        if (S, mode) not in compiled:
            compiled[(S, mode)] = rt.Module(rt.compile_source(band_probe_source(S, None, "probe", **modes[mode])))
        grid = 8 * NSL * (K // 8) * tiles
        args = [C.c_void_p(t.data_ptr()) for t in (X, Xp, W, Wg, G, Y, Yp, blist, bptr, rows, cols)] + \
               [C.c_uint64(E), C.c_uint64(N), C.c_int(K), C.c_int(SPG), C.c_int(NSL), C.c_int(tiles)]
        best = float("inf")
        for rep in range(4):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            compiled[(S, mode)].launch("probe", grid, 64, args, stream=stream)
            b.record()
            b.synchronize()
            if rep >= 1:
                best = min(best, a.elapsed_time(b))
        out["variants"].append({"channels_per_slice": S, "receiver_bands": K, "mode": mode, "ms": round(best, 3),
                                "dZ_slice_per_XCD_MB": round(N / K * S * 43 * 4 / 1e6, 2)})
        del Xp, Yp, blist, bptr, kk, q, band
    print(json.dumps(out))


MFMA_PROBE_SRC = r"""
// Wavefronts that do nothing but matrix-core instructions on NACC independent accumulators, with VALU dependent
// multiply-adds on the operand registers after each of them.  SHAPE 32: v_mfma_f32_32x32x2_f32, 16: v_mfma_f32_16x16x4_f32.
typedef float V4 __attribute__((ext_vector_type(4)));
typedef float V16 __attribute__((ext_vector_type(16)));
extern "C" __global__ void __launch_bounds__(64) oeq_mfma_probe(float* out, int iters) {
    const float a = (float)threadIdx.x * 1e-3f, b = (float)blockIdx.x * 1e-6f;
#if SHAPE == 32
    V16 acc[NACC];
    for (int i = 0; i < NACC; ++i) for (int r = 0; r < 16; ++r) acc[i][r] = 0;
#else
    V4 acc[NACC];
    for (int i = 0; i < NACC; ++i) for (int r = 0; r < 4; ++r) acc[i][r] = 0;
#endif
    float v[8] = {a, b, a + b, a - b, a * 2, b * 2, a + 1, b + 1};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < NACC; ++i) {
#if SHAPE == 32
            acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(v[i & 7], v[(i + 1) & 7], acc[i], 0, 0, 0);
#else
            acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(v[i & 7], v[(i + 1) & 7], acc[i], 0, 0, 0);
#endif
#pragma unroll
            for (int q = 0; q < VALU; ++q) v[(i + q) & 7] = v[(i + q) & 7] * 1.0001f + v[(i + q + 3) & 7];
        }
    }
    float s = 0;
    for (int i = 0; i < NACC; ++i) s += acc[i][0] + acc[i][3];
    for (int q = 0; q < 8; ++q) s += v[q];
    if (s == 12345.678f) out[0] = s;
}
"""


def mfma_rate_probe():
    """What the fp32 matrix cores sustain on this GPU, and what vector-ALU instructions between the matrix
    instructions cost: the yardstick for the dense uvw kernels (157.3 TFLOP/s is the datasheet figure at the
    peak clock).  Grid = wavefronts per SIMD x 4 SIMDs x compute units, one wavefront per workgroup."""
    import ctypes as C
    import torch
    from openequivariance_amd import runtime as rt
    out = torch.zeros(16, device="cuda")
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    stream = torch.cuda.current_stream().cuda_stream
    iters, nacc = 2000, 4
    rec = {"workload": "mfma_rate_probe", "unit": "TFLOP/s", "peak": MFMA_FP32_PEAK_TFLOPS, "compute_units": cus,
           "accumulators": nacc, "variants": []}
    for shape in (16, 32):
        for valu in (0, 1, 2, 4, 8):
            for wps in (1, 2, 3):
                opts = tuple(rt.DEFAULT_OPTIONS) + (f"-DSHAPE={shape}", f"-DNACC={nacc}", f"-DVALU={valu}")
                mod = rt.Module(rt.compile_source(MFMA_PROBE_SRC, options=opts))
                grid = cus * 4 * wps
                best = float("inf")
                for r in range(5):
                    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    a.record()
                    mod.launch("oeq_mfma_probe", grid, 64, [C.c_void_p(out.data_ptr()), C.c_int(iters)], stream=stream)
                    b.record()
                    b.synchronize()
                    if r >= 1:
                        best = min(best, a.elapsed_time(b))
                flops = (4096 if shape == 32 else 2048) * nacc * iters * grid
                rec["variants"].append({"mfma": "32x32x2" if shape == 32 else "16x16x4", "valu_per_mfma": valu,
                                        "wavefronts_per_simd": wps, "TFLOP/s": round(flops / best / 1e9, 1)})
    print(json.dumps(rec))


def measure_torch_op(case, ev, steps, warmup, raw_ms):
    """The operator a user calls (reference protocol: implementations/TensorProductBase.py:114-219 and
    convolution/ConvolutionBase.py:251-411 time the torch op when torch_op=True): ``steps`` forward +
    backward passes through the custom ops and autograd, output allocation and argument checks included.
    Reports the wall clock per step, the HIP-event time of each direction, and what one call costs on the
    host (time until the call returns, measured with the GPU idle before each call)."""
    import torch
    run_f, run_b = case.torch_step
    for _ in range(max(warmup, 3)):           # (the unsorted operator times its backward variants on first use)
        run_f()
        run_b()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        ev.wrap("torch_forward", run_f)
        ev.wrap("torch_backward", run_b)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    host = {"forward": [], "backward": []}
    for _ in range(min(steps, 20)):
        for name, fn in (("forward", run_f), ("backward", run_b)):
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            fn()
            host[name].append((time.perf_counter() - t1) * 1e6)
    torch.cuda.synchronize()
    f_ms, b_ms = ev.mean_ms("torch_forward"), ev.mean_ms("torch_backward")
    med = lambda v: sorted(v)[len(v) // 2]
    return {"ms_per_step": round(wall_ms, 5), "forward_ms": round(f_ms, 5), "backward_ms": round(b_ms, 5),
            "host_us_per_call": {"forward": round(med(host["forward"]), 1), "backward": round(med(host["backward"]), 1)},
            "vs_raw_entry_points": round(wall_ms / raw_ms, 3) if raw_ms > 0 else None}


def measure(name, steps, warmup, cold=True, cpu=True, cpu_sample=0, ceiling=True, cpu_seconds=10.0):
    """Build one workload, time ``steps`` forward+backward steps after ``warmup`` untimed ones and
    return (workload, record): whole-job throughput from the wall clock around the timed region, and
    the per-direction averages from HIP event pairs recorded around every launch inside it."""
    import torch
    from openequivariance_amd import workloads
    dev = torch.device("cuda:0")
    wl = workloads.get(name)
    case = wl.build(dev)                      # operator + device tensors + raw-call closures
    ev = Events()

    def step(timed):
        if timed:
            ev.wrap("forward", case.forward)
            ev.wrap("backward", case.backward)
        else:
            case.forward()
            case.backward()

    for _ in range(warmup):
        step(False)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step(True)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / steps
    value = wl.units / (ms_per_step * 1e-3)

    fwd_ms, bwd_ms = ev.mean_ms("forward"), ev.mean_ms("backward")
    dom = "backward" if bwd_ms >= fwd_ms else "forward"
    dom_ms = max(fwd_ms, bwd_ms)
    if wl.bound == "hbm":
        work, scale = wl.alg_bytes, 1e9
        peak, unit = HBM_PEAK_GBS, "GB/s"
    else:
        work, scale = wl.alg_flops, 1e12
        peak, unit = (MFMA_FP32_PEAK_TFLOPS if wl.dtype == "f32" else MFMA_FP64_PEAK_TFLOPS), "TFLOP/s"
    alg = work[dom]
    achieved = alg / (dom_ms * 1e-3) / scale
    roofline = {"bound": wl.bound, "kernel": f"{wl.name}:{dom}", "achieved": round(achieved, 2), "peak": peak,
                "unit": unit, "frac": round(achieved / peak, 4), "traffic": load_traffic(f"{wl.name}:{dom}"),
                "algorithmic_per_launch": alg, "algorithmic": {"forward": work["forward"], "backward": work["backward"]},
                "avg_launch_ms": round(dom_ms, 5),
                "forward_ms": round(fwd_ms, 5), "backward_ms": round(bwd_ms, 5),
                "fwd_bwd_frac": round((work["forward"] + work["backward"]) / ((fwd_ms + bwd_ms) * 1e-3) / scale / peak, 4),
                "forward_frac": round(work["forward"] / (fwd_ms * 1e-3) / scale / peak, 4),
                "backward_frac": round(work["backward"] / (bwd_ms * 1e-3) / scale / peak, 4)}

    if wl.bound == "hbm" and ceiling:
        # what plain streaming kernels with the dominant kernel's read:write mix sustain on this GPU
        # (best of a sweep over access width, cache policy and grid shape): the practical ceiling
        # under the 8 TB/s datasheet peak
        rd, wr = wl.read_write_split(dom)
        nr, nw = mix_of(rd, wr)
        ceil, label, _ = stream_probe(nr, nw)
        roofline["streaming_ceiling"] = {"mix": f"{nr} reads : {nw} writes", "GB/s": ceil, "variant": label,
                                         "frac_of_ceiling": round(achieved / ceil, 4)}

    if cold:
        # second leg, outside the timed region: the same launches with the caches flushed before
        # each one (a 512 MiB fill, twice the 256 MiB Infinity Cache), the protocol of the reference's
        # timers (openequivariance/extension/util/backend_hip.hpp:65-99 clears a 100 MB buffer)
        flush = torch.empty(512 << 20, dtype=torch.uint8, device=dev)
        for _ in range(min(steps, 30)):
            flush.fill_(1)
            ev.wrap("forward_cold", case.forward)
            flush.fill_(2)
            ev.wrap("backward_cold", case.backward)
        torch.cuda.synchronize()
        del flush
        fm, fmin = ev.median_min_ms("forward_cold")
        bm, bmin = ev.median_min_ms("backward_cold")
        roofline["flushed_caches"] = {
            "forward_ms_median": round(fm, 5), "forward_ms_min": round(fmin, 5),
            "backward_ms_median": round(bm, 5), "backward_ms_min": round(bmin, 5),
            "fwd_bwd_frac": round((work["forward"] + work["backward"]) / ((fm + bm) * 1e-3) / scale / peak, 4)}

    if wl.min_traffic:
        # compulsory bytes + the per-edge rows any schedule must gather (or spill) when no cache holds them
        mt = wl.min_traffic
        roofline["min_traffic"] = dict(mt)
        roofline["min_traffic_rate_GBs"] = {"forward": round(mt["forward"] / (fwd_ms * 1e-3) / 1e9, 1),
                                            "backward": round(mt["backward"] / (bwd_ms * 1e-3) / 1e9, 1)}

    if case.forward_prepared is not None:
        # the timed launches prepare the graph on every call (the operators' default: a caller may hand over
        # a new graph each time); the same launches with the preparation reused from the workspace, the
        # regime of an operator built with graph_cache=True inside a model that calls one graph many times
        for _ in range(min(steps, 10)):
            ev.wrap("forward_prepared", case.forward_prepared)
            ev.wrap("backward_prepared", case.backward_prepared)
        torch.cuda.synchronize()
        fp, bp = ev.mean_ms("forward_prepared"), ev.mean_ms("backward_prepared")
        roofline["prepared_graph"] = {"forward_ms": round(fp, 5), "backward_ms": round(bp, 5),
                                      "fwd_bwd_frac": round((work["forward"] + work["backward"]) / ((fp + bp) * 1e-3) / scale / peak, 4)}
        case.forward()
        case.backward()

    torch_op = None
    if case.torch_step is not None:
        torch_op = measure_torch_op(case, ev, steps, warmup, fwd_ms + bwd_ms)

    rec = {"value": round(value, 1), "unit": wl.unit, "ms_per_step": round(ms_per_step, 5), "dtype": wl.dtype,
           "data": wl.data_note, "config": {"workload": wl.description, **wl.config}, "roofline": roofline,
           "torch_op": torch_op,
           "cpu_baseline": cpu_baseline(wl, case, cpu_sample, cpu_seconds) if cpu else None}
    del case
    torch.cuda.empty_cache()
    return wl, rec


# every benchmark configuration besides the headline one (config 2 = mace_uvu), the MACE problem as a convolution in both
# precisions, and one problem of each of the other two uvw kernel families (per-row weights, few shared weights)
OTHER_WORKLOADS = ("readme_uvu", "nequip_conv_det", "nequip_conv_atomic", "dense_uvw_f32", "dense_uvw_f64",
                   "large_conv_det", "large_conv_atomic", "mace_conv_det", "mace_conv_det_f64", "diffdock_uvw_f32",
                   "tetris_poly1_uvw_f32")


def main():
    args = parse()
    if args.workload == "copy_calibration":
        copy_calibration(args.steps)
        return
    if args.workload == "stream_calibration":
        stream_calibration()
        return
    if args.workload == "conv_band_probe":
        conv_band_probe()
        return
    if args.workload == "mfma_rate_probe":
        mfma_rate_probe()
        return
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (the path shards over rows/edges "
              "without communication and is measured on one)", file=sys.stderr)
        sys.exit(2)

    import torch
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)

    headline = args.workload or "mace_uvu"
    wl, rec = measure(headline, args.steps, args.warmup, cold=not args.no_cold, cpu=not args.no_cpu,
                      cpu_sample=args.cpu_sample, ceiling=not args.no_cold)
    out = {"metric": "fwd+bwd edges/s and % HBM roofline, MACE-style uvu TP and fused conv",
           "value": rec["value"], "unit": rec["unit"], "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "ms_per_step": rec["ms_per_step"], "higher_is_better": True, "scaling": "weak",
           "vs_baseline": None, "dtype": rec["dtype"], "data": rec["data"], "config": rec["config"],
           "roofline": rec["roofline"], "torch_op": rec["torch_op"], "cpu_baseline": rec["cpu_baseline"],
           "device": torch.cuda.get_device_name(0)}
    if not args.workload and not args.headline_only:
        # the other benchmark configurations, same protocol (same steps and warm-up, HIP events around every
        # launch), with a shorter CPU leg each
        others = {}
        for name in OTHER_WORKLOADS:
            t0 = time.perf_counter()
            try:
                _, r = measure(name, args.steps, args.warmup, cold=not args.no_cold, cpu=not args.no_cpu,
                               ceiling=False, cpu_seconds=3.0)
                rf = r["roofline"]
                others[name] = {"value": r["value"], "unit": r["unit"], "ms_per_step": r["ms_per_step"],
                                "forward_ms": rf["forward_ms"], "backward_ms": rf["backward_ms"],
                                "dtype": r["dtype"], "data": r["data"], "config": r["config"], "bound": rf["bound"],
                                "dominant": rf["kernel"], "frac": rf["frac"], "fwd_bwd_frac": rf["fwd_bwd_frac"],
                                "forward_frac": rf["forward_frac"], "backward_frac": rf["backward_frac"],
                                "algorithmic_per_launch": rf["algorithmic"],
                                "traffic": {"forward": load_traffic(f"{name}:forward"), "backward": load_traffic(f"{name}:backward")},
                                "flushed_caches": rf.get("flushed_caches"),
                                "prepared_graph": rf.get("prepared_graph"), "min_traffic": rf.get("min_traffic"),
                                "min_traffic_rate_GBs": rf.get("min_traffic_rate_GBs"),
                                "torch_op": r.get("torch_op"), "cpu_baseline": r["cpu_baseline"],
                                "bench_seconds": None}
            except Exception as exc:          # one workload failing must not hide the others
                others[name] = {"error": f"{type(exc).__name__}: {exc}"}
            others[name]["bench_seconds"] = round(time.perf_counter() - t0, 1)
        out["workloads"] = others
    print(json.dumps(out))


if __name__ == "__main__":
    main()
