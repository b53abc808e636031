"""Headline benchmark: MACE-style uvu tensor product, forward + backward, on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload mace_uvu|nequip_conv_atomic|...]

A step is one forward and one backward pass of the hot path over one batch of synthetic,
seeded inputs that already live in HBM.  Prints ONE JSON line.  Besides the whole-job
throughput (edges/s) it reports, for the dominant kernel, the achieved algorithmic bandwidth
measured with HIP events around every launch of the timed region, and a CPU baseline (the
e3nn-equivalent torch implementation on the host cores, on a bounded sample).
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
    ap.add_argument("--workload", default="mace_uvu")
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


def cpu_baseline(wl, case, sample):
    """e3nn-equivalent torch implementation on the host cores, forward+backward, fp32, on a
    bounded sample of the same seeded inputs (the op is independent per row/edge, so the rate of
    the sample is the rate of the workload).  This is the only place where the oracle package is
    used by the benchmark: as the thing timed beside the GPU, never as the product."""
    from oracle import spec, torch_cpu
    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
    h = case.host
    if wl.mode == "uvw":
        oprob = spec.fully_connected(*wl.irreps, shared_weights=True)
    elif wl.name == "readme_uvu":
        oprob = spec.Problem(*wl.irreps, [(0, 0, 0, "uvu", True)], shared_weights=False)
    else:
        oprob = spec.channelwise(*wl.irreps)
    if wl.kind == "tp":
        n = sample or min(wl.units, {"mace_uvu": 1000, "readme_uvu": 1000}.get(wl.name, 2000))
        W = h["W"] if h["W"].ndim == 1 else h["W"][:n]
        args_ = (h["X"][:n], h["Y"][:n], W, h["G"][:n])
        sec = torch_cpu.time_forward_backward(oprob, *args_, threads=cores, repeats=1)
        reps = max(1, min(20, int(10.0 / max(sec, 1e-3))))
        sec = torch_cpu.time_forward_backward(oprob, *args_, threads=cores, repeats=reps)
        what = f"first {n} rows of the same seeded batch, {reps} repeats"
    else:
        n = sample or min(wl.units, 5000)
        rows, cols = h["rows"][:n], h["cols"][:n]
        args_ = (h["X"], h["Y"][:n], h["W"][:n], h["G"])
        sec = torch_cpu.time_forward_backward(oprob, *args_, threads=cores, repeats=1, rows=rows, cols=cols)
        reps = max(1, min(20, int(10.0 / max(sec, 1e-3))))
        sec = torch_cpu.time_forward_backward(oprob, *args_, threads=cores, repeats=reps, rows=rows, cols=cols)
        what = f"first {n} edges of the same seeded graph (all nodes), {reps} repeats"
    return {"value": round(n / sec, 1), "unit": wl.unit, "cores": cores, "kind": "port",
            "sample": what + "; torch CPU einsum + autograd, fp32 (e3nn itself is not installable offline)"}


COPY_SRC = r"""
// Plain streaming copy: reads n 16-byte vectors and writes n 16-byte vectors, nothing else.
extern "C" __global__ __launch_bounds__(256) void oeq_copy_calibration(const float4* __restrict__ in, float4* __restrict__ out, unsigned long long n) {
    for (unsigned long long i = (unsigned long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (unsigned long long)gridDim.x * 256)
        out[i] = in[i];
}
"""

STREAM_SRC = r"""
// Streaming probe with a fixed read:write mix: every thread reads NR 16-byte vectors (one from each
// of NR input streams) and writes NW (one to each of NW output streams), nothing else.
typedef float v4 __attribute__((ext_vector_type(4)));
extern "C" __global__ __launch_bounds__(256) void oeq_stream_probe(const v4* __restrict__ in, v4* __restrict__ out, unsigned long long n) {
    v4 keep = {0.f, 0.f, 0.f, 0.f};
    for (unsigned long long i = (unsigned long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (unsigned long long)gridDim.x * 256) {
        v4 acc = {1.f, 2.f, 3.f, 4.f};
#pragma unroll
        for (int r = 0; r < NR; ++r) acc += __builtin_nontemporal_load(in + r * n + i);
#pragma unroll
        for (int w = 0; w < NW; ++w) __builtin_nontemporal_store(acc, out + w * n + i);
        keep += acc;
    }
    if (NW == 0 && keep.x == 12345.678f) out[0] = keep;       // keeps the loads alive; never true for zero inputs
}
"""


def stream_probe(nr, nw, total_bytes=3 << 30, reps=5):
    """GB/s of a plain streaming kernel that reads ``nr`` and writes ``nw`` 16-byte vectors per
    thread (best of ``reps`` launches, 3 GiB per launch so that the 256 MiB Infinity Cache does not
    help): what HBM sustains for this read:write mix, the practical ceiling of a kernel with it."""
    import ctypes as C
    import torch
    from openequivariance_amd import runtime as rt
    n = total_bytes // 16 // (nr + nw)
    src = torch.zeros(max(nr, 1) * n * 4, dtype=torch.float32, device="cuda")
    dst = torch.empty(max(nw, 1) * n * 4, dtype=torch.float32, device="cuda")
    mod = rt.Module(rt.compile_source(STREAM_SRC, options=tuple(rt.DEFAULT_OPTIONS) + (f"-DNR={nr}", f"-DNW={nw}")))
    stream = torch.cuda.current_stream().cuda_stream
    args = [C.c_void_p(src.data_ptr()), C.c_void_p(dst.data_ptr()), C.c_uint64(n)]
    best = float("inf")
    for r in range(reps + 2):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        mod.launch("oeq_stream_probe", 32768, 256, args, stream=stream)
        b.record()
        b.synchronize()
        if r >= 2:
            best = min(best, a.elapsed_time(b))
    return (nr + nw) * n * 16 / (best * 1e-3) / 1e9


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


def stream_calibration():
    """Sustained HBM rate of plain streaming kernels for several read:write mixes."""
    out = {"workload": "stream_calibration", "unit": "GB/s", "peak": HBM_PEAK_GBS}
    for nr, nw in ((1, 0), (4, 1), (1, 1), (1, 3), (0, 1)):
        out[f"read{nr}_write{nw}"] = round(stream_probe(nr, nw), 1)
    print(json.dumps(out))


def main():
    args = parse()
    if args.workload == "copy_calibration":
        copy_calibration(args.steps)
        return
    if args.workload == "stream_calibration":
        stream_calibration()
        return
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (the path shards over rows/edges "
              "without communication and is measured on one)", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    import openequivariance_amd as oeq
    from openequivariance_amd import workloads

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    dev = torch.device("cuda:0")
    wl = workloads.get(args.workload)
    case = wl.build(dev)                      # operator + device tensors + raw-call closures
    ev = Events()

    def step(timed):
        if timed:
            ev.wrap("forward", case.forward)
            ev.wrap("backward", case.backward)
        else:
            case.forward()
            case.backward()

    for _ in range(args.warmup):
        step(False)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step(True)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    value = wl.units / (ms_per_step * 1e-3)

    fwd_ms, bwd_ms = ev.mean_ms("forward"), ev.mean_ms("backward")
    dom = "backward" if bwd_ms >= fwd_ms else "forward"
    dom_ms = max(fwd_ms, bwd_ms)
    if wl.bound == "hbm":
        alg = wl.alg_bytes[dom]
        achieved = alg / (dom_ms * 1e-3) / 1e9
        peak, unit = HBM_PEAK_GBS, "GB/s"
    else:
        alg = wl.alg_flops[dom]
        achieved = alg / (dom_ms * 1e-3) / 1e12
        peak, unit = (MFMA_FP32_PEAK_TFLOPS if wl.dtype == "f32" else MFMA_FP64_PEAK_TFLOPS), "TFLOP/s"
    roofline = {"bound": wl.bound, "kernel": f"{wl.name}:{dom}", "achieved": round(achieved, 2), "peak": peak,
                "unit": unit, "frac": round(achieved / peak, 4), "traffic": load_traffic(f"{wl.name}:{dom}"),
                "algorithmic_per_launch": alg, "avg_launch_ms": round(dom_ms, 5),
                "forward_ms": round(fwd_ms, 5), "backward_ms": round(bwd_ms, 5)}
    if wl.bound == "hbm":
        tot = wl.alg_bytes["forward"] + wl.alg_bytes["backward"]
        roofline["fwd_bwd_frac"] = round(tot / ((fwd_ms + bwd_ms) * 1e-3) / 1e9 / peak, 4)
        roofline["forward_frac"] = round(wl.alg_bytes["forward"] / (fwd_ms * 1e-3) / 1e9 / peak, 4)
        roofline["backward_frac"] = round(wl.alg_bytes["backward"] / (bwd_ms * 1e-3) / 1e9 / peak, 4)
    else:
        tot = wl.alg_flops["forward"] + wl.alg_flops["backward"]
        roofline["fwd_bwd_frac"] = round(tot / ((fwd_ms + bwd_ms) * 1e-3) / 1e12 / peak, 4)

    if wl.bound == "hbm" and not args.no_cold:
        # what a plain streaming kernel with the dominant kernel's read:write mix sustains on this
        # GPU: the practical ceiling under the 8 TB/s datasheet peak
        rd, wr = wl.read_write_split(dom)
        nr, nw = mix_of(rd, wr)
        ceil = stream_probe(nr, nw)
        roofline["streaming_ceiling"] = {"mix": f"{nr} reads : {nw} writes", "GB/s": round(ceil, 1),
                                         "frac_of_ceiling": round(achieved / ceil, 4)}

    if not args.no_cold:
        # second leg, outside the timed region: the same launches with the caches flushed before
        # each one (a 512 MiB fill, twice the 256 MiB Infinity Cache), the protocol of the reference's
        # timers (openequivariance/extension/util/backend_hip.hpp:65-99 clears a 100 MB buffer)
        flush = torch.empty(512 << 20, dtype=torch.uint8, device=dev)
        for _ in range(min(args.steps, 30)):
            flush.fill_(1)
            ev.wrap("forward_cold", case.forward)
            flush.fill_(2)
            ev.wrap("backward_cold", case.backward)
        torch.cuda.synchronize()
        del flush
        fm, fmin = ev.median_min_ms("forward_cold")
        bm, bmin = ev.median_min_ms("backward_cold")
        work = wl.alg_bytes if wl.bound == "hbm" else wl.alg_flops
        scale = 1e9 if wl.bound == "hbm" else 1e12
        roofline["flushed_caches"] = {
            "forward_ms_median": round(fm, 5), "forward_ms_min": round(fmin, 5),
            "backward_ms_median": round(bm, 5), "backward_ms_min": round(bmin, 5),
            "fwd_bwd_frac": round((work["forward"] + work["backward"]) / ((fm + bm) * 1e-3) / scale / peak, 4)}

    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline(wl, case, args.cpu_sample)

    out = {"metric": "fwd+bwd edges/s and % HBM roofline, MACE-style uvu TP and fused conv",
           "value": round(value, 1), "unit": wl.unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak",
           "vs_baseline": None, "dtype": wl.dtype, "data": "synthetic",
           "config": {"workload": wl.description, **wl.config},
           "roofline": roofline, "cpu_baseline": cpu,
           "device": torch.cuda.get_device_name(0)}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
