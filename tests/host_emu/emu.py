"""CPU emulation of the generated kernels (test infrastructure).

The kernel generator's output is ordinary C++ apart from a small prelude of
device helpers.  Here the same generated source is compiled for the host with a
prelude that maps one wavefront to 64 threads (LDS -> a static array, waits ->
a pthread barrier, lane shuffles -> an exchange buffer) and is linked with
AddressSanitizer, then run as a separate executable on files.  This checks
indexing, bounds and arithmetic of the generated code in the build container,
where there is no GPU; the numbers that count are still the ones the GPU tests
produce.
"""
from __future__ import annotations

import hashlib
import os
import pathlib
import subprocess
import tempfile
from typing import Dict, List, Sequence

import numpy as np

CACHE = pathlib.Path(tempfile.gettempdir()) / "oeq_host_emu"

EMU_PRELUDE = r"""
#include <algorithm>
#include <cassert>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <mutex>
#include <string>
#include <thread>
#include <vector>
#include <pthread.h>
using std::min; using std::max;
typedef @T@ T;
typedef long long i64;
typedef unsigned long long u64;
struct emu_dim3 { unsigned x, y, z; };
static thread_local emu_dim3 threadIdx, blockIdx;
static emu_dim3 gridDim, blockDim;
#define __global__
#define __device__
#define __forceinline__ inline
#define __launch_bounds__(x)
#define __shared__ static
static pthread_barrier_t g_bar;
static T g_xT[1024];
static int g_xi[1024];
static std::mutex g_atomic_mutex;
static pthread_barrier_t g_wbar[16];             // one per wavefront of the workgroup
static inline void oeq_sync() { pthread_barrier_wait(&g_wbar[threadIdx.x >> 6]); }
static inline T oeq_fma(T a, T b, T c) { return std::fma(a, b, c); }
static inline void oeq_atomic_add(T* p, T v) { std::lock_guard<std::mutex> g(g_atomic_mutex); *p += v; }
static inline T oeq_shfl_xor(T v, int mask) { g_xT[threadIdx.x] = v; oeq_sync(); T r = g_xT[threadIdx.x ^ mask]; oeq_sync(); return r; }
static inline int oeq_shfl_i32(int v, int src) { g_xi[threadIdx.x] = v; oeq_sync(); int r = g_xi[src & 63]; oeq_sync(); return r; }
static i64 g_xl[1024];
static inline i64 oeq_shfl_up_i64(i64 v, int delta) { g_xl[threadIdx.x] = v; oeq_sync(); const int l = threadIdx.x & 63; i64 r = l >= delta ? g_xl[threadIdx.x - delta] : v; oeq_sync(); return r; }
static inline int oeq_shfl_xor_i32(int v, int mask) { g_xi[threadIdx.x] = v; oeq_sync(); int r = g_xi[threadIdx.x ^ mask]; oeq_sync(); return r; }
#define __builtin_amdgcn_readfirstlane(x) oeq_shfl_i32((x), 0)
static inline u64 oeq_uniform_u64(u64 v) { return v; }
struct VT { T v[16 / sizeof(T)]; T& operator[](int i) { return v[i]; } const T& operator[](int i) const { return v[i]; } };
typedef VT VTU;
#define __builtin_nontemporal_store(v, p) (*(p) = (v))
#define __builtin_nontemporal_load(p) (*(p))
#define OEQ_DMA(BYTES, POLICY, g, lds_base) memcpy((char*)(lds_base) + ((BYTES) == 12 ? 16 : (BYTES)) * (threadIdx.x & 63), (g), (BYTES))
static inline void oeq_release_agent() {}
static inline void oeq_acquire_agent() {}
static inline int oeq_ticket_add(int* p) { std::lock_guard<std::mutex> g(g_atomic_mutex); return (*p)++; }
static inline i64 oeq_lds_claim(i64* slot, i64 key) { std::lock_guard<std::mutex> g(g_atomic_mutex); const i64 old = *slot; if (old == -1) *slot = key; return old; }
static inline void oeq_st_agent(T* p, T v) { *p = v; }
static inline T oeq_ld_agent(const T* p) { return *p; }
static inline int oeq_lds_add(int* p, int v) { std::lock_guard<std::mutex> g(g_atomic_mutex); const int o = *p; *p += v; return o; }
static inline void oeq_wait_vm() {}
static inline void oeq_wait_lds() {}
static inline T oeq_wave_sum63(T v) { g_xT[threadIdx.x] = v; oeq_sync(); T t = 0; for (int i = 0; i < 64; ++i) t += g_xT[(threadIdx.x & ~63) + i]; oeq_sync(); return t; }
static inline T oeq_lane_value(T v, int l) { g_xT[threadIdx.x] = v; oeq_sync(); const T r = g_xT[(threadIdx.x & ~63) + l]; oeq_sync(); return r; }
template <int P> static inline T oeq_group_sum(T v) { g_xT[threadIdx.x] = v; oeq_sync(); T t = 0; for (int i = 0; i < P; ++i) t += g_xT[(threadIdx.x & ~(P - 1)) + i]; oeq_sync(); return t; }
static inline T oeq_ldnt(const T* p) { return *p; }
static inline void oeq_stnt(T* p, T v) { *p = v; }
struct V2 { T v[2]; T& operator[](int i) { return v[i]; } const T& operator[](int i) const { return v[i]; } };
static inline V2 oeq_ldnt2(const T* p) { assert((uintptr_t)p % (2 * sizeof(T)) == 0); V2 r; r[0] = p[0]; r[1] = p[1]; return r; }
static inline void oeq_stnt2(T* p, V2 v) { assert((uintptr_t)p % (2 * sizeof(T)) == 0); p[0] = v[0]; p[1] = v[1]; }
static inline void oeq_block_sync() { pthread_barrier_wait(&g_bar); }
static inline void oeq_sched_fence() {}
#define OEQ_OPAQUE(x) ((void)0)
static inline void __syncthreads() { pthread_barrier_wait(&g_bar); }
#define __HIP_MEMORY_SCOPE_AGENT 0
#define __HIP_MEMORY_SCOPE_WORKGROUP 0
template <class V> static inline V __hip_atomic_fetch_add(V* p, V v, int, int) { std::lock_guard<std::mutex> g(g_atomic_mutex); V o = *p; *p += v; return o; }
// matrix-core step of one wavefront, emulated collectively by its 64 threads
struct V4 { T v[4]; T& operator[](int i) { return v[i]; } const T& operator[](int i) const { return v[i]; } };
static T g_mA[16][16][4], g_mB[16][4][16];
static inline V4 oeq_mfma(T a, T b, V4 c) {
    const int wv = threadIdx.x >> 6, l = threadIdx.x & 63;
    g_mA[wv][l & 15][l >> 4] = a; g_mB[wv][l >> 4][l & 15] = b;
    pthread_barrier_wait(&g_wbar[wv]);
    V4 d = c;
    for (int r = 0; r < 4; ++r) {
        const int i = (sizeof(T) == 4) ? 4 * (l >> 4) + r : 4 * r + (l >> 4), j = l & 15;
        T acc = 0;
        for (int k = 0; k < 4; ++k) acc += g_mA[wv][i][k] * g_mB[wv][k][j];
        d[r] = c[r] + acc;
    }
    pthread_barrier_wait(&g_wbar[wv]);
    return d;
}

static void emu_run(unsigned gx, unsigned gy, unsigned block, const std::function<void()>& kernel) {
    gridDim = {gx, gy, 1}; blockDim = {block, 1, 1};
    pthread_barrier_init(&g_bar, nullptr, block);
    for (unsigned w = 0; w < (block + 63) / 64; ++w) pthread_barrier_init(&g_wbar[w], nullptr, block < 64 ? block : 64);
    for (unsigned by = 0; by < gy; ++by)
        for (unsigned bx = 0; bx < gx; ++bx) {
            std::vector<std::thread> th;
            for (unsigned t = 0; t < block; ++t)
                th.emplace_back([&, t] { threadIdx = {t, 0, 0}; blockIdx = {bx, by, 0}; kernel(); });
            for (auto& x : th) x.join();
        }
    pthread_barrier_destroy(&g_bar);
}
static std::vector<char> emu_read(const std::string& path, size_t expect) {
    FILE* f = fopen(path.c_str(), "rb");
    if (!f) { fprintf(stderr, "cannot open %s\n", path.c_str()); exit(3); }
    std::vector<char> buf(expect);                 // exact size: ASan sees any overrun
    size_t got = expect ? fread(buf.data(), 1, expect, f) : 0;
    fclose(f);
    if (got != expect) { fprintf(stderr, "short read %s\n", path.c_str()); exit(3); }
    return buf;
}
static void emu_write(const std::string& path, const std::vector<char>& buf) {
    FILE* f = fopen(path.c_str(), "wb");
    if (buf.size()) fwrite(buf.data(), 1, buf.size(), f);
    fclose(f);
}
"""

# main() for the two operator families.  argv: dir; the directory holds job.txt:
#   line 1: sizes; following lines: "<kernel> <threads> <grid_x> <grid_y>"
TP_MAIN = r"""
int main(int argc, char** argv) {
    std::string d = argv[1];
    FILE* job = fopen((d + "/job.txt").c_str(), "r");
    unsigned long long n, d1, d2, d3, wrow, wsz, ws_bytes; int backward_pass;
    if (fscanf(job, "%llu %llu %llu %llu %llu %llu %llu %d", &n, &d1, &d2, &d3, &wrow, &wsz, &ws_bytes, &backward_pass) != 8) return 3;
    auto X = emu_read(d + "/X.bin", n * d1 * sizeof(T));
    auto Y = emu_read(d + "/Y.bin", n * d2 * sizeof(T));
    auto W = emu_read(d + "/W.bin", wsz * sizeof(T));
    std::vector<char> Z(n * d3 * sizeof(T), (char)0x7f), ws(ws_bytes, (char)0x7f);
    std::vector<char> G, Xg(n * d1 * sizeof(T), (char)0x7f), Yg(n * d2 * sizeof(T), (char)0x7f), Wg(wsz * sizeof(T), (char)0x7f);
    if (backward_pass) G = emu_read(d + "/G.bin", n * d3 * sizeof(T));
    char name[64]; unsigned threads, gx, gy;
    while (fscanf(job, "%63s %u %u %u", name, &threads, &gx, &gy) == 4) {
        std::string k = name;
        if (k == "forward") emu_run(gx, gy, threads, [&] { forward(n, (const T*)X.data(), (const T*)Y.data(), (T*)Z.data(), (const T*)W.data(), ws.data()); });
        else if (k == "backward") emu_run(gx, gy, threads, [&] { backward(n, (const T*)X.data(), (T*)Xg.data(), (const T*)Y.data(), (T*)Yg.data(), (const T*)W.data(), (T*)Wg.data(), (const T*)G.data(), ws.data()); });
@EXTRA@
        else { fprintf(stderr, "unknown kernel %s\n", name); return 3; }
    }
    fclose(job);
    emu_write(d + "/Z.bin", Z); emu_write(d + "/Xg.bin", Xg); emu_write(d + "/Yg.bin", Yg); emu_write(d + "/Wg.bin", Wg);
    return 0;
}
"""

TP_EXTRA_UVW = r"""
        else if (k == "prep_forward") emu_run(gx, gy, threads, [&] { prep_forward(n, (const T*)X.data(), (const T*)Y.data(), (T*)Z.data(), (const T*)W.data(), ws.data()); });
#define UVW_BWD(fn) emu_run(gx, gy, threads, [&] { fn(n, (const T*)X.data(), (T*)Xg.data(), (const T*)Y.data(), (T*)Yg.data(), (const T*)W.data(), (T*)Wg.data(), (const T*)G.data(), ws.data()); })
        else if (k == "prep_backward") UVW_BWD(prep_backward);
        else if (k == "backward_dw") UVW_BWD(backward_dw);
        else if (k == "backward_reduce") UVW_BWD(backward_reduce);
"""

TP_EXTRA_UVW_ROWS = r"""
#define UVW_BWD(fn) emu_run(gx, gy, threads, [&] { fn(n, (const T*)X.data(), (T*)Xg.data(), (const T*)Y.data(), (T*)Yg.data(), (const T*)W.data(), (T*)Wg.data(), (const T*)G.data(), ws.data()); })
        else if (k == "backward_dw") UVW_BWD(backward_dw);
        else if (k == "backward_reduce") UVW_BWD(backward_reduce);
"""

TP_EXTRA_SHARED = r"""
        else if (k == "backward_reduce") emu_run(gx, gy, threads, [&] { backward_reduce(n, (const T*)X.data(), (T*)Xg.data(), (const T*)Y.data(), (T*)Yg.data(), (const T*)W.data(), (T*)Wg.data(), (const T*)G.data(), ws.data()); });
"""

CONV_MAIN = r"""
int main(int argc, char** argv) {
    std::string d = argv[1];
    FILE* job = fopen((d + "/job.txt").c_str(), "r");
    unsigned long long nnz, nodes, d1, d2, d3, wn, ws_bytes; int backward_pass, has_tperm;
    if (fscanf(job, "%llu %llu %llu %llu %llu %llu %llu %d %d", &nnz, &nodes, &d1, &d2, &d3, &wn, &ws_bytes, &backward_pass, &has_tperm) != 9) return 3;
    auto X = emu_read(d + "/X.bin", nodes * d1 * sizeof(T));
    auto Y = emu_read(d + "/Y.bin", nnz * d2 * sizeof(T));
    auto W = emu_read(d + "/W.bin", nnz * wn * sizeof(T));
    auto rows = emu_read(d + "/rows.bin", nnz * 8);
    auto cols = emu_read(d + "/cols.bin", nnz * 8);
    std::vector<char> tperm;
    if (has_tperm) tperm = emu_read(d + "/tperm.bin", nnz * 8);
    // accumulation targets start at zero (caller contract of the atomic kernels); the
    // deterministic kernels overwrite them, so fill those with junk instead
    const char fill = has_tperm ? (char)0x7f : (char)0;
    std::vector<char> Z(nodes * d3 * sizeof(T), fill), ws(ws_bytes, (char)0x7f);
    std::vector<char> G, Xg(nodes * d1 * sizeof(T), fill), Yg(nnz * d2 * sizeof(T), (char)0x7f), Wg(nnz * wn * sizeof(T), (char)0x7f);
    if (backward_pass) G = emu_read(d + "/G.bin", nodes * d3 * sizeof(T));
    char name[64]; unsigned threads, gx, gy;
#define FWD_CALL(fn) emu_run(gx, gy, threads, [&] { fn((const T*)X.data(), (const T*)Y.data(), (const T*)W.data(), (T*)Z.data(), (const i64*)rows.data(), (const i64*)cols.data(), nnz, nodes, ws.data(), (const i64*)tperm.data()); })
#define BWD_CALL(fn) emu_run(gx, gy, threads, [&] { fn((const T*)X.data(), (T*)Xg.data(), (const T*)Y.data(), (T*)Yg.data(), (const T*)W.data(), (T*)Wg.data(), (const T*)G.data(), (const i64*)rows.data(), (const i64*)cols.data(), nnz, nodes, ws.data(), (const i64*)tperm.data()); })
    while (fscanf(job, "%63s %u %u %u", name, &threads, &gx, &gy) == 4) {
        std::string k = name;
        if (k == "forward") FWD_CALL(forward);
        else if (k == "backward") BWD_CALL(backward);
@EXTRA@
        else { fprintf(stderr, "unknown kernel %s\n", name); return 3; }
    }
    fclose(job);
    emu_write(d + "/Z.bin", Z); emu_write(d + "/Xg.bin", Xg); emu_write(d + "/Yg.bin", Yg); emu_write(d + "/Wg.bin", Wg);
    return 0;
}
"""

CONV_EXTRA_DET = r"""
        else if (k == "prep_forward") FWD_CALL(prep_forward);
        else if (k == "prep_backward") BWD_CALL(prep_backward);
"""
CONV_EXTRA_ORDER = r"""
        else if (k == "order_backward") BWD_CALL(order_backward);
"""
CONV_EXTRA_SORTED = r"""
        else if (k == "group_clear") FWD_CALL(group_clear);
        else if (k == "group_count") FWD_CALL(group_count);
        else if (k == "group_fill") FWD_CALL(group_fill);
"""
CONV_EXTRA_GROUPED_BWD = r"""
        else if (k == "group_clear_backward") BWD_CALL(group_clear_backward);
        else if (k == "group_count_backward") BWD_CALL(group_count_backward);
        else if (k == "group_fill_backward") BWD_CALL(group_fill_backward);
"""
CONV_EXTRA_DYRED = r"""
        else if (k == "backward_dy_reduce") BWD_CALL(backward_dy_reduce);
"""


def emu_prelude(ctype: str) -> str:
    return EMU_PRELUDE.replace("@T@", ctype)


def build(source: str, main: str) -> pathlib.Path:
    """Compile generated source (rendered with ``emu_prelude``) + ``main`` with ASan."""
    text = source + "\n" + main
    key = hashlib.sha256(text.encode()).hexdigest()[:24]
    CACHE.mkdir(parents=True, exist_ok=True)
    exe = CACHE / f"emu_{key}"
    if exe.exists():
        return exe
    # (per-process names: test workers running side by side may build the same source at the same time)
    src = CACHE / f"emu_{key}.{os.getpid()}.cpp"
    tmp = f"{exe}.{os.getpid()}.tmp"
    src.write_text(text)
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address", "-static-libasan", "-fno-omit-frame-pointer",
           "-Wno-unknown-pragmas", "-ffp-contract=off", str(src), "-o", tmp, "-lpthread"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("host build of generated kernel failed:\n" + res.stderr[-6000:])
    os.replace(tmp, exe)
    os.replace(src, CACHE / f"emu_{key}.cpp")
    return exe


def grid_of(step: Dict, rows: int, nodes: int) -> int:
    """Same rule as the C library's launch()."""
    kind = step.get("grid_kind", 1)
    if kind == 0:
        return step["num_blocks"]
    if kind == 3:                            # one workgroup per node, then two per tile of the edge list
        g = (nodes + step["work_per_block"] - 1) // step["work_per_block"]
        if step.get("num_blocks", 0) and rows > 0 and nodes > 0:
            t = max(32, step["num_blocks"] * ((rows + nodes - 1) // nodes))
            g += 2 * ((rows + t - 1) // t)
        return g
    work = rows if kind == 1 else nodes
    wpb = step["work_per_block"]
    g = (work + wpb - 1) // wpb
    if step.get("num_blocks", 0):
        g = min(g, step["num_blocks"])
    return g


def _run(exe: pathlib.Path, workdir: str) -> None:
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:verify_asan_link_order=0")
    res = subprocess.run([str(exe), workdir], capture_output=True, text=True, env=env, timeout=600)
    if res.returncode != 0:
        raise RuntimeError(f"emulated kernel failed (exit {res.returncode}):\n{res.stderr[-6000:]}")


def run_tp(gen, steps: Sequence[Dict], X, Y, W, G=None, ws_bytes: int = 0):
    """Run TP steps; returns dict of outputs (Z or dX, dY, dW)."""
    dt = np.float32 if gen.T == "float" else np.float64
    extra = TP_EXTRA_UVW if gen.kind == "uvw" else TP_EXTRA_UVW_ROWS if gen.kind == "uvw_rows" else (TP_EXTRA_SHARED if gen.shared else "")
    main = TP_MAIN.replace("@EXTRA@", extra)
    exe = build(gen.render(prelude=emu_prelude(gen.T)), main)
    n = X.shape[0]
    with tempfile.TemporaryDirectory() as d:
        for name, arr in (("X", X), ("Y", Y), ("W", W)) + ((("G", G),) if G is not None else ()):
            np.ascontiguousarray(arr, dtype=dt).tofile(os.path.join(d, name + ".bin"))
        with open(os.path.join(d, "job.txt"), "w") as f:
            f.write(f"{n} {gen.D1} {gen.D2} {gen.D3} {W.shape[-1]} {W.size} {ws_bytes} {int(G is not None)}\n")
            for s in steps:
                f.write(f"{s['kernel']} {s['num_threads']} {grid_of(s, n, 0)} {s.get('grid_y', 1)}\n")
        _run(exe, d)
        out = {}
        out["Z"] = np.fromfile(os.path.join(d, "Z.bin"), dtype=dt).reshape(n, gen.D3)
        out["Xg"] = np.fromfile(os.path.join(d, "Xg.bin"), dtype=dt).reshape(n, gen.D1)
        out["Yg"] = np.fromfile(os.path.join(d, "Yg.bin"), dtype=dt).reshape(n, gen.D2)
        out["Wg"] = np.fromfile(os.path.join(d, "Wg.bin"), dtype=dt).reshape(W.shape)
    return out


def run_conv(gen, steps: Sequence[Dict], X, Y, W, rows, cols, G=None, tperm=None, ws_bytes: int = 0):
    dt = np.float32 if gen.T == "float" else np.float64
    extra = ""
    det = None
    if gen.kind == "conv_det":
        extra += CONV_EXTRA_DET
        det = gen
    elif hasattr(gen, "fwd"):
        extra += CONV_EXTRA_SORTED
        if gen.grouped_backward:
            extra += CONV_EXTRA_GROUPED_BWD
            if gen.recv_backward:
                extra += CONV_EXTRA_GROUPED_BWD.replace("_backward", "_recv")
            det = gen.bwd
    fdet = gen if gen.kind == "conv_det" else getattr(gen, "fwd", None)
    if fdet is not None:
        for k in fdet.forward_kernels()[1:]:
            extra += f'        else if (k == "{k[0]}") FWD_CALL({k[0]});\n'
    if det is not None:
        if det.ordered_backward:
            extra += CONV_EXTRA_ORDER
        for k in det.backward_kernel_sources()[1:]:
            extra += f'        else if (k == "{k["name"]}") BWD_CALL({k["name"]});\n'
        if det.dy_slots > 1:
            extra += CONV_EXTRA_DYRED
    exe = build(gen.render(prelude=emu_prelude(gen.T)), CONV_MAIN.replace("@EXTRA@", extra))
    nodes, nnz = X.shape[0], rows.shape[0]
    with tempfile.TemporaryDirectory() as d:
        for name, arr in (("X", X), ("Y", Y), ("W", W)) + ((("G", G),) if G is not None else ()):
            np.ascontiguousarray(arr, dtype=dt).tofile(os.path.join(d, name + ".bin"))
        np.ascontiguousarray(rows, dtype=np.int64).tofile(os.path.join(d, "rows.bin"))
        np.ascontiguousarray(cols, dtype=np.int64).tofile(os.path.join(d, "cols.bin"))
        if tperm is not None:
            np.ascontiguousarray(tperm, dtype=np.int64).tofile(os.path.join(d, "tperm.bin"))
        with open(os.path.join(d, "job.txt"), "w") as f:
            f.write(f"{nnz} {nodes} {gen.D1} {gen.D2} {gen.D3} {gen.WN} {ws_bytes} {int(G is not None)} {int(tperm is not None)}\n")
            for s in steps:
                f.write(f"{s['kernel']} {s['num_threads']} {grid_of(s, nnz, nodes)} {s.get('grid_y', 1)}\n")
        _run(exe, d)
        out = {}
        out["Z"] = np.fromfile(os.path.join(d, "Z.bin"), dtype=dt).reshape(nodes, gen.D3)
        out["Xg"] = np.fromfile(os.path.join(d, "Xg.bin"), dtype=dt).reshape(nodes, gen.D1)
        out["Yg"] = np.fromfile(os.path.join(d, "Yg.bin"), dtype=dt).reshape(nnz, gen.D2)
        out["Wg"] = np.fromfile(os.path.join(d, "Wg.bin"), dtype=dt).reshape(nnz, gen.WN)
    return out
