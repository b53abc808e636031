// C-ABI runtime for the gfx950 tensor-product / fused-convolution kernels.
//
// Host-only code: hipRTC compilation, code-object loading, launches on the caller's stream,
// device properties, an event timer and a small device-buffer helper.  The kernels themselves
// are generated as HIP source by the Python kernel generator and arrive here as text
// (oeq_compile) or as code objects (oeq_*_create).  See include/oeq_hip.h for the contract and
// the reference interfaces each entry point replaces.
#include "../../include/oeq_hip.h"

#include <hip/hip_runtime.h>
#include <hip/hiprtc.h>

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

// Scratch of oeq_conv_forward_noalloc: device memory that exists from the moment the library is
// loaded, one copy per GPU.  Host code never uses this name as an address; it asks the runtime for
// the array's device address once per device (noalloc_scratch) and passes that to the kernels.
static __device__ __align__(256) unsigned char oeq_noalloc_scratch[OEQ_NOALLOC_SCRATCH_BYTES];

namespace {

thread_local std::string g_error;

int fail(const char* fmt, ...) {
    char buf[2048];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_error = buf;
    return 1;
}

#define OEQ_HIP_CHECK(expr)                                                                   \
    do {                                                                                      \
        hipError_t _e = (expr);                                                               \
        if (_e != hipSuccess)                                                                 \
            return fail("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), __FILE__, __LINE__); \
    } while (0)

struct Step {
    oeq_step desc;
    hipFunction_t fn;
};

struct Module {
    hipModule_t mod = nullptr;
    ~Module() {
        if (mod) (void)hipModuleUnload(mod);
    }
};

int load_steps(Module& m, const void* code, size_t code_size, const oeq_step* steps, int n,
               std::vector<Step>& out) {
    (void)code_size;
    if (!m.mod) OEQ_HIP_CHECK(hipModuleLoadData(&m.mod, code));
    for (int i = 0; i < n; ++i) {
        Step s;
        s.desc = steps[i];
        s.desc.kernel[sizeof(s.desc.kernel) - 1] = 0;
        if (s.desc.num_threads == 0 || s.desc.num_threads > 1024)
            return fail("step %d (%s): bad workgroup size %u", i, s.desc.kernel, s.desc.num_threads);
        if (s.desc.grid_kind > OEQ_GRID_PER_NODE_AND_PIECE)
            return fail("step %d (%s): unknown grid rule %u", i, s.desc.kernel, s.desc.grid_kind);
        if (s.desc.grid_kind != OEQ_GRID_FIXED && s.desc.work_per_block == 0)
            return fail("step %d (%s): work_per_block must be > 0", i, s.desc.kernel);
        if (s.desc.grid_kind == OEQ_GRID_FIXED && s.desc.num_blocks == 0)
            return fail("step %d (%s): fixed grid of 0 blocks", i, s.desc.kernel);
        hipError_t e = hipModuleGetFunction(&s.fn, m.mod, s.desc.kernel);
        if (e != hipSuccess)
            return fail("kernel '%s' not found in code object: %s", s.desc.kernel, hipGetErrorString(e));
        if (s.desc.smem > 64 * 1024) {
            // raise the dynamic-LDS ceiling above the 64 KB default (160 KB per workgroup on gfx950)
            e = hipFuncSetAttribute(reinterpret_cast<const void*>(s.fn),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)s.desc.smem);
            if (e != hipSuccess) (void)hipGetLastError();  // not fatal: the launch reports a real failure
        }
        out.push_back(s);
    }
    return 0;
}

// Edges per piece of a long node's edge list: the kernels compute the same number from nnz and node_count.
uint64_t piece_edges(uint64_t factor, uint64_t rows, uint64_t nodes) {
    const uint64_t mean = nodes ? (rows + nodes - 1) / nodes : 0;
    const uint64_t t = factor * mean;
    return t < OEQ_PIECE_MIN_EDGES ? OEQ_PIECE_MIN_EDGES : t;
}

uint64_t grid_of(const oeq_step& d, uint64_t rows, uint64_t nodes, bool pieces) {
    if (d.grid_kind == OEQ_GRID_FIXED) return d.num_blocks;
    if (d.grid_kind == OEQ_GRID_PER_NODE_AND_PIECE) {
        // one workgroup per node, then two per tile of the edge list (the piece of a long node that ends
        // in the tile and the piece of one that begins in it); num_blocks holds the long-node factor
        uint64_t g = (nodes + d.work_per_block - 1) / d.work_per_block;
        if (pieces && d.num_blocks != 0 && rows > 0 && nodes > 0) {
            const uint64_t t = piece_edges(d.num_blocks, rows, nodes);
            g += 2 * ((rows + t - 1) / t);
        }
        return g;
    }
    uint64_t work = (d.grid_kind == OEQ_GRID_PER_ROW) ? rows : nodes;
    uint64_t g = (work + d.work_per_block - 1) / d.work_per_block;
    if (d.num_blocks != 0 && g > d.num_blocks) g = d.num_blocks;
    return g;
}

int launch(const Step& s, uint64_t rows, uint64_t nodes, void** args, void* stream, bool pieces = true) {
    uint64_t g = grid_of(s.desc, rows, nodes, pieces);
    if (g == 0) return 0;
    if (g > 0x7fffffffull) return fail("grid of %llu workgroups is too large", (unsigned long long)g);
    const unsigned gy = s.desc.grid_y ? s.desc.grid_y : 1u;
    if (gy > 65535u) return fail("grid_y of %u is too large", gy);
    OEQ_HIP_CHECK(hipModuleLaunchKernel(s.fn, (unsigned)g, gy, 1, s.desc.num_threads, 1, 1, s.desc.smem,
                                        (hipStream_t)stream, args, nullptr));
    return 0;
}

// Rejects a NULL workspace / transpose permutation that a step of the plan would dereference.
int check_pointers(const std::vector<Step>& steps, const void* workspace, const void* tperm, const char* what) {
    for (auto& s : steps) {
        if ((s.desc.flags & OEQ_STEP_NEEDS_WORKSPACE) && !workspace)
            return fail("%s: kernel '%s' needs a workspace, but the workspace pointer is NULL", what, s.desc.kernel);
        if ((s.desc.flags & OEQ_STEP_NEEDS_TPERM) && !tperm)
            return fail("%s: kernel '%s' reads the transpose permutation, but that pointer is NULL", what, s.desc.kernel);
    }
    return 0;
}

}  // namespace

struct oeq_tp {
    Module mod;
    std::vector<Step> fwd, bwd;
};
struct oeq_conv {
    Module mod;
    std::vector<Step> fwd, bwd;
    // bytes of workspace the forward steps use when long nodes are not cut into pieces:
    // fixed + per_node * node_count + per_edge * nnz (oeq_conv_set_forward_workspace)
    uint64_t ws_fixed = 0, ws_per_node = 16, ws_per_edge = 8;
    bool ws_model_set = false;
};
struct oeq_module {
    Module mod;
};
struct oeq_timer {
    hipEvent_t start = nullptr, stop = nullptr;
    void* flush = nullptr;
    size_t flush_bytes = 0;
};

extern "C" {

const char* oeq_last_error(void) { return g_error.c_str(); }

int oeq_device_count(int* count) {
    if (!count) return fail("null argument");
    hipError_t e = hipGetDeviceCount(count);
    if (e != hipSuccess) {
        *count = 0;
        (void)hipGetLastError();
    }
    return 0;
}

int oeq_device_props(int device, oeq_device_prop* out) {
    if (!out) return fail("null argument");
    hipDeviceProp_t p;
    OEQ_HIP_CHECK(hipGetDeviceProperties(&p, device));
    memset(out, 0, sizeof(*out));
    snprintf(out->name, sizeof(out->name), "%s", p.name);
    snprintf(out->arch, sizeof(out->arch), "%s", p.gcnArchName);
    if (char* colon = strchr(out->arch, ':')) *colon = 0;
    out->warpsize = p.warpSize;
    out->major = p.major;
    out->minor = p.minor;
    out->multiprocessorCount = p.multiProcessorCount;
    out->maxSharedMemPerBlock = (int64_t)p.sharedMemPerBlock;
    int optin = 0;
    if (hipDeviceGetAttribute(&optin, hipDeviceAttributeMaxSharedMemoryPerBlock, device) == hipSuccess &&
        optin > out->maxSharedMemPerBlock)
        out->maxSharedMemPerBlock = optin;
    out->totalGlobalMem = (int64_t)p.totalGlobalMem;
    out->clockRateKHz = p.clockRate;
    out->memoryClockRateKHz = p.memoryClockRate;
    out->memoryBusWidth = p.memoryBusWidth;
    out->l2CacheSize = p.l2CacheSize;
    return 0;
}

int oeq_hiprtc_version(int* major, int* minor) {
    if (!major || !minor) return fail("null argument");
    hiprtcResult r = hiprtcVersion(major, minor);
    if (r != HIPRTC_SUCCESS) return fail("hiprtcVersion: %s", hiprtcGetErrorString(r));
    return 0;
}

int oeq_compile(const char* source, const char* arch, const char* const* options, int n_options,
                void** code, size_t* code_size) {
    if (!source || !code || !code_size) return fail("null argument");
    *code = nullptr;
    *code_size = 0;
    hiprtcProgram prog;
    hiprtcResult r = hiprtcCreateProgram(&prog, source, "oeq_kernel.hip", 0, nullptr, nullptr);
    if (r != HIPRTC_SUCCESS) return fail("hiprtcCreateProgram: %s", hiprtcGetErrorString(r));
    std::vector<std::string> store;
    if (arch && arch[0]) store.push_back(std::string("--offload-arch=") + arch);
    for (int i = 0; i < n_options; ++i) store.push_back(options[i]);
    std::vector<const char*> opts;
    for (auto& s : store) opts.push_back(s.c_str());
    r = hiprtcCompileProgram(prog, (int)opts.size(), opts.data());
    if (r != HIPRTC_SUCCESS) {
        size_t n = 0;
        hiprtcGetProgramLogSize(prog, &n);
        std::string log(n, '\0');
        if (n) hiprtcGetProgramLog(prog, &log[0]);
        hiprtcDestroyProgram(&prog);
        g_error = std::string("hipRTC compilation failed: ") + hiprtcGetErrorString(r) + "\n" + log;
        return 2;
    }
    size_t n = 0;
    r = hiprtcGetCodeSize(prog, &n);
    if (r != HIPRTC_SUCCESS || n == 0) {
        hiprtcDestroyProgram(&prog);
        return fail("hiprtcGetCodeSize: %s", hiprtcGetErrorString(r));
    }
    void* buf = malloc(n);
    if (!buf) {
        hiprtcDestroyProgram(&prog);
        return fail("out of host memory");
    }
    r = hiprtcGetCode(prog, (char*)buf);
    hiprtcDestroyProgram(&prog);
    if (r != HIPRTC_SUCCESS) {
        free(buf);
        return fail("hiprtcGetCode: %s", hiprtcGetErrorString(r));
    }
    *code = buf;
    *code_size = n;
    return 0;
}

void oeq_free(void* p) { free(p); }

// ---------------------------------------------------------------- batch TP
int oeq_tp_create(const void* code, size_t code_size, const oeq_step* fs, int nf, const oeq_step* bs,
                  int nb, oeq_tp** out) {
    if (!code || !out || nf < 0 || nb < 0 || (nf && !fs) || (nb && !bs)) return fail("bad argument");
    oeq_tp* tp = new oeq_tp();
    if (load_steps(tp->mod, code, code_size, fs, nf, tp->fwd) ||
        load_steps(tp->mod, code, code_size, bs, nb, tp->bwd)) {
        delete tp;
        return 1;
    }
    *out = tp;
    return 0;
}

void oeq_tp_destroy(oeq_tp* tp) { delete tp; }

int oeq_tp_forward(oeq_tp* tp, uint64_t n, const void* L1, const void* L2, void* L3, const void* W,
                   void* workspace, void* stream) {
    if (!tp) return fail("null handle");
    if (tp->fwd.empty()) return fail("this operator was built without a forward plan");
    if (n > 0 && check_pointers(tp->fwd, workspace, (const void*)1, "forward")) return 1;
    void* args[] = {&n, &L1, &L2, &L3, &W, &workspace};
    for (auto& s : tp->fwd)
        if (launch(s, n, 0, args, stream)) return 1;
    return 0;
}

int oeq_tp_backward(oeq_tp* tp, uint64_t n, const void* L1, void* L1g, const void* L2, void* L2g,
                    const void* W, void* Wg, const void* L3g, void* workspace, void* stream) {
    if (!tp) return fail("null handle");
    if (tp->bwd.empty()) return fail("this operator was built without a backward plan");
    if (n > 0 && check_pointers(tp->bwd, workspace, (const void*)1, "backward")) return 1;
    void* args[] = {&n, &L1, &L1g, &L2, &L2g, &W, &Wg, &L3g, &workspace};
    for (auto& s : tp->bwd)
        if (launch(s, n, 0, args, stream)) return 1;
    return 0;
}

// ------------------------------------------------------------------- conv
static int noalloc_scratch(void** out);

int oeq_conv_create(const void* code, size_t code_size, const oeq_step* fs, int nf, const oeq_step* bs,
                    int nb, oeq_conv** out) {
    if (!code || !out || nf < 0 || nb < 0 || (nf && !fs) || (nb && !bs)) return fail("bad argument");
    oeq_conv* c = new oeq_conv();
    if (load_steps(c->mod, code, code_size, fs, nf, c->fwd) ||
        load_steps(c->mod, code, code_size, bs, nb, c->bwd)) {
        delete c;
        return 1;
    }
    // Set-up is where the static scratch of oeq_conv_forward_noalloc is looked up on this device (the runtime
    // materialises the array on first use): the entry point itself must not be the first to touch it, it may
    // run under stream capture.  A failure here is reported by that entry point, not by this one.
    void* scratch = nullptr;
    if (noalloc_scratch(&scratch)) g_error.clear();
    *out = c;
    return 0;
}

void oeq_conv_destroy(oeq_conv* c) { delete c; }

// A step is skipped when the call says that the state it would build is already in the workspace.
static bool skipped(const oeq_step& d, uint32_t call_flags) {
    if ((call_flags & OEQ_CALL_PREPARED) && (d.flags & OEQ_STEP_GRAPH_PREP)) return true;
    if ((call_flags & OEQ_CALL_COUNTERS_ZERO) && (d.flags & OEQ_STEP_COUNTER_CLEAR)) return true;
    return false;
}

static int conv_forward(oeq_conv* c, const void* L1, const void* L2, const void* W, void* L3,
                        const void* rows, const void* cols, uint64_t nnz, uint64_t node_count,
                        void* workspace, const void* tperm, void* stream, uint32_t call_flags, bool pieces = true) {
    if (!c) return fail("null handle");
    if (c->fwd.empty()) return fail("this operator was built without a forward plan");
    if (nnz > 0 && node_count == 0) return fail("convolution called with %llu edges but no nodes", (unsigned long long)nnz);
    if (nnz > 0 && (!rows || !cols)) return fail("forward: rows / cols are NULL");
    // (an empty edge list has no transpose permutation to read: a NULL pointer is what an empty tensor gives)
    if ((nnz > 0 || node_count > 0) && check_pointers(c->fwd, workspace, nnz > 0 ? tperm : (const void*)1, "forward")) return 1;
    if (call_flags & ~(uint32_t)(OEQ_CALL_PREPARED | OEQ_CALL_COUNTERS_ZERO)) return fail("forward: unknown call flags 0x%x", call_flags);
    void* args[] = {&L1, &L2, &W, &L3, &rows, &cols, &nnz, &node_count, &workspace, &tperm};
    for (auto& s : c->fwd) {
        if (skipped(s.desc, call_flags)) continue;
        if (launch(s, nnz, node_count, args, stream, pieces)) return 1;
    }
    return 0;
}

static int conv_backward(oeq_conv* c, const void* L1, void* L1g, const void* L2, void* L2g, const void* W,
                         void* Wg, const void* L3g, const void* rows, const void* cols, uint64_t nnz,
                         uint64_t node_count, void* workspace, const void* tperm, void* stream, uint32_t call_flags) {
    if (!c) return fail("null handle");
    if (c->bwd.empty()) return fail("this operator was built without a backward plan");
    if (nnz > 0 && node_count == 0) return fail("convolution called with %llu edges but no nodes", (unsigned long long)nnz);
    if (nnz > 0 && (!rows || !cols)) return fail("backward: rows / cols are NULL");
    // (an empty edge list has no transpose permutation to read: a NULL pointer is what an empty tensor gives)
    if ((nnz > 0 || node_count > 0) && check_pointers(c->bwd, workspace, nnz > 0 ? tperm : (const void*)1, "backward")) return 1;
    if (call_flags & ~(uint32_t)(OEQ_CALL_PREPARED | OEQ_CALL_COUNTERS_ZERO)) return fail("backward: unknown call flags 0x%x", call_flags);
    void* args[] = {&L1, &L1g, &L2, &L2g, &W, &Wg, &L3g, &rows, &cols, &nnz, &node_count, &workspace, &tperm};
    for (auto& s : c->bwd) {
        if (skipped(s.desc, call_flags)) continue;
        if (launch(s, nnz, node_count, args, stream)) return 1;
    }
    return 0;
}

int oeq_conv_forward(oeq_conv* c, const void* L1, const void* L2, const void* W, void* L3,
                     const void* rows, const void* cols, uint64_t nnz, uint64_t node_count,
                     void* workspace, const void* tperm, void* stream) {
    return conv_forward(c, L1, L2, W, L3, rows, cols, nnz, node_count, workspace, tperm, stream, 0);
}

int oeq_conv_forward_ex(oeq_conv* c, const void* L1, const void* L2, const void* W, void* L3,
                        const void* rows, const void* cols, uint64_t nnz, uint64_t node_count,
                        void* workspace, const void* tperm, void* stream, uint32_t call_flags) {
    return conv_forward(c, L1, L2, W, L3, rows, cols, nnz, node_count, workspace, tperm, stream, call_flags);
}

int oeq_conv_backward(oeq_conv* c, const void* L1, void* L1g, const void* L2, void* L2g, const void* W,
                      void* Wg, const void* L3g, const void* rows, const void* cols, uint64_t nnz,
                      uint64_t node_count, void* workspace, const void* tperm, void* stream) {
    return conv_backward(c, L1, L1g, L2, L2g, W, Wg, L3g, rows, cols, nnz, node_count, workspace, tperm, stream, 0);
}

int oeq_conv_backward_ex(oeq_conv* c, const void* L1, void* L1g, const void* L2, void* L2g, const void* W,
                         void* Wg, const void* L3g, const void* rows, const void* cols, uint64_t nnz,
                         uint64_t node_count, void* workspace, const void* tperm, void* stream, uint32_t call_flags) {
    return conv_backward(c, L1, L1g, L2, L2g, W, Wg, L3g, rows, cols, nnz, node_count, workspace, tperm, stream, call_flags);
}

int oeq_conv_set_forward_workspace(oeq_conv* c, uint64_t fixed_bytes, uint64_t bytes_per_node, uint64_t bytes_per_edge) {
    if (!c) return fail("null handle");
    c->ws_fixed = fixed_bytes;
    c->ws_per_node = bytes_per_node;
    c->ws_per_edge = bytes_per_edge;
    c->ws_model_set = true;
    return 0;
}

// Device address of this GPU's copy of oeq_noalloc_scratch, looked up on first use per device.
static int noalloc_scratch(void** out) {
    enum { MAX_DEVICES = 64 };
    static void* ptrs[MAX_DEVICES] = {nullptr};
    static std::mutex mu;
    int dev = -1;
    OEQ_HIP_CHECK(hipGetDevice(&dev));
    if (dev < 0 || dev >= MAX_DEVICES) return fail("device ordinal %d is out of range", dev);
    std::lock_guard<std::mutex> lock(mu);
    if (!ptrs[dev]) {
        void* p = nullptr;
        OEQ_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(oeq_noalloc_scratch)));
        if (!p) return fail("hipGetSymbolAddress returned a null address for the static scratch");
        ptrs[dev] = p;
    }
    *out = ptrs[dev];
    return 0;
}

int oeq_conv_forward_noalloc(oeq_conv* c, const void* L1, const void* L2, const void* W, void* L3,
                             const void* rows, const void* cols, uint64_t nnz, uint64_t node_count,
                             const void* tperm, void* stream) {
    if (!c) return fail("null handle");
    if (!c->ws_model_set)
        return fail("oeq_conv_forward_noalloc: the operator's forward workspace size is unknown "
                    "(call oeq_conv_set_forward_workspace after oeq_conv_create)");
    if (nnz > (1ull << 40) || node_count > (1ull << 40)) return fail("graph too large");
    // what the forward steps of this operator's plan use with every node walked by one wavefront
    const uint64_t need = c->ws_fixed + c->ws_per_node * node_count + c->ws_per_edge * nnz;
    if (need > (uint64_t)OEQ_NOALLOC_SCRATCH_BYTES)
        return fail("oeq_conv_forward_noalloc: %llu edges and %llu nodes need %llu bytes of scratch, the static "
                    "scratch holds %llu (use oeq_conv_forward with a caller-owned workspace)",
                    (unsigned long long)nnz, (unsigned long long)node_count, (unsigned long long)need,
                    (unsigned long long)OEQ_NOALLOC_SCRATCH_BYTES);
    void* scratch = nullptr;
    if (noalloc_scratch(&scratch)) return 1;
    return conv_forward(c, L1, L2, W, L3, rows, cols, nnz, node_count, scratch, tperm, stream, 0, /*pieces=*/false);
}

// ---------------------------------------------------------- generic module
int oeq_module_load(const void* code, size_t code_size, oeq_module** out) {
    (void)code_size;
    if (!code || !out) return fail("null argument");
    oeq_module* m = new oeq_module();
    hipError_t e = hipModuleLoadData(&m->mod.mod, code);
    if (e != hipSuccess) {
        delete m;
        return fail("hipModuleLoadData: %s", hipGetErrorString(e));
    }
    *out = m;
    return 0;
}

void oeq_module_unload(oeq_module* m) { delete m; }

int oeq_module_launch(oeq_module* m, const char* kernel, uint32_t grid, uint32_t block, uint32_t smem,
                      void* stream, void** args) {
    if (!m || !kernel) return fail("null argument");
    if (grid == 0) return 0;
    hipFunction_t fn;
    hipError_t e = hipModuleGetFunction(&fn, m->mod.mod, kernel);
    if (e != hipSuccess) return fail("kernel '%s' not found: %s", kernel, hipGetErrorString(e));
    OEQ_HIP_CHECK(hipModuleLaunchKernel(fn, grid, 1, 1, block, 1, 1, smem, (hipStream_t)stream, args, nullptr));
    return 0;
}

// ------------------------------------------------------------------ timer
int oeq_timer_create(oeq_timer** out) {
    if (!out) return fail("null argument");
    oeq_timer* t = new oeq_timer();
    hipError_t e = hipEventCreate(&t->start);
    if (e == hipSuccess) e = hipEventCreate(&t->stop);
    if (e != hipSuccess) {
        delete t;
        return fail("hipEventCreate: %s", hipGetErrorString(e));
    }
    *out = t;
    return 0;
}

void oeq_timer_destroy(oeq_timer* t) {
    if (!t) return;
    if (t->start) (void)hipEventDestroy(t->start);
    if (t->stop) (void)hipEventDestroy(t->stop);
    if (t->flush) (void)hipFree(t->flush);
    delete t;
}

int oeq_timer_start(oeq_timer* t, void* stream) {
    if (!t) return fail("null handle");
    OEQ_HIP_CHECK(hipEventRecord(t->start, (hipStream_t)stream));
    return 0;
}

int oeq_timer_stop(oeq_timer* t, void* stream, float* ms) {
    if (!t || !ms) return fail("null argument");
    OEQ_HIP_CHECK(hipEventRecord(t->stop, (hipStream_t)stream));
    OEQ_HIP_CHECK(hipEventSynchronize(t->stop));
    OEQ_HIP_CHECK(hipEventElapsedTime(ms, t->start, t->stop));
    return 0;
}

int oeq_timer_clear_cache(oeq_timer* t, void* stream) {
    if (!t) return fail("null handle");
    if (!t->flush) {
        t->flush_bytes = (size_t)512 << 20;
        OEQ_HIP_CHECK(hipMalloc(&t->flush, t->flush_bytes));
    }
    OEQ_HIP_CHECK(hipMemsetAsync(t->flush, 42, t->flush_bytes, (hipStream_t)stream));
    return 0;
}

// ---------------------------------------------------------------- buffers
int oeq_buffer_alloc(size_t bytes, void** dptr) {
    if (!dptr) return fail("null argument");
    OEQ_HIP_CHECK(hipMalloc(dptr, bytes ? bytes : 1));
    return 0;
}
int oeq_buffer_free(void* dptr) {
    OEQ_HIP_CHECK(hipFree(dptr));
    return 0;
}
int oeq_buffer_h2d(void* dptr, const void* host, size_t bytes) {
    OEQ_HIP_CHECK(hipMemcpy(dptr, host, bytes, hipMemcpyHostToDevice));
    return 0;
}
int oeq_buffer_d2h(void* host, const void* dptr, size_t bytes) {
    OEQ_HIP_CHECK(hipMemcpy(host, dptr, bytes, hipMemcpyDeviceToHost));
    return 0;
}
int oeq_buffer_zero(void* dptr, size_t bytes, void* stream) {
    OEQ_HIP_CHECK(hipMemsetAsync(dptr, 0, bytes, (hipStream_t)stream));
    return 0;
}
int oeq_stream_synchronize(void* stream) {
    OEQ_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}

}  // extern "C"
