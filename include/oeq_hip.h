/*
 * oeq_hip.h - C ABI of the MI355X (gfx950) tensor-product / fused-convolution runtime.
 *
 * This is the boundary a host language binds to.  It replaces the pybind11 module
 * `kernel_wrapper` of the reference (openequivariance/extension/kernel_wrapper.cpp:23-66):
 * plain pointers and sizes only, no C++ or torch types.  Every function returns 0 on
 * success and a non-zero code on failure; oeq_last_error() then describes the failure
 * (the reference prints and calls exit(1): extension/util/backend_hip.hpp:11-41).
 *
 * Device pointers are passed as `void*` (the reference passes them as uint64_t:
 * extension/tensorproducts.hpp:14-22).  All launches are asynchronous on the caller's
 * stream (`hipStream_t` passed as void*; the reference uses the NULL stream:
 * extension/util/backend_hip.hpp:131).  The library never allocates tensors; workspaces
 * are owned by the caller.
 */
#ifndef OEQ_HIP_H
#define OEQ_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---------------------------------------------------------------- errors */
/* Thread-local description of the last failure in this thread. */
const char* oeq_last_error(void);

/* ------------------------------------------------------- device properties */
/* Replaces DeviceProp (extension/util/backend_hip.hpp:101-121). */
typedef struct {
    char     name[256];
    char     arch[64];              /* gcnArchName without feature suffixes, e.g. "gfx950" */
    int32_t  warpsize;
    int32_t  major, minor;
    int32_t  multiprocessorCount;   /* compute units */
    int64_t  maxSharedMemPerBlock;  /* LDS bytes per workgroup */
    int64_t  totalGlobalMem;
    int32_t  clockRateKHz;
    int32_t  memoryClockRateKHz;
    int32_t  memoryBusWidth;
    int32_t  l2CacheSize;
} oeq_device_prop;
int oeq_device_props(int device, oeq_device_prop* out);
int oeq_device_count(int* count);

/* ------------------------------------------------------------ JIT compile */
/* hipRTC compile of one HIP translation unit to a gfx code object.  Works without a GPU
 * when `arch` is given.  `options` are extra compiler flags.  On success *code is a
 * malloc'ed buffer to release with oeq_free(); on a compile error the compiler log is in
 * oeq_last_error().  Replaces HIPJITKernel::compile
 * (extension/util/backend_hip.hpp:167-247); kernels are looked up by their extern "C"
 * names, so no lowered-name bookkeeping is needed. */
int  oeq_compile(const char* source, const char* arch, const char* const* options, int n_options,
                 void** code, size_t* code_size);
void oeq_free(void* p);
/* Version string of the hipRTC in use (part of the code-object cache key). */
int  oeq_hiprtc_version(int* major, int* minor);

/* -------------------------------------------------------------- launch plan */
/* One kernel launch of an operator.  Replaces KernelLaunchConfig
 * (extension/util/backend_hip.hpp:123-133) and adds how the grid follows the work size. */
/* OEQ_GRID_PER_NODE_AND_PIECE: one workgroup per `work_per_block` nodes followed by two per tile of
 * T = max(OEQ_PIECE_MIN_EDGES, num_blocks * ceil(nnz / node_count)) consecutive positions of the edge
 * list; `num_blocks` holds the long-node factor instead of a bound (0: no piece workgroups).  The
 * extra workgroups walk the pieces of nodes whose edge list is longer than T, so that a hub does not
 * serialise one wavefront (the reference deals the edge list to its warps in equal shares and repairs
 * the seams: templates/loop_unroll_conv_det.cuh:33-133). */
enum { OEQ_GRID_FIXED = 0, OEQ_GRID_PER_ROW = 1, OEQ_GRID_PER_NODE = 2, OEQ_GRID_PER_NODE_AND_PIECE = 3 };
#define OEQ_PIECE_MIN_EDGES 32u
/* What a step dereferences and what it is for.  A call whose plan holds a step with
 * OEQ_STEP_NEEDS_WORKSPACE (OEQ_STEP_NEEDS_TPERM) is rejected, before anything is launched, when the
 * workspace (transpose permutation) pointer is NULL; a call with nnz == 0 has no transpose permutation
 * to read and may pass NULL for it.  OEQ_STEP_GRAPH_PREP marks the steps that only
 * derive graph structure (CSR pointers, position lists, node order) from rows / cols /
 * transpose_perm into the workspace: a call with OEQ_CALL_PREPARED skips them.  OEQ_STEP_COUNTER_CLEAR
 * marks a step that only zeroes counters in the workspace which the operator's later steps leave
 * zeroed again: a call with OEQ_CALL_COUNTERS_ZERO skips it. */
enum { OEQ_STEP_NEEDS_WORKSPACE = 1, OEQ_STEP_NEEDS_TPERM = 2, OEQ_STEP_GRAPH_PREP = 4, OEQ_STEP_COUNTER_CLEAR = 8 };
typedef struct {
    char     kernel[64];        /* extern "C" symbol in the code object */
    uint32_t num_threads;       /* workgroup size */
    uint32_t smem;              /* dynamic LDS bytes */
    uint32_t grid_kind;         /* OEQ_GRID_* */
    uint32_t work_per_block;    /* rows (edges) or nodes handled by one workgroup */
    uint32_t num_blocks;        /* OEQ_GRID_FIXED: the grid; otherwise an upper bound (0 = none) */
    uint32_t grid_y;            /* second grid dimension (0 or 1 = none), e.g. one 64-channel chunk each */
    uint32_t warp_size;         /* informational: 64 */
    uint32_t flags;             /* OEQ_STEP_* */
} oeq_step;

/* ------------------------------------------------------ batch tensor product */
/* Replaces JITTPImpl (extension/tensorproducts.hpp:50-98).  `code` is a code object from
 * oeq_compile.  Every forward step is launched with the argument list
 *   (uint64_t n, const void* L1, const void* L2, void* L3, const void* W, void* workspace)
 * and every backward step with
 *   (uint64_t n, const void* L1, void* L1g, const void* L2, void* L2g,
 *    const void* W, void* Wg, const void* L3g, void* workspace). */
typedef struct oeq_tp oeq_tp;
int  oeq_tp_create(const void* code, size_t code_size,
                   const oeq_step* forward_steps, int n_forward,
                   const oeq_step* backward_steps, int n_backward, oeq_tp** out);
void oeq_tp_destroy(oeq_tp* tp);
/* exec_tensor_product (extension/tensorproducts.hpp:76-85) */
int  oeq_tp_forward(oeq_tp* tp, uint64_t num_products, const void* L1_in, const void* L2_in,
                    void* L3_out, const void* weights, void* workspace, void* stream);
/* backward (extension/tensorproducts.hpp:87-95) */
int  oeq_tp_backward(oeq_tp* tp, uint64_t num_products, const void* L1_in, void* L1_grad,
                     const void* L2_in, void* L2_grad, const void* weights, void* weights_grad,
                     const void* L3_grad, void* workspace, void* stream);

/* -------------------------------------------------------- fused convolution */
/* Replaces JITConvImpl (extension/convolution.hpp:94-176).  rows = receivers (scatter
 * target), cols = senders (gather source), both int64[nnz].  Forward steps receive
 *   (const void* L1, const void* L2, const void* W, void* L3, const int64_t* rows,
 *    const int64_t* cols, uint64_t nnz, uint64_t node_count, void* workspace,
 *    const int64_t* transpose_perm)
 * and backward steps
 *   (const void* L1, void* L1g, const void* L2, void* L2g, const void* W, void* Wg,
 *    const void* L3g, const int64_t* rows, const int64_t* cols, uint64_t nnz,
 *    uint64_t node_count, void* workspace, const int64_t* transpose_perm).
 * The reference passes rows/cols/nnz/node_count as a by-value struct
 * (extension/convolution.hpp:87-92); they are flattened here. */
typedef struct oeq_conv oeq_conv;
int  oeq_conv_create(const void* code, size_t code_size,
                     const oeq_step* forward_steps, int n_forward,
                     const oeq_step* backward_steps, int n_backward, oeq_conv** out);
void oeq_conv_destroy(oeq_conv* conv);
/* exec_conv (extension/convolution.hpp:121-147) */
int  oeq_conv_forward(oeq_conv* conv, const void* L1_in, const void* L2_in, const void* weights,
                      void* L3_out, const void* rows, const void* cols, uint64_t nnz,
                      uint64_t node_count, void* workspace, const void* transpose_perm, void* stream);
/* backward (extension/convolution.hpp:149-173) */
int  oeq_conv_backward(oeq_conv* conv, const void* L1_in, void* L1_grad, const void* L2_in,
                       void* L2_grad, const void* weights, void* weights_grad, const void* L3_grad,
                       const void* rows, const void* cols, uint64_t nnz, uint64_t node_count,
                       void* workspace, const void* transpose_perm, void* stream);

/* The same two calls with what the caller knows about the workspace (OEQ_CALL_* flags, or 0).
 * OEQ_CALL_PREPARED: the workspace already holds this graph's preparation; the steps flagged
 * OEQ_STEP_GRAPH_PREP are skipped.  Valid only if the last forward (for _forward_ex) / backward (for
 * _backward_ex) call that used this workspace ran with the same rows, cols, transpose_perm contents,
 * nnz and node_count, and nothing else has written the workspace's preparation areas since (forward
 * and backward keep theirs in disjoint parts of the workspace).  A model calls one graph for the
 * forward, the backward and the seven launches of the double backward of every layer; the reference
 * allocates its workspace once and rebuilds nothing either
 * (implementations/convolution/ConvolutionBase.py:93-100).
 * OEQ_CALL_COUNTERS_ZERO: the counters that the operator keeps in the workspace are zero: the workspace
 * was zero-filled, or the last call that used it was a completed call of this operator with the same
 * node_count, and nothing else has written it since.  The steps flagged OEQ_STEP_COUNTER_CLEAR are
 * skipped (every call leaves its counters zeroed). */
enum { OEQ_CALL_PREPARED = 1, OEQ_CALL_COUNTERS_ZERO = 2 };
int  oeq_conv_forward_ex(oeq_conv* conv, const void* L1_in, const void* L2_in, const void* weights,
                         void* L3_out, const void* rows, const void* cols, uint64_t nnz,
                         uint64_t node_count, void* workspace, const void* transpose_perm, void* stream,
                         uint32_t call_flags);
int  oeq_conv_backward_ex(oeq_conv* conv, const void* L1_in, void* L1_grad, const void* L2_in,
                          void* L2_grad, const void* weights, void* weights_grad, const void* L3_grad,
                          const void* rows, const void* cols, uint64_t nnz, uint64_t node_count,
                          void* workspace, const void* transpose_perm, void* stream, uint32_t call_flags);

/* Workspace bytes the forward steps use when every node is walked by one wavefront (no pieces):
 * fixed_bytes + bytes_per_node * node_count + bytes_per_edge * nnz.  The host sets it from the plan it
 * built the operator with; oeq_conv_forward_noalloc checks graphs against it.  (The reference sizes
 * its workspace on the Python side as well: implementations/convolution/LoopUnrollConv.py:61-72.) */
int  oeq_conv_set_forward_workspace(oeq_conv* conv, uint64_t fixed_bytes, uint64_t bytes_per_node,
                                    uint64_t bytes_per_edge);

/* oeq_conv_forward for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * The workspace is a static device array of OEQ_NOALLOC_SCRATCH_BYTES inside the library (one copy
 * per GPU, held until the process ends); the call allocates and frees nothing.  The forward kernels
 * use what oeq_conv_set_forward_workspace declared (every node is walked by one wavefront here: the
 * pieces of long nodes would need partial rows beyond a static array); larger graphs are rejected
 * with an error.  All
 * calls on one GPU share the array: calls that overlap in time on one GPU (different streams or
 * threads) race on it, and a captured graph holding such a call must not replay concurrently with
 * another.  Inputs and outputs are the caller's, as in oeq_conv_forward. */
#define OEQ_NOALLOC_SCRATCH_BYTES (16u << 20)
int  oeq_conv_forward_noalloc(oeq_conv* conv, const void* L1_in, const void* L2_in, const void* weights,
                              void* L3_out, const void* rows, const void* cols, uint64_t nnz,
                              uint64_t node_count, const void* transpose_perm, void* stream);

/* ------------------------------------------------------------ generic module */
/* Thin access to a loaded code object, for callers that pack their own arguments
 * (HIPJITKernel::execute, extension/util/backend_hip.hpp:266-283). */
typedef struct oeq_module oeq_module;
int  oeq_module_load(const void* code, size_t code_size, oeq_module** out);
void oeq_module_unload(oeq_module* m);
int  oeq_module_launch(oeq_module* m, const char* kernel, uint32_t grid, uint32_t block,
                       uint32_t smem, void* stream, void** args);

/* -------------------------------------------------------------------- timer */
/* Replaces GPUTimer (extension/util/backend_hip.hpp:65-99): an event pair recorded on the
 * given stream, and a cache flush that overwrites a buffer larger than the 256 MB
 * Infinity Cache (the reference's 100 MB is sized for an A100's L2). */
typedef struct oeq_timer oeq_timer;
int  oeq_timer_create(oeq_timer** out);
void oeq_timer_destroy(oeq_timer* t);
int  oeq_timer_start(oeq_timer* t, void* stream);
int  oeq_timer_stop(oeq_timer* t, void* stream, float* elapsed_ms);   /* synchronises on the stop event */
int  oeq_timer_clear_cache(oeq_timer* t, void* stream);

/* ------------------------------------------------------------ device buffers */
/* Replaces DeviceBuffer (extension/util/buffer.hpp:8-45) for callers without torch. */
int  oeq_buffer_alloc(size_t bytes, void** dptr);
int  oeq_buffer_free(void* dptr);
int  oeq_buffer_h2d(void* dptr, const void* host, size_t bytes);
int  oeq_buffer_d2h(void* host, const void* dptr, size_t bytes);
int  oeq_buffer_zero(void* dptr, size_t bytes, void* stream);
int  oeq_stream_synchronize(void* stream);

#ifdef __cplusplus
}
#endif
#endif /* OEQ_HIP_H */
