"""ctypes binding of the C-ABI runtime (``csrc/liboeq_hip.so``, declared in ``include/oeq_hip.h``).

Python keeps only plumbing here: argument marshalling, the on-disk code-object
cache and error translation (a non-zero status becomes ``RuntimeError`` with
the library's message).  There is no fallback: if the shared object has not
been built, loading raises.
"""
from __future__ import annotations

import ctypes as C
import hashlib
import os
import pathlib
import threading
from typing import List, Optional, Sequence

from . import tunables

PKG_DIR = pathlib.Path(__file__).resolve().parent
LIB_PATH = PKG_DIR / "csrc" / "liboeq_hip.so"
CACHE_DIR = tunables.current.cache_dir
TARGET_ARCH = "gfx950"

GRID_FIXED, GRID_PER_ROW, GRID_PER_NODE, GRID_PER_NODE_AND_PIECE = 0, 1, 2, 3
STEP_NEEDS_WORKSPACE, STEP_NEEDS_TPERM, STEP_GRAPH_PREP, STEP_COUNTER_CLEAR = 1, 2, 4, 8
CALL_PREPARED, CALL_COUNTERS_ZERO = 1, 2
PIECE_MIN_EDGES = 32                     # OEQ_PIECE_MIN_EDGES
NOALLOC_SCRATCH_BYTES = 16 << 20        # OEQ_NOALLOC_SCRATCH_BYTES


class DeviceProp(C.Structure):
    """Mirror of ``oeq_device_prop`` (reference type: DeviceProp, backend_hip.hpp:101-121)."""
    _fields_ = [("name", C.c_char * 256), ("arch", C.c_char * 64), ("warpsize", C.c_int32),
                ("major", C.c_int32), ("minor", C.c_int32), ("multiprocessorCount", C.c_int32),
                ("maxSharedMemPerBlock", C.c_int64), ("totalGlobalMem", C.c_int64),
                ("clockRateKHz", C.c_int32), ("memoryClockRateKHz", C.c_int32),
                ("memoryBusWidth", C.c_int32), ("l2CacheSize", C.c_int32)]


class Step(C.Structure):
    """Mirror of ``oeq_step``: one kernel launch of an operator."""
    _fields_ = [("kernel", C.c_char * 64), ("num_threads", C.c_uint32), ("smem", C.c_uint32),
                ("grid_kind", C.c_uint32), ("work_per_block", C.c_uint32), ("num_blocks", C.c_uint32),
                ("grid_y", C.c_uint32), ("warp_size", C.c_uint32), ("flags", C.c_uint32)]

    @classmethod
    def make(cls, kernel: str, num_threads: int, smem: int = 0, grid_kind: int = GRID_PER_ROW,
             work_per_block: int = 1, num_blocks: int = 0, grid_y: int = 1, flags: int = 0) -> "Step":
        s = cls()
        s.kernel = kernel.encode()
        s.num_threads, s.smem, s.grid_kind = num_threads, smem, grid_kind
        s.work_per_block, s.num_blocks, s.grid_y, s.warp_size = work_per_block, num_blocks, grid_y, 64
        s.flags = flags
        return s


_lib = None
_lib_lock = threading.Lock()


def lib() -> C.CDLL:
    """Load the runtime library once.  torch is imported first so that the HIP runtime
    already mapped by torch is the one this library binds to."""
    global _lib
    if _lib is not None:
        return _lib
    with _lib_lock:
        if _lib is not None:
            return _lib
        if not LIB_PATH.exists():
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m openequivariance_amd.build_ext` "
                "(there is no CPU fallback)")
        try:
            import torch  # noqa: F401  (maps torch's libamdhip64 / libhiprtc first)
        except ImportError:
            pass
        L = C.CDLL(str(LIB_PATH))
        vp, u64, sz = C.c_void_p, C.c_uint64, C.c_size_t
        sig = {
            "oeq_last_error": (C.c_char_p, []),
            "oeq_device_props": (C.c_int, [C.c_int, C.POINTER(DeviceProp)]),
            "oeq_device_count": (C.c_int, [C.POINTER(C.c_int)]),
            "oeq_compile": (C.c_int, [C.c_char_p, C.c_char_p, C.POINTER(C.c_char_p), C.c_int,
                                      C.POINTER(vp), C.POINTER(sz)]),
            "oeq_free": (None, [vp]),
            "oeq_hiprtc_version": (C.c_int, [C.POINTER(C.c_int), C.POINTER(C.c_int)]),
            "oeq_tp_create": (C.c_int, [vp, sz, C.POINTER(Step), C.c_int, C.POINTER(Step), C.c_int, C.POINTER(vp)]),
            "oeq_tp_destroy": (None, [vp]),
            "oeq_tp_forward": (C.c_int, [vp, u64, vp, vp, vp, vp, vp, vp]),
            "oeq_tp_backward": (C.c_int, [vp, u64, vp, vp, vp, vp, vp, vp, vp, vp, vp]),
            "oeq_conv_create": (C.c_int, [vp, sz, C.POINTER(Step), C.c_int, C.POINTER(Step), C.c_int, C.POINTER(vp)]),
            "oeq_conv_destroy": (None, [vp]),
            "oeq_conv_forward": (C.c_int, [vp, vp, vp, vp, vp, vp, vp, u64, u64, vp, vp, vp]),
            "oeq_conv_backward": (C.c_int, [vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, u64, u64, vp, vp, vp]),
            "oeq_conv_forward_ex": (C.c_int, [vp, vp, vp, vp, vp, vp, vp, u64, u64, vp, vp, vp, C.c_uint32]),
            "oeq_conv_backward_ex": (C.c_int, [vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, u64, u64, vp, vp, vp, C.c_uint32]),
            "oeq_conv_set_forward_workspace": (C.c_int, [vp, u64, u64, u64]),
            "oeq_conv_forward_noalloc": (C.c_int, [vp, vp, vp, vp, vp, vp, vp, u64, u64, vp, vp]),
            "oeq_module_load": (C.c_int, [vp, sz, C.POINTER(vp)]),
            "oeq_module_unload": (None, [vp]),
            "oeq_module_launch": (C.c_int, [vp, C.c_char_p, C.c_uint32, C.c_uint32, C.c_uint32, vp, C.POINTER(vp)]),
            "oeq_timer_create": (C.c_int, [C.POINTER(vp)]),
            "oeq_timer_destroy": (None, [vp]),
            "oeq_timer_start": (C.c_int, [vp, vp]),
            "oeq_timer_stop": (C.c_int, [vp, vp, C.POINTER(C.c_float)]),
            "oeq_timer_clear_cache": (C.c_int, [vp, vp]),
            "oeq_buffer_alloc": (C.c_int, [sz, C.POINTER(vp)]),
            "oeq_buffer_free": (C.c_int, [vp]),
            "oeq_buffer_h2d": (C.c_int, [vp, vp, sz]),
            "oeq_buffer_d2h": (C.c_int, [vp, vp, sz]),
            "oeq_buffer_zero": (C.c_int, [vp, sz, vp]),
            "oeq_stream_synchronize": (C.c_int, [vp]),
        }
        for name, (res, args) in sig.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


EXPORTED_SYMBOLS = [
    "oeq_last_error", "oeq_device_props", "oeq_device_count", "oeq_compile", "oeq_free", "oeq_hiprtc_version",
    "oeq_tp_create", "oeq_tp_destroy", "oeq_tp_forward", "oeq_tp_backward",
    "oeq_conv_create", "oeq_conv_destroy", "oeq_conv_forward", "oeq_conv_backward",
    "oeq_conv_forward_ex", "oeq_conv_backward_ex", "oeq_conv_set_forward_workspace", "oeq_conv_forward_noalloc",
    "oeq_module_load", "oeq_module_unload", "oeq_module_launch",
    "oeq_timer_create", "oeq_timer_destroy", "oeq_timer_start", "oeq_timer_stop", "oeq_timer_clear_cache",
    "oeq_buffer_alloc", "oeq_buffer_free", "oeq_buffer_h2d", "oeq_buffer_d2h", "oeq_buffer_zero",
    "oeq_stream_synchronize",
]


def _check(status: int) -> None:
    if status != 0:
        raise RuntimeError(lib().oeq_last_error().decode(errors="replace"))


# --------------------------------------------------------------------------- device
def device_count() -> int:
    n = C.c_int(0)
    _check(lib().oeq_device_count(C.byref(n)))
    return n.value


def device_props(device: int = 0) -> DeviceProp:
    p = DeviceProp()
    _check(lib().oeq_device_props(device, C.byref(p)))
    return p


# -------------------------------------------------------------------------- compile
DEFAULT_OPTIONS = ("-O3", "-std=c++17", "-munsafe-fp-atomics",
                   "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops")


def hiprtc_version() -> str:
    a, b = C.c_int(0), C.c_int(0)
    _check(lib().oeq_hiprtc_version(C.byref(a), C.byref(b)))
    return f"{a.value}.{b.value}"


def compile_source(source: str, arch: str = TARGET_ARCH, options: Sequence[str] = DEFAULT_OPTIONS,
                   use_cache: bool = True, refresh: bool = False) -> bytes:
    """hipRTC-compile ``source`` for ``arch``; code objects are cached on disk keyed by
    (source, arch, options, hipRTC version).  ``refresh`` compiles even when the cache holds the
    code object and replaces it."""
    key = hashlib.sha256("\0".join([source, arch, *options, hiprtc_version()]).encode()).hexdigest()[:32]
    path = CACHE_DIR / f"{key}.hsaco"
    if use_cache and not refresh and path.exists():
        return path.read_bytes()
    opts = (C.c_char_p * len(options))(*[o.encode() for o in options])
    code, size = C.c_void_p(), C.c_size_t()
    _check(lib().oeq_compile(source.encode(), arch.encode(), opts, len(options), C.byref(code), C.byref(size)))
    try:
        blob = C.string_at(code.value, size.value)
    finally:
        lib().oeq_free(code)
    if use_cache:
        try:
            CACHE_DIR.mkdir(parents=True, exist_ok=True)
            tmp = path.with_suffix(f".tmp{os.getpid()}")
            tmp.write_bytes(blob)
            os.replace(tmp, path)
        except OSError:
            pass
    return blob


def kernel_metadata(code: bytes) -> dict:
    """{kernel name: metadata} from the AMDGPU note of a code object: ``.vgpr_count``, ``.agpr_count``,
    ``.sgpr_count``, ``.private_segment_fixed_size`` (scratch bytes per lane: register spills),
    ``.group_segment_fixed_size`` (static LDS bytes)."""
    import struct

    import msgpack
    if code[:4] != b"\x7fELF" or code[4] != 2:
        raise ValueError("not a 64-bit ELF code object")
    shoff, = struct.unpack_from("<Q", code, 0x28)
    shentsize, shnum = struct.unpack_from("<HH", code, 0x3A)
    out = {}
    for i in range(shnum):
        off = shoff + i * shentsize
        sh_type, = struct.unpack_from("<I", code, off + 4)
        sh_offset, sh_size = struct.unpack_from("<QQ", code, off + 0x18)
        if sh_type != 7:                                  # SHT_NOTE
            continue
        pos, end = sh_offset, sh_offset + sh_size
        while pos + 12 <= end:
            namesz, descsz, ntype = struct.unpack_from("<III", code, pos)
            pos += 12
            name = code[pos:pos + namesz].rstrip(b"\0")
            pos += (namesz + 3) & ~3
            desc = code[pos:pos + descsz]
            pos += (descsz + 3) & ~3
            if name == b"AMDGPU" and ntype == 32:         # NT_AMDGPU_METADATA
                for k in msgpack.unpackb(desc, raw=False, strict_map_key=False).get("amdhsa.kernels", []):
                    out[k[".name"]] = k
    return out


# ------------------------------------------------------------------------ operators
def _steps(steps: Sequence[Step]):
    arr = (Step * max(1, len(steps)))(*steps)
    return arr, len(steps)


class TPImpl:
    """Handle of a compiled batch tensor product (reference type: JITTPImpl,
    extension/tensorproducts.hpp:50-98)."""

    def __init__(self, code: bytes, forward_steps: Sequence[Step], backward_steps: Sequence[Step]):
        self._h = C.c_void_p()
        self._code = code
        fa, nf = _steps(forward_steps)
        ba, nb = _steps(backward_steps)
        _check(lib().oeq_tp_create(code, len(code), fa, nf, ba, nb, C.byref(self._h)))

    def exec_tensor_product(self, n, L1, L2, L3, W, workspace=0, stream=0):
        _check(lib().oeq_tp_forward(self._h, n, L1, L2, L3, W, workspace, stream))

    def backward(self, n, L1, L1g, L2, L2g, W, Wg, L3g, workspace=0, stream=0):
        _check(lib().oeq_tp_backward(self._h, n, L1, L1g, L2, L2g, W, Wg, L3g, workspace, stream))

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h and _lib is not None:
            _lib.oeq_tp_destroy(h)


class ConvImpl:
    """Handle of a compiled fused convolution (reference type: JITConvImpl,
    extension/convolution.hpp:94-176)."""

    def __init__(self, code: bytes, forward_steps: Sequence[Step], backward_steps: Sequence[Step]):
        self._h = C.c_void_p()
        self._code = code
        fa, nf = _steps(forward_steps)
        ba, nb = _steps(backward_steps)
        _check(lib().oeq_conv_create(code, len(code), fa, nf, ba, nb, C.byref(self._h)))

    def set_forward_workspace(self, fixed_bytes: int, bytes_per_node: int, bytes_per_edge: int) -> None:
        """Declares what the forward steps use of the workspace without piece workgroups (checked by
        exec_conv_noalloc against the static scratch)."""
        _check(lib().oeq_conv_set_forward_workspace(self._h, fixed_bytes, bytes_per_node, bytes_per_edge))

    def exec_conv_rawptrs(self, L1, L2, W, L3, rows, cols, nnz, node_count, workspace=0, tperm=0, stream=0,
                          prepared=False, counters_zero=False):
        """``prepared``: the workspace still holds this graph's forward preparation (OEQ_CALL_PREPARED); the
        preparation kernels are then not launched.  ``counters_zero``: the operator's counters in the
        workspace are known to be zero (OEQ_CALL_COUNTERS_ZERO); the step that clears them is skipped."""
        flags = (CALL_PREPARED if prepared else 0) | (CALL_COUNTERS_ZERO if counters_zero else 0)
        _check(lib().oeq_conv_forward_ex(self._h, L1, L2, W, L3, rows, cols, nnz, node_count, workspace, tperm, stream, flags))

    def exec_conv_noalloc(self, L1, L2, W, L3, rows, cols, nnz, node_count, tperm=0, stream=0):
        """The forward with the library's static scratch as its workspace: allocates nothing."""
        _check(lib().oeq_conv_forward_noalloc(self._h, L1, L2, W, L3, rows, cols, nnz, node_count, tperm, stream))

    def backward_rawptrs(self, L1, L1g, L2, L2g, W, Wg, L3g, rows, cols, nnz, node_count,
                         workspace=0, tperm=0, stream=0, prepared=False, counters_zero=False):
        flags = (CALL_PREPARED if prepared else 0) | (CALL_COUNTERS_ZERO if counters_zero else 0)
        _check(lib().oeq_conv_backward_ex(self._h, L1, L1g, L2, L2g, W, Wg, L3g, rows, cols, nnz, node_count, workspace,
                                          tperm, stream, flags))

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h and _lib is not None:
            _lib.oeq_conv_destroy(h)


class Module:
    """A loaded code object with caller-packed launches."""

    def __init__(self, code: bytes):
        self._h = C.c_void_p()
        self._code = code
        _check(lib().oeq_module_load(code, len(code), C.byref(self._h)))

    def launch(self, kernel: str, grid: int, block: int, args: Sequence, smem: int = 0, stream: int = 0):
        """``args`` are ctypes scalars (c_void_p, c_uint64, ...)."""
        holders = list(args)
        arr = (C.c_void_p * len(holders))(*[C.cast(C.pointer(a), C.c_void_p) for a in holders])
        _check(lib().oeq_module_launch(self._h, kernel.encode(), grid, block, smem, stream, arr))

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h and _lib is not None:
            _lib.oeq_module_unload(h)


class GPUTimer:
    """Event-pair timer on a stream plus a cache flush (reference type: GPUTimer,
    extension/util/backend_hip.hpp:65-99)."""

    def __init__(self, stream: int = 0):
        self._h = C.c_void_p()
        self.stream = stream
        _check(lib().oeq_timer_create(C.byref(self._h)))

    def start(self):
        _check(lib().oeq_timer_start(self._h, self.stream))

    def stop_clock_get_elapsed(self) -> float:
        ms = C.c_float()
        _check(lib().oeq_timer_stop(self._h, self.stream, C.byref(ms)))
        return ms.value

    def clear_L2_cache(self):
        _check(lib().oeq_timer_clear_cache(self._h, self.stream))

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h and _lib is not None:
            _lib.oeq_timer_destroy(h)


class DeviceBuffer:
    """Owning device allocation initialised from a numpy array (reference type:
    DeviceBuffer, extension/util/buffer.hpp:8-45).  For torch-free callers."""

    def __init__(self, host_or_bytes):
        import numpy as np
        self._p = C.c_void_p()
        if isinstance(host_or_bytes, (int, np.integer)):
            self.host, self.nbytes = None, int(host_or_bytes)
        else:
            self.host = np.ascontiguousarray(host_or_bytes)
            self.nbytes = self.host.nbytes
        _check(lib().oeq_buffer_alloc(self.nbytes, C.byref(self._p)))
        if self.host is not None and self.nbytes:
            _check(lib().oeq_buffer_h2d(self._p, self.host.ctypes.data, self.nbytes))

    def data_ptr(self) -> int:
        return self._p.value

    def zero(self, stream: int = 0) -> None:
        """Fill the allocation with zero bytes on ``stream``."""
        if self.nbytes:
            _check(lib().oeq_buffer_zero(self._p, self.nbytes, stream))

    def copy_to_host(self):
        if self.host is None:
            raise RuntimeError("buffer was created without a host array")
        if self.nbytes:
            _check(lib().oeq_buffer_d2h(self.host.ctypes.data, self._p, self.nbytes))
        return self.host

    def __del__(self):
        p, self._p = getattr(self, "_p", None), None
        if p and _lib is not None:
            _lib.oeq_buffer_free(p)


def stream_synchronize(stream: int = 0) -> None:
    _check(lib().oeq_stream_synchronize(stream))
