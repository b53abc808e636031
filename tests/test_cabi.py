"""The C-ABI library: builds in-tree, loads, exports every symbol the header declares.
No compute calls (there is no GPU here); error paths that need no device are exercised."""
import ctypes
import pathlib
import re

import pytest

from openequivariance_amd import runtime as rt

ROOT = pathlib.Path(__file__).resolve().parent.parent
HEADER = (ROOT / "include" / "oeq_hip.h").read_text()


def declared_functions():
    names = re.findall(r"^\s*(?:const\s+char\*|int|void)\s+(oeq_[a-z0-9_]+)\s*\(", HEADER, flags=re.M)
    return sorted(set(names))


def test_library_is_built_and_loads():
    assert rt.LIB_PATH.exists(), "run `python -m openequivariance_amd.build_ext` (or __graft_entry__.build())"
    assert rt.lib() is not None


def test_every_declared_symbol_is_exported():
    names = declared_functions()
    assert len(names) >= 28
    L = ctypes.CDLL(str(rt.LIB_PATH))
    for n in names:
        assert hasattr(L, n), f"{n} is declared in include/oeq_hip.h but not exported"
    assert sorted(rt.EXPORTED_SYMBOLS) == names, "runtime.py binds a different set than the header declares"


def test_step_struct_matches_header():
    fields = re.search(r"typedef struct \{(.*?)\} oeq_step;", HEADER, flags=re.S).group(1)
    order = re.findall(r"\b(kernel|num_threads|smem|grid_kind|work_per_block|num_blocks|grid_y|warp_size|flags)\b[\[;]", fields)
    assert order == [f[0] for f in rt.Step._fields_]
    assert ctypes.sizeof(rt.Step) == 64 + 8 * 4
    for name in ("OEQ_STEP_NEEDS_WORKSPACE", "OEQ_STEP_NEEDS_TPERM", "OEQ_STEP_GRAPH_PREP"):
        value = int(re.search(name + r"\s*=\s*(\d+)", HEADER).group(1))
        assert value == getattr(rt, name[4:])


def test_static_scratch_size_matches_header():
    shift = re.search(r"#define OEQ_NOALLOC_SCRATCH_BYTES \((\d+)u << (\d+)\)", HEADER)
    assert int(shift.group(1)) << int(shift.group(2)) == rt.NOALLOC_SCRATCH_BYTES


def test_hiprtc_compiles_for_gfx950_without_a_gpu_and_reports_errors():
    code = rt.compile_source('extern "C" __global__ void k(float* p) { p[threadIdx.x] = 1.0f; }', use_cache=False)
    assert code[:4] == b"\x7fELF"
    with pytest.raises(RuntimeError, match="hipRTC compilation failed"):
        rt.compile_source('extern "C" __global__ void k(float* p) { p[0] = undefined_symbol; }', use_cache=False)


def test_error_reporting_without_device():
    L = rt.lib()
    assert L.oeq_tp_forward(None, 1, None, None, None, None, None, None) != 0
    assert b"null handle" in L.oeq_last_error()
    assert L.oeq_conv_forward(None, None, None, None, None, None, None, 0, 0, None, None, None) != 0
    assert b"null handle" in L.oeq_last_error()
    assert L.oeq_conv_forward_ex(None, None, None, None, None, None, None, 0, 0, None, None, None, rt.CALL_PREPARED) != 0
    assert b"null handle" in L.oeq_last_error()
    assert L.oeq_conv_set_forward_workspace(None, 0, 0, 0) != 0
    assert L.oeq_conv_forward_noalloc(None, None, None, None, None, None, None, 0, 0, None, None) != 0
    assert b"null handle" in L.oeq_last_error()
    n = ctypes.c_int(-1)
    assert L.oeq_device_count(ctypes.byref(n)) == 0 and n.value >= 0
