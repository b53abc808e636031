"""In-tree build of the C-ABI runtime library ``liboeq_hip.so`` with hipcc.

``python -m openequivariance_amd.build_ext`` (or ``__graft_entry__.build()``)
compiles ``csrc/oeq_hip.cpp`` for gfx950 and leaves the shared object next to
the sources, where :mod:`openequivariance_amd.runtime` loads it from.  The
library is never built implicitly at import time.
"""
from __future__ import annotations

import os
import pathlib
import shutil
import subprocess
import sys

PKG_DIR = pathlib.Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_PATH = CSRC / "liboeq_hip.so"
ROCM = pathlib.Path(os.environ.get("ROCM_PATH", "/opt/rocm"))

# -packed-fp32-ops is switched off for every device compilation of this project
PACKED_FP32_OFF = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def hipcc_path() -> str:
    cand = shutil.which("hipcc") or str(ROCM / "bin" / "hipcc")
    if not os.path.exists(cand):
        raise RuntimeError("hipcc not found; set ROCM_PATH")
    return cand


def build_native(verbose: bool = True) -> pathlib.Path:
    cmd = [hipcc_path(), "--offload-arch=gfx950", "-O2", "-std=c++17", "-fPIC", "-shared",
           *PACKED_FP32_OFF,
           str(CSRC / "oeq_hip.cpp"), "-o", str(LIB_PATH),
           f"-L{ROCM / 'lib'}", "-lhiprtc", f"-Wl,-rpath,{ROCM / 'lib'}", "-Wl,--enable-new-dtags"]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed:\n{res.stdout}\n{res.stderr}")
    if verbose and res.stderr.strip():
        print(res.stderr, file=sys.stderr)
    return LIB_PATH


if __name__ == "__main__":
    print(build_native())
