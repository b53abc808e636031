"""Process-wide switches of the package, read from the environment ONCE, when the package is imported.

Every choice the kernels make by themselves (which schedule, how many wavefronts, what goes through LDS)
is a static rule in the generators with the measurement that set it beside it.  The entries below are the
few choices a user or a measurement run may want to override; nothing else in the package reads the
environment.  Code reads ``tunables.current``; tests and measurement scripts change its attributes
(before the operators they affect are constructed) instead of the environment.

=========================  =====================  ==========================================================
environment variable       attribute              meaning
=========================  =====================  ==========================================================
OEQ_AMD_CACHE              cache_dir              folder of the hipRTC code-object cache
OEQ_AMD_GRAPH_CACHE        graph_cache            1: the torch convolution operators reuse the graph
                                                  preparation left in their workspace while rows / cols /
                                                  transpose_perm are the same tensors (address, in-place
                                                  version counter) - only safe when nothing rewrites the
                                                  index memory behind torch's back; default 0
OEQ_AMD_AUTOTUNE           autotune               0: the unsorted convolution's backward keeps the
                                                  generator's rule of thumb instead of timing both variants
OEQ_AMD_CONV_FORWARD       conv_forward           ``sorted`` (default) | ``atomic``: forward of the unsorted
                                                  convolution
OEQ_AMD_CONV_BACKWARD      conv_backward          ``atomic`` | ``grouped``: backward of the unsorted
                                                  convolution (unset: rule of thumb, then first-use timing)
OEQ_AMD_DET_BACKWARD       det_backward           ``send`` | ``recv``: edge order of the deterministic
                                                  backward (unset: by the shape of the problem)
OEQ_AMD_DET_LDS            det_lds                0 | 1: LDS-staged edge loop of the deterministic kernels
                                                  off / wherever it fits (unset: static rule)
OEQ_AMD_DET_SPLIT          det_split              operand words per edge above which the deterministic
                                                  backward runs one launch per group of output blocks
                                                  (0: never)
OEQ_AMD_DET_PREFETCH       det_prefetch           0 | 1: second register set in the deterministic backward
OEQ_AMD_TP_NT              tp_nontemporal         accesses of the batch product that carry the
                                                  non-temporal hint: subset of ``fl,fs,bl,bs``
OEQ_AMD_LONG_NODE          long_node              a node whose edge list is longer than this multiple of
                                                  the mean is cut into pieces walked by separate
                                                  wavefronts (0: never)
=========================  =====================  ==========================================================
"""
from __future__ import annotations

import os
import pathlib
from dataclasses import dataclass
from typing import Mapping, Optional


def _flag(v: Optional[str]) -> Optional[bool]:
    return None if v in (None, "") else v not in ("0", "false", "False", "off")


def _choice(v: Optional[str], allowed, name: str) -> Optional[str]:
    if v in (None, ""):
        return None
    if v not in allowed:
        raise ValueError(f"{name}={v!r}: expected one of {', '.join(allowed)}")
    return v


@dataclass
class Tunables:
    cache_dir: pathlib.Path
    graph_cache: bool = False
    autotune: bool = True
    conv_forward: str = "sorted"
    conv_backward: Optional[str] = None
    det_backward: Optional[str] = None
    det_lds: Optional[bool] = None
    det_split: Optional[int] = None
    det_prefetch: Optional[bool] = None
    tp_nontemporal: str = "bl,bs"
    long_node: int = 2

    @classmethod
    def from_env(cls, env: Mapping[str, str] = os.environ) -> "Tunables":
        pkg = pathlib.Path(__file__).resolve().parent
        t = cls(cache_dir=pathlib.Path(env.get("OEQ_AMD_CACHE") or pkg / "_kcache"))
        t.graph_cache = bool(_flag(env.get("OEQ_AMD_GRAPH_CACHE")))
        t.autotune = _flag(env.get("OEQ_AMD_AUTOTUNE")) is not False
        t.conv_forward = _choice(env.get("OEQ_AMD_CONV_FORWARD"), ("sorted", "atomic"), "OEQ_AMD_CONV_FORWARD") or "sorted"
        t.conv_backward = _choice(env.get("OEQ_AMD_CONV_BACKWARD"), ("atomic", "grouped"), "OEQ_AMD_CONV_BACKWARD")
        t.det_backward = _choice(env.get("OEQ_AMD_DET_BACKWARD"), ("send", "recv"), "OEQ_AMD_DET_BACKWARD")
        t.det_lds = _flag(env.get("OEQ_AMD_DET_LDS"))
        t.det_split = int(env["OEQ_AMD_DET_SPLIT"]) if env.get("OEQ_AMD_DET_SPLIT", "").isdigit() else None
        t.det_prefetch = _flag(env.get("OEQ_AMD_DET_PREFETCH"))
        t.tp_nontemporal = env.get("OEQ_AMD_TP_NT", "bl,bs")
        t.long_node = int(env["OEQ_AMD_LONG_NODE"]) if env.get("OEQ_AMD_LONG_NODE", "").isdigit() else 2
        return t


current = Tunables.from_env()
