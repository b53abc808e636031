"""Ahead-of-time hipRTC compilation of the benchmark configurations' kernels.

hipRTC cross-compiles for gfx950 without a GPU, so the code objects of the five benchmark
problems can be produced where the package is built and picked up from the in-tree cache on the
GPU machine.  Problems outside this list are compiled on first construction as usual.
"""
from __future__ import annotations

import time

import numpy as np

from . import runtime as rt
from .codegen.uvu import UVUGenerator
from .codegen.uvu_det import UVUDetGenerator
from .codegen.uvu_direct import UVUDirectGenerator
from .codegen.uvu_fast import UVUFastGenerator
from .problem import ChannelwiseTPP, FullyConnectedTPProblem, TPProblem

MACE = ("128x0e+128x1o+128x2e", "1x0e+1x1o+1x2e+1x3o", "128x0e+128x1o+128x2e+128x3o")
NEQUIP = ("32x0e+32x1o+32x2e", "1x0e+1x1o+1x2e", "32x0e+32x1o+32x2e")
LARGE = ("256x0e+256x1o+256x2e", "1x0e+1x1o+1x2e+1x3o", "256x0e+256x1o+256x2e")
DENSE = ("64x0e+64x1o+64x2e", "1x0e+1x1o+1x2e", "64x0e+64x1o+64x2e")


def benchmark_generators():
    readme = TPProblem("1x2e", "1x3e", "1x2e", [(0, 0, 0, "uvu", True)], shared_weights=False, internal_weights=False)
    gens = [("readme/tp", UVUGenerator(readme, "tp")),
            ("mace/tp", UVUGenerator(ChannelwiseTPP(*MACE), "tp")),
            ("nequip/tp", UVUGenerator(ChannelwiseTPP(*NEQUIP), "tp")),
            ("nequip/conv_atomic", UVUGenerator(ChannelwiseTPP(*NEQUIP), "conv_atomic")),
            ("nequip/conv_det", UVUGenerator(ChannelwiseTPP(*NEQUIP), "conv_det")),
            ("large/conv_atomic", UVUGenerator(ChannelwiseTPP(*LARGE), "conv_atomic")),
            ("large/conv_det", UVUGenerator(ChannelwiseTPP(*LARGE), "conv_det"))]
    for name, g in list(gens):
        if g.kind != "conv_det" and not g.shared:
            gens.append((name + "/direct", UVUDirectGenerator(g.problem, g.kind)))
        elif g.kind == "conv_det":
            gens.append((name + "/direct", UVUDetGenerator(g.problem)))
    try:
        from .codegen.uvw import UVWGenerator
    except ImportError:
        UVWGenerator = None
    if UVWGenerator is not None:
        for dt in (np.float32, np.float64):
            p = FullyConnectedTPProblem(*DENSE, shared_weights=True, internal_weights=False,
                                        irrep_dtype=dt, weight_dtype=dt)
            gens.append((f"dense/uvw/{np.dtype(dt).name}", UVWGenerator(p)))
    return gens


def compile_benchmark_kernels(verbose: bool = False) -> None:
    for name, g in benchmark_generators():
        t = time.time()
        code = rt.compile_source(g.render())
        if verbose:
            print(f"hipRTC gfx950 {name}: {len(code) // 1024} KiB ({time.time() - t:.1f}s)", flush=True)
