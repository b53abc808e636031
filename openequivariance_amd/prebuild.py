"""Ahead-of-time hipRTC compilation of the benchmark configurations' kernels.

hipRTC cross-compiles for gfx950 without a GPU, so the code objects of the benchmark
problems can be produced where the package is built and picked up from the in-tree cache on the
GPU machine.  Problems outside this list are compiled on first construction as usual.
"""
from __future__ import annotations

import time

import numpy as np

from . import runtime as rt
from .conv import select_conv_generator
from .problem import ChannelwiseTPP, FullyConnectedTPProblem, TPProblem
from .tensor_product import select_generator
from .workloads import get as get_workload
from .workloads import DENSE, DIFFDOCK_L2, LARGE, MACE, MACE_ALL, NEQUIP, TETRIS_POLY


def benchmark_generators():
    """(label, generator) for every kernel set the benchmark workloads and the smoke test use,
    chosen by the same selection functions as the operators."""
    readme = TPProblem("1x2e", "1x3e", "1x2e", [(0, 0, 0, "uvu", True)], shared_weights=False, internal_weights=False)
    gens = [("readme/tp", select_generator(readme)),
            ("mace/tp", select_generator(ChannelwiseTPP(*MACE))),
            ("mace-all-parities/tp", select_generator(ChannelwiseTPP(*MACE_ALL))),
            ("nequip/tp", select_generator(ChannelwiseTPP(*NEQUIP)))]
    for label, irreps in (("nequip", NEQUIP), ("large", LARGE), ("mace", MACE)):
        for det in (False, True):
            gens.append((f"{label}/conv_{'det' if det else 'atomic'}", select_conv_generator(ChannelwiseTPP(*irreps), det)))
    for det in (False, True):
        p = ChannelwiseTPP(*MACE, irrep_dtype=np.float64, weight_dtype=np.float64)
        gens.append((f"mace/conv_{'det' if det else 'atomic'}/float64", select_conv_generator(p, det)))
    gens.append(("benzene/conv_det", select_conv_generator(get_workload("benzene_conv_det").problem(), True)))
    for dt in (np.float32, np.float64):
        p = FullyConnectedTPProblem(*DENSE, shared_weights=True, internal_weights=False, irrep_dtype=dt, weight_dtype=dt)
        gens.append((f"dense/uvw/{np.dtype(dt).name}", select_generator(p)))
        p = FullyConnectedTPProblem(*DIFFDOCK_L2, shared_weights=False, internal_weights=False, irrep_dtype=dt, weight_dtype=dt)
        gens.append((f"diffdock/uvw per-row weights/{np.dtype(dt).name}", select_generator(p)))
        for which, irreps in TETRIS_POLY.items():
            p = FullyConnectedTPProblem(*irreps, shared_weights=True, internal_weights=False, irrep_dtype=dt, weight_dtype=dt)
            gens.append((f"tetris-poly-{which}/uvw few weights/{np.dtype(dt).name}", select_generator(p)))
    return gens


def compile_benchmark_kernels(verbose: bool = False, refresh: bool = False) -> None:
    """``refresh``: compile every kernel set again even where the cache already holds its code object."""
    for name, g in benchmark_generators():
        t = time.time()
        code = rt.compile_source(g.render(), refresh=refresh)
        if verbose:
            print(f"hipRTC gfx950 {name}: {len(code) // 1024} KiB ({time.time() - t:.1f}s)", flush=True)
