"""Runs fused-convolution implementations over a graph and writes the reference's result files
(reference: openequivariance/benchmark/ConvBenchmarkSuite.py)."""
from __future__ import annotations

import json
import pathlib
import time

import numpy as np

from ..conv import CoordGraph
from .logging_utils import getLogger

logger = getLogger()


def load_graph(filename):
    """Graph from an ``.npz`` file with arrays ``coords``, ``row``, ``col`` (the reference reads a
    pickle with the same keys; a pickle executes code on load, so this loader takes the same
    content in numpy's own format)."""
    with np.load(filename, allow_pickle=False) as f:
        coords, rows, cols = f["coords"], f["row"], f["col"]
    name = pathlib.Path(filename).stem
    logger.info(f"graph {name}: {len(coords)} nodes, {len(rows)} edges")
    return CoordGraph(coords, rows.astype(np.int64), cols.astype(np.int64), name)


class ConvBenchmarkSuite:
    def __init__(self, configs, num_warmup=10, num_iter=30, reference_impl=None, torch_op=True, prng_seed=12345):
        self.configs = configs
        self.num_warmup, self.num_iter = num_warmup, num_iter
        self.reference_impl = reference_impl
        self.prng_seed = prng_seed
        self.correctness_threshold = 1e-5
        self.torch_op = torch_op
        self.exp_count = 0

    def run(self, graph, implementations, direction, output_folder=None, correctness=True,
            double_backward_correctness=False, benchmark=True):
        if output_folder is None:
            raise ValueError("output folder must be specified")
        output_folder = pathlib.Path(output_folder) / f"{round(time.time() * 1000)}"
        output_folder.mkdir(parents=True)
        if self.exp_count == 0:
            (output_folder / "metadata.json").write_text(json.dumps({
                "test_name": "Convolution", "configs": [str(c) for c in self.configs],
                "implementations": [impl.name() for impl in implementations], "graph": graph.name}, indent=2))
        for config in self.configs:
            for impl in implementations:
                logger.info(f"{config}, {impl.name()}, graph {graph.name}, {direction}")
                conv = impl(config, torch_op=self.torch_op)
                common = dict(thresh=self.correctness_threshold, prng_seed=self.prng_seed,
                              reference_implementation=self.reference_impl)
                record = {"correctness": correctness, "benchmark": benchmark,
                          "double_backward_correctness": double_backward_correctness}
                if double_backward_correctness:
                    record["double_backward_correctness"] = conv.test_correctness_double_backward(graph, **common)
                if correctness:
                    record["correctness"] = getattr(conv, f"test_correctness_{direction}")(graph, **common)
                if benchmark:
                    record["benchmark"] = getattr(conv, f"benchmark_{direction}")(self.num_warmup, self.num_iter, graph,
                                                                                  prng_seed=self.prng_seed)
                result = {"config": str(config), "irrep_dtype": str(config.irrep_dtype),
                          "weight_dtype": str(config.weight_dtype), "torch_overhead_included": self.torch_op,
                          "direction": direction, "graph": graph.name, "name": impl.name(), **record}
                (output_folder / f"{self.exp_count}_{impl.name()}_{graph.name}.json").write_text(json.dumps(result, indent=2))
                self.exp_count += 1
        return output_folder
