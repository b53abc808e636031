"""Runs a list of (implementation, problem, direction) tests and writes the reference's result
files: ``metadata.json`` and one ``<id>_<implementation>.json`` per test
(reference: openequivariance/benchmark/TestBenchmarkSuite.py)."""
from __future__ import annotations

import json
import pathlib
import time
from dataclasses import dataclass
from typing import Any, Literal, NamedTuple, Optional, get_args

from .. import runtime as rt
from ..problem import TPProblem
from ..tensor_product import TensorProductBase
from .benchmark_utils import benchmark_backward, benchmark_forward
from .correctness_utils import correctness_backward, correctness_double_backward, correctness_forward
from .logging_utils import getLogger

logger = getLogger()

Direction = Literal["forward", "backward", "double_backward"]


class TestDefinition(NamedTuple):
    implementation: type
    problem: TPProblem
    direction: str
    correctness: bool = True
    benchmark: bool = True


TestDefinition.__test__ = False          # not a pytest class, whatever its name suggests


def _unique(items):
    return list(dict.fromkeys(items))


@dataclass(init=True, repr=False, eq=False)
class TestBenchmarkSuite:
    __test__ = False

    num_warmup: int = 10
    num_iter: int = 30
    correctness_batch_size: int = 10_000
    bench_batch_size: int = 10_000_000
    prng_seed: int = 12345
    reference_implementation: Optional[type] = None
    correctness_threshold: float = 5e-7
    torch_op: bool = True

    @staticmethod
    def validate_inputs(test_list) -> None:
        assert isinstance(test_list, list) and len(test_list) != 0
        for test in test_list:
            assert isinstance(test, TestDefinition)
            assert issubclass(test.implementation, TensorProductBase)
            assert isinstance(test.problem, TPProblem)
            assert test.direction in get_args(Direction)
            assert isinstance(test.correctness, bool) and isinstance(test.benchmark, bool)

    @staticmethod
    def generate_metadata(test_list) -> dict[str, Any]:
        try:
            gpu_name = rt.device_props(0).name.decode()
        except Exception:                      # metadata can be generated where no GPU is visible
            gpu_name = "unknown"
        return {
            "config_strs": _unique(str(t.problem) for t in test_list),
            "config_reprs": _unique(repr(t.problem) for t in test_list),
            "config_labels": _unique(t.problem.label for t in test_list),
            "implementations": _unique(t.implementation.name() for t in test_list),
            "directions": _unique(t.direction for t in test_list),
            "did_correctness": any(t.correctness for t in test_list),
            "did_benchmark": any(t.benchmark for t in test_list),
            "gpu_name": gpu_name,
            "test details": {i: {"implementation": t.implementation.name(), "problem": repr(t.problem),
                                 "direction": t.direction, "correctness": t.correctness, "benchmark": t.benchmark}
                             for i, t in enumerate(test_list)},
        }

    def run(self, test_list, output_folder=None) -> pathlib.Path:
        if output_folder is None:
            raise ValueError("output folder must be specified")
        output_folder = pathlib.Path(output_folder) / f"{round(time.time() * 1000)}"
        TestBenchmarkSuite.validate_inputs(test_list)
        output_folder.mkdir(parents=True)
        (output_folder / "metadata.json").write_text(json.dumps(TestBenchmarkSuite.generate_metadata(test_list), indent=2))

        check = {"forward": correctness_forward, "backward": correctness_backward,
                 "double_backward": correctness_double_backward}
        bench = {"forward": benchmark_forward, "backward": benchmark_backward}
        for test_id, test in enumerate(test_list):
            impl, tpp = test.implementation, test.problem
            logger.info(f"test {test_id}: {tpp} [{tpp.label}] {impl.name()} {test.direction} "
                        f"({tpp.irrep_dtype.__name__}), torch overhead included: {self.torch_op}")
            result = {"config_str": str(tpp), "config_repr": repr(tpp), "config_label": tpp.label,
                      "direction": test.direction, "implementation_name": impl.name(),
                      "correctness": str(test.correctness), "benchmark": str(test.benchmark),
                      "torch_overhead_included": self.torch_op}
            if test.correctness:
                result["correctness results"] = check[test.direction](
                    problem=tpp, test_implementation=impl, reference_implementation=self.reference_implementation,
                    batch_size=self.correctness_batch_size, correctness_threshold=self.correctness_threshold,
                    prng_seed=self.prng_seed)
            if test.benchmark and test.direction in bench:
                result["benchmark results"] = bench[test.direction](
                    problem=tpp, implementation=impl, batch_size=self.bench_batch_size, num_warmup=self.num_warmup,
                    num_iter=self.num_iter, prng_seed=self.prng_seed, torch_op=self.torch_op)
            (output_folder / f"{test_id}_{impl.name()}.json").write_text(json.dumps(result, indent=2))
            logger.info(f"finished test {test_id}")
        return output_folder
