"""Timing of one implementation on one problem and the statistics record of the reference's
result files (reference: openequivariance/benchmark/benchmark_utils.py)."""
from __future__ import annotations

import numpy as np

from ..problem import TPProblem
from .logging_utils import getLogger
from .perf_metrics_utils import (calculate_minimum_flops_forward, calculate_minimum_memory_streamed_backward,
                                 calculate_minimum_memory_streamed_forward, calculate_total_nnz)
from .random_buffer_utils import get_random_buffers_backward, get_random_buffers_forward

logger = getLogger()


def calculate_performance_statistics(problem: TPProblem, batch_size: int, total_flops: int, total_memory_streamed: int,
                                     time_millis: np.ndarray) -> dict:
    t = np.asarray(time_millis, dtype=np.float64)
    gflops = [float(v) for v in total_flops / (t * 1e6)]
    gbps = [float(v) for v in total_memory_streamed / (t * 1e6)]
    logger.info(f"throughput {np.mean(gflops):.2f} +- {np.std(gflops):.2f} GFLOPS, "
                f"bandwidth {np.mean(gbps):.2f} +- {np.std(gbps):.2f} GB/s")
    return {
        "total_cg_nnz": calculate_total_nnz(problem),
        "flops_per_tp": total_flops / batch_size,
        "L1": str(problem.irreps_in1), "L2": str(problem.irreps_in2), "L3": str(problem.irreps_out),
        "L1_rep_len": problem.irreps_in1.dim, "L2_rep_len": problem.irreps_in2.dim, "L3_rep_len": problem.irreps_out.dim,
        "rep_dtype": str(problem.irrep_dtype), "weight_dtype": str(problem.weight_dtype),
        "arithmetic_intensity (FLOPs / byte)": total_flops / total_memory_streamed,
        "batch_size": batch_size,
        "time_millis": [float(v) for v in t],
        "throughputs_gflops": gflops,
        "bandwidth_gbps": gbps,
    }


def _model(tp, what: str, batch_size: int, fallback):
    try:
        return getattr(tp, what)(batch_size=batch_size)
    except NotImplementedError:
        logger.warning(f"{what} is not implemented by {type(tp).__name__}; using the minimum model")
        return fallback()


def _run(direction: str, problem, implementation, batch_size, num_warmup, num_iter, prng_seed, torch_op, time_it,
         flops, memory) -> dict:
    result = {"tp_direction": direction, "num_warmup": num_warmup, "num_iter": num_iter, "prng_seed": prng_seed}
    tp = implementation(problem, torch_op=torch_op)
    try:
        time_millis = time_it(tp)
    except NotImplementedError:
        logger.warning("benchmarking is not implemented for this implementation; times are -1")
        time_millis = np.full(num_iter, -1.0)
    result |= calculate_performance_statistics(problem, batch_size, flops(tp)["total"], memory(tp)["total"], time_millis)
    return result


def benchmark_forward(problem: TPProblem, implementation, batch_size: int, num_warmup: int, num_iter: int,
                      prng_seed: int, torch_op: bool) -> dict:
    in1, in2, weights, out = get_random_buffers_forward(problem, batch_size, prng_seed)
    return _run("forward", problem, implementation, batch_size, num_warmup, num_iter, prng_seed, torch_op,
                lambda tp: tp.benchmark_forward(num_warmup=num_warmup, num_iter=num_iter, L1_in=in1, L2_in=in2,
                                                weights=weights, L3_buffer=out),
                lambda tp: _model(tp, "calculate_flops_forward", batch_size,
                                  lambda: calculate_minimum_flops_forward(problem, batch_size)),
                lambda tp: _model(tp, "calculate_memory_streamed_forward", batch_size,
                                  lambda: calculate_minimum_memory_streamed_forward(problem, batch_size)))


def benchmark_backward(problem: TPProblem, implementation, batch_size: int, num_warmup: int, num_iter: int,
                       prng_seed: int, torch_op: bool) -> dict:
    in1, in2, out_grad, weights, wg, g1, g2 = get_random_buffers_backward(problem, batch_size, prng_seed)
    return _run("backward", problem, implementation, batch_size, num_warmup, num_iter, prng_seed, torch_op,
                lambda tp: tp.benchmark_backward(num_warmup=num_warmup, num_iter=num_iter, L1_in=in1, L2_in=in2,
                                                 L3_buffer=out_grad, weights=weights, L1_grad=g1, L2_grad=g2,
                                                 weights_grad=wg),
                lambda tp: _model(tp, "calculate_flops_backward", batch_size, lambda: {"total": -1}),
                lambda tp: _model(tp, "calculate_memory_streamed_backward", batch_size,
                                  lambda: calculate_minimum_memory_streamed_backward(problem, batch_size)))
