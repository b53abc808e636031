"""Comparison of an implementation against a reference implementation on seeded host buffers
(reference: openequivariance/benchmark/correctness_utils.py).  Both sides are objects with the
``forward_cpu`` / ``backward_cpu`` numpy entry points taking weights in e3nn order."""
from __future__ import annotations

from typing import Optional

import numpy as np

from ..problem import TPProblem
from .logging_utils import getLogger
from .random_buffer_utils import get_random_buffers_backward, get_random_buffers_forward

logger = getLogger()


def check_similiarity(name: str, to_check: np.ndarray, ground_truth: np.ndarray, correctness_threshold: float) -> dict:
    """{"shape_match", "diff_Linf_norm", "pass"}: absolute L-inf difference below the threshold."""
    if to_check.shape != ground_truth.shape:
        logger.error(f"{name}: shape {to_check.shape} differs from the reference's {ground_truth.shape}")
        return {"shape_match": False, "diff_Linf_norm": float("inf"), "pass": False}
    diff = float(np.max(np.abs(ground_truth.astype(np.float64) - to_check.astype(np.float64)))) if to_check.size else 0.0
    ok = bool(diff < correctness_threshold)
    (logger.info if ok else logger.error)(f"{name}: L-inf difference {diff:.3e} (threshold {correctness_threshold}) "
                                          + ("pass" if ok else "FAIL"))
    return {"shape_match": True, "diff_Linf_norm": diff, "pass": ok}


def default_reference():
    """The reference compares against e3nn (E3NNTensorProduct.py:30-41); that package is optional
    here, so the caller normally passes ``reference_implementation``."""
    raise NotImplementedError("pass reference_implementation=...: no CPU reference ships with this package "
                              "(the reference's default, e3nn, is an optional third-party dependency)")


def correctness_forward(problem: TPProblem, test_implementation, reference_implementation: Optional[type],
                        batch_size: int, correctness_threshold: float, prng_seed: int) -> dict:
    if reference_implementation is None:
        reference_implementation = default_reference()
    in1, in2, weights, out = get_random_buffers_forward(problem, batch_size, prng_seed)
    outs = []
    for impl in (reference_implementation, test_implementation):
        buf = out.copy()
        impl(problem).forward_cpu(L1_in=in1.copy(), L2_in=in2.copy(), L3_out=buf, weights=weights.copy())
        outs.append(buf)
    return {"thresh": correctness_threshold, "batch_size": batch_size,
            "output": check_similiarity("output", outs[1], outs[0], correctness_threshold)}


def correctness_backward(problem: TPProblem, test_implementation, reference_implementation: Optional[type],
                         batch_size: int, correctness_threshold: float, prng_seed: int) -> dict:
    if reference_implementation is None:
        reference_implementation = default_reference()
    in1, in2, out_grad, weights, wg, g1, g2 = get_random_buffers_backward(problem, batch_size, prng_seed)
    grads = []
    for impl in (reference_implementation, test_implementation):
        bufs = dict(weights_grad=wg.copy(), L1_grad=g1.copy(), L2_grad=g2.copy())
        impl(problem).backward_cpu(L1_in=in1.copy(), L2_in=in2.copy(), L3_grad=out_grad.copy(), weights=weights.copy(), **bufs)
        grads.append(bufs)
    result = {"thresh": correctness_threshold, "batch_size": batch_size}
    for name, key in (("weight_grad", "weights_grad"), ("in1_grad", "L1_grad"), ("in2_grad", "L2_grad")):
        result[name] = check_similiarity(name, grads[1][key], grads[0][key], correctness_threshold)
    return result


def correctness_double_backward(problem: TPProblem, test_implementation, reference_implementation: Optional[type],
                                batch_size: int, correctness_threshold: float, prng_seed: int) -> dict:
    """Second-order check of the torch ops: gradients of a scalar built from the first gradients,
    with respect to the output gradient and the three inputs (same protocol as the reference)."""
    import torch
    if reference_implementation is None:
        reference_implementation = default_reference()
    in1, in2, out_grad, weights, _, _, _ = get_random_buffers_backward(problem, batch_size, prng_seed)
    scale = float(np.random.default_rng(seed=prng_seed * 2).standard_normal(1)[0])
    got = []
    for impl in (test_implementation, reference_implementation):
        tp = impl(problem, torch_op=True)
        dev = getattr(tp, "device", "cuda")
        w_in = weights
        if impl is test_implementation and hasattr(tp, "reorder_weights_e3nn_to_oeq"):
            w_in = np.zeros_like(weights)
            tp.reorder_weights_e3nn_to_oeq(weights, w_in, not problem.shared_weights)
        a, b, w, g = (torch.tensor(t, device=dev, requires_grad=True) for t in (in1, in2, w_in, out_grad))
        out = tp.forward(a, b, w)
        out.backward(g, create_graph=True, retain_graph=True, inputs=[a, b, w])
        dummy = torch.norm(a.grad) + torch.norm(b.grad) + torch.norm(w.grad)
        dummy.backward(torch.tensor(scale, device=dev, dtype=dummy.dtype), retain_graph=True, inputs=[g, a, b, w])
        wgrad = w.grad.detach().cpu().numpy()
        if impl is test_implementation and hasattr(tp, "reorder_weights_oeq_to_e3nn"):
            tmp = wgrad.copy()
            tp.reorder_weights_oeq_to_e3nn(tmp, wgrad, not problem.shared_weights)
        got.append((g.grad.detach().cpu().numpy(), a.grad.detach().cpu().numpy(), b.grad.detach().cpu().numpy(), wgrad))
    result = {"thresh": correctness_threshold, "batch_size": batch_size}
    for i, name in enumerate(("output_grad", "in1_grad", "in2_grad", "weights_grad")):
        result[name] = check_similiarity(name, got[0][i], got[1][i], correctness_threshold)
    return result
