"""Seeded U[0,1) host buffers for the harness.  The draw order per seed is the reference's
(in1, in2, [out_grad,] weights), so the same seed gives the same problem instance
(reference: openequivariance/benchmark/random_buffer_utils.py)."""
from __future__ import annotations

import numpy as np

from ..problem import TPProblem


def _draw(rng, rows: int, dim: int, dtype):
    return rng.uniform(size=(rows, dim)).astype(dtype)


def _weights(rng, tpp: TPProblem, rows: int, dtype):
    shape = (tpp.weight_numel,) if tpp.shared_weights else (rows, tpp.weight_numel)
    return rng.uniform(size=shape).astype(dtype)


def _forward(tpp: TPProblem, n1: int, n2: int, seed: int):
    assert isinstance(tpp, TPProblem)
    rng = np.random.default_rng(seed)
    in1 = _draw(rng, n1, tpp.irreps_in1.dim, tpp.irrep_dtype)
    in2 = _draw(rng, n2, tpp.irreps_in2.dim, tpp.irrep_dtype)
    weights = _weights(rng, tpp, n2, tpp.weight_dtype)
    out = np.zeros((n1, tpp.irreps_out.dim), dtype=tpp.weight_dtype)
    return in1, in2, weights, out


def _backward(tpp: TPProblem, n1: int, n2: int, seed: int):
    assert isinstance(tpp, TPProblem)
    rng = np.random.default_rng(seed)
    in1 = _draw(rng, n1, tpp.irreps_in1.dim, tpp.irrep_dtype)
    in2 = _draw(rng, n2, tpp.irreps_in2.dim, tpp.irrep_dtype)
    out_grad = _draw(rng, n1, tpp.irreps_out.dim, tpp.irrep_dtype)
    weights = _weights(rng, tpp, n2, tpp.irrep_dtype)
    return in1, in2, out_grad, weights, np.zeros_like(weights), np.zeros_like(in1), np.zeros_like(in2)


def get_random_buffers_forward(tpp: TPProblem, batch_size: int, prng_seed: int):
    """(in1, in2, weights, out) for a batch product; weights are [weight_numel] when shared."""
    return _forward(tpp, batch_size, batch_size, prng_seed)


def get_random_buffers_backward(tpp: TPProblem, batch_size: int, prng_seed: int):
    """(in1, in2, out_grad, weights, weights_grad, in1_grad, in2_grad); the gradients are zeroed."""
    return _backward(tpp, batch_size, batch_size, prng_seed)


def get_random_buffers_forward_conv(tpp: TPProblem, node_count: int, edge_count: int, prng_seed: int):
    """Node features in1 [nodes], edge features in2 and weights [edges], output [nodes]."""
    return _forward(tpp, node_count, edge_count, prng_seed)


def get_random_buffers_backward_conv(tpp: TPProblem, node_count: int, edge_count: int, prng_seed: int):
    return _backward(tpp, node_count, edge_count, prng_seed)
