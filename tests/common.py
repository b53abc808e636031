"""Shared test helpers: the benchmark problems described once for the product and once for
the oracle (two independent code paths), seeded inputs and the comparison metric."""
import numpy as np

import openequivariance_amd as oeq
from openequivariance_amd.sh import random_unit_vectors, spherical_harmonics
from oracle import spec

FP32_TOL = 1e-5      # relative L-inf error allowed in fp32 (against the fp64 oracle)
FP64_TOL = 1e-12     # ... in fp64

MACE = ("128x0e+128x1o+128x2e", "1x0e+1x1o+1x2e+1x3o", "128x0e+128x1o+128x2e+128x3o")
NEQUIP = ("32x0e+32x1o+32x2e", "1x0e+1x1o+1x2e", "32x0e+32x1o+32x2e")
LARGE = ("256x0e+256x1o+256x2e", "1x0e+1x1o+1x2e+1x3o", "256x0e+256x1o+256x2e")
DENSE = ("64x0e+64x1o+64x2e", "1x0e+1x1o+1x2e", "64x0e+64x1o+64x2e")
README = ("1x2e", "1x3e", "1x2e")


def channelwise(irreps, dtype=np.float32):
    return (oeq.ChannelwiseTPP(*irreps, irrep_dtype=dtype, weight_dtype=dtype), spec.channelwise(*irreps))


def readme_problem(dtype=np.float32):
    ins = [(0, 0, 0, "uvu", True)]
    return (oeq.TPProblem(*README, ins, shared_weights=False, internal_weights=False,
                          irrep_dtype=dtype, weight_dtype=dtype),
            spec.Problem(*README, ins, shared_weights=False))


def fully_connected(irreps, shared=True, dtype=np.float32):
    return (oeq.FullyConnectedTPProblem(*irreps, shared_weights=shared, internal_weights=False,
                                        irrep_dtype=dtype, weight_dtype=dtype),
            spec.fully_connected(*irreps, shared_weights=shared))


def rel_err(a, b):
    a, b = np.asarray(a, dtype=np.float64), np.asarray(b, dtype=np.float64)
    if a.size == 0:
        return 0.0
    return float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-300))


def tp_inputs(prob, n, seed, dtype=np.float32, sh_lmax=None, w_scale=1.0):
    """X ~ N(0,1); Y = spherical harmonics of random unit vectors when ``sh_lmax`` is given,
    else N(0,1); W ~ N(0, w_scale^2); G ~ N(0,1).  Values are rounded to ``dtype`` so that the
    oracle sees exactly what the kernel sees."""
    rng = np.random.default_rng(seed)
    d1, d2, d3 = prob.irreps_in1.dim, prob.irreps_in2.dim, prob.irreps_out.dim
    X = rng.standard_normal((n, d1))
    if sh_lmax is not None:
        Y = spherical_harmonics(sh_lmax, random_unit_vectors(n, rng))
        assert Y.shape[1] == d2
    else:
        Y = rng.standard_normal((n, d2))
    wshape = (prob.weight_numel,) if prob.shared_weights else (n, prob.weight_numel)
    W = rng.standard_normal(wshape) * w_scale
    G = rng.standard_normal((n, d3))
    return tuple(np.ascontiguousarray(a.astype(dtype)) for a in (X, Y, W, G))


def random_graph(nodes, nnz, seed, self_loops=False):
    rng = np.random.default_rng(seed)
    rows = rng.integers(0, nodes, nnz)
    cols = rng.integers(0, nodes, nnz)
    if not self_loops and nodes > 1:
        clash = rows == cols
        cols[clash] = (cols[clash] + 1 + rng.integers(0, nodes - 1, clash.sum())) % nodes
    return rows.astype(np.int64), cols.astype(np.int64)


def conv_inputs(prob, nodes, nnz, seed, dtype=np.float32, sh_lmax=None):
    rng = np.random.default_rng(seed)
    d1, d2, d3 = prob.irreps_in1.dim, prob.irreps_in2.dim, prob.irreps_out.dim
    X = rng.standard_normal((nodes, d1))
    Y = spherical_harmonics(sh_lmax, random_unit_vectors(nnz, rng)) if sh_lmax is not None \
        else rng.standard_normal((nnz, d2))
    W = rng.standard_normal((nnz, prob.weight_numel))
    G = rng.standard_normal((nodes, d3))
    return tuple(np.ascontiguousarray(a.astype(dtype)) for a in (X, Y, W, G))


def hub_graph(nodes, nnz, seed, hub_in, hub_out, in_edges, out_edges):
    """A random graph of ``nnz`` edges in which node ``hub_in`` receives ``in_edges`` of them and node
    ``hub_out`` sends ``out_edges`` (the rest uniform): two long edge lists next to short ones."""
    rng = np.random.default_rng(seed)
    rows = rng.integers(0, nodes, nnz)
    cols = rng.integers(0, nodes, nnz)
    pick = rng.permutation(nnz)
    rows[pick[:in_edges]] = hub_in
    cols[pick[in_edges:in_edges + out_edges]] = hub_out
    return rows.astype(np.int64), cols.astype(np.int64)


def with_invalid_edges(rows, cols, nodes, seed, count=7):
    """A copy of the edge list in which ``count`` edges name a node that does not exist (sender or
    receiver negative or >= nodes), and the mask of the edges left valid."""
    rng = np.random.default_rng(seed)
    rows, cols = rows.copy(), cols.copy()
    bad = rng.choice(rows.size, size=min(count, rows.size), replace=False)
    for k, e in enumerate(bad):
        target = rows if k % 2 == 0 else cols
        target[e] = (-1 - k) if k % 3 == 0 else nodes + k
    valid = (rows >= 0) & (rows < nodes) & (cols >= 0) & (cols < nodes)
    return rows, cols, valid


def conv_reference_on_valid_edges(otp, oprob, X, Y, W, G, rows, cols, valid):
    """Oracle outputs when edges outside ``valid`` contribute nothing: Z and dX from the valid sub-graph,
    dY / dW rows of the other edges zero."""
    Z = otp.conv_forward(oprob, X, Y[valid], W[valid], rows[valid], cols[valid])
    dX, dYv, dWv = otp.conv_backward(oprob, X, Y[valid], W[valid], G, rows[valid], cols[valid])
    dY, dW = np.zeros_like(Y, dtype=np.float64), np.zeros_like(W, dtype=np.float64)
    dY[valid], dW[valid] = dYv, dWv
    return Z, dX, dY, dW
