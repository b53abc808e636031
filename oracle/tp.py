"""Oracle: the weighted tensor product and the fused convolution, fp64 numpy.

Test infrastructure.  Restates what the reference compares itself against:
``e3nn.o3.TensorProduct`` evaluated per instruction as
``coeff * einsum(w, C, x, y)`` and summed per output block
(call sites: openequivariance/implementations/E3NNTensorProduct.py:30-61; the
same contraction is written out for uvu in
openequivariance/implementations/NumpyTensorProduct.py:35-46), and the unfused
convolution ``gather -> product -> scatter-add``
(openequivariance/implementations/convolution/E3NNConv.py:38-64).

Weights are in e3nn order: instruction after instruction, ``[u][v]`` (uvu) or
``[u][v][w]`` (uvw), row-major; shape ``[wn]`` when shared, ``[B, wn]`` otherwise.
"""
from __future__ import annotations

from math import prod

import numpy as np

from .cg import wigner_3j
from .spec import Problem, offsets


def _blocks(prob: Problem, p):
    m1, l1, _ = prob.in1[p["i1"]]
    m2, l2, _ = prob.in2[p["i2"]]
    mo, l3, _ = prob.out[p["io"]]
    o1, o2, o3 = offsets(prob.in1)[p["i1"]], offsets(prob.in2)[p["i2"]], offsets(prob.out)[p["io"]]
    return (m1, l1, o1), (m2, l2, o2), (mo, l3, o3)


def _weights_of(prob: Problem, p, W, B):
    w = W[..., p["woff"]: p["woff"] + prod(p["shape"])]
    if w.ndim == 1:
        w = np.broadcast_to(w, (B,) + w.shape)
    return w.reshape((B,) + tuple(p["shape"]))


def forward(prob: Problem, X, Y, W):
    """Z[B, d3] in float64."""
    X, Y, W = (np.asarray(a, dtype=np.float64) for a in (X, Y, W))
    B = X.shape[0]
    Z = np.zeros((B, prob.d3))
    for p in prob.paths:
        (m1, l1, o1), (m2, l2, o2), (mo, l3, o3) = _blocks(prob, p)
        C = wigner_3j(l1, l2, l3)
        x = X[:, o1:o1 + m1 * (2 * l1 + 1)].reshape(B, m1, 2 * l1 + 1)
        y = Y[:, o2:o2 + m2 * (2 * l2 + 1)].reshape(B, m2, 2 * l2 + 1)
        w = _weights_of(prob, p, W, B)
        if p["mode"] == "uvu":
            out = np.einsum("zuv,ijk,zui,zvj->zuk", w, C, x, y, optimize=True)
        else:
            out = np.einsum("zuvw,ijk,zui,zvj->zwk", w, C, x, y, optimize=True)
        Z[:, o3:o3 + mo * (2 * l3 + 1)] += p["coeff"] * out.reshape(B, mo * (2 * l3 + 1))
    return Z


def backward(prob: Problem, X, Y, W, G):
    """(dX, dY, dW) of <G, Z>; dW has the shape of W (summed over rows when shared)."""
    X, Y, W, G = (np.asarray(a, dtype=np.float64) for a in (X, Y, W, G))
    B = X.shape[0]
    shared = (W.ndim == 1)
    dX, dY = np.zeros_like(X), np.zeros_like(Y)
    dW = np.zeros_like(W)
    for p in prob.paths:
        (m1, l1, o1), (m2, l2, o2), (mo, l3, o3) = _blocks(prob, p)
        C = wigner_3j(l1, l2, l3) * p["coeff"]
        x = X[:, o1:o1 + m1 * (2 * l1 + 1)].reshape(B, m1, 2 * l1 + 1)
        y = Y[:, o2:o2 + m2 * (2 * l2 + 1)].reshape(B, m2, 2 * l2 + 1)
        g = G[:, o3:o3 + mo * (2 * l3 + 1)].reshape(B, mo, 2 * l3 + 1)
        w = _weights_of(prob, p, W, B)
        if p["mode"] == "uvu":
            dx = np.einsum("zuv,ijk,zvj,zuk->zui", w, C, y, g, optimize=True)
            dy = np.einsum("zuv,ijk,zui,zuk->zvj", w, C, x, g, optimize=True)
            dw = np.einsum("ijk,zui,zvj,zuk->zuv", C, x, y, g, optimize=True)
        else:
            dx = np.einsum("zuvw,ijk,zvj,zwk->zui", w, C, y, g, optimize=True)
            dy = np.einsum("zuvw,ijk,zui,zwk->zvj", w, C, x, g, optimize=True)
            dw = np.einsum("ijk,zui,zvj,zwk->zuvw", C, x, y, g, optimize=True)
        dX[:, o1:o1 + m1 * (2 * l1 + 1)] += dx.reshape(B, m1 * (2 * l1 + 1))
        dY[:, o2:o2 + m2 * (2 * l2 + 1)] += dy.reshape(B, m2 * (2 * l2 + 1))
        sl = slice(p["woff"], p["woff"] + prod(p["shape"]))
        if shared:
            dW[sl] += dw.sum(axis=0).reshape(-1)
        else:
            dW[:, sl] += dw.reshape(B, sl.stop - sl.start)
    return dX, dY, dW


def shared_weight_gradient(prob: Problem, X, Y, G, chunk: int = 8192):
    """dW of <G, Z> for shared weights (e3nn order), accumulated in float64 over chunks of rows: the
    same contraction as ``backward`` split in two steps, ``T = C x y`` then ``dW = T . G`` over
    (row, k), so that a batch of 10^5 rows costs seconds and bounded memory.  Pinned against
    ``backward`` in tests/test_oracle.py."""
    assert prob.shared_weights
    X, Y, G = (np.asarray(a) for a in (X, Y, G))
    dW = np.zeros(prob.weight_numel)
    for b0 in range(0, X.shape[0], chunk):
        Xc, Yc, Gc = (np.asarray(a[b0:b0 + chunk], dtype=np.float64) for a in (X, Y, G))
        B = Xc.shape[0]
        for p in prob.paths:
            (m1, l1, o1), (m2, l2, o2), (mo, l3, o3) = _blocks(prob, p)
            C = wigner_3j(l1, l2, l3) * p["coeff"]
            x = Xc[:, o1:o1 + m1 * (2 * l1 + 1)].reshape(B, m1, 2 * l1 + 1)
            y = Yc[:, o2:o2 + m2 * (2 * l2 + 1)].reshape(B, m2, 2 * l2 + 1)
            g = Gc[:, o3:o3 + mo * (2 * l3 + 1)].reshape(B, mo, 2 * l3 + 1)
            T = np.einsum("ijk,zui,zvj->zuvk", C, x, y, optimize=True)
            if p["mode"] == "uvu":
                dw = np.einsum("zuvk,zuk->uv", T, g, optimize=True)
            else:
                dw = np.tensordot(T, g, axes=([0, 3], [0, 2]))            # [u, v, w]
            dW[p["woff"]: p["woff"] + prod(p["shape"])] += dw.reshape(-1)
    return dW


# ---------------------------------------------------------------------------
# fused convolution: Z[n] = sum over edges e with rows[e] == n of TP(X[cols[e]], Y[e], W[e])
# ---------------------------------------------------------------------------

def conv_forward(prob: Problem, X, Y, W, rows, cols):
    """E3NNConv.py:38-49: rows = receivers (scatter target), cols = senders (gather source)."""
    X = np.asarray(X, dtype=np.float64)
    Ze = forward(prob, X[cols], Y, W)
    Z = np.zeros((X.shape[0], prob.d3))
    np.add.at(Z, rows, Ze)
    return Z


def conv_backward(prob: Problem, X, Y, W, G, rows, cols):
    """E3NNConv.py:51-64: per-edge dY, dW; dX scatter-added by sender."""
    X = np.asarray(X, dtype=np.float64)
    G = np.asarray(G, dtype=np.float64)
    dXe, dY, dW = backward(prob, X[cols], Y, W, G[rows])
    dX = np.zeros_like(X)
    np.add.at(dX, cols, dXe)
    return dX, dY, dW


def coord_graph(rows, cols):
    """Receiver-sorted COO and the transpose permutation
    (openequivariance/implementations/convolution/ConvolutionBase.py:59-70):
    sort edges by (row, col); ``tperm[j]`` = position in that sorted list of the
    j-th edge when the sorted list is re-sorted by (col, row)."""
    rows, cols = np.asarray(rows), np.asarray(cols)
    order = np.lexsort((cols, rows))
    r, c = rows[order], cols[order]
    tperm = np.lexsort((np.arange(r.size), r, c))
    return r, c, tperm.astype(r.dtype), order
