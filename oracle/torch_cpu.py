"""Oracle: e3nn-equivalent tensor product on torch CPU, used as the timed CPU baseline.

Test/benchmark infrastructure.  e3nn itself cannot be installed here, so this restates the
computation its ``o3.TensorProduct`` performs (the reference wraps it in
openequivariance/implementations/E3NNTensorProduct.py:30-61): per instruction
``coeff * einsum(w, C, x, y)`` accumulated per output block, gradients by torch autograd;
the convolution is gather + ``index_add_``
(openequivariance/implementations/convolution/E3NNConv.py:38-64).  It is checked against
``oracle.tp`` in the tests and is never used by the product.
"""
from __future__ import annotations

from math import prod

import torch

from .cg import wigner_3j
from .spec import Problem, offsets


class TorchTP:
    def __init__(self, prob: Problem, dtype=torch.float32):
        self.prob, self.dtype = prob, dtype
        self.cg = [torch.tensor(wigner_3j(prob.in1[p["i1"]][1], prob.in2[p["i2"]][1], prob.out[p["io"]][1]) * p["coeff"],
                                dtype=dtype) for p in prob.paths]
        self.o1, self.o2, self.o3 = offsets(prob.in1), offsets(prob.in2), offsets(prob.out)

    def forward(self, X, Y, W):
        prob, B = self.prob, X.shape[0]
        outs = [None] * len(prob.out)
        for p, C in zip(prob.paths, self.cg):
            m1, l1, _ = prob.in1[p["i1"]]
            m2, l2, _ = prob.in2[p["i2"]]
            x = X[:, self.o1[p["i1"]]: self.o1[p["i1"]] + m1 * (2 * l1 + 1)].reshape(B, m1, 2 * l1 + 1)
            y = Y[:, self.o2[p["i2"]]: self.o2[p["i2"]] + m2 * (2 * l2 + 1)].reshape(B, m2, 2 * l2 + 1)
            w = W[..., p["woff"]: p["woff"] + prod(p["shape"])]
            if p["mode"] == "uvu":
                if w.ndim == 1:
                    r = torch.einsum("uv,ijk,zui,zvj->zuk", w.reshape(p["shape"]), C, x, y)
                else:
                    r = torch.einsum("zuv,ijk,zui,zvj->zuk", w.reshape((B,) + tuple(p["shape"])), C, x, y)
            else:
                if w.ndim == 1:
                    r = torch.einsum("uvw,ijk,zui,zvj->zwk", w.reshape(p["shape"]), C, x, y)
                else:
                    r = torch.einsum("zuvw,ijk,zui,zvj->zwk", w.reshape((B,) + tuple(p["shape"])), C, x, y)
            r = r.reshape(B, -1)
            outs[p["io"]] = r if outs[p["io"]] is None else outs[p["io"]] + r
        cols = []
        for i, (m, l, _) in enumerate(prob.out):
            cols.append(outs[i] if outs[i] is not None else X.new_zeros(B, m * (2 * l + 1)))
        return torch.cat(cols, dim=1)

    def conv_forward(self, X, Y, W, rows, cols):
        Ze = self.forward(X[cols], Y, W)
        Z = X.new_zeros(X.shape[0], self.prob.d3)
        return Z.index_add_(0, rows, Ze)


def time_forward_backward(prob: Problem, X, Y, W, G, threads: int, repeats: int = 1, rows=None, cols=None):
    """Seconds for ``repeats`` forward+backward passes on the CPU with ``threads`` threads."""
    import time
    torch.set_num_threads(threads)
    tp = TorchTP(prob)
    x, y, w = (torch.tensor(a, requires_grad=True) for a in (X, Y, W))
    g = torch.tensor(G)
    idx = None if rows is None else (torch.tensor(rows), torch.tensor(cols))

    def step():
        for t in (x, y, w):
            t.grad = None
        z = tp.forward(x, y, w) if idx is None else tp.conv_forward(x, y, w, *idx)
        z.backward(g)
    step()                                   # warm-up (einsum path planning, allocator)
    t0 = time.perf_counter()
    for _ in range(repeats):
        step()
    return (time.perf_counter() - t0) / repeats
