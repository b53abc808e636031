"""Seeded random problems through the operators against the fp64 oracle: irreps, multiplicities
(ragged, above and below a wavefront), parities, batch and graph sizes are drawn per seed, so that
kernel-generator paths which no hand-written case names still get exercised."""
import numpy as np
import pytest

import common
from common import FP32_TOL, FP64_TOL, rel_err
from oracle import tp as otp, weights as ow

pytestmark = pytest.mark.gpu


def _par(l):
    return "e" if l % 2 == 0 else "o"


def _channelwise(rng, muls):
    import openequivariance_amd as oeq
    ls = sorted(rng.choice(4, size=rng.integers(1, 4), replace=False))
    mul = int(rng.choice(muls))
    same = rng.random() < 0.6
    in1 = "+".join(f"{mul if same else int(rng.choice([1, 5, 16, 32, 70]))}x{l}{_par(l)}" for l in ls)
    in2 = "+".join(f"1x{l}{_par(l)}" for l in range(int(rng.integers(1, 4)) + 1))
    widest = max(m for m, _ in oeq.Irreps(in1))
    both = rng.random() < 0.3
    out = "+".join(f"{widest}x{l}{p}" for l in range(int(rng.integers(0, 4)) + 1) for p in "eo"
                   if both or p == _par(l))
    return in1, in2, out


@pytest.mark.parametrize("seed", range(3000, 3024))
def test_random_convolution(cuda, seed):
    import torch
    import openequivariance_amd as oeq
    rng = np.random.default_rng(seed)
    while True:                                   # drawn again until at least one path is allowed
        irreps = _channelwise(rng, [1, 3, 8, 16, 20, 32, 48, 64, 100, 128])
        prob, oprob = common.channelwise(irreps)
        if prob.instructions:
            break
    nodes, nnz = int(rng.integers(1, 80)), int(rng.integers(0, 2000))
    for deterministic in (True, False):
        rows, cols = common.random_graph(nodes, nnz, seed, self_loops=True)
        tperm = None
        if deterministic:
            rows, cols, tperm, _ = otp.coord_graph(rows, cols)
        X, Y, W, G = common.conv_inputs(prob, nodes, nnz, seed)
        print(f"seed={seed} {irreps} paths={len(prob.instructions)} nodes={nodes} nnz={nnz} det={deterministic}", flush=True)
        conv = oeq.TensorProductConv(prob, torch_op=True, deterministic=deterministic)
        x, y, w = (torch.tensor(a, device=cuda, requires_grad=True) for a in (X, Y, W))
        idx = [torch.tensor(a, device=cuda) for a in ((rows, cols, tperm) if deterministic else (rows, cols))]
        z = conv.forward(x, y, w, *idx)
        z.backward(torch.tensor(G, device=cuda))
        torch.cuda.synchronize()
        assert rel_err(z.detach().cpu().numpy(), otp.conv_forward(oprob, X, Y, W, rows, cols)) <= FP32_TOL
        for got, ref in zip((x.grad, y.grad, w.grad), otp.conv_backward(oprob, X, Y, W, G, rows, cols)):
            assert rel_err(got.cpu().numpy(), ref) <= FP32_TOL


@pytest.mark.parametrize("seed", range(4000, 4030))
def test_random_tensor_product(cuda, seed):
    import torch
    import openequivariance_amd as oeq
    rng = np.random.default_rng(seed)
    kind = rng.choice(["uvu", "uvw_shared", "uvw_rows"], p=[0.5, 0.3, 0.2])
    dtype = np.float64 if rng.random() < 0.25 else np.float32
    tol = FP32_TOL if dtype == np.float32 else FP64_TOL
    n = int(rng.choice([1, 5, 17, 64, 300, 1111]))
    while True:                                   # drawn again until at least one path is allowed
        if kind == "uvu":
            irreps = _channelwise(rng, [1, 3, 8, 16, 20, 32, 48, 64, 100, 128, 200])
            prob, oprob = common.channelwise(irreps, dtype=dtype)
        else:
            ls = sorted(rng.choice(4, size=rng.integers(1, 4), replace=False))
            mul = lambda: int(rng.choice([1, 4, 16, 20, 32, 48, 64, 96]))
            irreps = ("+".join(f"{mul()}x{l}{_par(l)}" for l in ls),
                      "+".join(f"1x{l}{_par(l)}" for l in range(int(rng.integers(0, 4)) + 1)),
                      "+".join(f"{mul()}x{l}{_par(l)}" for l in range(int(rng.integers(0, 4)) + 1)))
            prob, oprob = common.fully_connected(irreps, shared=(kind == "uvw_shared"), dtype=dtype)
        if prob.instructions:
            break
    print(f"seed={seed} {kind} {dtype.__name__} {irreps} paths={len(prob.instructions)} n={n}", flush=True)
    tp = oeq.TensorProduct(prob, torch_op=True)
    X, Y, We, G = common.tp_inputs(prob, n, seed, dtype, w_scale=0.3)
    W = We if kind == "uvu" else ow.e3nn_to_oeq(oprob, We)
    x, y, w = (torch.tensor(a, device=cuda, requires_grad=True) for a in (X, Y, W))
    z = tp(x, y, w)
    z.backward(torch.tensor(G, device=cuda))
    torch.cuda.synchronize()
    dW = w.grad.cpu().numpy()
    if kind != "uvu":
        dW = ow.oeq_to_e3nn(oprob, dW)
    assert rel_err(z.detach().cpu().numpy(), otp.forward(oprob, X, Y, We)) <= tol
    for got, ref in zip((x.grad.cpu().numpy(), y.grad.cpu().numpy(), dW), otp.backward(oprob, X, Y, We, G)):
        assert rel_err(got, ref) <= tol
