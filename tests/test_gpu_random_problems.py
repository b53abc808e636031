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


# (the second group: draws whose dZ rows are long enough for the receiver-order backward - deterministic and, for most of
# them, unsorted - with 16 to 64 lanes per row and one or two chunks, and draws that stage a multi-chunk forward)
@pytest.mark.parametrize("seed", list(range(3000, 3024)) + [4002, 4011, 4014, 4029, 4088, 4095, 4114, 4145, 4149, 4188])
def test_random_convolution(cuda, seed):
    _random_convolution(cuda, seed, np.float32)


# (fp64 has kernels of its own choice: no LDS stage, the receiver order with register loads in one launch per in1
# block, forward groups of 32 output words)
# (5001 - 5045: draws that take the receiver order; the others keep the sender order)
@pytest.mark.parametrize("seed", [5000, 5001, 5003, 5004, 5011, 5017, 5030, 5039, 5040, 5045])
def test_random_convolution_fp64(cuda, seed):
    _random_convolution(cuda, seed, np.float64)


def _random_convolution(cuda, seed, dtype):
    import torch
    import openequivariance_amd as oeq
    rng = np.random.default_rng(seed)
    tol = FP32_TOL if dtype == np.float32 else FP64_TOL
    while True:                                   # drawn again until at least one path is allowed
        irreps = _channelwise(rng, [1, 3, 8, 16, 20, 32, 48, 64, 100, 128])
        prob, oprob = common.channelwise(irreps, dtype=dtype)
        if prob.instructions:
            break
    nodes, nnz = int(rng.integers(1, 80)), int(rng.integers(0, 2000))
    for deterministic in (True, False):
        rows, cols = common.random_graph(nodes, nnz, seed, self_loops=True)
        tperm = None
        if deterministic:
            rows, cols, tperm, _ = otp.coord_graph(rows, cols)
        X, Y, W, G = common.conv_inputs(prob, nodes, nnz, seed, dtype)
        conv = oeq.TensorProductConv(prob, torch_op=True, deterministic=deterministic)
        print(f"seed={seed} {np.dtype(dtype).name} {irreps} paths={len(prob.instructions)} nodes={nodes} nnz={nnz} "
              f"det={deterministic} {type(conv.generator).__name__}", flush=True)
        x, y, w = (torch.tensor(a, device=cuda, requires_grad=True) for a in (X, Y, W))
        idx = [torch.tensor(a, device=cuda) for a in ((rows, cols, tperm) if deterministic else (rows, cols))]
        z = conv.forward(x, y, w, *idx)
        z.backward(torch.tensor(G, device=cuda))
        torch.cuda.synchronize()
        assert rel_err(z.detach().cpu().numpy(), otp.conv_forward(oprob, X, Y, W, rows, cols)) <= tol
        for got, ref in zip((x.grad, y.grad, w.grad), otp.conv_backward(oprob, X, Y, W, G, rows, cols)):
            assert rel_err(got.cpu().numpy(), ref) <= tol


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


@pytest.mark.parametrize("seed", range(5000, 5016))
def test_random_second_operand_multiplicities(cuda, seed):
    """Random multiplicities on the second operand as well (1 to 40 copies per irrep, unrolled and walked
    at run time), uvu and uvw, shared and per-row weights, through the chunk-of-32 external weight order."""
    import torch
    import openequivariance_amd as oeq
    rng = np.random.default_rng(seed)
    mode = rng.choice(["uvu", "uvw"])
    shared = bool(rng.random() < 0.5)
    dtype = np.float64 if rng.random() < 0.25 else np.float32
    tol = FP32_TOL if dtype == np.float32 else FP64_TOL
    n = int(rng.choice([1, 7, 40, 200]))
    l1 = sorted(rng.choice(3, size=rng.integers(1, 3), replace=False))
    l2 = sorted(rng.choice(3, size=rng.integers(1, 3), replace=False))
    mul1 = int(rng.choice([3, 16, 33, 70]))
    in1 = "+".join(f"{mul1}x{l}{_par(l)}" for l in l1)
    # (uvw unrolls one contraction per copy: fewer copies there keep the kernels small)
    copies = [1, 2, 5, 9, 12, 40] if mode == "uvu" else [1, 2, 3, 5, 9]
    in2 = "+".join(f"{int(rng.choice(copies))}x{l}{_par(l)}" for l in l2)
    lo = range(int(rng.integers(1, 4)))
    if mode == "uvu":
        out = "+".join(f"{mul1}x{l}{_par(l)}" for l in lo)
        ins = [(i, j, k, "uvu", True) for i, a in enumerate(l1) for j, b in enumerate(l2) for k, c in enumerate(lo)
               if abs(a - b) <= c <= a + b and (a + b + c) % 2 == 0]
        if not ins:
            ins, out = [(0, 0, 0, "uvu", True)], f"{mul1}x{abs(l1[0] - l2[0])}{_par(abs(l1[0] - l2[0]))}"
        prob = oeq.TPProblem(in1, in2, out, ins, shared_weights=shared, internal_weights=False,
                             irrep_dtype=dtype, weight_dtype=dtype)
        from oracle import spec
        oprob = spec.Problem(in1, in2, out, ins, shared_weights=shared)
    else:
        out = "+".join(f"{int(rng.choice([4, 20, 48]))}x{l}{_par(l)}" for l in range(3))
        prob, oprob = common.fully_connected((in1, in2, out), shared=shared, dtype=dtype)
    print(f"seed={seed} {mode} shared={shared} {dtype.__name__} {in1} (x) {in2} -> {out} paths={len(prob.instructions)} n={n}",
          flush=True)
    tp = oeq.TensorProduct(prob, torch_op=True)
    X, Y, We, G = common.tp_inputs(prob, n, seed, dtype, w_scale=0.2)
    W = ow.e3nn_to_oeq(oprob, We)
    x, y, w = (torch.tensor(a, device=cuda, requires_grad=True) for a in (X, Y, W))
    z = tp(x, y, w)
    z.backward(torch.tensor(G, device=cuda))
    torch.cuda.synchronize()
    assert rel_err(z.detach().cpu().numpy(), otp.forward(oprob, X, Y, We)) <= tol
    dW = ow.oeq_to_e3nn(oprob, w.grad.cpu().numpy())
    for got, ref in zip((x.grad.cpu().numpy(), y.grad.cpu().numpy(), dW), otp.backward(oprob, X, Y, We, G)):
        assert rel_err(got, ref) <= tol


@pytest.mark.parametrize("seed", range(6000, 6012))
def test_random_uvw_with_few_shared_weights(cuda, seed):
    """Fully connected problems with small, ragged multiplicities and shared weights: most draws are served by the
    vector-ALU kernels with a row per lane (one to several register groups per row on either side, one to four
    copies of the second operand, batches from one row to several tiles per wavefront), the rest by the MFMA kernels."""
    import torch
    import openequivariance_amd as oeq
    rng = np.random.default_rng(seed)
    dtype = np.float64 if rng.random() < 0.25 else np.float32
    tol = FP32_TOL if dtype == np.float32 else FP64_TOL
    n = int(rng.choice([1, 31, 64, 65, 200, 700]))
    mul = lambda: int(rng.choice([1, 2, 3, 5, 6, 7, 10, 24]))
    while True:
        l1 = sorted(rng.choice(4, size=rng.integers(1, 4), replace=False))
        irreps = ("+".join(f"{mul()}x{l}{_par(l)}" for l in l1),
                  "+".join(f"{int(rng.choice([1, 1, 2, 4]))}x{l}{_par(l)}" for l in range(int(rng.integers(0, 3)) + 1)),
                  "+".join(f"{mul()}x{l}{p}" for l in range(int(rng.integers(0, 4)) + 1) for p in "eo"
                           if p == _par(l) or rng.random() < 0.3))
        prob, oprob = common.fully_connected(irreps, shared=True, dtype=dtype)
        if prob.instructions:
            break
    tp = oeq.TensorProduct(prob, torch_op=True)
    print(f"seed={seed} {dtype.__name__} {irreps} paths={len(prob.instructions)} wn={prob.weight_numel} n={n} "
          f"{type(tp.generator).__name__}", flush=True)
    X, Y, We, G = common.tp_inputs(prob, n, seed, dtype, w_scale=0.3)
    W = ow.e3nn_to_oeq(oprob, We)
    x, y, w = (torch.tensor(a, device=cuda, requires_grad=True) for a in (X, Y, W))
    z = tp(x, y, w)
    z.backward(torch.tensor(G, device=cuda))
    torch.cuda.synchronize()
    assert rel_err(z.detach().cpu().numpy(), otp.forward(oprob, X, Y, We)) <= tol
    dW = ow.oeq_to_e3nn(oprob, w.grad.cpu().numpy())
    for got, ref in zip((x.grad.cpu().numpy(), y.grad.cpu().numpy(), dW), otp.backward(oprob, X, Y, We, G)):
        assert rel_err(got, ref) <= tol
