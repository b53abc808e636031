"""Second derivatives through the torch ops (needed for force training), checked against fp64
torch autograd through the oracle's e3nn-equivalent implementation
(reference formula: openequivariance/implementations/TensorProductBase.py:281-298)."""
import numpy as np
import pytest

import common
from common import rel_err
from oracle import torch_cpu

pytestmark = pytest.mark.gpu
TOL = 2e-5     # two chained fp32 kernels per term


def _second_order(f, x, y, w, g, probes):
    """Returns grads of L = <p1, dX> + <p2, dY> + <p3, dW> (with (dX,dY,dW) = grad <g, f(x,y,w)>)
    with respect to x, y, w, g."""
    import torch
    z = f(x, y, w)
    dx, dy, dw = torch.autograd.grad(z, (x, y, w), g, create_graph=True)
    L = (probes[0] * dx).sum() + (probes[1] * dy).sum() + (probes[2] * dw).sum()
    return torch.autograd.grad(L, (x, y, w, g))


def _check(op_fn, ref_fn, arrays, dev):
    import torch
    X, Y, W, G = arrays
    rng = np.random.default_rng(99)
    probes = [rng.standard_normal(a.shape).astype(np.float32) for a in (X, Y, W)]
    gpu = [torch.tensor(a, device=dev, requires_grad=True) for a in (X, Y, W, G)]
    got = _second_order(op_fn, *gpu, [torch.tensor(p, device=dev) for p in probes])
    cpu = [torch.tensor(a.astype(np.float64), requires_grad=True) for a in (X, Y, W, G)]
    ref = _second_order(ref_fn, *cpu, [torch.tensor(p.astype(np.float64)) for p in probes])
    for name, a, b in zip(("d/dX", "d/dY", "d/dW", "d/dG"), got, ref):
        err = rel_err(a.cpu().numpy(), b.numpy())
        print(name, err, flush=True)
        assert err <= TOL, f"{name}: {err:.3e}"


def test_tp_double_backward(cuda):
    import openequivariance_amd as oeq
    prob, oprob = common.channelwise(common.NEQUIP)
    tp = oeq.TensorProduct(prob, torch_op=True)
    ref = torch_cpu.TorchTP(oprob, dtype=__import__("torch").float64)
    _check(lambda x, y, w: tp(x, y, w), ref.forward, common.tp_inputs(prob, 150, 61, sh_lmax=2), cuda)


@pytest.mark.parametrize("deterministic", [False, True])
def test_conv_double_backward(cuda, deterministic):
    import torch
    import openequivariance_amd as oeq
    from oracle import tp as otp
    prob, oprob = common.channelwise(common.NEQUIP)
    nodes, nnz = 60, 900
    rows, cols = common.random_graph(nodes, nnz, 62)
    tperm = None
    if deterministic:
        rows, cols, tperm, _ = otp.coord_graph(rows, cols)
    conv = oeq.TensorProductConv(prob, torch_op=True, deterministic=deterministic)
    idx = [torch.tensor(a, device=cuda) for a in ((rows, cols, tperm) if deterministic else (rows, cols))]
    ref = torch_cpu.TorchTP(oprob, dtype=torch.float64)
    r, c = torch.tensor(rows), torch.tensor(cols)
    _check(lambda x, y, w: conv.forward(x, y, w, *idx), lambda x, y, w: ref.conv_forward(x, y, w, r, c),
           common.conv_inputs(prob, nodes, nnz, 63, sh_lmax=2), cuda)


@pytest.mark.parametrize("kind", ["few_shared_weights", "mfma", "per_row_weights"])
def test_uvw_double_backward(cuda, kind):
    """The same second-order check through the three uvw kernel families (multiplicities of at most 32 and one
    copy of the second operand: the external weight order is e3nn's there, so the oracle takes the same W)."""
    import openequivariance_amd as oeq
    from openequivariance_amd.codegen.uvw import UVWGenerator
    from openequivariance_amd.codegen.uvw_batched import UVWBatchedGenerator
    from openequivariance_amd.codegen.uvw_rows import UVWRowsGenerator
    irreps, shared, gen = {"few_shared_weights": (("6x0e+5x1o", "1x0e+1x1o", "1x0o+6x0e+3x1o"), True, UVWRowsGenerator),
                           "mfma": (("16x0e+16x1o", "1x0e+1x1o", "16x0e+16x1o"), True, UVWGenerator),
                           "per_row_weights": (("16x0e+16x1o", "1x0e+1x1o", "16x0e+16x1o"), False, UVWBatchedGenerator)}[kind]
    prob, oprob = common.fully_connected(irreps, shared=shared)
    tp = oeq.TensorProduct(prob, torch_op=True)
    assert type(tp.generator) is gen
    ref = torch_cpu.TorchTP(oprob, dtype=__import__("torch").float64)
    _check(lambda x, y, w: tp(x, y, w), ref.forward, common.tp_inputs(prob, 90, 63, w_scale=0.3), cuda)
