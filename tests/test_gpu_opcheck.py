"""The torch operators are registered so that torch.compile / export can use them: schemas, fake
(meta) kernels and autograd registration pass torch's own operator checks (the reference registers
fake kernels for this purpose: TensorProductBase.py:247-270, ConvolutionBase.py:575-616)."""
import numpy as np
import pytest

import common
from oracle import tp as otp

pytestmark = pytest.mark.gpu

TESTS = ("test_schema", "test_faketensor", "test_autograd_registration")


def test_tensor_product_ops(cuda):
    import torch
    import openequivariance_amd as oeq
    prob, _ = common.channelwise(common.NEQUIP)
    tp = oeq.TensorProduct(prob, torch_op=True)
    x, y, w = (torch.randn(20, d, device=cuda, requires_grad=True) for d in (288, 9, 352))
    g = torch.randn(20, 1120, device=cuda, requires_grad=True)
    torch.library.opcheck(tp.forward, (x, y, w), test_utils=TESTS)
    torch.library.opcheck(tp.backward_helper, (x, y, w, g), test_utils=TESTS)


@pytest.mark.parametrize("deterministic", [False, True])
def test_convolution_ops(cuda, deterministic):
    import torch
    import openequivariance_amd as oeq
    prob, _ = common.channelwise(common.NEQUIP)
    conv = oeq.TensorProductConv(prob, torch_op=True, deterministic=deterministic)
    rows, cols = common.random_graph(12, 90, 3)
    index = [rows, cols]
    if deterministic:
        rows, cols, tperm, _ = otp.coord_graph(rows, cols)
        index = [rows, cols, tperm]
    index = [torch.tensor(a, device=cuda) for a in index]
    x = torch.randn(12, 288, device=cuda, requires_grad=True)
    y, w = (torch.randn(90, d, device=cuda, requires_grad=True) for d in (9, 352))
    g = torch.randn(12, 1120, device=cuda, requires_grad=True)
    torch.library.opcheck(conv.forward, (x, y, w, *index), test_utils=TESTS)
    torch.library.opcheck(conv.backward_helper, (x, y, w, g, *index), test_utils=TESTS)


def test_fake_tensor_shapes_without_running_kernels(cuda):
    """Tracing with fake tensors goes through the registered fake kernels only."""
    import torch
    from torch._subclasses.fake_tensor import FakeTensorMode
    import openequivariance_amd as oeq
    prob, _ = common.channelwise(common.NEQUIP)
    tp = oeq.TensorProduct(prob, torch_op=True)
    with FakeTensorMode():
        x, y, w = (torch.empty(7, d, device="cuda") for d in (288, 9, 352))
        z = tp.forward(x, y, w)
        assert tuple(z.shape) == (7, 1120) and z.device.type == "cuda"
        gx, gy, gw = tp.backward_helper(x, y, w, z)
        assert gx.shape == x.shape and gy.shape == y.shape and gw.shape == w.shape


@pytest.mark.parametrize("deterministic", [False, True])
def test_compiled_function_matches_eager(cuda, deterministic):
    """torch.compile traces through the operators with their fake kernels and differentiates through
    their registered backward (backend aot_eager: tracing, functionalisation and the joint graph, no
    code generation): same numbers as eager."""
    import torch
    import openequivariance_amd as oeq
    prob, _ = common.channelwise(common.NEQUIP)
    tp = oeq.TensorProduct(prob, torch_op=True)
    conv = oeq.TensorProductConv(prob, torch_op=True, deterministic=deterministic)
    rows, cols = common.random_graph(12, 90, 3)
    index = [rows, cols]
    if deterministic:
        rows, cols, tperm, _ = otp.coord_graph(rows, cols)
        index = [rows, cols, tperm]
    index = [torch.tensor(a, device=cuda) for a in index]

    def model(x, y, w, xe):
        return conv.forward(x, y, w, *index).square().sum() + tp.forward(xe, y, w).sum()
    x = torch.randn(12, 288, device=cuda, requires_grad=True)
    xe = torch.randn(90, 288, device=cuda, requires_grad=True)
    y, w = (torch.randn(90, d, device=cuda, requires_grad=True) for d in (9, 352))
    eager = model(x, y, w, xe)
    g_eager = torch.autograd.grad(eager, (x, y, w, xe))
    compiled = torch.compile(model, backend="aot_eager", fullgraph=True)
    got = compiled(x, y, w, xe)
    g_got = torch.autograd.grad(got, (x, y, w, xe))
    torch.cuda.synchronize()
    assert torch.allclose(got, eager, rtol=1e-5, atol=1e-5)
    for a, b in zip(g_got, g_eager):
        assert torch.allclose(a, b, rtol=1e-4, atol=1e-4)
