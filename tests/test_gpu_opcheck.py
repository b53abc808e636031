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
