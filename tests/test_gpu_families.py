"""The reference's benchmark problem families beyond the five headline configurations
(test/benchmark.py:37-70 and benchmark/benchmark_configs.py of the reference): forward and
backward parity for each, small batches."""
import numpy as np
import pytest

import common
from common import FP32_TOL, rel_err
from oracle import spec, tp as otp, weights as ow

pytestmark = pytest.mark.gpu

CHANNELWISE = {
    "mace-medium": ("128x0e+128x1o", "1x0e+1x1o+1x2e+1x3o", "128x0e+128x1o+128x2e"),
    "nequip-lips": ("32x0o+32x0e+32x1o+32x1e+32x2o+32x2e", "0e+1o+2e", "32x0o+32x0e+32x1o+32x1e+32x2o+32x2e"),
    "nequip-revmd17-aspirin": ("64x0o+64x0e+64x1o+64x1e", "0e+1o", "64x0o+64x0e+64x1o+64x1e"),
    "nequip-revmd17-toluene": ("64x0o+64x0e+64x1o+64x1e+64x2o+64x2e", "0e+1o+2e", "64x0o+64x0e+64x1o+64x1e+64x2o+64x2e"),
    "nequip-revmd17-benzene": ("64x0o+64x0e+64x1o+64x1e+64x2o+64x2e+64x3o+64x3e", "0e+1o+2e+3o",
                               "64x0o+64x0e+64x1o+64x1e+64x2o+64x2e+64x3o+64x3e"),
    "nequip-water": ("32x0o+32x0e+32x1o+32x1e", "0e+1o", "32x0o+32x0e+32x1o+32x1e"),
}

# roofline set of the reference: single uvu instructions with l up to 7
SINGLE = [("128x1e", "1x1e", "128x1e"), ("128x2e", "1x1e", "128x2e"), ("128x3e", "1x3e", "128x3e"),
          ("128x5e", "1x5e", "128x3e"), ("128x5e", "1x3e", "128x5e"), ("128x6e", "1x3e", "128x6e"),
          ("128x7e", "1x4e", "128x7e"), ("128x7e", "1x7e", "128x7e")]

FULLY_CONNECTED = {
    "tetris-poly-1": ("1x0e+1x1o+1x2e+1x3o", "1x0e+1x1o+1x2e+1x3o", "64x0e+24x1e+24x1o+16x2e+16x2o"),
    "tetris-poly-2": ("64x0e+24x1e+24x1o+16x2e+16x2o", "1x0e+1x1o+1x2e+1x3o", "0o+6x0e"),
    # layers of e3nn's tetris example (benchmark/benchmark_configs.py:6-33 of the reference):
    # multiplicities that are no multiple of 16, up to 300 x 250 weight blocks, scalar second operand
    "tetris-0-sc": ("1x0e", "1x0e", "150x0e+50x1o+50x2e"),
    "tetris-1-sc": ("50x0e+50x1o+50x2e", "1x0e", "250x0e+50x1o+50x1e+50x2o+50x2e"),
    "tetris-2-lin2": ("100x0o+150x0e+300x1o+250x1e+250x2o+300x2e", "1x0e", "50x0o+250x0e+50x1o+50x1e+50x2o+50x2e"),
    "tetris-3-lin2": ("150x0o+150x0e", "1x0e", "1x0o+6x0e"),
}


@pytest.mark.parametrize("irreps", SINGLE, ids=[f"{a}x{b}" for a, b, _ in SINGLE])
def test_single_instruction_family(cuda, irreps):
    import torch
    import openequivariance_amd as oeq
    prob = oeq.SingleInstruction(*irreps, "uvu")
    oprob = spec.single_instruction(*irreps, "uvu")
    X, Y, W, G = common.tp_inputs(prob, 19, 72)
    tp = oeq.TensorProduct(prob, torch_op=True)
    x, y, w = (torch.tensor(a, device=cuda, requires_grad=True) for a in (X, Y, W))
    z = tp(x, y, w)
    z.backward(torch.tensor(G, device=cuda))
    refs = (otp.forward(oprob, X, Y, W),) + otp.backward(oprob, X, Y, W, G)
    for nm, a, b in zip(("Z", "dX", "dY", "dW"), (z.detach(), x.grad, y.grad, w.grad), refs):
        assert rel_err(a.cpu().numpy(), b) <= FP32_TOL, nm


@pytest.mark.parametrize("name", list(CHANNELWISE))
def test_channelwise_family(cuda, name):
    import torch
    import openequivariance_amd as oeq
    prob, oprob = common.channelwise(CHANNELWISE[name])
    X, Y, W, G = common.tp_inputs(prob, 37, 70)
    tp = oeq.TensorProduct(prob, torch_op=True)
    x, y, w = (torch.tensor(a, device=cuda, requires_grad=True) for a in (X, Y, W))
    z = tp(x, y, w)
    z.backward(torch.tensor(G, device=cuda))
    refs = (otp.forward(oprob, X, Y, W),) + otp.backward(oprob, X, Y, W, G)
    for nm, a, b in zip(("Z", "dX", "dY", "dW"), (z.detach(), x.grad, y.grad, w.grad), refs):
        assert rel_err(a.cpu().numpy(), b) <= FP32_TOL, nm


@pytest.mark.parametrize("name", list(FULLY_CONNECTED))
def test_fully_connected_family(cuda, name):
    import torch
    import openequivariance_amd as oeq
    prob, oprob = common.fully_connected(FULLY_CONNECTED[name], shared=True)
    X, Y, We, G = common.tp_inputs(prob, 41, 71, w_scale=0.3)
    tp = oeq.TensorProduct(prob, torch_op=True)
    W = ow.e3nn_to_oeq(oprob, We)
    x, y, w = (torch.tensor(a, device=cuda, requires_grad=True) for a in (X, Y, W))
    z = tp(x, y, w)
    z.backward(torch.tensor(G, device=cuda))
    dXr, dYr, dWr = otp.backward(oprob, X, Y, We, G)
    assert rel_err(z.detach().cpu().numpy(), otp.forward(oprob, X, Y, We)) <= FP32_TOL
    assert rel_err(x.grad.cpu().numpy(), dXr) <= FP32_TOL
    assert rel_err(y.grad.cpu().numpy(), dYr) <= FP32_TOL
    assert rel_err(ow.oeq_to_e3nn(oprob, w.grad.cpu().numpy()), dWr) <= FP32_TOL
