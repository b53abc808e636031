"""The torch-free entry points (host arrays in, host arrays out, weights in e3nn order):
``forward_cpu`` / ``backward_cpu`` of both operators, as the reference's correctness harness
calls them (openequivariance/benchmark/correctness_utils.py:33-157)."""
import numpy as np
import pytest

import common
from common import FP32_TOL, rel_err
from oracle import tp as otp

pytestmark = pytest.mark.gpu


def test_tp_forward_backward_cpu_uvu(cuda):
    import openequivariance_amd as oeq
    prob, oprob = common.channelwise(common.NEQUIP)
    X, Y, W, G = common.tp_inputs(prob, 100, 80)
    tp = oeq.TensorProduct(prob, torch_op=False)
    Z = np.zeros((100, prob.irreps_out.dim), dtype=np.float32)
    tp.forward_cpu(X, Y, Z, W)
    assert rel_err(Z, otp.forward(oprob, X, Y, W)) <= FP32_TOL
    dX, dY, dW = np.zeros_like(X), np.zeros_like(Y), np.zeros_like(W)
    tp.backward_cpu(X, dX, Y, dY, G, W, dW)
    for got, ref in zip((dX, dY, dW), otp.backward(oprob, X, Y, W, G)):
        assert rel_err(got, ref) <= FP32_TOL


def test_tp_forward_backward_cpu_uvw_reorders_weights(cuda):
    """uvw: the caller passes e3nn-ordered weights and gets the e3nn-ordered gradient back."""
    import openequivariance_amd as oeq
    prob, oprob = common.fully_connected(common.DENSE, shared=True)
    X, Y, We, G = common.tp_inputs(prob, 64, 81, w_scale=0.125)
    tp = oeq.TensorProduct(prob, torch_op=False)
    Z = np.zeros((64, 576), dtype=np.float32)
    tp.forward_cpu(X, Y, Z, We)
    assert rel_err(Z, otp.forward(oprob, X, Y, We)) <= FP32_TOL
    dX, dY, dW = np.zeros_like(X), np.zeros_like(Y), np.zeros_like(We)
    tp.backward_cpu(X, dX, Y, dY, G, We, dW)
    for got, ref in zip((dX, dY, dW), otp.backward(oprob, X, Y, We, G)):
        assert rel_err(got, ref) <= FP32_TOL


@pytest.mark.parametrize("deterministic", [False, True])
def test_conv_forward_backward_cpu(cuda, deterministic):
    import openequivariance_amd as oeq
    prob, oprob = common.channelwise(common.NEQUIP)
    nodes, nnz = 50, 600
    rows, cols = common.random_graph(nodes, nnz, 82)
    graph = oeq.CoordGraph(np.zeros((nodes, 3)), rows, cols, "test")      # receiver-sorted + transpose perm
    X, Y, W, G = common.conv_inputs(prob, nodes, nnz, 83)
    conv = oeq.TensorProductConv(prob, torch_op=False, deterministic=deterministic)
    Z = np.zeros((nodes, prob.irreps_out.dim), dtype=np.float32)
    conv.forward_cpu(X, Y, W, Z, graph)
    assert rel_err(Z, otp.conv_forward(oprob, X, Y, W, graph.rows, graph.cols)) <= FP32_TOL
    dX, dY, dW = np.zeros_like(X), np.zeros_like(Y), np.zeros_like(W)
    conv.backward_cpu(X, dX, Y, dY, G, W, dW, graph)
    for got, ref in zip((dX, dY, dW), otp.conv_backward(oprob, X, Y, W, G, graph.rows, graph.cols)):
        assert rel_err(got, ref) <= FP32_TOL
