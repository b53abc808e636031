"""The benchmark harness end to end on the GPU: result files in the reference's layout, with the
oracle standing in for e3nn as the reference implementation."""
import json

import numpy as np
import pytest

import common
import openequivariance_amd as oeq
from openequivariance_amd.benchmark.ConvBenchmarkSuite import ConvBenchmarkSuite
from openequivariance_amd.benchmark.TestBenchmarkSuite import TestBenchmarkSuite, TestDefinition
from reference_impl import OracleConv, OracleTensorProduct, TorchReferenceConv, TorchReferenceTP

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("torch_op", [True, False])
def test_tensor_product_suite(cuda, tmp_path, torch_op):
    uvu, _ = common.channelwise(common.NEQUIP)
    uvw, _ = common.fully_connected(("16x0e+16x1o", "1x0e+1x1o", "16x0e+16x1o"), shared=True)
    tests = [TestDefinition(oeq.TensorProduct, p, d) for p in (uvu, uvw) for d in ("forward", "backward")]
    suite = TestBenchmarkSuite(num_warmup=2, num_iter=3, correctness_batch_size=200, bench_batch_size=5000,
                               reference_implementation=OracleTensorProduct, correctness_threshold=5e-5,
                               torch_op=torch_op)
    out = suite.run(tests, output_folder=tmp_path)
    md = json.loads((out / "metadata.json").read_text())
    assert md["directions"] == ["forward", "backward"] and len(md["test details"]) == 4
    for i, t in enumerate(tests):
        r = json.loads((out / f"{i}_LoopUnrollTP.json").read_text())
        assert r["direction"] == t.direction and r["torch_overhead_included"] == torch_op
        checks = [v for v in r["correctness results"].values() if isinstance(v, dict)]
        assert checks and all(c["pass"] for c in checks), r["correctness results"]
        b = r["benchmark results"]
        assert b["batch_size"] == 5000 and len(b["time_millis"]) == 3 and min(b["time_millis"]) > 0
        assert len(b["throughputs_gflops"]) == 3 and len(b["bandwidth_gbps"]) == 3 and b["L1_rep_len"] == t.problem.irreps_in1.dim


def test_double_backward_check(cuda, tmp_path):
    uvu, _ = common.channelwise(("8x0e+8x1o", "1x0e+1x1o", "8x0e+8x1o"))
    suite = TestBenchmarkSuite(correctness_batch_size=50, reference_implementation=TorchReferenceTP,
                               correctness_threshold=5e-5)
    out = suite.run([TestDefinition(oeq.TensorProduct, uvu, "double_backward", benchmark=False)], output_folder=tmp_path)
    r = json.loads((out / "0_LoopUnrollTP.json").read_text())["correctness results"]
    assert all(r[k]["pass"] for k in ("output_grad", "in1_grad", "in2_grad", "weights_grad")), r


@pytest.mark.parametrize("deterministic", [False, True])
@pytest.mark.parametrize("torch_op", [True, False])
def test_conv_suite(cuda, tmp_path, deterministic, torch_op):
    prob, _ = common.channelwise(common.NEQUIP)
    rows, cols = common.random_graph(60, 900, 3)
    graph = oeq.CoordGraph(np.zeros((60, 3)), rows, cols, "random60")

    class Impl(oeq.TensorProductConv):
        def __init__(self, config, torch_op=False):
            super().__init__(config, torch_op=torch_op, deterministic=deterministic)

    suite = ConvBenchmarkSuite([prob], num_warmup=1, num_iter=2, reference_impl=OracleConv, torch_op=torch_op)
    suite.correctness_threshold = 5e-5
    for direction in ("forward", "backward"):
        out = suite.run(graph, [Impl], direction, output_folder=tmp_path / direction)
        r = json.loads(next(p for p in out.iterdir() if p.name != "metadata.json").read_text())
        assert r["direction"] == direction and r["graph"] == "random60" and r["name"] == "LoopUnrollConv"
        checks = [v for v in r["correctness"].values() if isinstance(v, dict)]
        assert checks and all(c["pass"] for c in checks), r["correctness"]
        if direction == "forward" and deterministic:
            assert r["correctness"]["output"]["bitwise_reproducible"]
        b = r["benchmark"]
        assert b["graph_adj_nnz"] == 900 and len(b["time_millis"]) == 2 and min(b["time_millis"]) > 0


def test_conv_double_backward_check(cuda):
    prob, _ = common.channelwise(("8x0e+8x1o", "1x0e+1x1o", "8x0e+8x1o"))
    rows, cols = common.random_graph(20, 150, 4)
    graph = oeq.CoordGraph(np.zeros((20, 3)), rows, cols, "random20")
    conv = oeq.TensorProductConv(prob, torch_op=True, deterministic=True)
    r = conv.test_correctness_double_backward(graph, 5e-5, 12345, reference_implementation=TorchReferenceConv)
    assert all(v["pass"] for v in r.values()), r


def test_conv_variants_agree(cuda):
    """The named variants of the reference (deterministic, atomic, unfused scatter-sum) on one graph."""
    import torch
    prob, oprob = common.channelwise(common.NEQUIP)
    nodes, nnz = 80, 1500
    rows, cols = common.random_graph(nodes, nnz, 9)
    graph = oeq.CoordGraph(np.zeros((nodes, 3)), rows, cols, "g")
    X, Y, W, G = common.conv_inputs(prob, nodes, nnz, 9, np.float32, 2)
    from oracle import tp as otp
    Zr = otp.conv_forward(oprob, X, Y, W, graph.rows, graph.cols)
    dXr, dYr, dWr = otp.conv_backward(oprob, X, Y, W, G, graph.rows, graph.cols)
    names = []
    for cls in (oeq.LoopUnrollConvDeterministic, oeq.LoopUnrollConvAtomic, oeq.LoopUnrollConvScatterSum):
        conv = cls(prob, torch_op=True)
        names.append(conv.name())
        x, y, w = (torch.tensor(a, device=cuda, requires_grad=True) for a in (X, Y, W))
        idx = [torch.tensor(a, device=cuda) for a in (graph.rows, graph.cols)]
        if conv.deterministic:
            idx.append(torch.tensor(graph.transpose_perm, device=cuda))
        z = conv.forward(x, y, w, *idx)
        z.backward(torch.tensor(G, device=cuda))
        for nm, a, b in (("Z", z.detach(), Zr), ("dX", x.grad, dXr), ("dY", y.grad, dYr), ("dW", w.grad, dWr)):
            assert common.rel_err(a.cpu().numpy(), b) <= common.FP32_TOL, (conv.name(), nm)
        # numpy entry points of the unfused baseline
        if cls is oeq.LoopUnrollConvScatterSum:
            out = np.zeros_like(Zr, dtype=np.float32)
            conv.forward_cpu(X, Y, W, out, graph)
            assert common.rel_err(out, Zr) <= common.FP32_TOL
            g1, g2, gw = np.zeros_like(X), np.zeros_like(Y), np.zeros_like(W)
            conv.backward_cpu(X, g1, Y, g2, G, W, gw, graph)
            for a, b in ((g1, dXr), (g2, dYr), (gw, dWr)):
                assert common.rel_err(a, b) <= common.FP32_TOL
    assert names == ["LoopUnrollConvDeterministic", "LoopUnrollConvAtomic", "LoopUnrollConvScatterSum"]
