"""HIP graph capture of the operators: the launches take the caller's stream, allocate nothing
and clear their scratch with kernels, so a captured forward + backward replays correctly.  Each
graph is replayed several times with eager work and synchronisations in between, and every replay
is compared with the eager result."""
import numpy as np
import pytest

import common
from common import FP32_TOL, rel_err
from oracle import tp as otp

pytestmark = pytest.mark.gpu


def _capture(torch, fn):
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for _ in range(2):
            fn()                                  # warm-up outside the capture: workspaces, module loads
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        fn()
    return graph


@pytest.mark.parametrize("kind", ["uvu", "uvu_shared", "uvw"])
def test_tensor_product_in_a_graph(cuda, kind):
    import torch
    import openequivariance_amd as oeq
    if kind == "uvw":
        prob, oprob = common.fully_connected(("16x0e+16x1o", "1x0e+1x1o", "16x0e+16x1o"), shared=True)
    elif kind == "uvu_shared":
        a = ("8x0e+8x1o", "1x0e+1x1o", "8x0e+8x1o+8x1o")
        ins = [(0, 0, 0, "uvu", True), (0, 1, 1, "uvu", True), (1, 0, 2, "uvu", True), (1, 1, 0, "uvu", True)]
        prob = oeq.TPProblem(*a, ins, shared_weights=True, internal_weights=False)
    else:
        prob, oprob = common.channelwise(common.NEQUIP)
    n = 333
    X, Y, W, G = common.tp_inputs(prob, n, 17, w_scale=0.3)
    tp = oeq.TensorProduct(prob, torch_op=True)
    x, y, w, g = (torch.tensor(a, device=cuda) for a in (X, Y, W, G))
    z, xg, yg, wg = torch.empty_like(g), torch.empty_like(x), torch.empty_like(y), torch.empty_like(w)

    def step():
        tp.forward_raw(n, x.data_ptr(), y.data_ptr(), z.data_ptr(), w.data_ptr())
        tp.backward_raw(n, x.data_ptr(), xg.data_ptr(), y.data_ptr(), yg.data_ptr(), w.data_ptr(), wg.data_ptr(), g.data_ptr())
    step()
    torch.cuda.synchronize()
    eager = [t.clone() for t in (z, xg, yg, wg)]
    graph = _capture(torch, step)
    for rep in range(4):
        for t in (z, xg, yg, wg):
            t.fill_(float("nan"))
        _ = (x * 2).sum().item()                  # eager work and a synchronisation between replays
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(("Z", "dX", "dY", "dW"), (z, xg, yg, wg), eager):
            assert torch.equal(a, b), (rep, name)
    # new inputs in the same buffers: the graph computes on what the buffers hold at replay time
    x.mul_(0.5)
    graph.replay()
    torch.cuda.synchronize()
    assert torch.allclose(z, 0.5 * eager[0], rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("deterministic", [True, False])
def test_convolution_in_a_graph(cuda, deterministic):
    import torch
    import openequivariance_amd as oeq
    prob, oprob = common.channelwise(common.NEQUIP)
    nodes, nnz = 150, 4000
    rows, cols = common.random_graph(nodes, nnz, 23)
    tperm = None
    if deterministic:
        rows, cols, tperm, _ = otp.coord_graph(rows, cols)
    X, Y, W, G = common.conv_inputs(prob, nodes, nnz, 23, np.float32, 2)
    conv = oeq.TensorProductConv(prob, torch_op=True, deterministic=deterministic)
    x, y, w, g = (torch.tensor(a, device=cuda) for a in (X, Y, W, G))
    r, c = torch.tensor(rows, device=cuda), torch.tensor(cols, device=cuda)
    tp_ptr = torch.tensor(tperm, device=cuda) if deterministic else None
    z, xg, yg, wg = torch.zeros_like(g), torch.zeros_like(x), torch.empty_like(y), torch.empty_like(w)
    ws = conv.workspace_ptr(nnz, nodes)

    def step():
        if not conv.forward_overwrites:
            z.zero_()
        conv.exec_conv_rawptrs(x.data_ptr(), y.data_ptr(), w.data_ptr(), z.data_ptr(), r.data_ptr(), c.data_ptr(), nnz, nodes,
                               ws, tp_ptr.data_ptr() if deterministic else 0)
        if not deterministic:
            xg.zero_()                            # the per-edge backward accumulates dX with atomics
        conv.backward_rawptrs(x.data_ptr(), xg.data_ptr(), y.data_ptr(), yg.data_ptr(), w.data_ptr(), wg.data_ptr(), g.data_ptr(),
                              r.data_ptr(), c.data_ptr(), nnz, nodes, ws, tp_ptr.data_ptr() if deterministic else 0)
    graph = _capture(torch, step)
    Zr = otp.conv_forward(oprob, X, Y, W, rows, cols)
    dXr, dYr, dWr = otp.conv_backward(oprob, X, Y, W, G, rows, cols)
    first = None
    for rep in range(4):
        for t in (z, xg, yg, wg):
            t.fill_(float("nan"))
        _ = (x * 2).sum().item()
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in (("Z", z, Zr), ("dX", xg, dXr), ("dY", yg, dYr), ("dW", wg, dWr)):
            assert rel_err(a.cpu().numpy(), b) <= FP32_TOL, (rep, name)
        if deterministic:
            now = [t.clone() for t in (z, xg, yg, wg)]
            if first is None:
                first = now
            assert all(torch.equal(p, q) for p, q in zip(first, now)), rep


@pytest.mark.parametrize("deterministic", [True, False])
def test_torch_operator_in_a_graph_prepares_the_graph_itself(cuda, deterministic):
    """The torch operator under capture: the capture always records the graph-preparation kernels (it
    does not rely on what an earlier eager call left in the workspace), so replays stay correct after
    eager calls with another graph, and eager calls stay correct after replays."""
    import torch
    import openequivariance_amd as oeq
    prob, oprob = common.channelwise(common.NEQUIP)
    conv = oeq.TensorProductConv(prob, torch_op=True, deterministic=deterministic)

    def make(nodes, nnz, seed):
        rows, cols = common.random_graph(nodes, nnz, seed)
        idx = (rows, cols)
        if deterministic:
            rows, cols, tperm, _ = otp.coord_graph(rows, cols)
            idx = (rows, cols, tperm)
        X, Y, W, _ = common.conv_inputs(prob, nodes, nnz, seed, np.float32, 2)
        ref = otp.conv_forward(oprob, X, Y, W, rows, cols)
        return [torch.tensor(a, device=cuda) for a in (X, Y, W)], [torch.tensor(a, device=cuda) for a in idx], ref
    (x, y, w), idx, ref = make(120, 3000, 51)
    (x2, y2, w2), idx2, ref2 = make(120, 3000, 52)          # same sizes, other graph: same workspace

    out = {}

    def step():
        out["z"] = conv.forward(x, y, w, *idx)
    graph = _capture(torch, step)
    for rep in range(3):
        out["z"].fill_(float("nan"))
        z_other = conv.forward(x2, y2, w2, *idx2)           # eager call between replays, other graph
        torch.cuda.synchronize()
        assert rel_err(z_other.cpu().numpy(), ref2) <= FP32_TOL, rep
        graph.replay()
        torch.cuda.synchronize()
        assert rel_err(out["z"].cpu().numpy(), ref) <= FP32_TOL, rep
    z_again = conv.forward(x2, y2, w2, *idx2)
    torch.cuda.synchronize()
    assert rel_err(z_again.cpu().numpy(), ref2) <= FP32_TOL
