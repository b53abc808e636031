"""oeq_conv_forward_noalloc: the forward with the library's static device scratch as its workspace,
against oeq_conv_forward with a caller-owned workspace, on two calls in a row, the second one on a
smaller graph (the scratch keeps the first call's contents)."""
import numpy as np
import pytest

import common
from common import FP32_TOL, rel_err
from oracle import tp as otp

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("deterministic", [True, False])
@pytest.mark.parametrize("irreps", [common.NEQUIP, common.LARGE], ids=["nequip", "large"])
def test_noalloc_forward_matches_forward(cuda, deterministic, irreps):
    import torch
    import openequivariance_amd as oeq
    prob, oprob = common.channelwise(irreps)
    conv = oeq.TensorProductConv(prob, torch_op=False, deterministic=deterministic)
    for nodes, nnz, seed in ((90, 2500, 41), (35, 600, 42)):
        rows, cols = common.random_graph(nodes, nnz, seed)
        tperm = None
        if deterministic:
            rows, cols, tperm, _ = otp.coord_graph(rows, cols)
        X, Y, W, _ = common.conv_inputs(prob, nodes, nnz, seed, np.float32, 2 if irreps is common.NEQUIP else 3)
        x, y, w = (torch.tensor(a, device=cuda) for a in (X, Y, W))
        r, c = torch.tensor(rows, device=cuda), torch.tensor(cols, device=cuda)
        tp = torch.tensor(tperm, device=cuda) if deterministic else None
        tp_ptr = tp.data_ptr() if deterministic else 0
        ws = torch.empty(conv._ws_bytes(nnz, nodes), dtype=torch.uint8, device=cuda)
        z_ref = torch.full((nodes, prob.irreps_out.dim), float("nan"), device=cuda)
        z_new = torch.full_like(z_ref, float("nan"))
        stream = torch.cuda.current_stream().cuda_stream
        print(f"det={deterministic} nodes={nodes} nnz={nnz}", flush=True)
        conv.internal.exec_conv_rawptrs(x.data_ptr(), y.data_ptr(), w.data_ptr(), z_ref.data_ptr(), r.data_ptr(),
                                        c.data_ptr(), nnz, nodes, ws.data_ptr(), tp_ptr, stream)
        torch.cuda.synchronize()
        before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
        conv.internal.exec_conv_noalloc(x.data_ptr(), y.data_ptr(), w.data_ptr(), z_new.data_ptr(), r.data_ptr(),
                                        c.data_ptr(), nnz, nodes, tp_ptr, stream)
        torch.cuda.synchronize()
        # neither torch's allocator nor the device as a whole (a hipMalloc inside the library) gave memory out
        assert torch.cuda.memory_allocated() == before and torch.cuda.mem_get_info()[0] == free_before
        if deterministic:
            assert torch.equal(z_new, z_ref)                  # fixed summation order: bit-equal
        else:
            assert rel_err(z_new.cpu().numpy(), z_ref.cpu().numpy()) <= FP32_TOL
        assert rel_err(z_new.cpu().numpy(), otp.conv_forward(oprob, X, Y, W, rows, cols)) <= FP32_TOL


@pytest.mark.parametrize("deterministic", [True, False])
def test_noalloc_forward_under_graph_capture(cuda, deterministic):
    """What the entry point is for: the call is captured into a HIP graph (after one call outside the
    capture, which looks up the scratch's address) and replayed, with eager work between the replays."""
    import torch
    import openequivariance_amd as oeq
    prob, oprob = common.channelwise(common.NEQUIP)
    conv = oeq.TensorProductConv(prob, torch_op=False, deterministic=deterministic)
    nodes, nnz = 70, 1800
    rows, cols = common.random_graph(nodes, nnz, 43)
    tperm = None
    if deterministic:
        rows, cols, tperm, _ = otp.coord_graph(rows, cols)
    X, Y, W, _ = common.conv_inputs(prob, nodes, nnz, 43, np.float32, 2)
    x, y, w = (torch.tensor(a, device=cuda) for a in (X, Y, W))
    r, c = torch.tensor(rows, device=cuda), torch.tensor(cols, device=cuda)
    tp = torch.tensor(tperm, device=cuda) if deterministic else None
    z = torch.zeros(nodes, prob.irreps_out.dim, device=cuda)
    Zr = otp.conv_forward(oprob, X, Y, W, rows, cols)

    def call(stream):
        conv.internal.exec_conv_noalloc(x.data_ptr(), y.data_ptr(), w.data_ptr(), z.data_ptr(), r.data_ptr(),
                                        c.data_ptr(), nnz, nodes, tp.data_ptr() if deterministic else 0, stream)
    call(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert rel_err(z.cpu().numpy(), Zr) <= FP32_TOL
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):          # (a hipMalloc inside the library would invalidate the capture)
        call(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    for k in range(3):
        z.fill_(float("nan"))
        x.mul_(1.0)                                   # eager work of the program between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert rel_err(z.cpu().numpy(), Zr) <= FP32_TOL, f"replay {k}"


def test_noalloc_rejects_graphs_beyond_the_scratch(cuda):
    import torch
    import openequivariance_amd as oeq
    from openequivariance_amd import runtime as rt
    prob, _ = common.channelwise(common.NEQUIP)
    conv = oeq.TensorProductConv(prob, torch_op=False, deterministic=False)
    nnz = rt.NOALLOC_SCRATCH_BYTES // 8          # two pointer arrays on top of this no longer fit
    one = torch.zeros(16, device=cuda)
    with pytest.raises(RuntimeError, match="static scratch holds"):
        conv.internal.exec_conv_noalloc(one.data_ptr(), one.data_ptr(), one.data_ptr(), one.data_ptr(), one.data_ptr(),
                                        one.data_ptr(), nnz, 10, 0, 0)
    torch.cuda.synchronize()
