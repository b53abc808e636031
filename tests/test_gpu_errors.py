"""Error behaviour of the operators: no silent fallback, shapes and dtypes are checked before any
kernel is launched."""
import numpy as np
import pytest

import common

pytestmark = pytest.mark.gpu


def test_tensor_product_rejects_bad_inputs(cuda):
    import torch
    import openequivariance_amd as oeq
    prob, _ = common.channelwise(common.NEQUIP)
    tp = oeq.TensorProduct(prob, torch_op=True)
    x, y, w = (torch.randn(10, d, device=cuda) for d in (288, 9, 352))
    assert tp(x, y, w).shape == (10, 1120)
    with pytest.raises(ValueError):
        tp(x[:, :-1], y, w)
    with pytest.raises(ValueError):
        tp(x, y[:5], w)
    with pytest.raises(ValueError):
        tp(x, y, w[0])                       # per-row weights expected
    with pytest.raises(TypeError):
        tp(x.double(), y.double(), w.double())
    with pytest.raises((NotImplementedError, RuntimeError)):
        tp(x.cpu(), y.cpu(), w.cpu())        # there is no CPU implementation
    assert tp(x[:0], y[:0], w[:0]).shape == (0, 1120)


@pytest.mark.parametrize("deterministic", [False, True])
def test_convolution_rejects_bad_inputs(cuda, deterministic):
    import torch
    import openequivariance_amd as oeq
    prob, _ = common.channelwise(common.NEQUIP)
    conv = oeq.TensorProductConv(prob, torch_op=True, deterministic=deterministic)
    x, y, w = torch.randn(6, 288, device=cuda), torch.randn(12, 9, device=cuda), torch.randn(12, 352, device=cuda)
    rows = torch.arange(12, device=cuda) // 2
    cols = (rows + 1) % 6
    extra = [torch.argsort(cols * 6 + rows, stable=True)] if deterministic else []
    assert conv.forward(x, y, w, rows, cols, *extra).shape == (6, 1120)
    with pytest.raises(ValueError):
        conv.forward(x, y[:5], w, rows, cols, *extra)
    with pytest.raises(ValueError):
        conv.forward(x, y, w[:, :-1], rows, cols, *extra)
    with pytest.raises(TypeError):
        conv.forward(x, y, w, rows.int(), cols.int(), *extra)
    with pytest.raises(TypeError):
        conv.forward(x.double(), y.double(), w.double(), rows, cols, *extra)
    # edges that name no node contribute nothing and do not fault
    bad = rows.clone()
    bad[0] = 99
    if not deterministic:
        z = conv.forward(x, y, w, bad, cols)
        assert torch.isfinite(z).all()


@pytest.mark.parametrize("deterministic", [False, True])
def test_pointers_that_kernels_would_dereference_are_checked_first(cuda, deterministic):
    """Host tensors among GPU tensors, a missing transpose permutation and a NULL workspace are
    rejected on the host, in Python and again behind the C ABI; no kernel is launched with them."""
    import torch
    import openequivariance_amd as oeq
    from openequivariance_amd import runtime as rt
    prob, _ = common.channelwise(common.NEQUIP)
    conv = oeq.TensorProductConv(prob, torch_op=True, deterministic=deterministic)
    x, y, w = torch.randn(6, 288, device=cuda), torch.randn(12, 9, device=cuda), torch.randn(12, 352, device=cuda)
    rows = torch.arange(12, device=cuda) // 2
    cols = (rows + 1) % 6
    extra = [torch.argsort(cols * 6 + rows, stable=True)] if deterministic else []
    with pytest.raises(ValueError, match="must be on the GPU"):
        conv.forward(x, y, w, rows.cpu(), cols, *extra)
    with pytest.raises(ValueError, match="must be on the GPU"):
        conv.forward(x, y.cpu(), w, rows, cols, *extra)
    if deterministic:
        with pytest.raises(ValueError, match="must be on the GPU"):
            conv.forward(x, y, w, rows, cols, extra[0].cpu())
        z, xg, yg, wg = torch.empty(6, 1120, device=cuda), torch.empty_like(x), torch.empty_like(y), torch.empty_like(w)
        with pytest.raises(ValueError, match="transpose_perm"):
            conv.backward_rawptrs(x.data_ptr(), xg.data_ptr(), y.data_ptr(), yg.data_ptr(), w.data_ptr(), wg.data_ptr(),
                                  z.data_ptr(), rows.data_ptr(), cols.data_ptr(), 12, 6)
        with pytest.raises(RuntimeError, match="transpose permutation"):      # the library checks again
            conv.internal.backward_rawptrs(x.data_ptr(), xg.data_ptr(), y.data_ptr(), yg.data_ptr(), w.data_ptr(),
                                           wg.data_ptr(), z.data_ptr(), rows.data_ptr(), cols.data_ptr(), 12, 6,
                                           conv.workspace_ptr(12, 6), 0, 0)
    z = torch.empty(6, 1120, device=cuda)
    with pytest.raises(RuntimeError, match="needs a workspace"):
        conv.internal.exec_conv_rawptrs(x.data_ptr(), y.data_ptr(), w.data_ptr(), z.data_ptr(), rows.data_ptr(),
                                        cols.data_ptr(), 12, 6, 0, extra[0].data_ptr() if extra else 0, 0)
    with pytest.raises(RuntimeError, match="rows / cols"):
        conv.internal.exec_conv_rawptrs(x.data_ptr(), y.data_ptr(), w.data_ptr(), z.data_ptr(), 0, 0, 12, 6,
                                        conv.workspace_ptr(12, 6), 0, 0)
    torch.cuda.synchronize()


def test_tensor_product_rejects_host_tensors_among_gpu_tensors(cuda):
    import torch
    import openequivariance_amd as oeq
    prob, _ = common.channelwise(common.NEQUIP)
    tp = oeq.TensorProduct(prob, torch_op=True)
    x, y, w = (torch.randn(10, d, device=cuda) for d in (288, 9, 352))
    with pytest.raises(ValueError, match="must be on the GPU"):
        tp(x, y.cpu(), w)
    shared = oeq.TensorProduct(oeq.FullyConnectedTPProblem("4x0e", "1x0e", "4x0e", shared_weights=True,
                                                           internal_weights=False), torch_op=True)
    xs, ys, ws_ = torch.randn(5, 4, device=cuda), torch.randn(5, 1, device=cuda), torch.randn(16, device=cuda)
    zs = torch.empty(5, 4, device=cuda)
    with pytest.raises(RuntimeError, match="needs a workspace"):     # behind the C ABI as well
        shared.internal.exec_tensor_product(5, xs.data_ptr(), ys.data_ptr(), zs.data_ptr(), ws_.data_ptr(), 0, 0)
    torch.cuda.synchronize()


@pytest.mark.parametrize("variant", ["det", "det_recv", "unsorted_atomic", "unsorted_grouped", "unsorted_grouped_recv"])
@pytest.mark.parametrize("irreps", [common.NEQUIP, common.LARGE], ids=["nequip", "large"])
def test_edges_naming_no_node_contribute_nothing(cuda, variant, irreps, monkeypatch):
    """Out-of-range senders / receivers: no fault, Z and dX as if those edges were absent, and their dW /
    dY rows are zeros from every backward variant."""
    import torch
    import openequivariance_amd as oeq
    from oracle import tp as otp
    from openequivariance_amd import tunables
    monkeypatch.setattr(tunables.current, "autotune", False)
    monkeypatch.setattr(tunables.current, "det_backward", "recv" if variant == "det_recv" else "send")
    if variant.startswith("unsorted"):
        from openequivariance_amd.codegen.uvu_sorted import UVUSortedGenerator
        monkeypatch.setattr(tunables.current, "conv_backward", variant.split("_")[1])
        # (the grouped backward in receiver order is chosen for long dZ rows; here for every shape, or for none)
        monkeypatch.setattr(UVUSortedGenerator, "RECV_ORDER_MIN_RATIO", 0 if variant.endswith("_recv") else 1e9)
    deterministic = variant.startswith("det")
    prob, oprob = common.channelwise(irreps)
    nodes, nnz = 40, 900
    rows, cols = common.random_graph(nodes, nnz, 71, self_loops=True)
    rows, cols, valid = common.with_invalid_edges(rows, cols, nodes, 72, count=9)
    index = [rows, cols]
    if deterministic:
        order = np.lexsort((cols, rows))
        rows, cols, valid = rows[order], cols[order], valid[order]
        index = [rows, cols, np.lexsort((np.arange(nnz), rows, cols)).astype(np.int64)]
    X, Y, W, G = common.conv_inputs(prob, nodes, nnz, 73)
    Zr, dXr, dYr, dWr = common.conv_reference_on_valid_edges(otp, oprob, X, Y, W, G, rows, cols, valid)
    conv = oeq.TensorProductConv(prob, torch_op=True, deterministic=deterministic)
    assert getattr(conv.generator, "recv_backward", False) == variant.endswith("grouped_recv")
    x, y, w = (torch.tensor(a, device=cuda, requires_grad=True) for a in (X, Y, W))
    idx = [torch.tensor(a, device=cuda) for a in index]
    for _ in range(2):                               # second pass: graph preparation reused
        for t in (x, y, w):
            t.grad = None
        z = conv.forward(x, y, w, *idx)
        z.backward(torch.tensor(G, device=cuda))
        torch.cuda.synchronize()
        assert common.rel_err(z.detach().cpu().numpy(), Zr) <= common.FP32_TOL
        assert common.rel_err(x.grad.cpu().numpy(), dXr) <= common.FP32_TOL
        assert common.rel_err(y.grad.cpu().numpy(), dYr) <= common.FP32_TOL
        assert common.rel_err(w.grad.cpu().numpy(), dWr) <= common.FP32_TOL
        bad = torch.tensor(~valid, device=cuda)
        assert not w.grad[bad].any() and not y.grad[bad].any()


def test_unsupported_problems_raise():
    import openequivariance_amd as oeq
    with pytest.raises(AssertionError):           # the convolution needs multiplicity 1 on the second operand
        oeq.TensorProductConv(oeq.TPProblem("2x0e", "2x0e", "2x0e", [(0, 0, 0, "uvu", True)], shared_weights=False,
                                            internal_weights=False))
    with pytest.raises(NotImplementedError):
        oeq.TensorProductConv(oeq.FullyConnectedTPProblem("4x0e", "1x0e", "4x0e", shared_weights=False, internal_weights=False))
