"""With ``graph_cache=True`` the convolution reuses the graph preparation (CSR pointers, position lists,
node order) that a call leaves in its workspace while the index tensors are unchanged, and rebuilds it
when they change: in place (version counter), by new tensors, or by sizes.  By default it prepares the
graph on every call, so writes that torch's version counter cannot see are always picked up.  Also: int32
index tensors, per-stream workspaces, and the raw entry points' ``prepared`` flag."""
import numpy as np
import pytest

import common
from common import FP32_TOL, rel_err
from oracle import tp as otp

pytestmark = pytest.mark.gpu


def _inputs(prob, nodes, nnz, seed, deterministic, cuda, idx=np.int64):
    import torch
    rows, cols = common.random_graph(nodes, nnz, seed)
    tperm = None
    if deterministic:
        rows, cols, tperm, _ = otp.coord_graph(rows, cols)
    X, Y, W, G = common.conv_inputs(prob, nodes, nnz, seed, np.float32)
    t = [torch.tensor(a, device=cuda, requires_grad=True) for a in (X, Y, W)]
    index = [torch.tensor(a.astype(idx), device=cuda) for a in ((rows, cols, tperm) if deterministic else (rows, cols))]
    return (X, Y, W, G), (rows, cols), t, index, torch.tensor(G, device=cuda)


def _check(oprob, host, graph, conv, t, index, g):
    import torch
    for a in t:
        a.grad = None
    z = conv.forward(*t, *index)
    z.backward(g)
    torch.cuda.synchronize()
    X, Y, W, G = host
    rows, cols = graph
    assert rel_err(z.detach().cpu().numpy(), otp.conv_forward(oprob, X, Y, W, rows, cols)) <= FP32_TOL
    for got, ref in zip((a.grad for a in t), otp.conv_backward(oprob, X, Y, W, G, rows, cols)):
        assert rel_err(got.cpu().numpy(), ref) <= FP32_TOL
    return z.detach().clone()


@pytest.mark.parametrize("deterministic", [True, False])
@pytest.mark.parametrize("irreps", [common.NEQUIP, common.LARGE], ids=["nequip", "large"])
def test_preparation_is_reused_and_rebuilt(cuda, deterministic, irreps):
    import torch
    import openequivariance_amd as oeq
    prob, oprob = common.channelwise(irreps)
    conv = oeq.TensorProductConv(prob, torch_op=True, deterministic=deterministic, graph_cache=True)
    nodes, nnz = 60, 900
    host, graph, t, index, g = _inputs(prob, nodes, nnz, 5, deterministic, cuda)
    rec = lambda: conv._workspace_record(nnz, nodes)
    _check(oprob, host, graph, conv, t, index, g)     # first call: the unsorted operator may compile a second backward
    z1 = _check(oprob, host, graph, conv, t, index, g)  # variant while timing, and grow its workspace for it
    assert rec().fwd_key is not None and rec().bwd_key is not None
    key = (rec().fwd_key, rec().bwd_key)
    # second call on the same tensors: the preparation kernels are skipped, results unchanged
    z2 = _check(oprob, host, graph, conv, t, index, g)
    assert (rec().fwd_key, rec().bwd_key) == key
    if deterministic:
        assert torch.equal(z1, z2)

    # in-place change of the edge list: same addresses, new contents -> rebuilt
    host2, graph2, _, index2, _ = _inputs(prob, nodes, nnz, 6, deterministic, cuda)
    for dst, src in zip(index, index2):
        dst.copy_(src)
    assert tuple(i.data_ptr() for i in index) == tuple(k[0] for k in key[0][3:])
    _check(oprob, (host[0], host[1], host[2], host[3]), graph2, conv, t, index, g)
    assert rec().fwd_key != key[0]

    # a smaller graph in new tensors, then the first graph's sizes again
    host3, graph3, t3, index3, g3 = _inputs(prob, nodes - 7, nnz // 3, 7, deterministic, cuda)
    _check(oprob, host3, graph3, conv, t3, index3, g3)
    _check(oprob, host, graph2, conv, t, index, g)


@pytest.mark.parametrize("deterministic", [True, False])
def test_cache_is_off_by_default_and_sees_writes_behind_torchs_back(cuda, deterministic):
    """The default operator prepares the graph on every call.  The index tensors are rewritten through an
    alias that does not bump their version counter (a view made by from_dlpack of the same memory: the
    hazard of neighbour lists written by another library): results must follow the new contents.  The same
    alias goes unnoticed by an operator built with graph_cache=True, which is why that is opt-in."""
    import torch
    import openequivariance_amd as oeq
    from openequivariance_amd import tunables
    assert tunables.current.graph_cache is False
    prob, oprob = common.channelwise(common.NEQUIP)
    conv = oeq.TensorProductConv(prob, torch_op=True, deterministic=deterministic)
    assert conv.graph_cache is False
    nodes, nnz = 40, 500
    host, graph, t, index, g = _inputs(prob, nodes, nnz, 8, deterministic, cuda)
    _check(oprob, host, graph, conv, t, index, g)
    assert conv._workspace_record(nnz, nodes).fwd_key is None
    _, graph2, _, index2, _ = _inputs(prob, nodes, nnz, 9, deterministic, cuda)
    versions = [i._version for i in index]
    for dst, src in zip(index, index2):
        torch.utils.dlpack.from_dlpack(torch.utils.dlpack.to_dlpack(dst)).copy_(src)
    torch.cuda.synchronize()
    assert [i._version for i in index] == versions, "the alias must not bump the version counters"
    _check(oprob, host, graph2, conv, t, index, g)           # fresh results from the rewritten edge list


@pytest.mark.parametrize("deterministic", [True, False])
@pytest.mark.parametrize("irreps", [common.NEQUIP, common.LARGE, common.MACE], ids=["nequip", "large", "mace"])
def test_int32_indices(cuda, deterministic, irreps):
    """reference: LoopUnrollConv.py:53,78 accepts int32 and int64 index tensors.  (The MACE problem takes the
    receiver-order backward when deterministic.)"""
    import torch
    import openequivariance_amd as oeq
    prob, oprob = common.channelwise(irreps)
    conv = oeq.TensorProductConv(prob, torch_op=True, deterministic=deterministic, idx_dtype=np.int32)
    host, graph, t, index, g = _inputs(prob, 50, 800, 9, deterministic, cuda, idx=np.int32)
    assert all(i.dtype == torch.int32 for i in index)
    _check(oprob, host, graph, conv, t, index, g)
    _check(oprob, host, graph, conv, t, index, g)
    with pytest.raises(TypeError):
        conv.forward(*t, *[i.long() for i in index])


def test_streams_have_their_own_workspaces(cuda):
    import torch
    import openequivariance_amd as oeq
    prob, oprob = common.channelwise(common.NEQUIP)
    conv = oeq.TensorProductConv(prob, torch_op=True, deterministic=True)
    a = _inputs(prob, 50, 700, 10, True, cuda)
    b = _inputs(prob, 45, 650, 11, True, cuda)
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    za = conv.forward(*a[2], *a[3])
    with torch.cuda.stream(side):
        zb = conv.forward(*b[2], *b[3])
    torch.cuda.synchronize()
    assert len(conv._workspaces) == 2
    for (host, graph, *_), z in ((a, za), (b, zb)):
        X, Y, W, _ = host
        assert rel_err(z.detach().cpu().numpy(), otp.conv_forward(oprob, X, Y, W, *graph)) <= FP32_TOL


@pytest.mark.parametrize("deterministic", [True, False])
def test_raw_entry_points_with_prepared_workspace(cuda, deterministic):
    """Through the C ABI: a full call prepares the caller's workspace, *_prepared calls reuse it."""
    import torch
    import openequivariance_amd as oeq
    prob, oprob = common.channelwise(common.LARGE)          # grouped backward when unsorted
    conv = oeq.TensorProductConv(prob, torch_op=False, deterministic=deterministic)
    nodes, nnz = 30, 400
    host, graph, t, index, g = _inputs(prob, nodes, nnz, 12, deterministic, cuda)
    x, y, w = (a.detach() for a in t)
    tp = index[2].data_ptr() if deterministic else 0
    ws = torch.empty(conv._ws_bytes(nnz, nodes), dtype=torch.uint8, device=cuda)
    outs = []
    for prepared in (False, True, True):
        z = torch.full((nodes, prob.irreps_out.dim), float("nan"), device=cuda)
        xg, yg, wg = (torch.full_like(a, float("nan")) for a in (x, y, w))
        if not conv.backward_overwrites:
            xg.zero_()
        conv.exec_conv_rawptrs(x.data_ptr(), y.data_ptr(), w.data_ptr(), z.data_ptr(), index[0].data_ptr(),
                               index[1].data_ptr(), nnz, nodes, ws.data_ptr(), tp, prepared=prepared)
        conv.backward_rawptrs(x.data_ptr(), xg.data_ptr(), y.data_ptr(), yg.data_ptr(), w.data_ptr(), wg.data_ptr(),
                              g.data_ptr(), index[0].data_ptr(), index[1].data_ptr(), nnz, nodes, ws.data_ptr(), tp,
                              prepared=prepared)
        torch.cuda.synchronize()
        outs.append((z, xg, yg, wg))
    X, Y, W, G = host
    refs = (otp.conv_forward(oprob, X, Y, W, *graph),) + tuple(otp.conv_backward(oprob, X, Y, W, G, *graph))
    for got in outs:
        for a, b in zip(got, refs):
            assert rel_err(a.cpu().numpy(), b) <= FP32_TOL
    if deterministic:
        for a, b in zip(outs[0], outs[2]):
            assert torch.equal(a, b)


def test_unsorted_backward_variant_is_chosen_by_measurement(cuda, monkeypatch):
    """The first backward call of a size class times the atomic and the grouped backward on the caller's
    tensors and keeps the faster; both give the oracle's gradients; overrides switch the timing off."""
    import openequivariance_amd as oeq
    from openequivariance_amd import tunables
    monkeypatch.setattr(tunables.current, "conv_backward", None)
    monkeypatch.setattr(tunables.current, "autotune", True)
    prob, oprob = common.channelwise(common.NEQUIP)
    conv = oeq.TensorProductConv(prob, torch_op=True, deterministic=False)
    assert conv.autotune and conv._bwd_default == "grouped"
    host, graph, t, index, g = _inputs(prob, 70, 1500, 13, False, cuda)
    _check(oprob, host, graph, conv, t, index, g)
    assert set(conv.last_tuning) == {"atomic", "grouped"} and len(conv._bwd_choice) == 1
    chosen = next(iter(conv._bwd_choice.values()))
    assert chosen == min(conv.last_tuning, key=conv.last_tuning.get)
    conv.last_tuning = None
    _check(oprob, host, graph, conv, t, index, g)            # same size class: no second measurement
    assert conv.last_tuning is None
    for name in ("atomic", "grouped"):                       # either variant, forced, against the oracle
        conv._bwd_choice = {k: name for k in conv._bwd_choice}
        _check(oprob, host, graph, conv, t, index, g)
    monkeypatch.setattr(tunables.current, "autotune", False)
    assert not oeq.TensorProductConv(prob, torch_op=True, deterministic=False).autotune
    assert not oeq.TensorProductConv(prob, torch_op=True, deterministic=True).autotune
