"""Fused convolution at the full sizes of the benchmark configurations 3 and 5.

The oracle cannot run 800 000 edges of the large problem in seconds, so the full-size runs are
checked through what does not depend on the size: every output row of a node depends only on the
edges of that node, and every per-edge output only on that edge, so sampled nodes and edges are
compared with the oracle on the sub-graph that determines them; the deterministic variant must
repeat bit for bit; and the two variants must agree with each other on the same inputs.
"""
import numpy as np
import pytest

import common
from common import FP32_TOL, rel_err
from oracle import tp as otp

pytestmark = pytest.mark.gpu


def _device_inputs(prob, nodes, rows, sh_lmax, seed, dev):
    """Inputs generated on the GPU (the large problem's weights are 10.6 GB); Y on the host from
    seeded unit vectors."""
    import torch
    from openequivariance_amd.sh import random_unit_vectors, spherical_harmonics
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    nnz = rows.shape[0]
    d1, d3, wn = prob.irreps_in1.dim, prob.irreps_out.dim, prob.weight_numel
    x = torch.randn(nodes, d1, device=dev, generator=gen)
    w = torch.randn(nnz, wn, device=dev, generator=gen)
    g = torch.randn(nodes, d3, device=dev, generator=gen)
    Y = spherical_harmonics(sh_lmax, random_unit_vectors(nnz, np.random.default_rng(seed))).astype(np.float32)
    return x, torch.from_numpy(Y).to(dev), w, g


def _check_sampled(oprob, x, y, w, g, rows, cols, z, dx, dy, dw, seed, n_nodes=12):
    """Sampled receivers (forward rows), sampled senders (dX rows) and their edges (dW, dY rows)
    against the oracle run on exactly the edges that determine them."""
    import torch
    rng = np.random.default_rng(seed)
    nodes = x.shape[0]
    X = x.cpu().numpy()
    G = g.cpu().numpy()
    dev = x.device

    def edge_subset(mask):
        idx = np.nonzero(mask)[0]
        t = torch.from_numpy(idx).to(dev)
        return idx, y[t].cpu().numpy(), w[t].cpu().numpy()

    rcv = rng.choice(nodes, n_nodes, replace=False)
    idx, Ys, Ws = edge_subset(np.isin(rows, rcv))
    Zr = otp.conv_forward(oprob, X, Ys, Ws, rows[idx], cols[idx])
    err = {"Z": rel_err(z[torch.from_numpy(rcv).to(dev)].cpu().numpy(), Zr[rcv])}
    snd = rng.choice(nodes, n_nodes, replace=False)
    idx, Ys, Ws = edge_subset(np.isin(cols, snd))
    dXr, dYr, dWr = otp.conv_backward(oprob, X, Ys, Ws, G, rows[idx], cols[idx])
    t = torch.from_numpy(idx).to(dev)
    err["dX"] = rel_err(dx[torch.from_numpy(snd).to(dev)].cpu().numpy(), dXr[snd])
    err["dY"] = rel_err(dy[t].cpu().numpy(), dYr)
    err["dW"] = rel_err(dw[t].cpu().numpy(), dWr)
    print(f"sampled {n_nodes} receivers / {n_nodes} senders ({len(idx)} edges): {err}", flush=True)
    for k, v in err.items():
        assert v <= FP32_TOL, f"{k}: relative error {v:.3e}"


def _run(conv, x, y, w, g, idx):
    for t in (x, y, w):
        t.grad = None
        t.requires_grad_(True)
    z = conv.forward(x, y, w, *idx)
    z.backward(g)
    return z.detach(), x.grad, y.grad, w.grad


def _full_size(name, irreps, sh_lmax, cuda, n_nodes):
    import torch
    import openequivariance_amd as oeq
    from openequivariance_amd import workloads
    wl = workloads.get(name)
    prob, oprob = common.channelwise(irreps)
    rows, cols, tperm = wl.graph(np.random.default_rng(wl.seed))
    nodes = wl.nodes
    print(f"{name}: {nodes} nodes, {rows.size} edges", flush=True)
    x, y, w, g = _device_inputs(prob, nodes, rows, sh_lmax, wl.seed, cuda)
    r, c, tp = (torch.from_numpy(a).to(cuda) for a in (rows, cols, tperm))

    det = oeq.TensorProductConv(prob, torch_op=True, deterministic=True)
    z, dx, dy, dw = _run(det, x, y, w, g, (r, c, tp))
    torch.cuda.synchronize()
    _check_sampled(oprob, x.detach(), y.detach(), w.detach(), g, rows, cols, z, dx, dy, dw, wl.seed, n_nodes)

    # bit-reproducible (reference protocol: convolution/ConvolutionBase.py:229-247)
    z2, dx2, dy2, dw2 = _run(det, x, y, w, g, (r, c, tp))
    for a, b in ((z, z2), (dx, dx2), (dy, dy2), (dw, dw2)):
        assert torch.equal(a, b)
    del z2, dx2, dy2, dw2

    # the variant for unsorted graphs on the same edges, handed over in a shuffled order
    perm = torch.randperm(rows.size, device=cuda, generator=torch.Generator(device=cuda).manual_seed(1))
    free = oeq.TensorProductConv(prob, torch_op=True, deterministic=False)
    ys, ws_ = y.detach()[perm].clone(), w.detach()[perm].clone()
    zf, dxf, dyf, dwf = _run(free, x, ys, ws_, g, (r[perm], c[perm]))
    torch.cuda.synchronize()

    def close(a, b, what):
        e = float((a - b).abs().max() / b.abs().max())
        assert e <= FP32_TOL, f"{what}: variants differ by {e:.3e}"
    close(zf, z, "Z")
    close(dxf, dx, "dX")
    close(dyf, dy[perm], "dY")
    close(dwf, dw[perm], "dW")


def test_nequip_conv_full_size(cuda):
    """benchmark configuration 3: 5 000 nodes, 150 000 edges."""
    _full_size("nequip_conv_det", common.NEQUIP, 2, cuda, 40)


def test_large_conv_full_size(cuda):
    """benchmark configuration 5: 20 000 nodes, Poisson(40) in-degree (about 800 000 edges)."""
    _full_size("large_conv_det", common.LARGE, 3, cuda, 6)
