"""GPU parity of the fused convolution (atomic and deterministic) against the fp64 oracle."""
import numpy as np
import pytest

import common
from common import FP32_TOL, FP64_TOL, rel_err
from oracle import tp as otp

pytestmark = pytest.mark.gpu


def _graph(nodes, nnz, seed, sort):
    rows, cols = common.random_graph(nodes, nnz, seed)
    tperm = None
    if sort:
        rows, cols, tperm, _ = otp.coord_graph(rows, cols)
    return rows, cols, tperm


def _run(prob, oprob, nodes, nnz, seed, deterministic, dtype=np.float32, sh_lmax=None, graph=None):
    import torch
    import openequivariance_amd as oeq
    tol = FP32_TOL if dtype == np.float32 else FP64_TOL
    rows, cols, tperm = graph if graph is not None else _graph(nodes, nnz, seed, deterministic)
    nnz = len(rows)
    X, Y, W, G = common.conv_inputs(prob, nodes, nnz, seed, dtype, sh_lmax)
    conv = oeq.TensorProductConv(prob, torch_op=True, deterministic=deterministic)
    dev = torch.device("cuda:0")
    x, y, w = (torch.tensor(a, device=dev, requires_grad=True) for a in (X, Y, W))
    idx = [torch.tensor(a, device=dev) for a in ((rows, cols, tperm) if deterministic else (rows, cols))]
    z = conv.forward(x, y, w, *idx)
    z.backward(torch.tensor(G, device=dev))
    torch.cuda.synchronize()
    Zr = otp.conv_forward(oprob, X, Y, W, rows, cols)
    dXr, dYr, dWr = otp.conv_backward(oprob, X, Y, W, G, rows, cols)
    errs = dict(Z=rel_err(z.detach().cpu().numpy(), Zr), dX=rel_err(x.grad.cpu().numpy(), dXr),
                dY=rel_err(y.grad.cpu().numpy(), dYr), dW=rel_err(w.grad.cpu().numpy(), dWr))
    print(f"nodes={nodes} nnz={nnz} det={deterministic} {errs}", flush=True)
    for k, v in errs.items():
        assert v <= tol, f"{k}: relative error {v:.3e} > {tol}"
    return conv, (x, y, w, idx, z, torch.tensor(G, device=dev))


@pytest.mark.parametrize("deterministic", [False, True])
def test_nequip_conv(cuda, deterministic):
    """benchmark configuration 3 problem on a scaled-down random graph (no self loops)."""
    prob, oprob = common.channelwise(common.NEQUIP)
    _run(prob, oprob, 300, 9001, 31, deterministic, sh_lmax=2)


@pytest.mark.parametrize("deterministic", [False, True])
def test_large_conv(cuda, deterministic):
    """benchmark configuration 5 problem (mul 256 = four chunks) on a small graph."""
    prob, oprob = common.channelwise(common.LARGE)
    _run(prob, oprob, 40, 700, 32, deterministic, sh_lmax=3)


@pytest.mark.parametrize("deterministic", [False, True])
def test_readme_conv(cuda, deterministic):
    prob, oprob = common.readme_problem()
    _run(prob, oprob, 130, 1000, 33, deterministic)


@pytest.mark.parametrize("deterministic", [False, True])
def test_ragged_conv(cuda, deterministic):
    irreps = ("5x0e+3x1o+70x2e", "1x0e+1x1o+1x2e", "5x0e+3x1o+70x2e+7x3o")
    prob, oprob = common.channelwise(irreps)
    _run(prob, oprob, 50, 333, 34, deterministic)


@pytest.mark.parametrize("deterministic", [False, True])
@pytest.mark.parametrize("which", ["nequip", "large"])
def test_conv_outputs_of_either_parity(cuda, which, deterministic):
    """The literal reading of the benchmark configurations 3 and 5: every triangle-allowed l3 <= 2 with the
    output parity p1 * p2, which adds the 1e and 2o outputs (15 and 18 paths)."""
    from openequivariance_amd import workloads
    irreps = workloads.NEQUIP_ALL if which == "nequip" else workloads.LARGE_ALL
    prob, oprob = common.channelwise(irreps)
    assert len(prob.instructions) == (15 if which == "nequip" else 18)
    if which == "nequip":
        _run(prob, oprob, 200, 5000, 37, deterministic, sh_lmax=2)
    else:
        _run(prob, oprob, 30, 400, 38, deterministic, sh_lmax=3)


def test_deterministic_backward_order_is_chosen_by_shape(cuda):
    """Static rule: the two-pass receiver-order backward when a dZ row is at least 5.5 times as long as an X row
    and pass 1 can stage its operands through LDS (fp32, at least as many channels per row group as Y
    components): the MACE problem (7.9) and configs 3 and 5 with outputs of either parity (5.7, 7.1) take it,
    configs 3 and 5 themselves (3.9, 4.8) keep the sender order.  fp64 has no stage: the receiver order is taken where
    pass 1 can run as one launch per in1 block with at most 32 dZ words held (the MACE problem), not otherwise."""
    from openequivariance_amd import workloads
    from openequivariance_amd.codegen.uvu_recv import UVURecvGenerator
    from openequivariance_amd.conv import select_conv_generator
    for irreps in (common.MACE, workloads.NEQUIP_ALL, workloads.LARGE_ALL):
        g = select_conv_generator(common.channelwise(irreps)[0], True)
        assert isinstance(g, UVURecvGenerator) and g.staged_edges and g.regroup_pairs
    for irreps in (common.NEQUIP, common.LARGE):
        assert not isinstance(select_conv_generator(common.channelwise(irreps)[0], True), UVURecvGenerator)
    g = select_conv_generator(common.channelwise(common.MACE, dtype=np.float64)[0], True)
    assert isinstance(g, UVURecvGenerator) and not g.staged_edges and g.HR == 3
    for irreps in (common.NEQUIP, workloads.MACE_ALL):
        assert not isinstance(select_conv_generator(common.channelwise(irreps, dtype=np.float64)[0], True), UVURecvGenerator)
    prob, oprob = common.channelwise(common.MACE)
    _run(prob, oprob, 60, 900, 40, True, sh_lmax=3)
    prob, oprob = common.channelwise(common.MACE, dtype=np.float64)
    _run(prob, oprob, 60, 900, 41, True, dtype=np.float64, sh_lmax=3)


def test_unsorted_mace_conv_backward_in_receiver_order(cuda, monkeypatch):
    """The unsorted operator's grouped backward takes the receiver order for long dZ rows: it then builds both
    groupings (by receiver for pass 1, by sender for pass 2) in the backward call."""
    from openequivariance_amd import tunables
    monkeypatch.setattr(tunables.current, "autotune", False)
    prob, oprob = common.channelwise(common.MACE)
    conv, _ = _run(prob, oprob, 60, 900, 42, False, sh_lmax=3)
    assert conv.generator.grouped_backward and conv.generator.recv_backward
    prob, oprob = common.channelwise(common.NEQUIP)
    conv, _ = _run(prob, oprob, 60, 900, 43, False, sh_lmax=2)
    assert not conv.generator.recv_backward


def test_unsorted_fp64_conv_backward_in_receiver_order_on_request(cuda, monkeypatch):
    """fp64 over an unsorted edge list keeps the sender order by default; the receiver order with register loads (one
    launch of pass 1 per in1 block, over the receiver-grouped position list) runs when the generator is asked for it."""
    import openequivariance_amd.conv as conv_mod
    from openequivariance_amd import tunables
    from openequivariance_amd.codegen.uvu_sorted import UVUSortedGenerator
    monkeypatch.setattr(tunables.current, "autotune", False)
    prob, oprob = common.channelwise(common.MACE, dtype=np.float64)
    conv, _ = _run(prob, oprob, 60, 900, 44, False, dtype=np.float64, sh_lmax=3)
    assert not conv.generator.recv_backward

    def pick(config, deterministic, vector_stores=True, idx_dtype=np.int64):
        assert not deterministic
        return UVUSortedGenerator(config, vector_stores=vector_stores, grouped_backward=True, recv_backward=True,
                                  idx_ctype="i64" if np.dtype(idx_dtype) == np.dtype(np.int64) else "int")
    monkeypatch.setattr(conv_mod, "select_conv_generator", pick)
    rows, cols = common.hub_graph(59, 900, 45, hub_in=3, hub_out=5, in_edges=300, out_edges=200)
    conv, _ = _run(prob, oprob, 60, 900, 45, False, dtype=np.float64, sh_lmax=3, graph=(rows, cols, None))
    b = conv.generator.bwd
    assert conv.generator.recv_backward and not b.staged_edges and b.HR == 3


@pytest.mark.parametrize("deterministic", [False, True])
def test_mace_conv_backward_split_over_output_blocks(cuda, deterministic, monkeypatch):
    """The MACE problem as a convolution in sender order: 104 registers of operands per edge, so the backward
    runs as two launches over two groups of output blocks (the second adds to dX; dY through per-group partials)."""
    from openequivariance_amd import tunables
    from openequivariance_amd.conv import select_conv_generator
    from openequivariance_amd.codegen.uvu_sorted import UVUSortedGenerator
    monkeypatch.setattr(tunables.current, "det_backward", "send")
    monkeypatch.setattr(UVUSortedGenerator, "RECV_ORDER_MIN_RATIO", 1e9)
    prob, oprob = common.channelwise(common.MACE)
    gen = select_conv_generator(prob, True)
    assert gen.H == 2 and sorted(sum(gen.out_groups, [])) == gen.used_out
    _run(prob, oprob, 60, 900, 39, deterministic, sh_lmax=3)


@pytest.mark.parametrize("staged", [True, False])
@pytest.mark.parametrize("which", ["nequip", "large", "mace", "ragged", "few_channels"])
def test_receiver_order_backward(cuda, which, staged, monkeypatch):
    """The two-pass backward of the deterministic variant, forced for every shape here, pass 1 with the next
    edge's operands staged through LDS and with plain register loads (what fp64 problems and rows with fewer
    channels than Y components get): parity, and bit-equal repeats."""
    import torch
    from openequivariance_amd import tunables
    from openequivariance_amd.codegen.uvu_recv import UVURecvGenerator
    monkeypatch.setattr(tunables.current, "det_backward", "recv")
    if not staged:
        init = UVURecvGenerator.__init__
        monkeypatch.setattr(UVURecvGenerator, "__init__", lambda self, *a, **k: init(self, *a, **{**k, "staged": False}))
    irreps = {"nequip": common.NEQUIP, "large": common.LARGE, "mace": common.MACE,
              "ragged": ("5x0e+3x1o+70x2e", "1x0e+1x1o+1x2e", "5x0e+3x1o+70x2e+7x3o"),
              "few_channels": ("8x0e+8x1o", "1x0e+1x1o+1x2e", "8x0e+8x1o+8x2e")}[which]
    prob, oprob = common.channelwise(irreps)
    nodes, nnz = (300, 9001) if which == "nequip" else (50, 1500)
    conv, (x, y, w, idx, z, g) = _run(prob, oprob, nodes, nnz, 61, True)
    assert isinstance(conv.generator, UVURecvGenerator)
    assert conv.generator.staged_edges == (staged and which != "few_channels")
    first = [t.grad.clone() for t in (x, y, w)]
    for t in (x, y, w):
        t.grad = None
    conv.forward(x, y, w, *idx).backward(g)
    torch.cuda.synchronize()
    for a, b in zip(first, (x.grad, y.grad, w.grad)):
        assert torch.equal(a, b)


STAGED_SHAPES = {
    # one full 64-channel list, a single path, D = 1 output: every staged Y read has a constant LDS address,
    # which the compiler once moved behind the next transfer into the same slab
    "mul64_single_path_l1": ("64x1o", "1x0e+1x1o+1x2e+1x3o", "64x0e"),
    "mul64_single_path_l2": ("64x2e", "1x0e+1x1o+1x2e", "64x0e"),
    "mul16_four_sublists": ("16x0e+16x1o", "1x0e+1x1o+1x2e", "16x0e+16x1o+16x2e"),
    "mul8_eight_sublists": ("8x0e+8x1o", "1x0e+1x1o", "8x0e+8x1o"),
    "mul64_one_list": ("64x0e+64x1o", "1x0e+1x1o", "64x0e+64x1o"),
    "ragged_multiplicities": ("20x0e+9x1o+3x2e", "1x0e+1x1o+1x2e", "20x0e+9x1o+3x2e"),
    "l3_seven_word_records": ("16x0e+16x3o", "1x0e+1x1o+1x2e+1x3o", "16x0e+16x1o+16x3o"),
}


@pytest.mark.parametrize("shape", sorted(STAGED_SHAPES))
@pytest.mark.parametrize("variant", ["unsorted", "det_send", "det_recv"])
def test_lds_staged_edge_loop_shapes(cuda, shape, variant, monkeypatch):
    """Single-chunk fp32 problems run the edge loop that stages operands through LDS (deterministic:
    forward and backward, in sender order and in pass 1 of the receiver order; unsorted: forward): every
    sub-list count, ragged multiplicities, and records of 1, 3, 5 and 7 words (one, one, two and two LDS-DMA
    transfers), with long and empty edge lists."""
    from openequivariance_amd import tunables
    from openequivariance_amd.conv import select_conv_generator
    deterministic = variant != "unsorted"
    if deterministic:
        monkeypatch.setattr(tunables.current, "det_backward", variant[4:])
    prob, oprob = common.channelwise(STAGED_SHAPES[shape])
    gen = select_conv_generator(prob, deterministic)
    staged = gen if deterministic else gen.fwd
    assert staged.lds_forward
    assert {"unsorted": True, "det_send": staged.lds_backward, "det_recv": getattr(staged, "staged_edges", False)}[variant]
    _run(prob, oprob, 23, 700, 40, deterministic)        # about 30 edges per node
    _run(prob, oprob, 200, 150, 41, deterministic)       # most nodes have no edge or a single one


def test_conv_fp64(cuda):
    prob, oprob = common.channelwise(common.NEQUIP, dtype=np.float64)
    _run(prob, oprob, 64, 900, 35, True, dtype=np.float64, sh_lmax=2)
    _run(prob, oprob, 64, 900, 36, False, dtype=np.float64, sh_lmax=2)


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["fp32", "fp64"])
@pytest.mark.parametrize("deterministic", [False, True])
@pytest.mark.parametrize("which", ["nequip-lips", "nequip-revmd17-benzene"])
def test_conv_forward_in_groups_of_output_blocks(cuda, which, deterministic, dtype):
    """The reference's NequIP convolution problems with 30 and 68 paths (outputs of either parity up to l = 2 and
    3: 102 and 312 output words per channel): the forward runs one launch per group of output blocks, the backward
    likewise (fp32: receiver order, pass 1 per group of blocks sharing no in1 block; fp64: the same with register loads
    for the 30-path problem, sender order for the 68-path one); a hub node makes one edge list long enough to be walked in pieces."""
    from openequivariance_amd.benchmark import benchmark_configs as bc
    irreps = [c[:3] for c in bc.nequip_conv if c[3] == which][0]
    prob, oprob = common.channelwise(irreps, dtype=dtype)
    nodes, nnz = 40, 900
    rows, cols = common.hub_graph(nodes - 1, nnz, 61, hub_in=3, hub_out=5, in_edges=300, out_edges=200)
    tperm = None
    if deterministic:
        rows, cols, tperm, _ = otp.coord_graph(rows, cols)
    conv, _ = _run(prob, oprob, nodes, nnz, 62, deterministic, dtype=dtype, graph=(rows, cols, tperm))
    f = getattr(conv.generator, "fwd", conv.generator)
    assert len(f.fwd_groups) >= 2 and f.piece_tiles(nnz, nodes) > 0


@pytest.mark.parametrize("deterministic", [False, True])
def test_conv_fp64_ragged_chunks(cuda, deterministic):
    """fp64 with multiplicities above one wavefront (two chunks, the second partly filled) and below it."""
    irreps = ("70x0e+100x1o+5x2e", "1x0e+1x1o+1x2e", "70x0e+100x1o+70x1o+5x2e+100x2e")
    prob, oprob = common.channelwise(irreps, dtype=np.float64)
    _run(prob, oprob, 30, 500, 37, deterministic, dtype=np.float64, sh_lmax=2)


def test_isolated_nodes_and_asymmetric_graph(cuda):
    """Nodes without incoming or outgoing edges get zero rows; the graph is not symmetric."""
    prob, oprob = common.channelwise(common.NEQUIP)
    nodes = 40
    rng = np.random.default_rng(5)
    rows = rng.integers(10, 20, 200).astype(np.int64)          # receivers only in [10, 20)
    cols = rng.integers(25, 40, 200).astype(np.int64)          # senders only in [25, 40)
    for det in (False, True):
        r, c, t = rows, cols, None
        if det:
            r, c, t, _ = otp.coord_graph(rows, cols)
        conv, (x, y, w, idx, z, g) = _run(prob, oprob, nodes, len(r), 37, det, graph=(r, c, t))
        assert float(z.detach()[:10].abs().max()) == 0.0 and float(z.detach()[20:].abs().max()) == 0.0
        assert float(x.grad[:25].abs().max()) == 0.0


@pytest.mark.parametrize("deterministic", [False, True])
def test_star_graph_with_self_loops(cuda, deterministic):
    """Half of the edges start or end at node 0 (about 750 edges each way: far more than the 255 the
    launch-order bins distinguish, and hundreds of iterations of the edge pipeline), with self loops and
    repeated edges."""
    rng = np.random.default_rng(42)
    nodes, nnz = 50, 3000
    rows = rng.integers(0, nodes, nnz)
    cols = rng.integers(0, nodes, nnz)
    rows[: nnz // 4] = 0
    cols[nnz // 4: nnz // 2] = 0
    cols[-20:] = rows[-20:]                       # self loops
    rows[-40:-20], cols[-40:-20] = rows[-60:-40], cols[-60:-40]      # repeated edges
    rows, cols = rows.astype(np.int64), cols.astype(np.int64)
    tperm = None
    if deterministic:
        rows, cols, tperm, _ = otp.coord_graph(rows, cols)
    prob, oprob = common.channelwise(common.NEQUIP)
    _run(prob, oprob, nodes, nnz, 43, deterministic, sh_lmax=2, graph=(rows, cols, tperm))
    prob, oprob = common.channelwise(common.LARGE)
    _run(prob, oprob, nodes, nnz, 44, deterministic, sh_lmax=3, graph=(rows, cols, tperm))


@pytest.mark.parametrize("deterministic", [False, True])
def test_blocks_no_path_touches(cuda, deterministic):
    """A wide in1 block that no path reads (and narrow blocks in use): its dX columns are zeros."""
    irreps = ("1x0e+1x1o+16x3o", "1x0e+1x1o", "16x0e+16x0o+16x1e+16x1o")
    prob, oprob = common.channelwise(irreps)
    _, (x, *_rest) = _run(prob, oprob, 21, 265, 2038, deterministic)
    assert not x.grad[:, 4:].any()


def test_no_edges(cuda):
    import torch
    import openequivariance_amd as oeq
    prob, _ = common.channelwise(common.NEQUIP)
    e = torch.zeros(0, dtype=torch.int64, device=cuda)
    for det in (False, True):
        conv = oeq.TensorProductConv(prob, torch_op=True, deterministic=det)
        args = [torch.randn(7, 288, device=cuda), torch.zeros(0, 9, device=cuda), torch.zeros(0, 352, device=cuda), e, e]
        if det:
            args.append(e)
        z = conv.forward(*args)
        assert z.shape == (7, 1120) and float(z.abs().max()) == 0.0
        # the backward of an empty edge list: dX = 0, empty dY and dW (an empty transpose permutation is a NULL pointer)
        x, y, w = (a.clone().requires_grad_(True) for a in args[:3])
        conv.forward(x, y, w, *args[3:]).backward(torch.randn(7, 1120, device=cuda))
        torch.cuda.synchronize()
        assert x.grad.shape == (7, 288) and float(x.grad.abs().max()) == 0.0
        assert y.grad.shape == (0, 9) and w.grad.shape == (0, 352)


def test_deterministic_bit_reproducible(cuda):
    """Five repeats of forward and backward give identical bits (reference protocol:
    convolution/ConvolutionBase.py:229-247)."""
    import torch
    prob, oprob = common.channelwise(common.NEQUIP)
    conv, (x, y, w, idx, z, g) = _run(prob, oprob, 500, 15000, 38, True, sh_lmax=2)
    z0 = z.detach().clone()
    grads0 = [t.grad.clone() for t in (x, y, w)]
    for _ in range(5):
        for t in (x, y, w):
            t.grad = None
        z1 = conv.forward(x, y, w, *idx)
        z1.backward(g)
        assert torch.equal(z1.detach(), z0)
        for a, b in zip(grads0, (x.grad, y.grad, w.grad)):
            assert torch.equal(a, b)


def test_device_graph_preparation(cuda):
    """The README recipe for deterministic=True without torch_geometric: an unsorted edge list is
    sorted on the GPU with sort_by_receiver; the result equals the oracle on the unsorted graph."""
    import torch
    import openequivariance_amd as oeq
    prob, oprob = common.channelwise(common.NEQUIP)
    nodes, nnz = 200, 5000
    rows, cols = common.random_graph(nodes, nnz, 41)
    X, Y, W, G = common.conv_inputs(prob, nodes, nnz, 41, np.float32, 2)
    dev = torch.device("cuda:0")
    x, y, w = (torch.tensor(a, device=dev, requires_grad=True) for a in (X, Y, W))
    r, c, rperm, tperm = oeq.sort_by_receiver(torch.tensor(rows, device=dev), torch.tensor(cols, device=dev), nodes)
    conv = oeq.TensorProductConv(prob, torch_op=True, deterministic=True)
    z = conv.forward(x, y[rperm], w[rperm], r, c, tperm)
    z.backward(torch.tensor(G, device=dev))
    torch.cuda.synchronize()
    Zr = otp.conv_forward(oprob, X, Y, W, rows, cols)
    dXr, dYr, dWr = otp.conv_backward(oprob, X, Y, W, G, rows, cols)
    errs = dict(Z=rel_err(z.detach().cpu().numpy(), Zr), dX=rel_err(x.grad.cpu().numpy(), dXr),
                dY=rel_err(y.grad.cpu().numpy(), dYr), dW=rel_err(w.grad.cpu().numpy(), dWr))
    print(errs, flush=True)
    for k, v in errs.items():
        assert v <= FP32_TOL, f"{k}: relative error {v:.3e}"


@pytest.mark.parametrize("deterministic", [False, True])
def test_misaligned_tensors(cuda, deterministic):
    """Every float tensor starts 4 bytes past a 16-byte boundary: kernels without vector stores."""
    import torch
    import openequivariance_amd as oeq
    prob, oprob = common.channelwise(common.LARGE)          # 64-channel chunks: the vector-store path
    nodes, nnz = 30, 400
    rows, cols, tperm = _graph(nodes, nnz, 51, deterministic)
    X, Y, W, G = common.conv_inputs(prob, nodes, nnz, 51, np.float32, 3)

    def shifted(a):
        flat = torch.empty(a.size + 1, dtype=torch.float32, device=cuda)
        view = flat[1:].view(a.shape)
        view.copy_(torch.from_numpy(a))
        assert view.data_ptr() % 16 == 4
        return view
    conv = oeq.TensorProductConv(prob, torch_op=True, deterministic=deterministic)
    x, y, w = (shifted(a).requires_grad_(True) for a in (X, Y, W))
    idx = [torch.tensor(a, device=cuda) for a in ((rows, cols, tperm) if deterministic else (rows, cols))]
    z = conv.forward(x, y, w, *idx)
    z.backward(shifted(G))
    zraw = shifted(np.zeros_like(G))
    conv.exec_conv_rawptrs(x.data_ptr(), y.data_ptr(), w.data_ptr(), zraw.data_ptr(), idx[0].data_ptr(), idx[1].data_ptr(),
                           nnz, nodes, 0, idx[2].data_ptr() if deterministic else 0)
    torch.cuda.synchronize()
    Zr = otp.conv_forward(oprob, X, Y, W, rows, cols)
    dXr, dYr, dWr = otp.conv_backward(oprob, X, Y, W, G, rows, cols)
    for nm, a, b in (("Z", z.detach(), Zr), ("Zraw", zraw, Zr), ("dX", x.grad, dXr), ("dY", y.grad, dYr), ("dW", w.grad, dWr)):
        assert rel_err(a.cpu().numpy(), b) <= FP32_TOL, nm
