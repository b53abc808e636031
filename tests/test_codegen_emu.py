"""The generated kernel source, compiled for the host and run under AddressSanitizer
(tests/host_emu): checks indexing, bounds and arithmetic of every kernel family against the
oracle without a GPU.  Sizes are tiny because 64 host threads stand in for one wavefront."""
import numpy as np
import pytest

import openequivariance_amd as oeq
from openequivariance_amd.codegen.uvu import UVUGenerator
from openequivariance_amd.codegen.uvu_det import UVUDetGenerator
from openequivariance_amd.codegen.uvu_direct import UVUDirectGenerator
from openequivariance_amd.codegen.uvu_sorted import UVUSortedGenerator
from openequivariance_amd.codegen.uvw import UVWGenerator
from host_emu import emu
from oracle import spec, tp as otp, weights as ow

import common
from common import rel_err

TOL = 2e-6     # fp32 arithmetic against the fp64 oracle on O(1) data


def _tp(gen_cls, irreps, n, seed, **kw):
    prob, oprob = common.channelwise(irreps)
    g = gen_cls(prob, "tp", **kw)
    X, Y, W, G = common.tp_inputs(prob, n, seed)
    fwd, bwd, ws = g.plan()
    out = emu.run_tp(g, fwd, X, Y, W, ws_bytes=ws())
    assert rel_err(out["Z"], otp.forward(oprob, X, Y, W)) < TOL
    out = emu.run_tp(g, bwd, X, Y, W, G, ws_bytes=ws())
    for got, ref in zip((out["Xg"], out["Yg"], out["Wg"]), otp.backward(oprob, X, Y, W, G)):
        assert rel_err(got, ref) < TOL


def test_direct_tp_two_rows_per_wave():
    _tp(UVUDirectGenerator, common.NEQUIP, 5, 1)


def test_direct_tp_ragged_two_chunks():
    _tp(UVUDirectGenerator, ("5x0e+3x1o+70x2e", "1x0e+1x1o+1x2e", "5x0e+3x1o+70x2e+7x3o"), 3, 2)


def test_direct_tp_record_stores_only():
    _tp(UVUDirectGenerator, common.NEQUIP, 3, 3, vector_stores=False)


@pytest.mark.parametrize("irreps,n", [(("128x3e", "1x3e", "128x3e"), 5),              # two full chunks, one path
                                      (("20x5e+70x0e", "1x5e+1x0e", "70x3e+70x0e"), 7),  # 11-word records, ragged chunks
                                      (("8x7e", "1x4e", "8x7e"), 9)],                     # eight rows per wavefront
                         ids=["one_path_l3", "long_records_among_short_ones", "l7_eight_rows_per_wave"])
def test_direct_tp_dx_through_the_lds_slot(irreps, n):
    """Backward of the batch product with dX blocks that leave through the LDS slot (long records, single paths):
    every lane count per row, chunks that are not full, blocks that keep their record stores beside them."""
    prob, _ = common.channelwise(irreps)
    g = UVUDirectGenerator(prob, "tp")
    assert any(g.dx_through_slot(g.in1[i]) for i in g.used_in1)
    _tp(UVUDirectGenerator, irreps, n, 31)


@pytest.mark.parametrize("irreps,n", [(common.NEQUIP, 5),
                                      (("5x0e+3x1o+70x2e", "1x0e+1x1o+1x2e", "5x0e+3x1o+70x2e+7x3o"), 3),
                                      (("64x0o+64x0e+64x1o+64x1e", "1x0e+1x1o", "64x0o+64x0e+64x1o+64x1e"), 2)],
                         ids=["two_rows_per_wave", "ragged_two_chunks", "both_parities"])
def test_direct_tp_operands_one_output_block_ahead(irreps, n, monkeypatch):
    """The batch product with dZ and the weights requested one output block ahead and the shared x_i y_j
    products formed per block (the form many-path problems take), forced here on small problems."""
    monkeypatch.setattr(UVUDirectGenerator, "LAZY_OPERANDS", True)
    _tp(UVUDirectGenerator, irreps, n, 41)


def test_generic_tp_shared_weights():
    ins = [(0, 0, 0, "uvu", True), (1, 1, 0, "uvu", True), (1, 0, 1, "uvu", True)]
    a = ("24x0e+24x1o", "1x0e+1x1o", "24x0e+24x1o")
    prob = oeq.TPProblem(*a, ins, shared_weights=True, internal_weights=False)
    oprob = spec.Problem(*a, ins, shared_weights=True)
    g = UVUGenerator(prob, "tp", dw_partials=3)
    X, Y, W, G = common.tp_inputs(prob, 9, 4)
    fwd, bwd, ws = g.plan()
    out = emu.run_tp(g, fwd, X, Y, W, ws_bytes=ws())
    assert rel_err(out["Z"], otp.forward(oprob, X, Y, W)) < TOL
    out = emu.run_tp(g, bwd, X, Y, W, G, ws_bytes=ws())
    for got, ref in zip((out["Xg"], out["Yg"], out["Wg"]), otp.backward(oprob, X, Y, W, G)):
        assert rel_err(got, ref) < TOL


@pytest.mark.parametrize("variant", ["atomic", "det", "sorted", "sorted_grouped_backward", "sorted_recv_backward"])
def test_conv(variant):
    prob, oprob = common.channelwise(common.NEQUIP)
    det = variant == "det"
    g = {"det": UVUDetGenerator, "sorted": lambda p: UVUSortedGenerator(p, grouped_backward=False),
         "sorted_grouped_backward": lambda p: UVUSortedGenerator(p, grouped_backward=True, recv_backward=False),
         "sorted_recv_backward": lambda p: UVUSortedGenerator(p, grouped_backward=True, recv_backward=True),
         "atomic": lambda p: UVUDirectGenerator(p, "conv_atomic")}[variant](prob)
    nodes, nnz = 7, 19
    rows, cols = common.random_graph(nodes, nnz, 5)
    tperm = None
    if det:
        rows, cols, tperm, _ = otp.coord_graph(rows, cols)
    X, Y, W, G = common.conv_inputs(prob, nodes, nnz, 6)
    fwd, bwd, ws = g.plan()
    # (a transpose permutation makes the emulator start from a junk-filled Z: the deterministic and
    # the sorted forward must write every row themselves; the sorted kernels never read it)
    junk = np.arange(nnz)
    out = emu.run_conv(g, fwd, X, Y, W, rows, cols, tperm=junk if variant.startswith("sorted") else tperm,
                       ws_bytes=ws(nnz, nodes))
    assert rel_err(out["Z"], otp.conv_forward(oprob, X, Y, W, rows, cols)) < TOL
    out = emu.run_conv(g, bwd, X, Y, W, rows, cols, G=G, tperm=junk if variant.endswith("_backward") else tperm,
                       ws_bytes=ws(nnz, nodes))
    for got, ref in zip((out["Xg"], out["Yg"], out["Wg"]), otp.conv_backward(oprob, X, Y, W, G, rows, cols)):
        assert rel_err(got, ref) < TOL
    assert getattr(g, "recv_backward", False) == (variant == "sorted_recv_backward")


HUB_CASES = {
    # name: (irreps, generator factory, deterministic?)
    "det_two_sublists_lds": (common.NEQUIP, lambda p: UVUDetGenerator(p, lds=True), True),
    "det_two_sublists_registers": (common.NEQUIP, lambda p: UVUDetGenerator(p, lds=False), True),
    "det_two_chunks_two_groups": (("70x0e+70x1o+70x2e", "1x0e+1x1o+1x2e+1x3o", "70x0e+70x1o+70x2e+70x3o"), UVUDetGenerator, True),
    "det_receiver_order": (common.NEQUIP, None, True),
    "unsorted_grouped": (common.NEQUIP, lambda p: UVUSortedGenerator(p, grouped_backward=True, recv_backward=False), False),
    "unsorted_receiver_order": (common.NEQUIP, lambda p: UVUSortedGenerator(p, grouped_backward=True, recv_backward=True), False),
    "unsorted_atomic_backward": (common.NEQUIP, lambda p: UVUSortedGenerator(p, grouped_backward=False), False),
}


@pytest.mark.parametrize("case", sorted(HUB_CASES))
def test_conv_long_nodes_walked_in_pieces(case):
    """A receiver with 150 incoming and a sender with 130 outgoing edges among 12 nodes and 400 edges (mean 34:
    pieces of 68 edges): the hubs' lists are cut at multiples of 68 list positions, each piece is walked by a
    wavefront of its own into a partial row, the piece finishing last adds them; short nodes, nodes spanning
    a cut without being long, and the zero-filled rows of nodes without edges are as before."""
    from openequivariance_amd.codegen.uvu_recv import UVURecvGenerator
    irreps, make, det = HUB_CASES[case]
    prob, oprob = common.channelwise(irreps)
    g = (make or UVURecvGenerator)(prob)
    nodes, nnz = 12, 400
    rows, cols = common.hub_graph(nodes - 1, nnz, 21, hub_in=3, hub_out=5, in_edges=150, out_edges=130)   # node 11: no edges
    tperm = None
    if det:
        rows, cols, tperm, _ = otp.coord_graph(rows, cols)
    X, Y, W, G = common.conv_inputs(prob, nodes, nnz, 22)
    fwd, bwd, ws = g.plan()
    f = g.fwd if hasattr(g, "fwd") else g
    assert f.LONG == 2 and f.piece_tiles(nnz, nodes) == 6
    assert emu.grid_of([s for s in fwd if s["kernel"] == "forward"][0], nnz, nodes) == nodes + 12
    junk = np.arange(nnz)
    out = emu.run_conv(g, fwd, X, Y, W, rows, cols, tperm=tperm if det else junk, ws_bytes=ws(nnz, nodes))
    assert rel_err(out["Z"], otp.conv_forward(oprob, X, Y, W, rows, cols)) < TOL
    assert not out["Z"][11].any()
    bt = tperm if det else (junk if g.grouped_backward else None)
    out = emu.run_conv(g, bwd, X, Y, W, rows, cols, G=G, tperm=bt, ws_bytes=ws(nnz, nodes))
    for got, ref in zip((out["Xg"], out["Yg"], out["Wg"]), otp.conv_backward(oprob, X, Y, W, G, rows, cols)):
        assert rel_err(got, ref) < TOL


def test_conv_long_node_of_more_pieces_than_one_group():
    """A receiver with 1250 of 1600 edges among 100 nodes: 40 pieces of 32 edges, added in two levels (groups of
    32 pieces, then the two groups)."""
    prob, oprob = common.channelwise(common.NEQUIP)
    g = UVUDetGenerator(prob)
    nodes, nnz = 100, 1600
    rows, cols = common.hub_graph(nodes, nnz, 23, hub_in=41, hub_out=17, in_edges=1250, out_edges=0)
    rows, cols, tperm, _ = otp.coord_graph(rows, cols)
    assert g.piece_tiles(nnz, nodes) == 50 and (rows == 41).sum() > 32 * g.PIECE_GROUP
    X, Y, W, G = common.conv_inputs(prob, nodes, nnz, 24)
    fwd, _, ws = g.plan()
    out = emu.run_conv(g, fwd, X, Y, W, rows, cols, tperm=tperm, ws_bytes=ws(nnz, nodes))
    assert rel_err(out["Z"], otp.conv_forward(oprob, X, Y, W, rows, cols)) < TOL


@pytest.mark.parametrize("case", ["det_registers", "det_lds", "det_two_chunks", "unsorted", "det_hubs", "unsorted_hubs",
                                  "untouched_output_block"])
def test_conv_forward_one_launch_per_group_of_output_blocks(case, monkeypatch):
    """The forward of problems with more output words than a wavefront keeps in registers runs once per group of
    output blocks: forced here on small problems (a group per 4 words), on a junk-filled Z, with hubs
    walked in pieces, with an output block that no path writes, over a position list built on the fly."""
    from openequivariance_amd.codegen.uvu_recv import UVURecvGenerator
    monkeypatch.setattr(UVUDetGenerator, "FWD_SPLIT_WORDS", {"float": 4, "double": 4})
    irreps = {"det_two_chunks": ("5x0e+3x1o+70x2e", "1x0e+1x1o+1x2e", "5x0e+3x1o+70x2e+7x3o"),
              }.get(case, common.NEQUIP)
    prob, oprob = common.channelwise(irreps)
    if case == "untouched_output_block":
        a = ("16x0e+16x1o", "1x0e+1x1o", "16x0e+16x1o+16x2e+16x1e")
        ins = [(0, 0, 0, "uvu", True), (1, 1, 0, "uvu", True), (0, 1, 1, "uvu", True), (1, 0, 1, "uvu", True),
               (1, 1, 3, "uvu", True)]
        prob = oeq.TPProblem(*a, ins, shared_weights=False, internal_weights=False)
        oprob = spec.Problem(*a, ins, shared_weights=False)
    det = case.startswith("det") or case == "untouched_output_block"
    if case in ("det_registers", "det_lds"):
        g = UVUDetGenerator(prob, lds=case == "det_lds")
        assert g.lds_forward == (case == "det_lds")
    elif det:
        g = UVUDetGenerator(prob)
    else:
        g = UVUSortedGenerator(prob, grouped_backward=False)
    f = g.fwd if hasattr(g, "fwd") else g
    assert len(f.fwd_groups) >= 2 and sorted(o for grp in f.fwd_groups for o in grp) == f.used_out
    if case.endswith("hubs"):
        nodes, nnz = 12, 400
        rows, cols = common.hub_graph(nodes - 1, nnz, 21, hub_in=3, hub_out=5, in_edges=150, out_edges=130)
    else:
        nodes, nnz = 7, 45
        rows, cols = common.random_graph(nodes - 1, nnz, 5)               # the last node has no edges
    tperm = np.arange(nnz)
    if det:
        rows, cols, tperm, _ = otp.coord_graph(rows, cols)
    X, Y, W, G = common.conv_inputs(prob, nodes, nnz, 6)
    fwd, bwd, ws = g.plan()
    assert [s["kernel"] for s in fwd if s["kernel"].startswith("forward")] == [k for k, _ in f.forward_kernels()]
    out = emu.run_conv(g, fwd, X, Y, W, rows, cols, tperm=tperm, ws_bytes=ws(nnz, nodes))
    assert rel_err(out["Z"], otp.conv_forward(oprob, X, Y, W, rows, cols)) < TOL
    assert not out["Z"][nodes - 1].any()
    if case == "untouched_output_block":
        blk = [b for b in f.out if b.idx not in f.used_out]
        assert blk and not out["Z"][:, blk[0].off:blk[0].off + blk[0].dim].any()


@pytest.mark.parametrize("case", ["det", "det_two_chunks", "det_four_lane_groups", "unsorted", "unsorted_invalid_edges",
                                  "det_fp64_register_loads", "det_fp64_two_chunks_invalid_edges", "unsorted_fp64",
                                  "unsorted_fp64_invalid_edges"])
def test_conv_receiver_order_pass_one_per_group_of_output_blocks(case, monkeypatch):
    """Pass 1 of the receiver-order backward in several launches (forced here: a launch per 4 dZ words): the groups
    share no in1 block, so each launch writes its own words of the per-edge dX rows and its own rows of dW; dY is
    summed from one partial row per (chunk, launch)."""
    from openequivariance_amd.codegen.uvu_recv import UVURecvGenerator
    monkeypatch.setattr(UVURecvGenerator, "RECV_SPLIT_WORDS", 4)
    monkeypatch.setattr(UVURecvGenerator, "RECV_SPLIT_WORDS_ONE_GROUP", 4)
    monkeypatch.setattr(UVURecvGenerator, "RECV_SPLIT_WORDS_REGISTER_LOADS", {"float": 4, "double": 4})
    irreps = {"det_two_chunks": ("5x0e+3x1o+70x2e", "1x0e+1x1o+1x2e", "5x0e+3x1o+70x2e+7x3o"),
              "det_fp64_two_chunks_invalid_edges": ("5x0e+3x1o+70x2e", "1x0e+1x1o+1x2e", "5x0e+3x1o+70x2e+7x3o"),
              "det_four_lane_groups": ("16x0e+16x1o", "1x0e+1x1o", "16x0e+16x0o+16x1e+16x1o")}.get(case, common.NEQUIP)
    fp64 = "fp64" in case
    prob, oprob = common.channelwise(irreps, dtype=np.float64 if fp64 else np.float32)
    det = case.startswith("det")
    g = UVURecvGenerator(prob) if det else UVUSortedGenerator(prob, grouped_backward=True, recv_backward=True)
    b = g if det else g.bwd
    assert b.staged_edges == (not fp64) and b.HR >= 2 and sorted(sum(b.recv_groups, [])) == b.used_out
    ins = [{p.a.idx for p in b.paths if p.o.idx in grp} for grp in b.recv_groups]
    assert all(not (x & y) for k, x in enumerate(ins) for y in ins[k + 1:])
    nodes, nnz = 9, 70
    rows, cols = common.random_graph(nodes - 1, nnz, 15, self_loops=True)
    valid = np.ones(nnz, dtype=bool)
    if case.endswith("invalid_edges"):
        rows, cols, valid = common.with_invalid_edges(rows, cols, nodes, 16)
    tperm = np.arange(nnz)
    if det:
        rows, cols, tperm, _ = otp.coord_graph(rows, cols)
    valid = (rows >= 0) & (rows < nodes) & (cols >= 0) & (cols < nodes)
    X, Y, W, G = common.conv_inputs(prob, nodes, nnz, 17, dtype=np.float64 if fp64 else np.float32)
    _, bwd, ws = g.plan()
    assert [s["kernel"] for s in bwd if s["kernel"].startswith("backward")][:b.HR + 1] == \
        ["backward"] + [f"backward_g{h}" for h in range(1, b.HR)] + ["backward_dx"]
    out = emu.run_conv(g, bwd, X, Y, W, rows, cols, G=G, tperm=tperm, ws_bytes=ws(nnz, nodes))
    ref = common.conv_reference_on_valid_edges(otp, oprob, X, Y, W, G, rows, cols, valid)[1:]
    for got, want in zip((out["Xg"], out["Yg"], out["Wg"]), ref):
        assert rel_err(got, want) < TOL


@pytest.mark.parametrize("staged", [True, False])
def test_conv_det_long_edge_lists(staged):
    """Edge lists of about 13 edges per node (6-7 iterations of two sub-lists) reach the steady state of
    the edge pipeline, with the next edge's operands staged through LDS and with register prefetch; the
    last node has no edges."""
    prob, oprob = common.channelwise(common.NEQUIP)
    g = UVUDetGenerator(prob, lds=staged)
    assert g.lds_backward == staged and g.lds_forward == staged
    nodes, nnz = 4, 40
    rows, cols = common.random_graph(nodes - 1, nnz, 11)          # node 3 has no edges
    rows, cols, tperm, _ = otp.coord_graph(rows, cols)
    X, Y, W, G = common.conv_inputs(prob, nodes, nnz, 12)
    fwd, bwd, ws = g.plan()
    out = emu.run_conv(g, fwd, X, Y, W, rows, cols, tperm=tperm, ws_bytes=ws(nnz, nodes))
    assert rel_err(out["Z"], otp.conv_forward(oprob, X, Y, W, rows, cols)) < TOL
    assert not out["Z"][3].any()
    out = emu.run_conv(g, bwd, X, Y, W, rows, cols, G=G, tperm=tperm, ws_bytes=ws(nnz, nodes))
    for got, ref in zip((out["Xg"], out["Yg"], out["Wg"]), otp.conv_backward(oprob, X, Y, W, G, rows, cols)):
        assert rel_err(got, ref) < TOL


def test_conv_long_runs_of_nodes_without_edges():
    """Receivers only among the first three nodes and senders only among the last ten of 700: the CSR pointers of
    the 690 nodes in between are written by the whole workgroup of the preparation kernels, not by one thread."""
    prob, oprob = common.channelwise(("8x0e+8x1o", "1x0e+1x1o", "8x0e+8x1o"))
    g = UVUDetGenerator(prob)
    nodes, nnz = 700, 90
    rng = np.random.default_rng(5)
    rows, cols = rng.integers(0, 3, nnz), rng.integers(690, 700, nnz)
    rows, cols, tperm, _ = otp.coord_graph(rows, cols)
    X, Y, W, G = common.conv_inputs(prob, nodes, nnz, 6)
    fwd, bwd, ws = g.plan()
    out = emu.run_conv(g, fwd, X, Y, W, rows, cols, tperm=tperm, ws_bytes=ws(nnz, nodes))
    assert rel_err(out["Z"], otp.conv_forward(oprob, X, Y, W, rows, cols)) < TOL
    assert not out["Z"][3:].any()
    out = emu.run_conv(g, bwd, X, Y, W, rows, cols, G=G, tperm=tperm, ws_bytes=ws(nnz, nodes))
    for got, ref in zip((out["Xg"], out["Yg"], out["Wg"]), otp.conv_backward(oprob, X, Y, W, G, rows, cols)):
        assert rel_err(got, ref) < TOL
    assert not out["Xg"][:690].any()


def test_conv_blocks_no_path_touches_are_zero_filled():
    """in1 holds a 16-channel l = 3 block that no path reads while the blocks in use have one channel: its
    dX columns must come out as zeros (the emulator starts the deterministic outputs from junk)."""
    irreps = ("1x0e+1x1o+16x3o", "1x0e+1x1o", "16x0e+16x0o+16x1e+16x1o")
    prob, oprob = common.channelwise(irreps)
    g = UVUDetGenerator(prob)
    assert g.used_in1 == [0, 1] and g.P == 16
    nodes, nnz = 21, 265
    rows, cols, tperm, _ = otp.coord_graph(*common.random_graph(nodes, nnz, 2038, self_loops=True))
    X, Y, W, G = common.conv_inputs(prob, nodes, nnz, 2038)
    fwd, bwd, ws = g.plan()
    out = emu.run_conv(g, fwd, X, Y, W, rows, cols, tperm=tperm, ws_bytes=ws(nnz, nodes))
    assert rel_err(out["Z"], otp.conv_forward(oprob, X, Y, W, rows, cols)) < TOL
    out = emu.run_conv(g, bwd, X, Y, W, rows, cols, G=G, tperm=tperm, ws_bytes=ws(nnz, nodes))
    assert not out["Xg"][:, 4:].any()
    for got, ref in zip((out["Xg"], out["Yg"], out["Wg"]), otp.conv_backward(oprob, X, Y, W, G, rows, cols)):
        assert rel_err(got, ref) < TOL


@pytest.mark.parametrize("staged", [False, True])
@pytest.mark.parametrize("irreps,nodes,nnz,prefetch", [
    (("5x0e+3x1o+70x2e", "1x0e+1x1o+1x2e", "5x0e+3x1o+70x2e+7x3o"), 5, 11, None),      # two chunks, ragged
    (("1x0e+1x1o+16x3o", "1x0e+1x1o", "16x0e+16x0o+16x1e+16x1o"), 21, 265, None),    # four lane groups, unused block
    (("8x0e+8x1o", "1x0e+1x1o", "8x0e+8x1o"), 9, 100, False)])                       # eight lane groups, one register set
def test_conv_receiver_order_backward(irreps, nodes, nnz, prefetch, staged):
    """The two-pass backward (per-edge dX rows spilled in receiver order, summed per sender in the order
    of the transpose permutation): tiles that end inside a receiver's edges, idle lane groups in the last
    iteration of a tile, self loops, nodes without edges; pass 1 with register loads and with the next
    edge's operands staged through LDS."""
    from openequivariance_amd.codegen.uvu_recv import UVURecvGenerator
    prob, oprob = common.channelwise(irreps)
    g = UVURecvGenerator(prob, prefetch=prefetch, staged=staged)
    assert g.staged_edges == (staged and g.P >= g.D2)
    rows, cols, tperm, _ = otp.coord_graph(*common.random_graph(nodes, nnz, 7, self_loops=True))
    X, Y, W, G = common.conv_inputs(prob, nodes, nnz, 8)
    _, bwd, ws = g.plan()
    assert [s["kernel"] for s in bwd][:3] == ["prep_backward", "backward", "backward_dx"]
    out = emu.run_conv(g, bwd, X, Y, W, rows, cols, G=G, tperm=tperm, ws_bytes=ws(nnz, nodes))
    for got, ref in zip((out["Xg"], out["Yg"], out["Wg"]), otp.conv_backward(oprob, X, Y, W, G, rows, cols)):
        assert rel_err(got, ref) < TOL


@pytest.mark.parametrize("variant", ["det", "det_two_chunks", "grouped", "grouped_recv", "recv", "recv_staged"])
def test_conv_edges_naming_no_node(variant):
    """Edges whose sender or receiver is out of range contribute nothing, and their dW / dY rows come
    out as zeros from every backward variant (the emulator starts all outputs from junk)."""
    from openequivariance_amd.codegen.uvu_recv import UVURecvGenerator
    irreps = ("70x0e+70x1o", "1x0e+1x1o", "70x0e+70x1o") if variant == "det_two_chunks" else \
        ("16x0e+16x1o", "1x0e+1x1o+1x2e", "16x0e+16x1o+16x2e") if variant in ("recv_staged", "grouped_recv") else \
        ("8x0e+8x1o", "1x0e+1x1o+1x2e", "8x0e+8x1o+8x2e")
    prob, oprob = common.channelwise(irreps)
    nodes, nnz = 9, 300 if variant != "det_two_chunks" else 40
    rows, cols = common.random_graph(nodes, nnz, 5, self_loops=True)
    rows, cols, valid = common.with_invalid_edges(rows, cols, nodes, 6)
    tperm = None
    if not variant.startswith("grouped"):
        order = np.lexsort((cols, rows))
        rows, cols, valid = rows[order], cols[order], valid[order]
        tperm = np.lexsort((np.arange(nnz), rows, cols)).astype(np.int64)
    g = {"det": UVUDetGenerator, "det_two_chunks": UVUDetGenerator, "recv": UVURecvGenerator,
         "recv_staged": lambda p: UVURecvGenerator(p, staged=True),
         "grouped": lambda p: UVUSortedGenerator(p, grouped_backward=True, recv_backward=False),
         "grouped_recv": lambda p: UVUSortedGenerator(p, grouped_backward=True, recv_backward=True)}[variant](prob)
    X, Y, W, G = common.conv_inputs(prob, nodes, nnz, 8)
    Zr, dXr, dYr, dWr = common.conv_reference_on_valid_edges(otp, oprob, X, Y, W, G, rows, cols, valid)
    fwd, bwd, ws = g.plan()
    junk = np.full(nnz, 12345, dtype=np.int64)
    tp = junk if variant.startswith("grouped") else tperm
    out = emu.run_conv(g, fwd, X, Y, W, rows, cols, tperm=tp, ws_bytes=ws(nnz, nodes))
    assert rel_err(out["Z"], Zr) < TOL
    out = emu.run_conv(g, bwd, X, Y, W, rows, cols, G=G, tperm=tp, ws_bytes=ws(nnz, nodes))
    assert rel_err(out["Xg"], dXr) < TOL and rel_err(out["Yg"], dYr) < TOL and rel_err(out["Wg"], dWr) < TOL
    assert not out["Wg"][~valid].any() and not out["Yg"][~valid].any()


def test_conv_det_chunked_ragged():
    irreps = ("5x0e+3x1o+70x2e", "1x0e+1x1o+1x2e", "5x0e+3x1o+70x2e+7x3o")
    prob, oprob = common.channelwise(irreps)
    g = UVUDetGenerator(prob)
    nodes, nnz = 5, 11
    rows, cols, tperm, _ = otp.coord_graph(*common.random_graph(nodes, nnz, 7))
    X, Y, W, G = common.conv_inputs(prob, nodes, nnz, 8)
    fwd, bwd, ws = g.plan()
    out = emu.run_conv(g, fwd, X, Y, W, rows, cols, tperm=tperm, ws_bytes=ws(nnz, nodes))
    assert rel_err(out["Z"], otp.conv_forward(oprob, X, Y, W, rows, cols)) < TOL
    out = emu.run_conv(g, bwd, X, Y, W, rows, cols, G=G, tperm=tperm, ws_bytes=ws(nnz, nodes))
    for got, ref in zip((out["Xg"], out["Yg"], out["Wg"]), otp.conv_backward(oprob, X, Y, W, G, rows, cols)):
        assert rel_err(got, ref) < TOL


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_uvw_matrix_core_kernels(dtype, monkeypatch):
    monkeypatch.setattr(UVWGenerator, "DW_WORKGROUPS", 3)
    a = ("5x0e+21x1o", "1x0e+1x1o+1x2e", "18x0e+7x1o+3x2e")
    prob, oprob = common.fully_connected(a, shared=True, dtype=dtype)
    g = UVWGenerator(prob)
    X, Y, We, G = common.tp_inputs(prob, 21, 9, dtype, w_scale=0.3)
    W = ow.e3nn_to_oeq(oprob, We)
    fwd, bwd, ws = g.plan()
    tol = TOL if dtype == np.float32 else 1e-13
    out = emu.run_tp(g, fwd, X, Y, W, ws_bytes=ws())
    assert rel_err(out["Z"], otp.forward(oprob, X, Y, We)) < tol
    out = emu.run_tp(g, bwd, X, Y, W, G, ws_bytes=ws())
    dX, dY, dW = otp.backward(oprob, X, Y, We, G)
    assert rel_err(out["Xg"], dX) < tol and rel_err(out["Yg"], dY) < tol
    assert rel_err(ow.oeq_to_e3nn(oprob, out["Wg"]), dW) < tol


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_uvw_dw_single_path_beyond_the_accumulator_budget(dtype, monkeypatch):
    """One path whose accumulators alone exceed what a dW pass may hold is cut by ranges of its w tiles: with
    the budget lowered to two tiles' worth, 70 x 40 channels take three passes for the first path."""
    monkeypatch.setattr(UVWGenerator, "DW_WORKGROUPS", 2)
    per_tile = 4 if dtype == np.float32 else 8
    monkeypatch.setattr(UVWGenerator, "DW_ACC_BUDGET", {4: 4 * per_tile, 8: 4 * per_tile})     # ceil(5 / 4) = 2 u groups x 2 w tiles
    a = ("70x0e+5x1o", "1x0e+1x1o", "40x0e+9x1o")
    prob, oprob = common.fully_connected(a, shared=True, dtype=dtype)
    g = UVWGenerator(prob)
    passes = g.dw_passes()
    assert max(sum(-(-p.NTU // 4) * (hi - lo) * per_tile for p, lo, hi in segs) for _, segs in passes) <= 4 * per_tile
    assert sum(1 for _, segs in passes for p, lo, hi in segs if p.t == 0) >= 2
    X, Y, We, G = common.tp_inputs(prob, 19, 13, dtype, w_scale=0.3)
    W = ow.e3nn_to_oeq(oprob, We)
    _, bwd, ws = g.plan()
    out = emu.run_tp(g, bwd, X, Y, W, G, ws_bytes=ws())
    tol = TOL if dtype == np.float32 else 1e-13
    assert rel_err(ow.oeq_to_e3nn(oprob, out["Wg"]), otp.backward(oprob, X, Y, We, G)[2]) < tol


def test_uvw_forward_work_item_mapping_over_many_tiles():
    """19 batch tiles: 16 of them in groups of 8 with the items of a tile 8 workgroup ids apart, the last three
    item-major; every (tile, item) pair must be visited exactly once."""
    a = ("4x0e+4x1o", "1x0e+1x1o", "4x0e+4x1o+4x1e")
    prob, oprob = common.fully_connected(a, shared=True)
    g = UVWGenerator(prob)
    X, Y, We, _ = common.tp_inputs(prob, 300, 12, w_scale=0.3)
    fwd, _, ws = g.plan()
    out = emu.run_tp(g, fwd, X, Y, ow.e3nn_to_oeq(oprob, We), ws_bytes=ws())
    assert rel_err(out["Z"], otp.forward(oprob, X, Y, We)) < TOL


@pytest.mark.parametrize("shared", [False, True])
def test_uvu_run_time_loop_over_second_operand_copies(shared, monkeypatch):
    """mul(in2) = 11 > 8: v is walked at run time; dY sums through the LDS accumulator, shared dW through
    the workgroup's partial row."""
    from openequivariance_amd.tensor_product import select_generator
    import openequivariance_amd as oeq
    ins = [(0, 0, 0, "uvu", True), (0, 1, 1, "uvu", True), (1, 0, 2, "uvu", True), (1, 1, 0, "uvu", True)]
    a = ("12x0e+12x1o", "11x0e+3x1o", "12x0e+12x1o+12x1o")
    prob = oeq.TPProblem(*a, ins, shared_weights=shared, internal_weights=False)
    oprob = spec.Problem(*a, ins, shared_weights=shared)
    g = select_generator(prob)
    assert [p.looped for p in g.paths] == [True, False, True, False]
    X, Y, We, G = common.tp_inputs(prob, 9, 1, w_scale=0.3)
    W = ow.e3nn_to_oeq(oprob, We)
    fwd, bwd, ws = g.plan()
    if shared:
        g.dw_partials = 3
        for s in bwd:
            if s["kernel"] == "backward":
                s["num_blocks"] = 3
    out = emu.run_tp(g, fwd, X, Y, W, ws_bytes=ws())
    assert rel_err(out["Z"], otp.forward(oprob, X, Y, We)) < TOL
    out = emu.run_tp(g, bwd, X, Y, W, G, ws_bytes=ws())
    dX, dY, dW = otp.backward(oprob, X, Y, We, G)
    assert rel_err(out["Xg"], dX) < TOL and rel_err(out["Yg"], dY) < TOL
    assert rel_err(ow.oeq_to_e3nn(oprob, out["Wg"]), dW) < TOL


@pytest.mark.parametrize("shared", [True, False])
def test_uvw_several_copies_of_the_second_operand(shared, monkeypatch):
    monkeypatch.setattr(UVWGenerator, "DW_WORKGROUPS", 3)
    from openequivariance_amd.tensor_product import select_generator
    a = ("5x0e+21x1o", "3x0e+2x1o", "18x0e+7x1o")
    prob, oprob = common.fully_connected(a, shared=shared)
    g = select_generator(prob)
    assert len(g.paths) == 10 and {p.mv for p in g.paths} == {2, 3}
    X, Y, We, G = common.tp_inputs(prob, 21 if shared else 5, 9, w_scale=0.3)
    W = ow.e3nn_to_oeq(oprob, We)
    fwd, bwd, ws = g.plan()
    out = emu.run_tp(g, fwd, X, Y, W, ws_bytes=ws())
    assert rel_err(out["Z"], otp.forward(oprob, X, Y, We)) < TOL
    out = emu.run_tp(g, bwd, X, Y, W, G, ws_bytes=ws())
    dX, dY, dW = otp.backward(oprob, X, Y, We, G)
    assert rel_err(out["Xg"], dX) < TOL and rel_err(out["Yg"], dY) < TOL
    assert rel_err(ow.oeq_to_e3nn(oprob, out["Wg"]), dW) < TOL


@pytest.mark.parametrize("a", [("5x0e+21x1o", "1x0e+1x1o+1x2e", "18x0e+7x1o+3x2e"),
                               ("70x0e+35x1o", "1x0e+1x1o", "48x0e+33x1o"),
                               ("10x0e+40x1o", "3x0e+2x1o", "36x0e+10x1o"),
                               ("6x0e+20x1o", "1x0e+1x1o+1x2e", "18x0e+7x1o+4x2e")],
                         ids=["narrow", "ragged_32_blocks", "several_copies", "even_and_odd_chunks"])
@pytest.mark.parametrize("t_words", [4096, 150], ids=["one_phase", "several_phases"])
def test_uvw_per_row_weights(a, t_words, monkeypatch):
    from openequivariance_amd.codegen.uvw_batched import UVWBatchedGenerator
    monkeypatch.setattr(UVWBatchedGenerator, "T_LDS_WORDS", t_words)
    prob, oprob = common.fully_connected(a, shared=False)
    g = UVWBatchedGenerator(prob)
    X, Y, We, G = common.tp_inputs(prob, 5, 10, w_scale=0.3)
    W = ow.e3nn_to_oeq(oprob, We)
    fwd, bwd, ws = g.plan()
    out = emu.run_tp(g, fwd, X, Y, W)
    assert rel_err(out["Z"], otp.forward(oprob, X, Y, We)) < TOL
    out = emu.run_tp(g, bwd, X, Y, W, G)
    dX, dY, dW = otp.backward(oprob, X, Y, We, G)
    assert rel_err(out["Xg"], dX) < TOL and rel_err(out["Yg"], dY) < TOL
    assert rel_err(ow.oeq_to_e3nn(oprob, out["Wg"]), dW) < TOL


@pytest.mark.parametrize("a,n", [(("1x0e+1x1o+1x2e+1x3o", "1x0e+1x1o+1x2e+1x3o", "64x0e+24x1e+24x1o+16x2e+16x2o"), 70),
                                 (("64x0e+24x1e+24x1o+16x2e+16x2o", "1x0e+1x1o+1x2e+1x3o", "1x0o+6x0e"), 130),
                                 (("3x0e+2x1o", "2x0e+1x1o", "5x0e+4x1o+1x2e"), 64),
                                 (("8x0e+10x1o", "1x0e+1x1o", "9x0e+11x1o"), 97),
                                 (("2x0e+9x4e", "1x0e+1x2e", "8x4e+3x2e"), 70)],
                         ids=["tetris_poly_1", "tetris_poly_2", "several_copies", "several_groups_on_both_sides",
                              "four_records_longer_than_a_group"])
def test_uvw_shared_weights_one_row_per_lane(a, n, monkeypatch):
    """The vector-ALU kernels for uvw problems with few weights: ragged last tile, several tiles per wavefront
    (the grid bound is lowered to 2 so that a wavefront accumulates dW over more than one tile)."""
    from openequivariance_amd.codegen.uvw_rows import UVWRowsGenerator
    monkeypatch.setattr(UVWRowsGenerator, "WAVES", 2)
    prob, oprob = common.fully_connected(a, shared=True)
    assert UVWRowsGenerator.suits(prob)
    g = UVWRowsGenerator(prob)
    X, Y, We, G = common.tp_inputs(prob, n, 11, w_scale=0.3)
    W = ow.e3nn_to_oeq(oprob, We)
    fwd, bwd, ws = g.plan()
    out = emu.run_tp(g, fwd, X, Y, W, ws_bytes=ws())
    assert rel_err(out["Z"], otp.forward(oprob, X, Y, We)) < TOL
    out = emu.run_tp(g, bwd, X, Y, W, G, ws_bytes=ws())
    dX, dY, dW = otp.backward(oprob, X, Y, We, G)
    assert rel_err(out["Xg"], dX) < TOL and rel_err(out["Yg"], dY) < TOL
    assert rel_err(ow.oeq_to_e3nn(oprob, out["Wg"]), dW) < TOL
