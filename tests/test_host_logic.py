"""Host-side logic that needs no GPU: validation errors, launch plans, byte/FLOP models, bench contract."""
import json
import subprocess
import sys

import numpy as np
import pytest

import openequivariance_amd as oeq
from openequivariance_amd import workloads
from openequivariance_amd.codegen.uvu import UVUGenerator
from openequivariance_amd.codegen.uvu_direct import UVUDirectGenerator
from openequivariance_amd.codegen.uvw import UVWGenerator
from openequivariance_amd.conv import flops_data_per_tp
from openequivariance_amd.tensor_product import validate_problem

import common


def test_validation_mirrors_reference_constraints():
    with pytest.raises(ValueError, match="no valid"):
        validate_problem(oeq.TPProblem("1x0e", "1x0e", "1x0e", []))
    mixed = oeq.TPProblem("2x0e", "1x0e", "2x0e", [(0, 0, 0, "uvu", True), (0, 0, 0, "uvw", True)])
    with pytest.raises(AssertionError):
        validate_problem(mixed)
    with pytest.raises(AssertionError):
        validate_problem(oeq.TPProblem("2x0e", "2x0e", "2x0e", [(0, 0, 0, "uuu", True)]))
    with pytest.raises(AssertionError):
        validate_problem(oeq.TPProblem("2x0e", "1x0e", "2x0e", [(0, 0, 0, "uvu", True)], irrep_dtype=np.float64))
    with pytest.raises(AssertionError):                      # conv needs mul 1 on the second operand
        UVUDirectGenerator(oeq.TPProblem("2x0e", "2x0e", "2x0e", [(0, 0, 0, "uvu", True)], shared_weights=False,
                                         internal_weights=False), "conv_atomic")


def test_launch_plans():
    prob, _ = common.channelwise(common.MACE)
    fwd, bwd, ws = UVUDirectGenerator(prob, "tp").plan()
    assert [s["kernel"] for s in fwd] == ["forward"] and fwd[0]["work_per_block"] == 1 and ws() == 0
    prob, _ = common.channelwise(common.NEQUIP)
    assert UVUDirectGenerator(prob, "tp").plan()[0][0]["work_per_block"] == 2       # two rows per wavefront
    prob, _ = common.channelwise(common.LARGE)
    from openequivariance_amd.codegen.uvu_det import UVUDetGenerator
    g = UVUDetGenerator(prob)
    fwd, bwd, ws = g.plan()
    assert [s["kernel"] for s in fwd] == ["prep_forward", "forward"] and fwd[1]["grid_y"] == 4
    assert [s["kernel"] for s in bwd] == ["prep_backward", "order_backward", "backward", "backward_dy_reduce"]
    assert bwd[1]["num_blocks"] == 1
    flags = 8 + 4 * 4                                                   # one int per 256 edges (+ alignment slack)
    main = 2 * 11 * 8 + 10 * 8 + 4 * 1000 * 16 * 4 + flags               # pointers | node order | dY partials | flags
    tiles = -(-1000 // 200)                                             # long nodes: pieces of twice the mean of 100 edges
    pieces = 256 + ((16 * 4 * tiles + 255) & ~255) + 2 * tiles * g.D3 * 4   # four counters per tile and chunk | two partial rows per tile
    assert fwd[1]["grid_kind"] == bwd[2]["grid_kind"] == 3 and fwd[1]["num_blocks"] == g.LONG == 2
    assert ws(1000, 10) == ((main + 255) & ~255) + pieces
    assert g.forward_workspace_model() == (8, 8, 0)                     # the forward alone, every node walked whole
    prob, _ = common.fully_connected(common.DENSE)
    fwd, bwd, ws = UVWGenerator(prob).plan()
    assert [s["kernel"] for s in bwd] == ["prep_backward", "backward", "backward_dw", "backward_reduce"]


def test_generated_source_bakes_cg_constants():
    prob, _ = common.readme_problem()
    src = UVUDirectGenerator(prob, "tp").render()
    assert src.count("oeq_fma(0x") + src.count("= 0x") + src.count("= -0x") >= 28      # 28 nonzeros of C(2,3,2)
    assert "__global__" in src and "#ifdef" not in src


def test_work_models_match_the_documented_numbers():
    mace = workloads.get("mace_uvu")
    assert mace.alg_bytes["forward"] == 50000 * 49728 and mace.alg_bytes["backward"] == 50000 * 63104
    dense = workloads.get("dense_uvw_f32")
    assert dense.alg_flops["forward"] == 100000 * 286720 and dense.alg_flops["backward"] == 100000 * 573440
    prob, _ = common.channelwise(common.NEQUIP)
    ops_f, bytes_f, nnz = flops_data_per_tp(prob, "forward")
    ops_b, bytes_b, _ = flops_data_per_tp(prob, "backward")
    assert (bytes_f, bytes_b, nnz) == (7076, 9672, 83)


def test_bench_refuses_more_than_one_gpu():
    res = subprocess.run([sys.executable, "bench.py", "--gpus", "2"], capture_output=True, text=True,
                         cwd=str(common.__file__).rsplit("/tests", 1)[0])
    assert res.returncode != 0 and "one GPU" in res.stderr


def test_spherical_harmonics_inputs():
    from openequivariance_amd.sh import spherical_harmonics
    v = np.random.default_rng(0).standard_normal((20, 3))
    Y = spherical_harmonics(3, v)
    assert Y.shape == (20, 16)
    n = v / np.linalg.norm(v, axis=1, keepdims=True)
    np.testing.assert_allclose(Y[:, 0], 1.0)
    np.testing.assert_allclose(Y[:, 1:4], np.sqrt(3) * n, atol=1e-13)
    for l in range(4):
        np.testing.assert_allclose((Y[:, l * l:(l + 1) ** 2] ** 2).sum(1), 2 * l + 1, atol=1e-12)


def test_lds_dma_transfer_plan():
    """Records are moved global -> LDS in transfers of 4, 3 or 1 words per lane, as few as possible, and
    a 3-word transfer occupies a 4-word lane stride in LDS."""
    from openequivariance_amd.codegen.uvu_det import UVUDetGenerator as G
    assert G.dma_pieces(1) == [(0, 1)]
    assert G.dma_pieces(3) == [(0, 3)]
    assert G.dma_pieces(5) in ([(0, 4), (4, 1)], [(0, 1), (1, 4)])
    assert sorted(w for _, w in G.dma_pieces(7)) == [3, 4]
    assert sorted(w for _, w in G.dma_pieces(6)) == [3, 3]
    for D in range(1, 12):
        pieces = G.dma_pieces(D)
        assert [k for k, _ in pieces] == [sum(w for _, w in pieces[:i]) for i in range(len(pieces))]
        assert sum(w for _, w in pieces) == D
    assert [G.dma_stride(w) for w in (1, 3, 4)] == [1, 4, 4]


def test_staged_conv_selection(monkeypatch):
    """The LDS-staged edge pipeline is used for fp32 problems whose multiplicity fits one chunk and
    whose stage leaves room for three wavefronts per SIMD; other problems keep the register pipeline."""
    from openequivariance_amd.codegen.uvu_det import UVUDetGenerator
    from openequivariance_amd.problem import ChannelwiseTPP
    from openequivariance_amd import tunables
    monkeypatch.setattr(tunables.current, "det_lds", None)
    small = UVUDetGenerator(ChannelwiseTPP("32x0e+32x1o+32x2e", "1x0e+1x1o+1x2e", "32x0e+32x1o+32x2e"))
    assert small.lds_forward and small.lds_backward and 12 * small.stage_words * 4 <= 160 * 1024
    large = UVUDetGenerator(ChannelwiseTPP("256x0e+256x1o+256x2e", "1x0e+1x1o+1x2e+1x3o", "256x0e+256x1o+256x2e"))
    assert not large.lds_forward and not large.lds_backward
    import numpy as np
    dbl = UVUDetGenerator(ChannelwiseTPP("32x0e+32x1o+32x2e", "1x0e+1x1o+1x2e", "32x0e+32x1o+32x2e",
                                         irrep_dtype=np.float64, weight_dtype=np.float64))
    assert not dbl.lds_forward and not dbl.lds_backward


def test_unsorted_conv_backward_selection(monkeypatch):
    """Unsorted edge lists: the backward scatters dX with atomics while a row of X is very short, and groups
    the edges by sender (three more grouping launches - the first of them only clears counters and may be
    skipped -, the segmented backward, larger workspace) from 128 values per edge on."""
    from openequivariance_amd.codegen.uvu_sorted import UVUSortedGenerator
    from openequivariance_amd.problem import ChannelwiseTPP
    from openequivariance_amd import tunables
    monkeypatch.setattr(tunables.current, "conv_backward", None)
    small = UVUSortedGenerator(ChannelwiseTPP("8x0e+8x1o+8x2e", "1x0e+1x1o+1x2e", "8x0e+8x1o+8x2e"))
    assert UVUSortedGenerator(ChannelwiseTPP("32x0e+32x1o+32x2e", "1x0e+1x1o+1x2e", "32x0e+32x1o+32x2e")).grouped_backward
    large = UVUSortedGenerator(ChannelwiseTPP("256x0e+256x1o+256x2e", "1x0e+1x1o+1x2e+1x3o", "256x0e+256x1o+256x2e"))
    assert not small.grouped_backward and large.grouped_backward
    _, bwd, ws = small.plan()
    assert [s["kernel"] for s in bwd] == ["backward"]
    group = (3 * 11 + 1000 + 1) * 8           # pointers, cursors, counters (11 each), position list, ticket
    tiles = -(-1000 // 200)                   # pieces of 2 x the mean of 100 edges per node
    pieces = lambda g, chunks: 256 + ((16 * chunks * tiles + 255) & ~255) + 2 * tiles * max(g.D1, g.D3) * 4
    assert ws(1000, 10) == ((group + 255) & ~255) + pieces(small, 1)
    fwd, bwd, ws = large.plan()
    assert [s["kernel"] for s in fwd] == ["group_clear", "group_count", "group_fill", "forward"]
    assert [bool(s.get("counter_clear")) for s in fwd] == [True, False, False, False]
    assert [s["kernel"] for s in bwd] == ["group_clear_backward", "group_count_backward", "group_fill_backward",
                                          "order_backward", "backward", "backward_dy_reduce"]
    assert bwd[4]["grid_y"] == 4 and bwd[4]["work_per_block"] == 1 and bwd[4]["grid_kind"] == 3
    # the forward's grouping and the backward's lie side by side (a prepared workspace serves both)
    main = 2 * group + 10 * 8 + 4 * 1000 * 16 * 4 + 8 + 4 * 4
    assert ws(1000, 10) == ((main + 255) & ~255) + pieces(large, 4)
    assert all(s.get("prep") for s in bwd[:4]) and not any(s.get("prep") for s in bwd[4:])
    src = large.render()
    for name in ("group_fill_backward", "backward_dy_reduce", "void backward("):
        assert name in src


def test_backward_split_over_output_block_groups():
    """Problems whose per-edge operands exceed 80 registers run the segmented backward as one launch per
    group of output blocks; the groups partition the output blocks and balance their operand counts."""
    from openequivariance_amd.codegen.uvu_det import UVUDetGenerator
    from openequivariance_amd.problem import ChannelwiseTPP
    large = UVUDetGenerator(ChannelwiseTPP("256x0e+256x1o+256x2e", "1x0e+1x1o+1x2e+1x3o", "256x0e+256x1o+256x2e"))
    assert large.H == 1 and [k for k, _ in large.backward_kernels()] == ["backward"] and large.dy_slots == 4
    mace = UVUDetGenerator(ChannelwiseTPP("128x0e+128x1o+128x2e", "1x0e+1x1o+1x2e+1x3o", "128x0e+128x1o+128x2e+128x3o"))
    assert mace.H == 2 and mace.dy_slots == 4 and mace.prefetch_backward
    assert sorted(sum(mace.out_groups, [])) == mace.used_out and all(mace.out_groups)
    _, bwd, ws = mace.plan()
    assert [s["kernel"] for s in bwd] == ["prep_backward", "order_backward", "backward", "backward_g1", "backward_dy_reduce"]
    assert mace.main_bytes(1000, 10) == (((2 * 11 + 10) * 8 + 4 * 1000 * 16 * 4 + 8 + 4 * 4) + 255) & ~255
    assert ws(1000, 10) == mace.main_bytes(1000, 10) + mace.piece_bytes(1000, 10)
    src = mace.render()
    assert "void backward_g1(" in src and "c * 2 + 1" in src
    with mace._group(1):
        assert {p.o.idx for p in mace.paths} == set(mace.out_groups[1])
    assert len(mace.paths) == 17                         # restored after the group context


def test_forward_split_over_output_block_groups():
    """The convolution forward keeps a node's output words in registers: beyond 100 (fp32) / 32 (fp64) words per
    channel it runs as one launch per group of output blocks.  The groups partition the output blocks, stay near
    the limit, and are cut along the in1 blocks; none of the benchmark configurations is split; fp64 splits the
    backward into groups of about 24 words."""
    from openequivariance_amd.benchmark import benchmark_configs as bc
    from openequivariance_amd.codegen.uvu_det import UVUDetGenerator
    from openequivariance_amd.codegen.uvu_sorted import UVUSortedGenerator
    from openequivariance_amd.problem import ChannelwiseTPP
    want = {"mace-large": (1, 3), "mace-medium": (1, 1), "nequip-lips": (2, 4), "nequip-revmd17-aspirin": (1, 1),
            "nequip-revmd17-toluene": (2, 4), "nequip-revmd17-benzene": (4, 10), "nequip-water": (1, 1)}
    for cfg in bc.mace_conv + bc.nequip_conv:
        for k, dt in enumerate((np.float32, np.float64)):
            g = UVUDetGenerator(ChannelwiseTPP(*cfg[:3], irrep_dtype=dt, weight_dtype=dt))
            words = lambda grp: sum(g.out[i].D for i in grp)
            assert len(g.fwd_groups) == want[cfg[3]][k], (cfg[3], dt)
            assert sorted(sum(g.fwd_groups, [])) == g.used_out and all(g.fwd_groups)
            assert max(map(words, g.fwd_groups)) <= 1.1 * g.FWD_SPLIT_WORDS[g.T] or len(g.fwd_groups) == 1
            fwd, _, _ = g.plan()
            names = [s["kernel"] for s in fwd if s["kernel"].startswith("forward")]
            assert names == ["forward"] + [f"forward_g{h}" for h in range(1, len(g.fwd_groups))]
            steps = [s for s in fwd if s["kernel"].startswith("forward")]
            assert all({k_: v for k_, v in s.items() if k_ != "kernel"} == {k_: v for k_, v in steps[0].items() if k_ != "kernel"}
                       for s in steps)
    for irreps in (workloads.NEQUIP, workloads.LARGE, workloads.MACE, workloads.NEQUIP_ALL, workloads.LARGE_ALL):
        assert len(UVUDetGenerator(ChannelwiseTPP(*irreps)).fwd_groups) == 1
    benz = ChannelwiseTPP(*[c for c in bc.nequip_conv if c[3] == "nequip-revmd17-benzene"][0][:3])
    g = UVUDetGenerator(benz)
    gathered = lambda groups: sum(sum(g.in1[a].D for a in {p.a.idx for p in g.paths if p.o.idx in grp}) for grp in groups)
    assert gathered(g.fwd_groups) < 0.5 * gathered(g.dealt_groups(4, lambda grp: sum(g.out[i].D for i in grp)))
    s = UVUSortedGenerator(benz)
    assert [st["kernel"] for st in s.plan()[0]][-4:] == ["forward", "forward_g1", "forward_g2", "forward_g3"]
    assert all(f"void {n}(" in s.render() for n in ("forward", "forward_g1", "forward_g2", "forward_g3"))
    mace64 = UVUDetGenerator(ChannelwiseTPP(*workloads.MACE, irrep_dtype=np.float64, weight_dtype=np.float64))
    assert mace64.H == 5 and not mace64.prefetch_backward


def test_receiver_order_pass_one_groups_share_no_in1_block():
    """Above 100 dZ words per lane (128 with 64 channels per wavefront) pass 1 of the receiver-order backward runs per
    group of output blocks; the
    groups partition the output blocks and no in1 block feeds two of them, so the launches write disjoint words of
    the per-edge dX rows.  The benchmark configurations stay one launch."""
    from openequivariance_amd.benchmark import benchmark_configs as bc
    from openequivariance_amd.codegen.uvu_recv import UVURecvGenerator
    from openequivariance_amd.problem import ChannelwiseTPP, TPProblem
    want = {"mace-large": 1, "mace-medium": 1, "nequip-lips": 2, "nequip-revmd17-aspirin": 1, "nequip-revmd17-toluene": 1,
            "nequip-revmd17-benzene": 3, "nequip-water": 1}
    for cfg in bc.mace_conv + bc.nequip_conv:
        g = UVURecvGenerator(ChannelwiseTPP(*cfg[:3]))
        assert g.HR == want[cfg[3]] and g.dy_slots == g.NCH * g.HR, cfg[3]
        assert sorted(sum(g.recv_groups, [])) == g.used_out
        ins = [{p.a.idx for p in g.paths if p.o.idx in grp} for grp in g.recv_groups]
        assert all(not (x & y) for k, x in enumerate(ins) for y in ins[k + 1:])
        words = sorted(g.spill_word.values())
        assert words == list(range(g.NW))
        names = [s["kernel"] for s in g.plan()[1]]
        assert names[names.index("backward"):][:g.HR + 1] == [k for k, _ in g.backward_kernels()] + ["backward_dx"]
        assert ("backward_dy_reduce" in names) == (g.dy_slots > 1)
    for irreps in (workloads.MACE, workloads.NEQUIP_ALL, workloads.LARGE_ALL):
        assert UVURecvGenerator(ChannelwiseTPP(*irreps)).HR == 1
    # every output block reads the one in1 block: nothing to split along
    ins = [(0, k, k, "uvu", True) for k in range(4)]
    one = UVURecvGenerator(TPProblem("64x3e", "1x0e+1x2e+1x4e+1x6e", "64x3e+64x3e+64x3e+64x3e", ins, shared_weights=False,
                                     internal_weights=False), recv_split=8)
    assert one.HR == 1
    assert UVURecvGenerator(ChannelwiseTPP(*workloads.NEQUIP), recv_split=4).HR == 3
    # fp64 has no LDS stage: pass 1 with register loads, a launch per in1 block, chosen where every launch holds at
    # most 32 dZ words
    from openequivariance_amd.conv import select_conv_generator
    f64 = lambda irreps: ChannelwiseTPP(*irreps, irrep_dtype=np.float64, weight_dtype=np.float64)
    mace64 = select_conv_generator(f64(workloads.MACE), True)
    assert isinstance(mace64, UVURecvGenerator) and not mace64.staged_edges and mace64.register_loads_fit
    assert [sum(mace64.out[i].D for i in grp) for grp in mace64.recv_groups] == [16, 24, 31]
    for irreps in (workloads.NEQUIP, workloads.LARGE, workloads.MACE_ALL):
        assert not isinstance(select_conv_generator(f64(irreps), True), UVURecvGenerator)
    assert not UVURecvGenerator(f64(workloads.MACE_ALL)).register_loads_fit
    # the operator over unsorted edge lists can run it as well (pass 1 then walks the receiver-grouped position list),
    # on request only: the second counting sort costs what the order gains
    from openequivariance_amd.codegen.uvu_sorted import UVUSortedGenerator
    assert not UVUSortedGenerator(f64(workloads.MACE)).recv_backward
    s64 = UVUSortedGenerator(f64(workloads.MACE), grouped_backward=True, recv_backward=True)
    assert s64.recv_backward and s64.bwd.register_loads_fit and s64.bwd.HR == 3 and not s64.bwd.staged_edges
