"""Problem description: normalisation, instruction enumeration, layouts - product vs oracle vs hand values."""
import numpy as np
import pytest

import openequivariance_amd as oeq
from openequivariance_amd.codegen.uvu import UVUGenerator
from oracle import spec

import common


def test_irreps_parsing_and_sort():
    ir = oeq.Irreps("128x0e+128x1o + 2e")
    assert ir.dim == 128 + 384 + 5 and len(ir) == 3 and repr(ir) == "128x0e+128x1o+1x2e"
    assert [s.start for s in ir.slices()] == [0, 128, 512]
    assert oeq.Irrep("3o").dim == 7 and oeq.Irrep("1e") in oeq.Irreps("2x1e")
    assert [repr(x) for x in oeq.Irrep("1o") * oeq.Irrep("2e")] == ["1o", "2o", "3o"]
    srt = oeq.Irreps("2x1o+3x0e+1x1o").sort()
    assert repr(srt.irreps) == "3x0e+2x1o+1x1o" and srt.inv == (1, 0, 2) and srt.p == (1, 0, 2)
    assert repr(oeq.Irreps("2x1o+1x1o+0x0e").simplify()) == "3x1o"
    with pytest.raises(ValueError):
        oeq.Irreps("2x1z")
    assert repr(oeq.Irreps.spherical_harmonics(3)) == "1x0e+1x1o+1x2e+1x3o"


def test_hand_values_of_path_coefficients():
    prob, oprob = common.readme_problem()
    assert prob.instructions[0].path_weight == pytest.approx(np.sqrt(5)) == pytest.approx(oprob.paths[0]["coeff"])
    prob, oprob = common.channelwise(common.MACE)
    for ins, p in zip(prob.instructions, oprob.paths):
        l3 = prob.irreps_out[ins.i_out].ir.l
        assert ins.path_weight == pytest.approx(np.sqrt(2 * l3 + 1)) == pytest.approx(p["coeff"])
    prob, oprob = common.fully_connected(common.DENSE)
    want = {0: np.sqrt(1 / 192), 1: np.sqrt(3 / 256), 2: np.sqrt(5 / 256)}
    for ins, p in zip(prob.instructions, oprob.paths):
        assert ins.path_weight == pytest.approx(want[prob.irreps_out[ins.i_out].ir.l]) == pytest.approx(p["coeff"])


@pytest.mark.parametrize("irr,paths,d1,d2,d3,wn,nnz", [
    (common.MACE, 17, 1152, 16, 9088, 2176, 215),
    (common.NEQUIP, 11, 288, 9, 1120, 352, 83),
    (common.LARGE, 13, 2304, 16, 11008, 3328, 125),
])
def test_channelwise_counts(irr, paths, d1, d2, d3, wn, nnz):
    prob, oprob = common.channelwise(irr)
    assert (len(prob.instructions), prob.irreps_in1.dim, prob.irreps_in2.dim, prob.irreps_out.dim, prob.weight_numel) \
        == (paths, d1, d2, d3, wn) == (len(oprob.paths), oprob.d1, oprob.d2, oprob.d3, oprob.weight_numel)
    assert sum(p.nnz for p in UVUGenerator(prob, "tp").paths) == nnz
    # same instruction order and output layout on both sides
    for ins, p in zip(prob.instructions, oprob.paths):
        assert (ins.i_in1, ins.i_in2, ins.i_out) == (p["i1"], p["i2"], p["io"])
    assert [(m.mul, m.ir.l, m.ir.p) for m in prob.irreps_out] == list(oprob.out)


def test_mace_column_table():
    """Explicit Z / W column table of the MACE problem (instruction -> in1 l, in2 l, out l, Z start)."""
    prob, _ = common.channelwise(common.MACE)
    table = [(0, 0, 0, 0), (1, 1, 0, 128), (2, 2, 0, 256), (0, 1, 1, 384), (1, 0, 1, 768), (1, 2, 1, 1152),
             (2, 1, 1, 1536), (2, 3, 1, 1920), (0, 2, 2, 2304), (1, 1, 2, 2944), (1, 3, 2, 3584), (2, 0, 2, 4224),
             (2, 2, 2, 4864), (0, 3, 3, 5504), (1, 2, 3, 6400), (2, 1, 3, 7296), (2, 3, 3, 8192)]
    offs = prob.irreps_out.offsets()
    for t, (l1, l2, l3, zoff) in enumerate(table):
        ins = prob.instructions[t]
        assert (prob.irreps_in1[ins.i_in1].ir.l, prob.irreps_in2[ins.i_in2].ir.l, prob.irreps_out[ins.i_out].ir.l,
                offs[ins.i_out]) == (l1, l2, l3, zoff)
        assert prob.weight_range_and_shape_for_instruction(t) == (128 * t, 128 * (t + 1), (128, 1))


def test_fully_connected_order_and_counts():
    prob, oprob = common.fully_connected(common.DENSE)
    order = [(0, 0, 0), (0, 1, 1), (0, 2, 2), (1, 0, 1), (1, 1, 0), (1, 1, 2), (1, 2, 1), (2, 0, 2), (2, 1, 1),
             (2, 2, 0), (2, 2, 2)]
    assert [(i.i_in1, i.i_in2, i.i_out) for i in prob.instructions] == order == \
        [(p["i1"], p["i2"], p["io"]) for p in oprob.paths]
    assert prob.weight_numel == 45056 == oprob.weight_numel
    assert prob.shared_weights and not prob.internal_weights


@pytest.mark.parametrize("inorm", ["component", "norm", "none"])
@pytest.mark.parametrize("pnorm", ["element", "path", "none"])
def test_normalisation_modes_agree_with_oracle(inorm, pnorm):
    a = ("3x0e+2x1o", "2x0e+1x1o", "4x0e+3x1o")
    ins = [(0, 0, 0, "uvw", True, 1.0), (1, 1, 0, "uvw", True, 2.0), (0, 1, 1, "uvw", True, 0.5), (1, 0, 1, "uvw", True)]
    kw = dict(irrep_normalization=inorm, path_normalization=pnorm, in1_var=[1.0, 2.0], in2_var=[0.5, 1.0],
              out_var=[1.0, 3.0])
    prob = oeq.TPProblem(*a, ins, shared_weights=True, internal_weights=False, **kw)
    oprob = spec.Problem(*a, ins, shared_weights=True, **kw)
    for i, p in zip(prob.instructions, oprob.paths):
        assert i.path_weight == pytest.approx(p["coeff"], rel=1e-14)
    # one value by hand: component/element, instruction 0: alpha = 1 / (1*0.5*3*2 + 2*1*2*1) * 1 * 1
    if (inorm, pnorm) == ("component", "element"):
        assert prob.instructions[0].path_weight == pytest.approx(np.sqrt(1.0 / (3.0 + 4.0)))


def test_constructor_errors():
    with pytest.raises(AssertionError):
        oeq.TPProblem("1x1o", "1x1o", "1x1o", [(0, 0, 0, "uvu", True)])          # parity
    with pytest.raises(AssertionError):
        oeq.TPProblem("1x0e", "1x1o", "1x3o", [(0, 0, 0, "uvu", True)])          # triangle rule
    p = oeq.TPProblem("1x0e", "1x0e", "1x0e", [(0, 0, 0, "uvu", False)])
    with pytest.raises(ValueError):
        p.weight_range_and_shape_for_instruction(0)


# ------------------------------------------------------------------ golden vectors of the reference's TPProblem
import json
import pathlib

GOLDEN_PROBLEMS = json.loads((pathlib.Path(__file__).parent / "golden" / "tpproblem.json").read_text())


@pytest.mark.parametrize("case", GOLDEN_PROBLEMS, ids=[c["name"] for c in GOLDEN_PROBLEMS])
def test_normalisation_matches_reference_golden(case):
    """Final path coefficients, weight shapes and sizes as computed by the reference's own TPProblem
    (tests/golden/make_golden.py), for the product's TPProblem and for the oracle's restatement."""
    from oracle import spec
    ins = [tuple(t) for t in case["instructions"]]
    exp = case["expect"]
    tpp = oeq.TPProblem(case["irreps_in1"], case["irreps_in2"], case["irreps_out"], ins, **case["kwargs"])
    assert [list(t.path_shape) for t in tpp.instructions] == exp["path_shapes"]
    assert np.allclose([t.path_weight for t in tpp.instructions], exp["path_weights"], rtol=1e-14, atol=0)
    assert tpp.weight_numel == exp["weight_numel"]
    assert [tpp.irreps_in1.dim, tpp.irreps_in2.dim, tpp.irreps_out.dim] == exp["dims"]
    assert bool(tpp.shared_weights) == exp["shared_weights"] and bool(tpp.internal_weights) == exp["internal_weights"]
    kw = {k: v for k, v in case["kwargs"].items() if k != "shared_weights"}
    op = spec.Problem(case["irreps_in1"], case["irreps_in2"], case["irreps_out"], ins,
                      shared_weights=exp["shared_weights"], **kw)
    assert np.allclose([p["coeff"] for p in op.paths], exp["path_weights"], rtol=1e-14, atol=0)
    assert [list(p["shape"]) for p in op.paths] == exp["path_shapes"]
    assert op.weight_numel == exp["weight_numel"] and [op.d1, op.d2, op.d3] == exp["dims"]


@pytest.mark.parametrize("name,irreps", [("mace", common.MACE), ("nequip", common.NEQUIP), ("large", common.LARGE),
                                         ("mace_all_parities", ("128x0e+128x1o+128x2e", "1x0e+1x1o+1x2e+1x3o",
                                                                "128x0e+128x1o+128x1e+128x2e+128x2o+128x3o+128x3e"))])
def test_channelwise_enumeration_matches_the_fixture(name, irreps):
    """The instruction order and output layout spelled out in the fixture (a literal enumeration,
    accepted by the reference's TPProblem) are what ChannelwiseTPP and the oracle produce."""
    from oracle import spec
    case = next(c for c in GOLDEN_PROBLEMS if c["name"] == name)
    prob = oeq.ChannelwiseTPP(*irreps)
    got = [(t.i_in1, t.i_in2, t.i_out) for t in prob.instructions]
    assert got == [tuple(t[:3]) for t in case["instructions"]]
    assert str(prob.irreps_out).replace(" ", "") == case["irreps_out"]
    op = spec.channelwise(*irreps)
    assert [(p["i1"], p["i2"], p["io"]) for p in op.paths] == got


def test_fully_connected_enumeration_matches_the_fixture():
    from oracle import spec
    case = next(c for c in GOLDEN_PROBLEMS if c["name"] == "dense_uvw")
    prob = oeq.FullyConnectedTPProblem(*common.DENSE, shared_weights=True, internal_weights=False)
    got = [(t.i_in1, t.i_in2, t.i_out, t.connection_mode) for t in prob.instructions]
    assert got == [tuple(t[:4]) for t in case["instructions"]]
    assert [(p["i1"], p["i2"], p["io"], p["mode"]) for p in spec.fully_connected(*common.DENSE, shared_weights=True).paths] == got


GOLDEN_IRREPS = json.loads((pathlib.Path(__file__).parent / "golden" / "irreps.json").read_text())


@pytest.mark.parametrize("case", GOLDEN_IRREPS["irreps"], ids=[c["text"] for c in GOLDEN_IRREPS["irreps"]])
def test_irreps_behave_like_the_reference(case):
    """Text form, sizes, slices and derived forms recorded from the reference's Irreps."""
    ir = oeq.Irreps(case["text"])
    assert repr(ir) == case["repr"] and ir.dim == case["dim"] and ir.num_irreps == case["num_irreps"]
    assert list(ir.ls) == case["ls"] and ir.lmax == case["lmax"] and len(ir) == case["length"]
    assert [m for m, _ in ir] == case["muls"] and [i.p for _, i in ir] == case["parities"]
    assert [[s.start, s.stop] for s in ir.slices()] == case["slices"]
    assert repr(ir.simplify()) == case["simplify"] and repr(ir.remove_zero_multiplicities()) == case["remove_zero"]
    srt = ir.sort()
    assert repr(srt.irreps) == case["sort"] and list(srt.p) == case["sort_p"] and list(srt.inv) == case["sort_inv"]
    assert repr(ir.regroup()) == case["regroup"]
    assert ir.count("1o") == case["count_1o"] and ("2e" in ir) == case["contains_2e"]
    assert repr(ir * 2) == case["times2"] and repr(ir + oeq.Irreps("1x3e")) == case["plus"]


def test_irrep_products_and_spherical_harmonics_like_the_reference():
    from openequivariance_amd.irreps import Irrep
    for key, want in GOLDEN_IRREPS["products"].items():
        a, b = key.split("*")
        assert [repr(x) for x in Irrep(a) * Irrep(b)] == want
    for l, want in GOLDEN_IRREPS["spherical_harmonics"].items():
        assert repr(oeq.Irreps.spherical_harmonics(int(l))) == want


@pytest.mark.parametrize("case", GOLDEN_PROBLEMS, ids=[c["name"] for c in GOLDEN_PROBLEMS])
def test_problem_text_and_weight_ranges_like_the_reference(case):
    tpp = oeq.TPProblem(case["irreps_in1"], case["irreps_in2"], case["irreps_out"], [tuple(t) for t in case["instructions"]],
                        **case["kwargs"])
    exp = case["expect"]
    assert str(tpp) == exp["text"]
    got = [tpp.weight_range_and_shape_for_instruction(i) for i in range(len(tpp.instructions))]
    assert [[a, b, list(sh)] for a, b, sh in got] == exp["weight_ranges"]
