"""The external ("oeq") weight order: product permutation vs the oracle's procedural restatement."""
import numpy as np
import pytest

import openequivariance_amd as oeq
from openequivariance_amd.weight_order import WeightReorder, is_identity, oeq_from_e3nn_permutation
from oracle import spec, weights as ow

import common


def test_identity_for_uvu_with_single_multiplicity_second_operand():
    for irr in (common.MACE, common.NEQUIP, common.LARGE):
        prob, oprob = common.channelwise(irr)
        assert is_identity(oeq_from_e3nn_permutation(prob))
        w = np.arange(oprob.weight_numel, dtype=np.float64)
        assert np.array_equal(ow.e3nn_to_oeq(oprob, w), w)


def test_dense_uvw_closed_form_index():
    """64 x 1 x 64 blocks: oeq = 4096 p + (u//32) 2048 + (w//32) 1024 + (u%32) 32 + (w%32)."""
    prob, oprob = common.fully_connected(common.DENSE)
    perm = oeq_from_e3nn_permutation(prob)
    p, u, w = np.meshgrid(np.arange(11), np.arange(64), np.arange(64), indexing="ij")
    e3nn = 4096 * p + 64 * u + w
    oeq_idx = 4096 * p + (u // 32) * 2048 + (w // 32) * 1024 + (u % 32) * 32 + (w % 32)
    expect = np.empty(45056, dtype=np.int64)
    expect[oeq_idx.ravel()] = e3nn.ravel()
    assert np.array_equal(perm, expect)
    wv = np.random.default_rng(0).standard_normal(45056)
    assert np.array_equal(ow.e3nn_to_oeq(oprob, wv), wv[perm])


def test_hand_case_chunked_transpose():
    """uvu, u = 2, v = 3 (one chunk each): e3nn [u][v] -> oeq [v][u]."""
    ins = [(0, 0, 0, "uvu", True)]
    prob = oeq.TPProblem("2x1e", "3x0e", "2x1e", ins, shared_weights=False, internal_weights=False)
    assert list(oeq_from_e3nn_permutation(prob)) == [0, 3, 1, 4, 2, 5]


@pytest.mark.parametrize("case", ["uvu_ragged", "uvw_ragged", "uvw_v"])
def test_ragged_chunks_roundtrip_and_agreement(case):
    if case == "uvu_ragged":
        a = ("40x0e+70x1o", "3x0e+35x1o", "40x0e+70x1o")
        ins = [(0, 0, 0, "uvu", True), (1, 1, 0, "uvu", True), (1, 0, 1, "uvu", True)]
        ins = [(0, 0, 0, "uvu", True), (1, 0, 1, "uvu", True)]
        prob = oeq.TPProblem(*a, ins, shared_weights=False, internal_weights=False)
        oprob = spec.Problem(*a, ins, shared_weights=False)
    elif case == "uvw_ragged":
        a = ("40x0e+70x1o", "1x0e+1x1o", "33x0e+65x1o")
        prob, oprob = common.fully_connected(a)
    else:
        a = ("5x0e+34x1o", "3x0e+2x1o", "36x0e+7x1o")
        prob, oprob = common.fully_connected(a)
    r = WeightReorder(prob)
    rng = np.random.default_rng(1)
    for batch in ((), (3,)):
        w = rng.standard_normal(batch + (prob.weight_numel,))
        out = np.zeros_like(w)
        r.e3nn_to_oeq(w, out, bool(batch))
        assert np.array_equal(out, ow.e3nn_to_oeq(oprob, w))
        back = np.zeros_like(w)
        r.oeq_to_e3nn(out, back, bool(batch))
        assert np.array_equal(back, w)
        assert np.array_equal(ow.oeq_to_e3nn(oprob, out), w)
