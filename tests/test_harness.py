"""Benchmark/correctness harness: host-side pieces (buffers, work models, comparison, metadata)."""
import json

import numpy as np
import pytest

import common
import openequivariance_amd as oeq
from openequivariance_amd.benchmark import perf_metrics_utils as pm
from openequivariance_amd.benchmark import random_buffer_utils as rb
from openequivariance_amd.benchmark.correctness_utils import check_similiarity, correctness_forward
from openequivariance_amd.benchmark.TestBenchmarkSuite import TestBenchmarkSuite, TestDefinition


def test_random_buffers_follow_the_seeded_draw_order():
    prob, _ = common.channelwise(common.NEQUIP)
    in1, in2, w, out = rb.get_random_buffers_forward(prob, 7, 12345)
    rng = np.random.default_rng(12345)            # in1, in2, weights: the order of the reference's generator
    assert np.array_equal(in1, rng.uniform(size=(7, 288)).astype(np.float32))
    assert np.array_equal(in2, rng.uniform(size=(7, 9)).astype(np.float32))
    assert np.array_equal(w, rng.uniform(size=(7, 352)).astype(np.float32))
    assert out.shape == (7, 1120) and not out.any()
    b = rb.get_random_buffers_backward(prob, 7, 12345)
    assert np.array_equal(b[0], in1) and np.array_equal(b[1], in2)          # same seed, same leading draws
    assert b[2].shape == (7, 1120) and b[3].shape == (7, 352)
    assert all(not g.any() for g in b[4:]) and [g.shape for g in b[4:]] == [(7, 352), (7, 288), (7, 9)]
    shared, _ = common.fully_connected(("4x0e", "1x0e", "4x0e"), shared=True)
    assert rb.get_random_buffers_forward(shared, 5, 1)[2].shape == (16,)
    c = rb.get_random_buffers_backward_conv(prob, 4, 9, 3)
    assert [a.shape for a in c] == [(4, 288), (9, 9), (4, 1120), (9, 352), (9, 352), (4, 288), (9, 9)]


def test_work_models():
    prob, _ = common.channelwise(common.MACE)
    assert pm.calculate_minimum_memory_streamed_forward(prob, 10)["total"] == 49728 * 10
    assert pm.calculate_minimum_memory_streamed_backward(prob, 10)["total"] == 63104 * 10
    # distinct (l1, l2, l3) triples counted once; (2,3,2) alone has 28 nonzeros
    one, _ = common.readme_problem()
    assert pm.calculate_total_nnz(one) == 28 == pm.count_cg_non_zero(2, 3, 2)
    f = pm.calculate_minimum_flops_forward(one, 3)
    pairs = pm.sparse_outer_product_work(oeq.wigner_3j(2, 3, 2))
    assert f == {"outer_products": pairs * 3, "CG_decomposition": 2 * 28 * 3, "linear_combination": 2 * 5 * 3,
                 "total": (pairs + 56 + 10) * 3}
    with pytest.raises(NotImplementedError):
        pm.calculate_minimum_flops_backward(one, 3)


def test_check_similiarity():
    a = np.zeros((3, 2), dtype=np.float32)
    b = a.copy()
    b[1, 1] = 1e-3
    assert check_similiarity("x", a, a, 1e-6) == {"shape_match": True, "diff_Linf_norm": 0.0, "pass": True}
    r = check_similiarity("x", b, a, 1e-6)
    assert r["shape_match"] and not r["pass"] and abs(r["diff_Linf_norm"] - 1e-3) < 1e-9
    r = check_similiarity("x", a[:2], a, 1e-6)
    assert r == {"shape_match": False, "diff_Linf_norm": float("inf"), "pass": False}


def test_suite_metadata_and_validation():
    prob, _ = common.channelwise(common.NEQUIP)
    prob.label = "nequip"
    tests = [TestDefinition(oeq.TensorProduct, prob, "forward"),
             TestDefinition(oeq.TensorProduct, prob, "backward", correctness=False)]
    TestBenchmarkSuite.validate_inputs(tests)
    md = TestBenchmarkSuite.generate_metadata(tests)
    json.dumps(md)
    assert md["implementations"] == ["LoopUnrollTP"] and md["directions"] == ["forward", "backward"]
    assert md["config_labels"] == ["nequip"] and md["did_correctness"] and md["did_benchmark"]
    assert md["test details"][1] == {"implementation": "LoopUnrollTP", "problem": repr(prob), "direction": "backward",
                                     "correctness": False, "benchmark": True}
    with pytest.raises(AssertionError):
        TestBenchmarkSuite.validate_inputs([TestDefinition(oeq.TensorProduct, prob, "sideways")])
    with pytest.raises(AssertionError):
        TestBenchmarkSuite.validate_inputs([])
    with pytest.raises(ValueError):
        TestBenchmarkSuite().run(tests)            # an output folder is required


def test_correctness_needs_a_reference_implementation():
    prob, _ = common.readme_problem()
    with pytest.raises(NotImplementedError):
        correctness_forward(prob, oeq.TensorProduct, None, 4, 1e-5, 1)
