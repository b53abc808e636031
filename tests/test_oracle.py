"""Pins the oracle's contraction and gradients by means that do not share its formulas."""
import numpy as np
import pytest

from oracle import spec, tp as otp, torch_cpu
from oracle.cg import wigner_3j
from oracle.spec import offsets

import common


def brute_forward(prob, X, Y, W):
    """Explicit loops over every index (tiny inputs only)."""
    B = X.shape[0]
    Z = np.zeros((B, prob.d3))
    o1, o2, o3 = offsets(prob.in1), offsets(prob.in2), offsets(prob.out)
    for b in range(B):
        for p in prob.paths:
            m1, l1, _ = prob.in1[p["i1"]]; m2, l2, _ = prob.in2[p["i2"]]; mo, l3, _ = prob.out[p["io"]]
            C = wigner_3j(l1, l2, l3)
            wrow = W if W.ndim == 1 else W[b]
            for u in range(m1):
                for v in range(m2):
                    for i in range(2 * l1 + 1):
                        for j in range(2 * l2 + 1):
                            xy = X[b, o1[p["i1"]] + u * (2 * l1 + 1) + i] * Y[b, o2[p["i2"]] + v * (2 * l2 + 1) + j]
                            for k in range(2 * l3 + 1):
                                if C[i, j, k] == 0.0:
                                    continue
                                if p["mode"] == "uvu":
                                    w = wrow[p["woff"] + u * m2 + v]
                                    Z[b, o3[p["io"]] + u * (2 * l3 + 1) + k] += p["coeff"] * w * C[i, j, k] * xy
                                else:
                                    for wi in range(mo):
                                        w = wrow[p["woff"] + (u * m2 + v) * mo + wi]
                                        Z[b, o3[p["io"]] + wi * (2 * l3 + 1) + k] += p["coeff"] * w * C[i, j, k] * xy
    return Z


PROBLEMS = {
    "uvu": lambda: spec.channelwise("2x0e+3x1o", "1x0e+1x1o+1x2e", "2x0e+3x1o+3x2e"),
    "uvu_v2": lambda: spec.Problem("3x0e+3x1o", "2x0e+2x1o", "3x0e+3x1o",
                                   [(0, 0, 0, "uvu", True), (1, 1, 0, "uvu", True), (1, 0, 1, "uvu", True)],
                                   shared_weights=False),
    "uvw_shared": lambda: spec.fully_connected("2x0e+3x1o", "1x0e+1x1o", "3x0e+2x1o", shared_weights=True),
    "uvw_batched": lambda: spec.fully_connected("2x0e+2x1o", "2x0e+1x1o", "2x0e+2x1o", shared_weights=False),
}


def _inputs(prob, B, seed):
    rng = np.random.default_rng(seed)
    W = rng.standard_normal(prob.weight_numel if prob.shared_weights else (B, prob.weight_numel))
    return rng.standard_normal((B, prob.d1)), rng.standard_normal((B, prob.d2)), W, rng.standard_normal((B, prob.d3))


@pytest.mark.parametrize("name", list(PROBLEMS))
def test_forward_against_brute_force(name):
    prob = PROBLEMS[name]()
    X, Y, W, _ = _inputs(prob, 3, 0)
    np.testing.assert_allclose(otp.forward(prob, X, Y, W), brute_forward(prob, X, Y, W), atol=1e-12)


@pytest.mark.parametrize("name", list(PROBLEMS))
def test_backward_against_finite_differences(name):
    prob = PROBLEMS[name]()
    X, Y, W, G = _inputs(prob, 2, 1)
    dX, dY, dW = otp.backward(prob, X, Y, W, G)
    f = lambda x, y, w: float((otp.forward(prob, x, y, w) * G).sum())
    rng = np.random.default_rng(2)
    h = 1e-6
    for arr, grad, which in ((X, dX, 0), (Y, dY, 1), (W, dW, 2)):
        for _ in range(6):
            idx = tuple(rng.integers(0, s) for s in arr.shape)
            plus, minus = arr.copy(), arr.copy()
            plus[idx] += h; minus[idx] -= h
            args_p = [X, Y, W]; args_m = [X, Y, W]
            args_p[which] = plus; args_m[which] = minus
            fd = (f(*args_p) - f(*args_m)) / (2 * h)
            assert grad[idx] == pytest.approx(fd, rel=1e-6, abs=1e-7)


@pytest.mark.parametrize("name", list(PROBLEMS))
def test_backward_against_torch_autograd_and_adjoint_identity(name):
    import torch
    prob = PROBLEMS[name]()
    X, Y, W, G = _inputs(prob, 4, 3)
    dX, dY, dW = otp.backward(prob, X, Y, W, G)
    t = torch_cpu.TorchTP(prob, torch.float64)
    x, y, w = (torch.tensor(a, requires_grad=True) for a in (X, Y, W))
    z = t.forward(x, y, w)
    np.testing.assert_allclose(z.detach().numpy(), otp.forward(prob, X, Y, W), atol=1e-12)
    z.backward(torch.tensor(G))
    for got, ref in ((dX, x.grad), (dY, y.grad), (dW, w.grad)):
        np.testing.assert_allclose(got, ref.numpy(), atol=1e-11)
    gz = float((G * otp.forward(prob, X, Y, W)).sum())          # tri-linearity: <G,Z> = <X,dX> = <Y,dY> = <W,dW>
    for a, g in ((X, dX), (Y, dY), (W, dW)):
        assert float((a * g).sum()) == pytest.approx(gz, rel=1e-11)


@pytest.mark.parametrize("name", ["uvw_shared", "uvu_shared_v2", "dense"])
def test_shared_weight_gradient_against_backward_and_finite_differences(name):
    """The chunked dW-only routine (used where the full backward is too slow) against ``backward`` on a
    batch that spans several chunks with a ragged last one, and against a central finite difference."""
    prob = {"uvw_shared": PROBLEMS["uvw_shared"],
            "uvu_shared_v2": lambda: spec.Problem("3x0e+3x1o", "2x0e+2x1o", "3x0e+3x1o",
                                                  [(0, 0, 0, "uvu", True), (1, 1, 0, "uvu", True), (1, 0, 1, "uvu", True)],
                                                  shared_weights=True),
            "dense": lambda: spec.fully_connected(*common.DENSE, shared_weights=True)}[name]()
    X, Y, W, G = _inputs(prob, 23, 5)
    dW = otp.shared_weight_gradient(prob, X, Y, G, chunk=7)
    np.testing.assert_allclose(dW, otp.backward(prob, X, Y, W, G)[2], rtol=1e-12, atol=1e-12)
    rng = np.random.default_rng(6)
    h = 1e-6
    for _ in range(4):
        q = int(rng.integers(0, prob.weight_numel))
        plus, minus = W.copy(), W.copy()
        plus[q] += h; minus[q] -= h
        fd = float(((otp.forward(prob, X, Y, plus) - otp.forward(prob, X, Y, minus)) * G).sum()) / (2 * h)
        assert dW[q] == pytest.approx(fd, rel=1e-6, abs=1e-7)


def test_equivariance_under_rotation_and_inversion():
    """Z(D1 x, D2 y) = D3 Z(x, y) with Wigner matrices generated from the coupling tensors' own
    invariance generators (rotation) and parity signs (inversion)."""
    from scipy.linalg import expm, block_diag
    from test_wigner import _rotation_generators
    prob = spec.channelwise("2x0e+2x1o+2x2e", "1x0e+1x1o+1x2e", "2x0e+2x1o+2x2e+2x3o")
    X, Y, W, _ = _inputs(prob, 3, 5)
    ang = np.array([0.3, -1.1, 0.7])

    def rep(irreps, parity):
        blocks = []
        for m, l, p in irreps:
            g = _rotation_generators(l)
            d = expm(sum(a * gi for a, gi in zip(ang, g)))
            if parity:
                d = d * p
            blocks += [d] * m
        return block_diag(*blocks)
    for parity in (False, True):
        D1, D2, D3 = rep(prob.in1, parity), rep(prob.in2, parity), rep(prob.out, parity)
        lhs = otp.forward(prob, X @ D1.T, Y @ D2.T, W)
        rhs = otp.forward(prob, X, Y, W) @ D3.T
        np.testing.assert_allclose(lhs, rhs, atol=1e-11)


def test_readme_example_structure():
    """1x2e (x) 1x3e -> 1x2e with one weight: Z = sqrt(5) * w * C(2,3,2) . x . y."""
    prob = spec.Problem("1x2e", "1x3e", "1x2e", [(0, 0, 0, "uvu", True)], shared_weights=False)
    rng = np.random.default_rng(0)
    X, Y, W = rng.uniform(size=(4, 5)), rng.uniform(size=(4, 7)), rng.uniform(size=(4, 1))
    ref = np.sqrt(5) * W * np.einsum("ijk,zi,zj->zk", wigner_3j(2, 3, 2), X, Y)
    np.testing.assert_allclose(otp.forward(prob, X, Y, W), ref, atol=1e-13)


def test_conv_against_edge_loop():
    prob = spec.channelwise("2x0e+2x1o", "1x0e+1x1o", "2x0e+2x1o")
    rng = np.random.default_rng(7)
    N, E = 6, 20
    rows, cols = common.random_graph(N, E, 3)
    X, Y, W, G = rng.standard_normal((N, prob.d1)), rng.standard_normal((E, prob.d2)), \
        rng.standard_normal((E, prob.weight_numel)), rng.standard_normal((N, prob.d3))
    Z = np.zeros((N, prob.d3)); dX = np.zeros_like(X); dY = np.zeros_like(Y); dW = np.zeros_like(W)
    for e in range(E):
        Z[rows[e]] += otp.forward(prob, X[cols[e]][None], Y[e][None], W[e][None])[0]
        gx, gy, gw = otp.backward(prob, X[cols[e]][None], Y[e][None], W[e][None], G[rows[e]][None])
        dX[cols[e]] += gx[0]; dY[e] = gy[0]; dW[e] = gw[0]
    np.testing.assert_allclose(otp.conv_forward(prob, X, Y, W, rows, cols), Z, atol=1e-12)
    for got, ref in zip(otp.conv_backward(prob, X, Y, W, G, rows, cols), (dX, dY, dW)):
        np.testing.assert_allclose(got, ref, atol=1e-12)


def test_coord_graph_and_transpose_perm():
    rows, cols = common.random_graph(9, 40, 11)
    r, c, tperm, order = otp.coord_graph(rows, cols)
    assert np.all(np.diff(r) >= 0) and sorted(zip(r, c)) == sorted(zip(rows, cols))
    # tperm walks the receiver-sorted list in (sender, receiver) order and is a permutation
    assert sorted(tperm) == list(range(40))
    key = list(zip(c[tperm], r[tperm]))
    assert key == sorted(key)
    # product's CoordGraph builds the same thing
    import openequivariance_amd as oeq
    gph = oeq.CoordGraph(np.zeros((9, 3)), rows, cols)
    assert np.array_equal(gph.rows, r) and np.array_equal(gph.cols, c) and np.array_equal(gph.transpose_perm, tperm)


def test_sort_by_receiver_matches_coord_graph():
    """The torch graph preparation (any device; CPU tensors here) gives the oracle's sorted edge
    list and transpose permutation, also with duplicate edges and isolated nodes."""
    import torch
    import openequivariance_amd as oeq
    rows, cols = common.random_graph(9, 40, 11)
    rows = np.concatenate([rows, rows[:5]])            # duplicate edges: ties broken by position
    cols = np.concatenate([cols, cols[:5]])
    r, c, tperm, order = otp.coord_graph(rows, cols)
    rs, cs, rperm, tp = oeq.sort_by_receiver(torch.from_numpy(rows), torch.from_numpy(cols), 12)
    assert np.array_equal(rs.numpy(), r) and np.array_equal(cs.numpy(), c)
    assert np.array_equal(rows[rperm.numpy()], r) and np.array_equal(cols[rperm.numpy()], c)
    key = list(zip(cs.numpy()[tp.numpy()], rs.numpy()[tp.numpy()]))
    assert key == sorted(key) and sorted(tp.tolist()) == list(range(45))
    assert np.array_equal(tp.numpy(), tperm)
    e = torch.zeros(0, dtype=torch.int64)
    assert all(t.numel() == 0 for t in oeq.sort_by_receiver(e, e))
