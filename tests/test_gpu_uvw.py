"""GPU parity of the dense uvw tensor product (shared weights, matrix cores) against the fp64
oracle; weights and their gradient are compared after the documented e3nn <-> oeq reordering."""
import numpy as np
import pytest

import common
from common import FP32_TOL, FP64_TOL, rel_err
from oracle import spec, tp as otp, weights as ow

pytestmark = pytest.mark.gpu


def _run(irreps, n, seed, dtype, w_scale=0.125, sh_lmax=None):
    import torch
    import openequivariance_amd as oeq
    tol = FP32_TOL if dtype == np.float32 else FP64_TOL
    prob, oprob = common.fully_connected(irreps, shared=True, dtype=dtype)
    X, Y, We, G = common.tp_inputs(prob, n, seed, dtype, sh_lmax, w_scale=w_scale)
    tp = oeq.TensorProduct(prob, torch_op=True)
    W = np.zeros_like(We)
    tp.reorder_weights_e3nn_to_oeq(We, W, False)
    assert np.array_equal(W, ow.e3nn_to_oeq(oprob, We))          # product permutation == oracle's procedure
    dev = torch.device("cuda:0")
    x, y, w = (torch.tensor(a, device=dev, requires_grad=True) for a in (X, Y, W))
    z = tp(x, y, w)
    z.backward(torch.tensor(G, device=dev))
    torch.cuda.synchronize()
    Zr = otp.forward(oprob, X, Y, We)
    dXr, dYr, dWr = otp.backward(oprob, X, Y, We, G)
    dW = np.zeros_like(We)
    tp.reorder_weights_oeq_to_e3nn(w.grad.cpu().numpy(), dW, False)
    errs = dict(Z=rel_err(z.detach().cpu().numpy(), Zr), dX=rel_err(x.grad.cpu().numpy(), dXr),
                dY=rel_err(y.grad.cpu().numpy(), dYr), dW=rel_err(dW, dWr))
    print(f"n={n} {errs}", flush=True)
    for k, v in errs.items():
        assert v <= tol, f"{k}: relative error {v:.3e} > {tol}"
    return tp, (x, y, w, torch.tensor(G, device=dev))


@pytest.mark.parametrize("n", [1, 16, 1000])
def test_dense_uvw_fp32(cuda, n):
    """benchmark configuration 4 problem: 64x0e+64x1o+64x2e (x) SH(lmax 2) -> same, 11 paths, shared W ~ N(0, 1/64)."""
    _run(common.DENSE, n, 40 + n, np.float32, sh_lmax=2)


def test_dense_uvw_fp64(cuda):
    _run(common.DENSE, 333, 41, np.float64, sh_lmax=2)


def test_ragged_uvw(cuda):
    """Multiplicities that are not multiples of the 16 x 4 MFMA tile."""
    _run(("5x0e+21x1o", "1x0e+1x1o+1x2e", "18x0e+7x1o+3x2e"), 77, 42, np.float32)
    _run(("5x0e+21x1o", "1x0e+1x1o+1x2e", "18x0e+7x1o+3x2e"), 50, 43, np.float64)


def test_large_multiplicity_uvw(cuda):
    """mul 96 > 64: more than four 16-channel subtiles per block."""
    _run(("96x0e+96x1o", "1x0e+1x1o", "80x0e+40x1o"), 100, 44, np.float32)


def test_dw_bit_reproducible_and_full_batch(cuda):
    """Full batch of config 4 (100 000 rows): dW is a deterministic two-stage sum, and the adjoint
    identity <G, Z> = <X, dX> = <Y, dY> = <W, dW> holds (size-independent check)."""
    import torch
    import openequivariance_amd as oeq
    prob, oprob = common.fully_connected(common.DENSE, shared=True)
    n = 100000
    X, Y, We, G = common.tp_inputs(prob, n, 12348, np.float32, 2, w_scale=0.125)
    tp = oeq.TensorProduct(prob, torch_op=True)
    x, y, w = (torch.tensor(a, device=cuda, requires_grad=True) for a in (X, Y, We))
    g = torch.tensor(G, device=cuda)
    z = tp(x, y, w)
    z.backward(g)
    gz = (g.double() * z.detach().double()).sum().item()
    for name, a in (("X", x), ("Y", y), ("W", w)):
        v = (a.detach().double() * a.grad.double()).sum().item()
        assert abs(v - gz) <= 2e-5 * abs(gz), f"<{name}, d{name}> = {v} vs <G, Z> = {gz}"
    w2 = w.detach().clone().requires_grad_(True)
    tp(x.detach(), y.detach(), w2).backward(g)
    assert torch.equal(w.grad, w2.grad)
    # rows against the oracle (W here is already in oeq order; map it back for the oracle)
    We_ = ow.oeq_to_e3nn(oprob, We)
    sl = slice(99990, 100000)
    assert rel_err(z.detach()[sl].cpu().numpy(), otp.forward(oprob, X[sl], Y[sl], We_)) <= FP32_TOL


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_full_batch_dw_element_wise(cuda, dtype):
    """dW of the full config-4 batch (100 000 rows) element by element against the oracle's dW accumulated in
    fp64 over chunks of rows on the CPU, plus the last rows of Z, dX and dY against the oracle."""
    import torch
    import openequivariance_amd as oeq
    tol = FP32_TOL if dtype == np.float32 else FP64_TOL
    prob, oprob = common.fully_connected(common.DENSE, shared=True, dtype=dtype)
    n = 100000
    X, Y, We, G = common.tp_inputs(prob, n, 12349, dtype, 2, w_scale=0.125)
    tp = oeq.TensorProduct(prob, torch_op=True)
    W = ow.e3nn_to_oeq(oprob, We)
    x, y, w = (torch.tensor(a, device=cuda, requires_grad=True) for a in (X, Y, W))
    z = tp(x, y, w)
    z.backward(torch.tensor(G, device=cuda))
    torch.cuda.synchronize()
    dWr = otp.shared_weight_gradient(oprob, X, Y, G)
    errs = dict(dW=rel_err(ow.oeq_to_e3nn(oprob, w.grad.cpu().numpy()), dWr))
    sl = slice(n - 24, n)
    dXr, dYr, _ = otp.backward(oprob, X[sl], Y[sl], We, G[sl])
    errs.update(Z=rel_err(z.detach()[sl].cpu().numpy(), otp.forward(oprob, X[sl], Y[sl], We)),
                dX=rel_err(x.grad[sl].cpu().numpy(), dXr), dY=rel_err(y.grad[sl].cpu().numpy(), dYr))
    print(f"n={n} {np.dtype(dtype).name} {errs}", flush=True)
    for k, v in errs.items():
        assert v <= tol, f"{k}: relative error {v:.3e} > {tol}"


def test_uvw_tensors_beyond_two_giga_elements(cuda):
    """3.8 M rows of the config-4 problem: X, Z and their gradients have more than 2^31 elements each.
    Sampled rows (start, around element 2^31, end) of Z, dX, dY against the oracle; dW, which sums over
    all rows, against the sum of the dW of the two halves of the batch (each below 2^31 elements)."""
    import torch
    import openequivariance_amd as oeq
    from openequivariance_amd.sh import random_unit_vectors, spherical_harmonics
    prob, oprob = common.fully_connected(common.DENSE, shared=True)
    n = 3_800_000
    d1, d3, wn = prob.irreps_in1.dim, prob.irreps_out.dim, prob.weight_numel
    assert n * d1 > 2 ** 31 and n * d3 > 2 ** 31
    gen = torch.Generator(device=cuda)
    gen.manual_seed(98)
    x = torch.randn(n, d1, device=cuda, generator=gen, requires_grad=True)
    g = torch.randn(n, d3, device=cuda, generator=gen)
    w = (0.125 * torch.randn(wn, device=cuda, generator=gen)).requires_grad_(True)
    Y = spherical_harmonics(2, random_unit_vectors(n, np.random.default_rng(98))).astype(np.float32)
    y = torch.tensor(Y, device=cuda, requires_grad=True)
    tp = oeq.TensorProduct(prob, torch_op=True)
    z = tp(x, y, w)
    z.backward(g)
    torch.cuda.synchronize()
    mid = 2 ** 31 // d1
    rows = np.r_[0:20, mid - 10:mid + 10, n - 20:n]
    t = torch.from_numpy(rows).to(cuda)
    We = ow.oeq_to_e3nn(oprob, w.detach().cpu().numpy())
    Xs, Gs = x.detach()[t].cpu().numpy(), g[t].cpu().numpy()
    Zr = otp.forward(oprob, Xs, Y[rows], We)
    dXr, dYr, _ = otp.backward(oprob, Xs, Y[rows], We, Gs)
    errs = dict(Z=rel_err(z.detach()[t].cpu().numpy(), Zr), dX=rel_err(x.grad[t].cpu().numpy(), dXr),
                dY=rel_err(y.grad[t].cpu().numpy(), dYr))
    half = n // 2
    parts = []
    for sl in (slice(0, half), slice(half, n)):
        wh = w.detach().clone().requires_grad_(True)
        tp(x.detach()[sl], y.detach()[sl], wh).backward(g[sl])
        parts.append(wh.grad.double())
    errs["dW"] = float(((parts[0] + parts[1]) - w.grad.double()).abs().max() / w.grad.double().abs().max())
    print(f"n={n} rows sampled={rows.size} {errs}", flush=True)
    for k, v in errs.items():
        assert v <= FP32_TOL, f"{k}: relative error {v:.3e}"


UVW_MUL2 = {
    "small": ("5x0e+21x1o", "3x0e+2x1o", "18x0e+7x1o"),
    "ragged_v_3x0e+35x1o": ("20x0e+33x1o", "3x0e+35x1o", "17x0e+40x1o"),        # v beyond one 32-chunk
    "wide": ("70x0e", "4x0e+2x1o", "66x0e+33x1o"),
}


@pytest.mark.parametrize("name", sorted(UVW_MUL2))
@pytest.mark.parametrize("shared", [True, False])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_uvw_several_copies_of_the_second_operand(cuda, name, shared, dtype):
    """uvw with mul(in2) > 1, shared and per-row weights, through reorder_weights_e3nn_to_oeq: the external
    order stores each 32-chunk block [v][u][w] (reference: ComputationSchedule.py:146-230, :427-471;
    loop_unroll_tp.cuh:48-60 walks v)."""
    import torch
    import openequivariance_amd as oeq
    tol = FP32_TOL if dtype == np.float32 else FP64_TOL
    prob, oprob = common.fully_connected(UVW_MUL2[name], shared=shared, dtype=dtype)
    n = 37
    X, Y, We, G = common.tp_inputs(prob, n, 47, dtype, w_scale=0.1)
    tp = oeq.TensorProduct(prob, torch_op=True)
    W = np.zeros_like(We)
    tp.reorder_weights_e3nn_to_oeq(We, W, not shared)
    assert np.array_equal(W, ow.e3nn_to_oeq(oprob, We))
    x, y, w = (torch.tensor(a, device=cuda, requires_grad=True) for a in (X, Y, W))
    z = tp(x, y, w)
    z.backward(torch.tensor(G, device=cuda))
    torch.cuda.synchronize()
    dXr, dYr, dWr = otp.backward(oprob, X, Y, We, G)
    assert rel_err(z.detach().cpu().numpy(), otp.forward(oprob, X, Y, We)) <= tol
    assert rel_err(x.grad.cpu().numpy(), dXr) <= tol
    assert rel_err(y.grad.cpu().numpy(), dYr) <= tol
    assert rel_err(ow.oeq_to_e3nn(oprob, w.grad.cpu().numpy()), dWr) <= tol


DIFFDOCK = {"DiffDock-L=1": ("10x1o+10x1e+48x0e+48x0o", "1x0e+1x1o", "10x1o+10x1e+48x0e+48x0o"),
            "DiffDock-L=2": ("10x1o+10x1e+48x0e+48x0o", "1x0e+1x1o+1x2e", "10x1o+10x1e+48x0e+48x0o")}


@pytest.mark.parametrize("name", list(DIFFDOCK))
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_uvw_per_row_weights_diffdock(cuda, name, dtype):
    """uvw with shared_weights=False (reference: benchmark/benchmark_configs.py:44-48)."""
    import torch
    import openequivariance_amd as oeq
    tol = FP32_TOL if dtype == np.float32 else FP64_TOL
    prob, oprob = common.fully_connected(DIFFDOCK[name], shared=False, dtype=dtype)
    X, Y, We, G = common.tp_inputs(prob, 129, 45, dtype, w_scale=0.2)
    tp = oeq.TensorProduct(prob, torch_op=True)
    W = ow.e3nn_to_oeq(oprob, We)
    x, y, w = (torch.tensor(a, device=cuda, requires_grad=True) for a in (X, Y, W))
    z = tp(x, y, w)
    z.backward(torch.tensor(G, device=cuda))
    dXr, dYr, dWr = otp.backward(oprob, X, Y, We, G)
    assert rel_err(z.detach().cpu().numpy(), otp.forward(oprob, X, Y, We)) <= tol
    assert rel_err(x.grad.cpu().numpy(), dXr) <= tol
    assert rel_err(y.grad.cpu().numpy(), dYr) <= tol
    assert rel_err(ow.oeq_to_e3nn(oprob, w.grad.cpu().numpy()), dWr) <= tol


def test_uvw_per_row_weights_wide(cuda):
    """Multiplicities above 64 on both sides (several lane chunks), ragged 32-blocks in the weight order."""
    import torch
    import openequivariance_amd as oeq
    prob, oprob = common.fully_connected(("70x0e+40x1o", "1x0e+1x1o", "66x0e+33x1o"), shared=False)
    X, Y, We, G = common.tp_inputs(prob, 33, 46, w_scale=0.2)
    tp = oeq.TensorProduct(prob, torch_op=True)
    W = ow.e3nn_to_oeq(oprob, We)
    x, y, w = (torch.tensor(a, device=cuda, requires_grad=True) for a in (X, Y, W))
    z = tp(x, y, w)
    z.backward(torch.tensor(G, device=cuda))
    dXr, dYr, dWr = otp.backward(oprob, X, Y, We, G)
    assert rel_err(z.detach().cpu().numpy(), otp.forward(oprob, X, Y, We)) <= FP32_TOL
    assert rel_err(x.grad.cpu().numpy(), dXr) <= FP32_TOL
    assert rel_err(y.grad.cpu().numpy(), dYr) <= FP32_TOL
    assert rel_err(ow.oeq_to_e3nn(oprob, w.grad.cpu().numpy()), dWr) <= FP32_TOL


def test_uvw_per_row_weights_misaligned(cuda):
    """fp32 per-row weights move two words per lane; tensors that start 4 bytes past an 8-byte boundary take the
    kernels with one-word accesses (raw entry points, every tensor shifted)."""
    import torch
    import openequivariance_amd as oeq
    prob, oprob = common.fully_connected(DIFFDOCK["DiffDock-L=1"], shared=False)
    n = 41
    X, Y, We, G = common.tp_inputs(prob, n, 47, w_scale=0.2)
    W = ow.e3nn_to_oeq(oprob, We)
    tp = oeq.TensorProduct(prob, torch_op=False)
    assert tp.generator.pairs

    def shifted(a):
        flat = torch.empty(a.size + 1, dtype=torch.float32, device=cuda)
        view = flat[1:].view(a.shape)
        view.copy_(torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)))
        assert view.data_ptr() % 8 == 4
        return view
    x, y, w, g = (shifted(a) for a in (X, Y, W, G))
    z, xg, yg, wg = (shifted(np.zeros_like(a)) for a in (G, X, Y, W))
    tp.forward_raw(n, x.data_ptr(), y.data_ptr(), z.data_ptr(), w.data_ptr())
    tp.backward_raw(n, x.data_ptr(), xg.data_ptr(), y.data_ptr(), yg.data_ptr(), w.data_ptr(), wg.data_ptr(), g.data_ptr())
    torch.cuda.synchronize()
    dXr, dYr, dWr = otp.backward(oprob, X, Y, We, G)
    assert rel_err(z.cpu().numpy(), otp.forward(oprob, X, Y, We)) <= FP32_TOL
    assert rel_err(xg.cpu().numpy(), dXr) <= FP32_TOL
    assert rel_err(yg.cpu().numpy(), dYr) <= FP32_TOL
    assert rel_err(ow.oeq_to_e3nn(oprob, wg.cpu().numpy()), dWr) <= FP32_TOL


TETRIS_POLY = {"tetris-poly-1": ("1x0e+1x1o+1x2e+1x3o", "1x0e+1x1o+1x2e+1x3o", "64x0e+24x1e+24x1o+16x2e+16x2o"),
               "tetris-poly-2": ("64x0e+24x1e+24x1o+16x2e+16x2o", "1x0e+1x1o+1x2e+1x3o", "1x0o+6x0e"),
               # rows longer than a register group on both sides, a last group that is no whole number of vectors,
               # two copies of the second operand
               "several-groups": ("8x0e+10x1o", "2x0e+1x1o", "9x0e+11x1o")}


@pytest.mark.parametrize("name", list(TETRIS_POLY))
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("waves", [1024, 3], ids=["one_tile_per_wavefront", "several_tiles_per_wavefront"])
def test_uvw_few_weights_one_row_per_lane(cuda, name, dtype, waves, monkeypatch):
    """The two shared-weight problems of the reference's uvw benchmark (benchmark/benchmark_configs.py:38-41): few
    weights on multiplicities of 1 or 6, served by the vector-ALU kernels with a row per lane.  517 rows = 8 full
    tiles and a ragged one; with 3 wavefronts each accumulates dW over three tiles."""
    import torch
    import openequivariance_amd as oeq
    from openequivariance_amd.codegen.uvw_rows import UVWRowsGenerator
    monkeypatch.setattr(UVWRowsGenerator, "WAVES", waves)
    tol = FP32_TOL if dtype == np.float32 else FP64_TOL
    prob, oprob = common.fully_connected(TETRIS_POLY[name], shared=True, dtype=dtype)
    X, Y, We, G = common.tp_inputs(prob, 517, 48, dtype, w_scale=0.2)
    tp = oeq.TensorProduct(prob, torch_op=True)
    assert isinstance(tp.generator, UVWRowsGenerator)
    W = ow.e3nn_to_oeq(oprob, We)
    x, y, w = (torch.tensor(a, device=cuda, requires_grad=True) for a in (X, Y, W))
    z = tp(x, y, w)
    z.backward(torch.tensor(G, device=cuda))
    dXr, dYr, dWr = otp.backward(oprob, X, Y, We, G)
    assert rel_err(z.detach().cpu().numpy(), otp.forward(oprob, X, Y, We)) <= tol
    assert rel_err(x.grad.cpu().numpy(), dXr) <= tol
    assert rel_err(y.grad.cpu().numpy(), dYr) <= tol
    assert rel_err(ow.oeq_to_e3nn(oprob, w.grad.cpu().numpy()), dWr) <= tol
    # the sums over the batch run in a fixed order: a second backward repeats bit for bit
    x2, y2, w2 = (t.detach().clone().requires_grad_(True) for t in (x, y, w))
    tp(x2, y2, w2).backward(torch.tensor(G, device=cuda))
    assert torch.equal(w2.grad, w.grad)


@pytest.mark.parametrize("name", ["DiffDock-L=1", "tetris-poly-1", "dense"])
def test_uvw_empty_batch(cuda, name):
    """No rows: an empty output, empty dX and dY, and - for shared weights - a dW of zeros, from all three uvw
    kernel families (per-row weights, few shared weights, MFMA)."""
    import torch
    import openequivariance_amd as oeq
    shared = name != "DiffDock-L=1"
    irreps = {"DiffDock-L=1": DIFFDOCK["DiffDock-L=1"], "tetris-poly-1": TETRIS_POLY["tetris-poly-1"],
              "dense": ("16x0e+16x1o", "1x0e+1x1o", "16x0e+16x1o")}[name]
    prob, _ = common.fully_connected(irreps, shared=shared)
    tp = oeq.TensorProduct(prob, torch_op=True)
    d1, d2, d3, wn = prob.irreps_in1.dim, prob.irreps_in2.dim, prob.irreps_out.dim, prob.weight_numel
    x = torch.zeros(0, d1, device=cuda, requires_grad=True)
    y = torch.zeros(0, d2, device=cuda, requires_grad=True)
    w = (torch.randn(wn, device=cuda) if shared else torch.zeros(0, wn, device=cuda)).requires_grad_(True)
    z = tp(x, y, w)
    assert z.shape == (0, d3)
    z.backward(torch.zeros(0, d3, device=cuda))
    torch.cuda.synchronize()
    assert x.grad.shape == (0, d1) and y.grad.shape == (0, d2)
    assert w.grad.shape == w.shape and not w.grad.abs().any()
