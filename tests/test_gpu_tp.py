"""GPU parity of the batch tensor product (uvu) against the fp64 oracle, through the C ABI."""
import numpy as np
import pytest

import common
from common import FP32_TOL, FP64_TOL, rel_err
from oracle import tp as otp

pytestmark = pytest.mark.gpu


def _run(prob, oprob, n, seed, dtype, sh_lmax=None):
    import torch
    import openequivariance_amd as oeq
    tol = FP32_TOL if dtype == np.float32 else FP64_TOL
    X, Y, W, G = common.tp_inputs(prob, n, seed, dtype, sh_lmax)
    tp = oeq.TensorProduct(prob, torch_op=True)
    dev = torch.device("cuda:0")
    x, y, w = (torch.tensor(a, device=dev, requires_grad=True) for a in (X, Y, W))
    z = tp(x, y, w)
    z.backward(torch.tensor(G, device=dev))
    torch.cuda.synchronize()
    Zr = otp.forward(oprob, X, Y, W)
    dXr, dYr, dWr = otp.backward(oprob, X, Y, W, G)
    errs = dict(Z=rel_err(z.detach().cpu().numpy(), Zr), dX=rel_err(x.grad.cpu().numpy(), dXr),
                dY=rel_err(y.grad.cpu().numpy(), dYr), dW=rel_err(w.grad.cpu().numpy(), dWr))
    print(f"n={n} {errs}", flush=True)
    for k, v in errs.items():
        assert v <= tol, f"{k}: relative error {v:.3e} > {tol}"
    return tp


def test_readme_single_path(cuda):
    """benchmark configuration 1: 1x2e (x) 1x3e -> 1x2e, batch 1000, inputs U[0,1), forward."""
    import torch
    import openequivariance_amd as oeq
    prob, oprob = common.readme_problem()
    rng = np.random.default_rng(12345)
    X, Y, W = (rng.uniform(size=(1000, d)).astype(np.float32) for d in (5, 7, 1))
    tp = oeq.TensorProduct(prob, torch_op=True)
    z = tp(*(torch.tensor(a, device=cuda) for a in (X, Y, W)))
    assert rel_err(z.cpu().numpy(), otp.forward(oprob, X, Y, W)) <= FP32_TOL
    # path coefficient sqrt(5): a hand value
    assert abs(prob.instructions[0].path_weight - 5 ** 0.5) < 1e-12


@pytest.mark.parametrize("n", [1, 257])
def test_readme_fwd_bwd(cuda, n):
    prob, oprob = common.readme_problem()
    _run(prob, oprob, n, 1, np.float32)


@pytest.mark.parametrize("n", [1, 130])
def test_mace_uvu(cuda, n):
    """benchmark configuration 2 problem (17 paths, mul 128 = two 64-channel chunks)."""
    prob, oprob = common.channelwise(common.MACE)
    _run(prob, oprob, n, 2, np.float32, sh_lmax=3)


def test_nequip_uvu_two_rows_per_wave(cuda):
    """mul 32: two rows share a wavefront; odd batch leaves a half-empty tile."""
    prob, oprob = common.channelwise(common.NEQUIP)
    _run(prob, oprob, 301, 3, np.float32, sh_lmax=2)


def test_large_uvu_four_chunks(cuda):
    prob, oprob = common.channelwise(common.LARGE)
    _run(prob, oprob, 33, 4, np.float32, sh_lmax=3)


def test_ragged_multiplicities(cuda):
    """Multiplicities that are not multiples of the lane tile, and an output nobody writes."""
    import openequivariance_amd as oeq
    from oracle import spec
    irreps = ("5x0e+3x1o+70x2e", "1x0e+1x1o+1x2e", "5x0e+3x1o+70x2e+7x3o")
    prob, oprob = common.channelwise(irreps)
    _run(prob, oprob, 77, 5, np.float32)


def test_mace_uvu_fp64(cuda):
    prob, oprob = common.channelwise(common.MACE, dtype=np.float64)
    _run(prob, oprob, 65, 6, np.float64, sh_lmax=3)


def test_mul2_greater_than_one(cuda):
    """uvu with mul(in2) = 3: exercises the chunked [v][u] external weight order."""
    import openequivariance_amd as oeq
    from oracle import spec, weights as ow
    import torch
    ins = [(0, 0, 0, "uvu", True), (1, 1, 0, "uvu", True), (1, 0, 1, "uvu", True), (0, 1, 1, "uvu", True)]
    a = ("40x0e+40x1o", "3x0e+3x1o", "40x0e+40x1o")
    prob = oeq.TPProblem(*a, ins, shared_weights=False, internal_weights=False)
    oprob = spec.Problem(*a, ins, shared_weights=False)
    X, Y, W, G = common.tp_inputs(prob, 50, 7)
    tp = oeq.TensorProduct(prob, torch_op=True)
    W_oeq = np.zeros_like(W)
    tp.reorder_weights_e3nn_to_oeq(W, W_oeq, True)
    assert np.array_equal(W_oeq, ow.e3nn_to_oeq(oprob, W))
    x, y, w = (torch.tensor(t, device=cuda, requires_grad=True) for t in (X, Y, W_oeq))
    z = tp(x, y, w)
    z.backward(torch.tensor(G, device=cuda))
    dXr, dYr, dWr = otp.backward(oprob, X, Y, W, G)
    assert rel_err(z.detach().cpu().numpy(), otp.forward(oprob, X, Y, W)) <= FP32_TOL
    assert rel_err(x.grad.cpu().numpy(), dXr) <= FP32_TOL
    assert rel_err(y.grad.cpu().numpy(), dYr) <= FP32_TOL
    assert rel_err(ow.oeq_to_e3nn(oprob, w.grad.cpu().numpy()), dWr) <= FP32_TOL


UVU_LOOPED = {
    # more than 8 copies of a second-operand irrep: the kernels walk v with a run-time loop
    "11_copies_two_rows_per_wave": ("12x0e+12x1o", "11x0e+3x1o", "12x0e+12x1o+12x1o"),
    "ragged_v_3x0e+35x1o": ("40x0e+40x1o", "3x0e+35x1o", "40x0e+40x1o+40x1o"),
    "two_chunks_35_copies": ("70x0e+70x1o", "35x0e+2x1o", "70x0e+70x1o+70x1o"),
}


@pytest.mark.parametrize("name", sorted(UVU_LOOPED))
@pytest.mark.parametrize("shared", [False, True])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_uvu_many_copies_of_the_second_operand(cuda, name, shared, dtype):
    """uvu with mul(in2) > 8 (reference: ComputationSchedule.py:146-230 chunks v as well as u,
    loop_unroll_tp.cuh:48-60 and :140-175 loop over it), per-row and shared weights, through the
    chunk-of-32 [v][u] external weight order."""
    import openequivariance_amd as oeq
    from oracle import spec, weights as ow
    import torch
    tol = FP32_TOL if dtype == np.float32 else 1e-12
    ins = [(0, 0, 0, "uvu", True), (0, 1, 1, "uvu", True), (1, 0, 2, "uvu", True), (1, 1, 0, "uvu", True)]
    a = UVU_LOOPED[name]
    prob = oeq.TPProblem(*a, ins, shared_weights=shared, internal_weights=False, irrep_dtype=dtype, weight_dtype=dtype)
    oprob = spec.Problem(*a, ins, shared_weights=shared)
    n = 2100 if shared else 61                       # shared: more rows than persistent workgroups
    X, Y, W, G = common.tp_inputs(prob, n, 17, dtype, w_scale=0.2)
    tp = oeq.TensorProduct(prob, torch_op=True)
    assert any(p.looped for p in tp.generator.paths)
    W_oeq = np.zeros_like(W)
    tp.reorder_weights_e3nn_to_oeq(W, W_oeq, not shared)
    assert np.array_equal(W_oeq, ow.e3nn_to_oeq(oprob, W))
    x, y, w = (torch.tensor(t, device=cuda, requires_grad=True) for t in (X, Y, W_oeq))
    z = tp(x, y, w)
    z.backward(torch.tensor(G, device=cuda))
    torch.cuda.synchronize()
    dXr, dYr, dWr = otp.backward(oprob, X, Y, W, G)
    assert rel_err(z.detach().cpu().numpy(), otp.forward(oprob, X, Y, W)) <= tol
    assert rel_err(x.grad.cpu().numpy(), dXr) <= tol
    assert rel_err(y.grad.cpu().numpy(), dYr) <= tol
    assert rel_err(ow.oeq_to_e3nn(oprob, w.grad.cpu().numpy()), dWr) <= tol
    if shared:
        w2 = w.detach().clone().requires_grad_(True)
        tp(x.detach(), y.detach(), w2).backward(torch.tensor(G, device=cuda))
        assert torch.equal(w.grad, w2.grad), "shared-weight dW must be bit-reproducible"


def test_shared_weights_uvu(cuda):
    """shared_weights=True: dW is the sum over the batch (deterministic two-stage reduction)."""
    import openequivariance_amd as oeq
    from oracle import spec
    import torch
    ins = [(0, 0, 0, "uvu", True), (1, 1, 0, "uvu", True), (1, 0, 1, "uvu", True)]
    a = ("96x0e+96x1o", "1x0e+1x1o", "96x0e+96x1o")
    prob = oeq.TPProblem(*a, ins, shared_weights=True, internal_weights=False)
    oprob = spec.Problem(*a, ins, shared_weights=True)
    X, Y, W, G = common.tp_inputs(prob, 3000, 8)
    tp = oeq.TensorProduct(prob, torch_op=True)
    x, y, w = (torch.tensor(t, device=cuda, requires_grad=True) for t in (X, Y, W))
    z = tp(x, y, w)
    z.backward(torch.tensor(G, device=cuda))
    dXr, dYr, dWr = otp.backward(oprob, X, Y, W, G)
    assert rel_err(z.detach().cpu().numpy(), otp.forward(oprob, X, Y, W)) <= FP32_TOL
    assert rel_err(x.grad.cpu().numpy(), dXr) <= FP32_TOL
    assert rel_err(y.grad.cpu().numpy(), dYr) <= FP32_TOL
    assert rel_err(w.grad.cpu().numpy(), dWr) <= FP32_TOL
    w2 = w.detach().clone().requires_grad_(True)
    tp(x.detach(), y.detach(), w2).backward(torch.tensor(G, device=cuda))
    assert torch.equal(w.grad, w2.grad), "shared-weight dW must be bit-reproducible"


def test_blocks_no_path_touches(cuda):
    """A wide in1 block that no path reads (and narrow blocks in use): its dX columns are zeros."""
    irreps = ("1x0e+1x1o+16x3o", "1x0e+1x1o", "16x0e+16x0o+16x1e+16x1o")
    prob, oprob = common.channelwise(irreps)
    _run(prob, oprob, 300, 51, np.float32)


def test_empty_batch(cuda):
    import torch
    import openequivariance_amd as oeq
    prob, _ = common.channelwise(common.NEQUIP)
    tp = oeq.TensorProduct(prob, torch_op=True)
    z = tp(torch.zeros(0, 288, device=cuda), torch.zeros(0, 9, device=cuda), torch.zeros(0, 352, device=cuda))
    assert z.shape == (0, 1120)


def test_full_size_properties(cuda):
    """benchmark configuration 2 at its full batch (50 000): size-independent checks.
    Tri-linearity in W, and the adjoint identity <G, Z> = <X, dX> = <Y, dY> = <W, dW>."""
    import torch
    import openequivariance_amd as oeq
    prob, oprob = common.channelwise(common.MACE)
    n = 50000
    X, Y, W, G = common.tp_inputs(prob, n, 12346, sh_lmax=3)
    tp = oeq.TensorProduct(prob, torch_op=True)
    x, y, w = (torch.tensor(t, device=cuda, requires_grad=True) for t in (X, Y, W))
    g = torch.tensor(G, device=cuda)
    z = tp(x, y, w)
    z.backward(g)
    gz = (g.double() * z.detach().double()).sum().item()
    for name, a, b in (("X", x, x.grad), ("Y", y, y.grad), ("W", w, w.grad)):
        v = (a.detach().double() * b.double()).sum().item()
        assert abs(v - gz) <= 1e-5 * abs(gz), f"<{name}, d{name}> = {v} vs <G, Z> = {gz}"
    z2 = tp(x.detach(), y.detach(), 2.0 * w.detach())
    assert torch.allclose(z2, 2.0 * z.detach(), rtol=1e-6, atol=1e-6)
    # a slice of rows against the oracle
    sl = slice(49900, 50000)
    assert rel_err(z.detach()[sl].cpu().numpy(), otp.forward(oprob, X[sl], Y[sl], W[sl])) <= FP32_TOL


def test_tensors_beyond_two_giga_elements(cuda):
    """A batch whose weight tensor has more than 2^31 elements (1.8 M rows of the MACE problem: W and dW
    9.2 GB each): row offsets must be 64-bit everywhere.  Rows at the start, around element 2^31 and at
    the end are compared with the oracle on the same inputs (each row depends on that row only)."""
    import torch
    import openequivariance_amd as oeq
    from openequivariance_amd.sh import random_unit_vectors, spherical_harmonics
    prob, oprob = common.channelwise(common.MACE)
    n = 1_800_000
    d1, d3, wn = prob.irreps_in1.dim, prob.irreps_out.dim, prob.weight_numel
    assert n * wn > 2 ** 31 and n * d3 > 2 ** 31
    gen = torch.Generator(device=cuda)
    gen.manual_seed(99)
    x = torch.randn(n, d1, device=cuda, generator=gen, requires_grad=True)
    w = torch.randn(n, wn, device=cuda, generator=gen, requires_grad=True)
    g = torch.randn(n, d3, device=cuda, generator=gen)
    Y = spherical_harmonics(3, random_unit_vectors(n, np.random.default_rng(99))).astype(np.float32)
    y = torch.tensor(Y, device=cuda, requires_grad=True)
    tp = oeq.TensorProduct(prob, torch_op=True)
    z = tp(x, y, w)
    z.backward(g)
    torch.cuda.synchronize()
    mid = 2 ** 31 // wn
    rows = np.r_[0:40, mid - 20:mid + 20, n - 40:n]
    t = torch.from_numpy(rows).to(cuda)
    Xs, Ws, Gs = (a.detach()[t].cpu().numpy() for a in (x, w, g))
    Zr = otp.forward(oprob, Xs, Y[rows], Ws)
    dXr, dYr, dWr = otp.backward(oprob, Xs, Y[rows], Ws, Gs)
    errs = dict(Z=rel_err(z.detach()[t].cpu().numpy(), Zr), dX=rel_err(x.grad[t].cpu().numpy(), dXr),
                dY=rel_err(y.grad[t].cpu().numpy(), dYr), dW=rel_err(w.grad[t].cpu().numpy(), dWr))
    print(f"n={n} rows sampled={rows.size} {errs}", flush=True)
    for k, v in errs.items():
        assert v <= FP32_TOL, f"{k}: relative error {v:.3e}"


def _misaligned(a, dev):
    """Contiguous device copy of ``a`` whose storage starts 4 bytes past a 16-byte boundary."""
    import torch
    flat = torch.empty(a.size + 1, dtype=torch.float32, device=dev)
    view = flat[1:].view(a.shape)
    view.copy_(torch.from_numpy(a))
    assert view.data_ptr() % 16 == 4 and view.is_contiguous()
    return view


def test_misaligned_tensors(cuda):
    """Views with an odd storage offset: the operator switches to kernels without 16-byte vector
    stores (inputs through the torch op, the output through the raw entry point)."""
    import torch
    import openequivariance_amd as oeq
    prob, oprob = common.channelwise(common.MACE)
    n = 37
    X, Y, W, G = common.tp_inputs(prob, n, 5, sh_lmax=3)
    tp = oeq.TensorProduct(prob, torch_op=True)
    x, y, w = (_misaligned(a, cuda).requires_grad_(True) for a in (X, Y, W))
    z = tp(x, y, w)
    z.backward(_misaligned(G, cuda))
    refs = (otp.forward(oprob, X, Y, W),) + otp.backward(oprob, X, Y, W, G)
    for nm, a, b in zip(("Z", "dX", "dY", "dW"), (z.detach(), x.grad, y.grad, w.grad), refs):
        assert rel_err(a.cpu().numpy(), b) <= FP32_TOL, nm
    zraw = _misaligned(np.zeros_like(G), cuda)
    tp.forward_raw(n, x.data_ptr(), y.data_ptr(), zraw.data_ptr(), w.data_ptr())
    torch.cuda.synchronize()
    assert rel_err(zraw.cpu().numpy(), refs[0]) <= FP32_TOL
