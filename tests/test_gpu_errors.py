"""Error behaviour of the operators: no silent fallback, shapes and dtypes are checked before any
kernel is launched."""
import numpy as np
import pytest

import common

pytestmark = pytest.mark.gpu


def test_tensor_product_rejects_bad_inputs(cuda):
    import torch
    import openequivariance_amd as oeq
    prob, _ = common.channelwise(common.NEQUIP)
    tp = oeq.TensorProduct(prob, torch_op=True)
    x, y, w = (torch.randn(10, d, device=cuda) for d in (288, 9, 352))
    assert tp(x, y, w).shape == (10, 1120)
    with pytest.raises(ValueError):
        tp(x[:, :-1], y, w)
    with pytest.raises(ValueError):
        tp(x, y[:5], w)
    with pytest.raises(ValueError):
        tp(x, y, w[0])                       # per-row weights expected
    with pytest.raises(TypeError):
        tp(x.double(), y.double(), w.double())
    with pytest.raises((NotImplementedError, RuntimeError)):
        tp(x.cpu(), y.cpu(), w.cpu())        # there is no CPU implementation
    assert tp(x[:0], y[:0], w[:0]).shape == (0, 1120)


@pytest.mark.parametrize("deterministic", [False, True])
def test_convolution_rejects_bad_inputs(cuda, deterministic):
    import torch
    import openequivariance_amd as oeq
    prob, _ = common.channelwise(common.NEQUIP)
    conv = oeq.TensorProductConv(prob, torch_op=True, deterministic=deterministic)
    x, y, w = torch.randn(6, 288, device=cuda), torch.randn(12, 9, device=cuda), torch.randn(12, 352, device=cuda)
    rows = torch.arange(12, device=cuda) // 2
    cols = (rows + 1) % 6
    extra = [torch.argsort(cols * 6 + rows, stable=True)] if deterministic else []
    assert conv.forward(x, y, w, rows, cols, *extra).shape == (6, 1120)
    with pytest.raises(ValueError):
        conv.forward(x, y[:5], w, rows, cols, *extra)
    with pytest.raises(ValueError):
        conv.forward(x, y, w[:, :-1], rows, cols, *extra)
    with pytest.raises(TypeError):
        conv.forward(x, y, w, rows.int(), cols.int(), *extra)
    with pytest.raises(TypeError):
        conv.forward(x.double(), y.double(), w.double(), rows, cols, *extra)
    # edges that name no node contribute nothing and do not fault
    bad = rows.clone()
    bad[0] = 99
    if not deterministic:
        z = conv.forward(x, y, w, bad, cols)
        assert torch.isfinite(z).all()


def test_unsupported_problems_raise():
    import openequivariance_amd as oeq
    with pytest.raises(NotImplementedError):      # uvw needs multiplicity 1 on the second operand
        oeq.TensorProduct(oeq.FullyConnectedTPProblem("4x0e", "2x0e", "4x0e", shared_weights=True, internal_weights=False))
    with pytest.raises(AssertionError):           # the convolution too
        oeq.TensorProductConv(oeq.TPProblem("2x0e", "2x0e", "2x0e", [(0, 0, 0, "uvu", True)], shared_weights=False,
                                            internal_weights=False))
    with pytest.raises(NotImplementedError):
        oeq.TensorProductConv(oeq.FullyConnectedTPProblem("4x0e", "1x0e", "4x0e", shared_weights=False, internal_weights=False))
