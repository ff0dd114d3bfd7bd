"""The float64 batch-norm restatement against torch's own batch norm and autograd on CPU."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import batch_norm as o_bn


@pytest.mark.parametrize("shape", [(4, 3, 5, 7), (8, 6, 4), (2, 5, 3, 2, 2), (16, 10)])
@pytest.mark.parametrize("affine", [True, False])
def test_forward_and_backward_match_torch(shape, affine):
    g = torch.Generator().manual_seed(sum(shape))
    x = (torch.randn(*shape, generator=g, dtype=torch.float64) * 2 + 0.7).requires_grad_(True)
    C = shape[1]
    w = (torch.rand(C, generator=g, dtype=torch.float64) + 0.5).requires_grad_(True) if affine else None
    b = torch.randn(C, generator=g, dtype=torch.float64).requires_grad_(True) if affine else None
    rm = torch.randn(C, generator=g, dtype=torch.float64)
    rv = torch.rand(C, generator=g, dtype=torch.float64) + 0.5
    rm0, rv0 = rm.clone(), rv.clone()
    y = F.batch_norm(x, rm, rv, w, b, True, 0.1, 1e-5)
    dy = torch.randn(*shape, generator=g, dtype=torch.float64)
    y.backward(dy)
    yo, mean, invstd, nrm, nrv = o_bn.forward(x.detach().numpy(), None if w is None else w.detach().numpy(),
                                              None if b is None else b.detach().numpy(),
                                              rm0.numpy(), rv0.numpy(), 0.1, 1e-5)
    assert np.allclose(yo, y.detach().numpy(), rtol=1e-10, atol=1e-10)
    assert np.allclose(nrm, rm.numpy(), rtol=1e-12) and np.allclose(nrv, rv.numpy(), rtol=1e-12)
    axes = (0,) + tuple(range(2, len(shape)))
    assert np.allclose(mean, x.detach().numpy().mean(axes))
    assert np.allclose(invstd, 1 / np.sqrt(x.detach().numpy().var(axes) + 1e-5))
    gi, gw, gb = o_bn.backward(x.detach().numpy(), dy.numpy(), None if w is None else w.detach().numpy(), 1e-5)
    assert np.allclose(gi, x.grad.numpy(), rtol=1e-9, atol=1e-10)
    if affine:
        assert np.allclose(gw, w.grad.numpy(), rtol=1e-10) and np.allclose(gb, b.grad.numpy(), rtol=1e-10)


def test_constant_channel_and_single_position():
    x = np.zeros((4, 2, 3))
    x[:, 1] = 5.0
    y, mean, invstd, _, _ = o_bn.forward(x, None, None, None, None, 0.1, 1e-5)
    assert np.allclose(mean, [0, 5]) and np.allclose(invstd, 1 / np.sqrt(1e-5)) and np.allclose(y, 0)


@pytest.mark.parametrize("shape", [(4, 3, 5, 7), (16, 10), (3, 6, 4)])
def test_evaluation_mode_matches_torch(shape):
    g = torch.Generator().manual_seed(sum(shape) + 1)
    x = (torch.randn(*shape, generator=g, dtype=torch.float64) * 2 + 0.7).requires_grad_(True)
    C = shape[1]
    w = (torch.rand(C, generator=g, dtype=torch.float64) + 0.5).requires_grad_(True)
    b = torch.randn(C, generator=g, dtype=torch.float64).requires_grad_(True)
    rm = torch.randn(C, generator=g, dtype=torch.float64)
    rv = torch.rand(C, generator=g, dtype=torch.float64) + 0.5
    y = F.batch_norm(x, rm, rv, w, b, False, 0.1, 1e-5)
    dy = torch.randn(*shape, generator=g, dtype=torch.float64)
    y.backward(dy)
    yo, mean, invstd = o_bn.forward_eval(x.detach().numpy(), w.detach().numpy(), b.detach().numpy(),
                                         rm.numpy(), rv.numpy(), 1e-5)
    assert np.allclose(yo, y.detach().numpy(), rtol=1e-10, atol=1e-10)
    assert np.allclose(mean, rm.numpy()) and np.allclose(invstd, 1 / np.sqrt(rv.numpy() + 1e-5))
    gi, gw, gb = o_bn.backward_eval(x.detach().numpy(), dy.numpy(), w.detach().numpy(), rm.numpy(), rv.numpy(), 1e-5)
    assert np.allclose(gi, x.grad.numpy(), rtol=1e-10, atol=1e-12)
    assert np.allclose(gw, w.grad.numpy(), rtol=1e-10) and np.allclose(gb, b.grad.numpy(), rtol=1e-10)
