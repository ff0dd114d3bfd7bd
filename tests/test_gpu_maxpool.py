"""act_quantized_max_pool2d vs F.max_pool2d forward/backward (reference test:
tests/test_act_quantized_ops.py:206-232, atol/rtol 1e-4) and vs the oracle's index rule."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import actnn_amd.cpp_extension.quantization as ext_q
from oracle import pool
from _util import DEV

pytestmark = pytest.mark.gpu

GEOMS = [((3, 3), (2, 2), (1, 1)), ((2, 2), (2, 2), (0, 0)), ((3, 3), (1, 1), (1, 1)),
         ((3, 2), (1, 2), (1, 0)), ((1, 1), (1, 1), (0, 0)), ((3, 5), (2, 3), (1, 2))]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("k,s,p", GEOMS)
@pytest.mark.parametrize("shape", [(4, 8, 28, 28), (2, 3, 13, 17), (1, 1, 5, 5), (3, 5, 32, 24),
                                   (2, 3, 16, 8), (1, 2, 224, 224)])
def test_forward_backward(dtype, k, s, p, shape):
    torch.manual_seed(sum(shape))
    x = torch.randn(*shape).to(dtype)
    xd = x.to(DEV).requires_grad_(True)
    y = ext_q.act_quantized_max_pool2d(xd, k, s, p, (1, 1), False, False)
    xr = x.to(DEV).requires_grad_(True)
    yr = F.max_pool2d(xr, k, s, p)
    assert torch.equal(y, yr)
    g = torch.randn_like(yr)
    y.backward(g)
    yr.backward(g)
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    assert torch.allclose(xd.grad.float(), xr.grad.float(), atol=tol, rtol=tol)
    # index rule against the oracle
    _, idx = ext_q.max_pool2d_forward(x.to(DEV), k, s, p, (1, 1))
    out_o, idx_o = pool.max_pool2d_forward(x.float().numpy(), k, s, p)
    assert idx.dtype == torch.int8 and np.array_equal(idx.cpu().numpy(), idx_o)
    gin_o = pool.max_pool2d_backward(g.float().cpu().numpy(), idx_o, shape, k, s, p)
    assert np.allclose(xd.grad.float().cpu().numpy(), gin_o, atol=tol, rtol=tol)


def test_ties_take_the_first_position():
    x = torch.zeros(1, 1, 8, 8, device=DEV)
    _, idx = ext_q.max_pool2d_forward(x, (3, 3), (2, 2), (1, 1), (1, 1))
    _, idx_o = pool.max_pool2d_forward(np.zeros((1, 1, 8, 8), np.float32), (3, 3), (2, 2), (1, 1))
    assert np.array_equal(idx.cpu().numpy(), idx_o)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("k,s,p", [((3, 3), (2, 2), (1, 1)), ((2, 2), (2, 2), (0, 0))])
@pytest.mark.parametrize("shape", [(2, 3, 16, 24), (2, 3, 14, 18)])
def test_special_values_follow_the_strict_compare(dtype, k, s, p, shape):
    """-inf, NaN, +-0 and values below the -1e10 start never win a strict '>' from the start
    value: output and index must follow the reference's scan (.cu:656-666) exactly, on the
    stride-2 kernels (W % 8 == 0) and on the general ones."""
    rng = np.random.default_rng(7)
    npdt = np.float32 if dtype == torch.float32 else np.float16
    x = rng.standard_normal(shape).astype(npdt)
    special = np.array([-np.inf, np.nan, 0.0, -0.0, -3e10 if npdt == np.float32 else -65504.0, np.inf], npdt)
    pick = rng.integers(0, 12, size=shape)
    x = np.where(pick < 6, special[np.minimum(pick, 5)], x)
    x[0, 0] = -np.inf                                    # whole windows of -inf / NaN
    x[0, 1] = np.nan
    y, idx = ext_q.max_pool2d_forward(torch.from_numpy(x).to(DEV), k, s, p, (1, 1))
    out_o, idx_o = pool.max_pool2d_forward_literal(x, k, s, p)
    assert np.array_equal(idx.cpu().numpy(), idx_o)
    assert np.array_equal(y.cpu().numpy(), out_o, equal_nan=True)
    assert np.array_equal(np.signbit(y.cpu().numpy()), np.signbit(out_o))


def test_rejected_arguments():
    x = torch.randn(1, 1, 8, 8, device=DEV)
    with pytest.raises(RuntimeError):
        ext_q.act_quantized_max_pool2d(x, (3, 3), (2, 2), (1, 1), (1, 1), True, False)    # ceil_mode
    with pytest.raises(RuntimeError):
        ext_q.act_quantized_max_pool2d(x, (3, 3), (2, 2), (1, 1), (1, 1), False, True)    # return_indices
    with pytest.raises(RuntimeError):
        ext_q.act_quantized_max_pool2d(x, (4, 4), (2, 2), (1, 1), (1, 1), False, False)   # KH*KW >= 16
    with pytest.raises(RuntimeError):
        ext_q.act_quantized_max_pool2d(x, (3,), (2, 2), (1, 1), (1, 1), False, False)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("k,s,p", GEOMS)
@pytest.mark.parametrize("shape", [(4, 8, 28, 28), (2, 16, 13, 17), (1, 64, 5, 5), (3, 24, 32, 24), (2, 8, 224, 224)])
def test_channels_last_equals_default_layout(dtype, k, s, p, shape):
    """[N, H, W, C] kernels: values, indices and gradients are those of the default-layout kernels
    on the same logical tensor; outputs keep the channels-last strides."""
    torch.manual_seed(sum(shape) + 1)
    x = torch.randn(*shape).to(dtype).to(DEV)
    x_cl = x.contiguous(memory_format=torch.channels_last)
    assert ext_q.pool_takes_channels_last(x_cl)
    y, idx = ext_q.max_pool2d_forward(x, k, s, p, (1, 1))
    y_cl, idx_cl = ext_q.max_pool2d_forward(x_cl, k, s, p, (1, 1))
    assert y_cl.is_contiguous(memory_format=torch.channels_last) and idx_cl.is_contiguous(memory_format=torch.channels_last)
    assert torch.equal(y_cl, y) and torch.equal(idx_cl, idx)
    g = torch.randn_like(y)
    gin = ext_q.max_pool2d_backward(g, idx, x.shape, k, s, p)
    gin_cl = ext_q.max_pool2d_backward(g.contiguous(memory_format=torch.channels_last), idx_cl, x.shape, k, s, p)
    assert gin_cl.is_contiguous(memory_format=torch.channels_last)
    tol = 1e-5 if dtype == torch.float32 else 2e-2          # the two kernels add overlapping windows in the same order
    assert torch.allclose(gin_cl.float(), gin.float(), atol=tol, rtol=tol)
    # and through autograd, against torch's own channels-last max-pool
    xa = x_cl.clone(memory_format=torch.preserve_format).requires_grad_(True)
    ya = ext_q.act_quantized_max_pool2d(xa, k, s, p, (1, 1), False, False)
    ya.backward(g)
    xr = x.clone().requires_grad_(True)
    F.max_pool2d(xr, k, s, p).backward(g)
    assert torch.equal(ya, F.max_pool2d(x, k, s, p))
    assert torch.allclose(xa.grad.float(), xr.grad.float(), atol=tol if dtype != torch.float32 else 1e-4, rtol=tol)


def test_channels_last_special_values():
    rng = np.random.default_rng(9)
    x = rng.standard_normal((2, 16, 14, 18)).astype(np.float16)
    special = np.array([-np.inf, np.nan, 0.0, -0.0, -65504.0, np.inf], np.float16)
    pick = rng.integers(0, 12, size=x.shape)
    x = np.where(pick < 6, special[np.minimum(pick, 5)], x)
    xt = torch.from_numpy(x).to(DEV).contiguous(memory_format=torch.channels_last)
    y, idx = ext_q.max_pool2d_forward(xt, (3, 3), (2, 2), (1, 1), (1, 1))
    out_o, idx_o = pool.max_pool2d_forward_literal(x, (3, 3), (2, 2), (1, 1))
    assert np.array_equal(idx.cpu().numpy(), idx_o)
    assert np.array_equal(y.cpu().numpy(), out_o, equal_nan=True)


def _memory_order(t):
    """the elements of a 4-d tensor in the order of its memory (default or channels-last)"""
    if t.is_contiguous():
        return t.reshape(-1)
    return t.permute(0, 2, 3, 1).reshape(-1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("k,s,p", GEOMS)
@pytest.mark.parametrize("shape", [(4, 8, 28, 28), (2, 3, 13, 17), (1, 1, 5, 5), (3, 5, 32, 24), (2, 3, 16, 8),
                                   (1, 2, 224, 224), (3, 1, 7, 9), (1, 16, 31, 30)])
def test_two_indices_per_byte_equal_the_int8_operators(dtype, k, s, p, shape):
    """The *_nibble operators: same values; the packed indices are the int8 indices (checked against
    the oracle above) packed two per byte in memory order, spare half byte 0; the gradient is
    bit-identical to the int8 operators' gradient.  The shapes reach the stride-2 kernels, the
    LDS-tiled ones (even output width), the one-thread-per-output ones (odd width, odd count) and,
    with 8 or 16 channels, the channels-last ones."""
    torch.manual_seed(sum(shape) + 5)
    x = torch.randn(*shape).to(dtype).to(DEV)
    layouts = [x]
    if shape[1] % 8 == 0:
        layouts.append(x.contiguous(memory_format=torch.channels_last))
    for xin in layouts:
        cl = xin is not x
        assert ext_q.pool_takes_channels_last(xin) == cl
        y, idx = ext_q.max_pool2d_forward(xin, k, s, p, (1, 1))
        y4, idx4 = ext_q.max_pool2d_forward(xin, k, s, p, (1, 1), nibble_indices=True)
        assert torch.equal(y4, y) and y4.stride() == y.stride()
        assert idx4.dtype == torch.uint8 and idx4.shape == ((y.numel() + 1) // 2,)
        want = pool.pack_index_nibbles(_memory_order(idx).cpu().numpy())
        assert np.array_equal(idx4.cpu().numpy(), want)
        g = torch.randn_like(y)
        gin = ext_q.max_pool2d_backward(g, idx, x.shape, k, s, p)
        gin4 = ext_q.max_pool2d_backward(g, idx4, x.shape, k, s, p, channels_last=cl)
        assert torch.equal(gin4, gin) and gin4.stride() == gin.stride()


@pytest.mark.parametrize("channels_last", [False, True])
def test_layer_keeps_half_a_byte_per_output(channels_last):
    """QMaxPool2d under config.pool_index_nibbles saves (numel + 1) // 2 bytes and gives torch's gradient."""
    from actnn_amd.conf import config
    from actnn_amd.layers import QMaxPool2d
    x = torch.randn(4, 16, 28, 28, device=DEV, dtype=torch.float16)
    if channels_last:
        x = x.contiguous(memory_format=torch.channels_last)
    saved = {}
    g = torch.randn(4, 16, 14, 14, device=DEV, dtype=torch.float16)
    if channels_last:
        g = g.contiguous(memory_format=torch.channels_last)
    for flag in (True, False):
        config.pool_index_nibbles = flag
        try:
            xa = x.clone(memory_format=torch.preserve_format).requires_grad_(True)
            sizes = []
            with torch.autograd.graph.saved_tensors_hooks(lambda t: (sizes.append(t.numel() * t.element_size()), t)[1],
                                                          lambda t: t):
                y = QMaxPool2d(3, 2, 1)(xa)
            y.backward(g)
            saved[flag] = (sizes, xa.grad.clone())
        finally:
            config.pool_index_nibbles = True
    n_out = 4 * 16 * 14 * 14
    assert saved[True][0] == [n_out // 2] and saved[False][0] == [n_out]
    assert torch.equal(saved[True][1], saved[False][1])
    xr = x.clone().requires_grad_(True)
    F.max_pool2d(xr, 3, 2, 1).backward(g)
    assert torch.allclose(saved[True][1].float(), xr.grad.float(), atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("k,s,p", [((3, 3), (2, 2), (1, 1)), ((2, 2), (2, 2), (0, 0))])
@pytest.mark.parametrize("shape", [(2, 8, 8, 8), (3, 16, 14, 18), (1, 64, 112, 112), (2, 8, 4, 4), (2, 24, 6, 4)])
def test_channels_last_stride2_backward_adds_in_the_order_of_the_default_layout(dtype, k, s, p, shape):
    """Even H and W with a stride-2 window take the channels-last kernel that owns 2x2 input blocks;
    it adds the windows of a pixel in the same order as the default-layout kernels, so the gradient is
    the same bit for bit (heavily tied inputs make several windows point at one pixel)."""
    torch.manual_seed(sum(shape) + 11)
    x = torch.randint(-2, 3, shape).to(dtype).to(DEV)          # many ties
    x_cl = x.contiguous(memory_format=torch.channels_last)
    y, idx = ext_q.max_pool2d_forward(x, k, s, p, (1, 1))
    _, idx_cl = ext_q.max_pool2d_forward(x_cl, k, s, p, (1, 1))
    g = torch.randn_like(y)
    gin = ext_q.max_pool2d_backward(g, idx, x.shape, k, s, p)
    gin_cl = ext_q.max_pool2d_backward(g.contiguous(memory_format=torch.channels_last), idx_cl, x.shape, k, s, p)
    assert gin_cl.is_contiguous(memory_format=torch.channels_last)
    assert torch.equal(gin_cl, gin)
    xr = x.clone().requires_grad_(True)
    F.max_pool2d(xr, k, s, p).backward(g)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    # torch picks the first maximum too, so the sums hold the same terms
    assert torch.allclose(gin_cl.float(), xr.grad.float(), atol=tol, rtol=tol)
