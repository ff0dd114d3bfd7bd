"""ReLU / Dropout with 1-bit masks: values vs torch (exact, as tests/test_act_quantized_ops.py:17-36
of the reference does for ReLU), mask words vs the oracle's layout."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import actnn_amd.cpp_extension.quantization as ext_q
from oracle import layouts, philox
from _util import DEV

pytestmark = pytest.mark.gpu

SHAPES = [(128, 56, 56, 31), (4, 512), (1, 1), (7,), (3, 171), (2, 8192), (5, 1025), (3, 6659)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", SHAPES)
def test_relu_forward_backward(dtype, shape):
    torch.manual_seed(len(shape))
    x = torch.randn(*shape).to(dtype)
    x.view(-1)[::97] = 0.0
    xd = x.to(DEV).requires_grad_(True)
    y = ext_q.act_quantized_relu(xd)
    ref = F.relu(x.to(DEV))
    assert torch.equal(y, ref)
    y.backward(torch.ones_like(y))
    xr = x.to(DEV).requires_grad_(True)
    F.relu(xr).backward(torch.ones_like(ref))
    assert torch.equal(xd.grad, xr.grad)
    # mask words follow the reference layout, tail block fully materialised
    _, mask = ext_q.relu_forward(x.to(DEV))
    exp = layouts.mask_words((x.view(-1) > 0).numpy())
    assert mask.dtype == torch.int32 and mask.numel() == exp.size
    assert np.array_equal(mask.cpu().numpy(), exp)
    # backward with a random upstream gradient
    g = torch.randn(*shape).to(dtype).to(DEV)
    gi = ext_q.relu_backward(g, mask)
    assert torch.equal(gi, torch.where(x.to(DEV) > 0, g, torch.zeros_like(g)))


def test_relu_rejects_bad_arguments():
    with pytest.raises(RuntimeError):
        ext_q.act_quantized_relu(torch.randn(8))
    with pytest.raises(RuntimeError):
        ext_q.act_quantized_relu(torch.randn(8, 8, device=DEV).t())
    with pytest.raises(RuntimeError):
        ext_q.act_quantized_relu(torch.zeros(8, dtype=torch.int32, device=DEV))
    assert ext_q.act_quantized_relu(torch.empty(0, device=DEV)).numel() == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("p", [0.5, 0.1, 0.0, 1.0])
def test_dropout(dtype, p):
    n = 1_000_003
    torch.manual_seed(1)
    x = (torch.randn(n) + 3.0).to(dtype).to(DEV).requires_grad_(True)
    torch.cuda.manual_seed(2024)
    offset = torch.cuda.default_generators[0].get_offset()
    y = ext_q.act_quantized_dropout(x, p)
    # keep flags are the oracle's Philox bits: r16 >= round(p * 2^16)
    r = philox.noise16(np.arange(n, dtype=np.uint64), 2024, offset)
    keep = r >= np.uint32(min(max(int(p * 65536.0 + 0.5), 0), 65536))
    keep_t = torch.from_numpy(keep).to(DEV)
    assert abs(keep.mean() - (1.0 - p)) < 3e-3
    # reference on the host in numpy: true fp32 division by float(1 - p) (torch's device division by
    # a python scalar multiplies by the reciprocal, which is not the same rounding)
    div = np.float32(1.0 - float(np.float32(p)))

    def expect(t):
        v = t.detach().float().cpu().numpy()
        with np.errstate(divide="ignore", invalid="ignore"):
            r_ = np.where(keep, v / div, np.float32(0)).astype(np.float32)
        return torch.from_numpy(r_).to(dtype)

    assert torch.equal(y.detach().cpu(), expect(x))
    g = torch.randn(n).to(dtype).to(DEV)
    y.backward(g)
    assert torch.equal(x.grad.cpu(), expect(g))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("n", [2048, 2048 * 37, 8 * 64 * 56 * 56])
def test_relu_forward_with_group_min_max(dtype, n):
    """The ReLU pass that also reduces its output per group of 256: output and mask as the plain
    operator, min / max bit-identical to minimax on the output."""
    import actnn_amd.cpp_extension.minimax as ext_minimax
    g = torch.Generator(device=DEV).manual_seed(n)
    x = (torch.randn(n, generator=g, device=DEV) * 2 - 0.3).to(dtype)
    x[:256] = -1.0                                                  # a group that is all zero after ReLU
    x[256:512] = torch.linspace(0.5, 3, 256, device=DEV).to(dtype)     # a group without zeros
    assert ext_q.relu_minmax_applies(x)
    y0, mask0 = ext_q.relu_forward(x)
    y, mask, mn, mx = ext_q.relu_forward_minmax(x)
    assert torch.equal(y, y0) and torch.equal(mask, mask0)
    mn_ref, mx_ref = ext_minimax.minimax(y.view(-1, 256))
    assert torch.equal(mn, mn_ref) and torch.equal(mx, mx_ref)
    assert not ext_q.relu_minmax_applies(x[:1024]) and not ext_q.relu_minmax_applies(x.float())


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", SHAPES + [(4, 64, 16, 16)])
def test_relu_of_a_sum_equals_the_addition_followed_by_relu(dtype, shape):
    """Values, mask words and both gradients of the fused pass are those of torch's addition (which
    rounds the sum to the tensors' dtype) followed by the ReLU above.  The operands are drawn so that
    sums cancel exactly, round to zero-adjacent values and differ widely in magnitude."""
    torch.manual_seed(len(shape) + 7)
    a = torch.randn(*shape).to(dtype)
    b = torch.randn(*shape).to(dtype)
    flat_a, flat_b = a.view(-1), b.view(-1)
    flat_b[::5] = -flat_a[::5]                              # exact cancellation
    flat_b[1::7] = flat_b[1::7] * 2.0 ** -12                # one operand far below the other's ulp
    flat_a[2::11] = flat_a[2::11] * 2.0 ** -14
    flat_b[2::11] = flat_b[2::11] * 2.0 ** -14              # tiny sums of either sign
    ad, bd = a.to(DEV).requires_grad_(True), b.to(DEV).requires_grad_(True)
    y = ext_q.ActQuantizedAddReLU.apply(ad, bd)
    total = a.to(DEV) + b.to(DEV)
    assert torch.equal(y, F.relu(total))
    y2, mask = ext_q.relu_add_forward(a.to(DEV), b.to(DEV))
    _, ref_mask = ext_q.relu_forward(total)
    assert torch.equal(y2, y.detach()) and torch.equal(mask, ref_mask)
    assert np.array_equal(mask.cpu().numpy(), layouts.mask_words((total.view(-1) > 0).cpu().numpy()))
    g = torch.randn(*shape).to(dtype).to(DEV)
    y.backward(g)
    expected = torch.where(total > 0, g, torch.zeros_like(g))
    assert torch.equal(ad.grad, expected) and torch.equal(bd.grad, expected)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", SHAPES + [(4, 64, 16, 16), (3, 8192 + 40)])
def test_masked_gradient_added_to_another_equals_the_two_steps(dtype, shape):
    """actnn_relu_backward_add: other + relu_backward(grad, mask) in one pass is torch's addition of
    the masked gradient (which rounds the sum to the tensors' dtype), for cancelling sums, operands
    of very different magnitude and negative zeros on either side."""
    from actnn_amd import _lib
    torch.manual_seed(len(shape) + 19)
    x = torch.randn(*shape).to(dtype).to(DEV)
    grad = torch.randn(*shape).to(dtype)
    other = torch.randn(*shape).to(dtype)
    fg, fo = grad.view(-1), other.view(-1)
    fo[::5] = -fg[::5]
    fo[1::7] = fo[1::7] * 2.0 ** -12
    fo[3::13] = -0.0
    fg[4::17] = -0.0
    grad, other = grad.to(DEV), other.to(DEV)
    _, mask = ext_q.relu_forward(x)
    expected = other + ext_q.relu_backward(grad, mask)
    got = ext_q.relu_backward_add(grad, mask, other)
    assert torch.equal(got.view(torch.int16 if dtype != torch.float32 else torch.int32),
                       expected.view(torch.int16 if dtype != torch.float32 else torch.int32))
    assert torch.equal(expected, other + torch.where(x > 0, grad, torch.zeros_like(grad)))
    lib = _lib.load()
    code = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dtype]
    n = grad.numel()
    assert lib.actnn_relu_backward_add(grad.data_ptr(), mask.data_ptr(), None, got.data_ptr(), n, code, None) != 0
    if n > 8:
        assert lib.actnn_relu_backward_add(grad.data_ptr(), mask.data_ptr(), other.data_ptr() + other.element_size(),
                                           got.data_ptr(), n - 8, code, None) != 0
    assert lib.actnn_relu_backward_add(None, None, None, None, 0, code, None) == 0
    torch.cuda.synchronize()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_relu_of_a_sum_with_group_min_max(dtype):
    torch.manual_seed(3)
    a = torch.randn(6, 2048 * 3).to(dtype).to(DEV)
    b = torch.randn(6, 2048 * 3).to(dtype).to(DEV)
    b[:, ::3] = -a[:, ::3]
    y, mask, mn, mx = ext_q.relu_add_forward(a, b, minmax=True)
    ref = F.relu(a + b)
    y1, mask1, mn1, mx1 = ext_q.relu_forward_minmax(a + b)
    assert torch.equal(y, ref) and torch.equal(mask, mask1)
    assert torch.equal(mn, mn1) and torch.equal(mx, mx1)
    groups = ref.view(-1, 256)
    assert torch.equal(mn, groups.min(1).values) and torch.equal(mx, groups.max(1).values)


def test_relu_of_a_sum_rejects_bad_arguments():
    from actnn_amd import _lib
    lib = _lib.load()
    x = torch.zeros(4096, dtype=torch.bfloat16, device=DEV)
    y = torch.empty_like(x)
    mask = torch.empty(ext_q.mask_words(4096), dtype=torch.int32, device=DEV)
    mn = torch.empty(16, dtype=torch.bfloat16, device=DEV)
    args = lambda **k: (k.get("x", x.data_ptr()), k.get("r", x.data_ptr()), y.data_ptr(), mask.data_ptr(),
                        k.get("mn", None), k.get("mx", None), k.get("n", 4096), k.get("dtype", 2), None)
    assert lib.actnn_relu_add_forward(*args()) == 0
    assert lib.actnn_relu_add_forward(*args(r=None)) != 0                       # no second operand
    assert lib.actnn_relu_add_forward(*args(mn=mn.data_ptr())) != 0             # one statistic without the other
    assert lib.actnn_relu_add_forward(*args(r=x.data_ptr() + 2)) != 0           # misaligned
    assert lib.actnn_relu_add_forward(*args(mn=mn.data_ptr(), mx=mn.data_ptr(), n=4096 - 512)) != 0
    assert lib.actnn_relu_add_forward(*args(mn=mn.data_ptr(), mx=mn.data_ptr(), dtype=0)) != 0
    assert lib.actnn_relu_add_forward(*args(n=0)) == 0
    torch.cuda.synchronize()
