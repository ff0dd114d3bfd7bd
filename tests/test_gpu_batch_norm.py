"""The library's training-mode batch norm (actnn_batch_norm_forward / _backward) against the
float64 restatement and against torch's own batch norm.  Floating point: the tolerances below are
a few units of the output type's rounding (fp32: 2^-19 of |y| + 4, the rounding of a*x + b on inputs a few standard deviations from a mean of order 1; 16-bit types one
rounding step of the result, 2^-8 for bf16 and 2^-11 for fp16, plus the fp32 error)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import actnn_amd.cpp_extension.backward_func as ext_bf
import actnn_amd.cpp_extension.minimax as ext_minimax
from oracle import batch_norm as o_bn
from _util import DEV

pytestmark = pytest.mark.gpu

# (N, C, spatial): ResNet-50 planes (112^2 ... 7^2), channel boundaries inside a 16-byte chunk
# (49, 196, 12, 10), several spans per channel, one span over many channels, ragged batch splits
SHAPES = [(8, 64, (112, 112)), (8, 16, (56, 56)), (5, 32, (28, 28)), (37, 24, (14, 14)),
          (16, 256, (7, 7)), (3, 6, (4, 3)), (9, 4, (10,)), (2, 8, (3, 4, 5)), (70, 8, (8, 8)),
          (4, 2048, (7, 7)), (1, 8, (16, 16)),
          # [N, C] inputs (the channels-last kernels with one pixel per sample), and shapes that are
          # not whole 16-byte chunks per row or per plane (element by element)
          (32, 512, ()), (64, 104, ()), (300, 8, ()), (33, 10, ()), (4, 3, (7, 7)), (6, 5, (3,)), (5, 4, (1, 1)),
          (70000, 3, (1,))]
RND = {torch.float32: 2.0 ** -19, torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}


def _inputs(N, C, spatial, dtype, seed):
    g = torch.Generator(device=DEV).manual_seed(seed)
    x = torch.randn(N, C, *spatial, generator=g, device=DEV)
    x = x * (0.5 + torch.rand(1, C, *([1] * len(spatial)), generator=g, device=DEV) * 2)
    x = (x + torch.randn(1, C, *([1] * len(spatial)), generator=g, device=DEV)).to(dtype)
    w = torch.rand(C, generator=g, device=DEV) + 0.5
    b = torch.randn(C, generator=g, device=DEV)
    rm = torch.randn(C, generator=g, device=DEV)
    rv = torch.rand(C, generator=g, device=DEV) + 0.5
    dy = torch.randn(N, C, *spatial, generator=g, device=DEV).to(dtype)
    return x, w, b, rm, rv, dy


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("N,C,spatial", SHAPES)
def test_forward_backward_against_float64(N, C, spatial, dtype):
    x, w, b, rm, rv, dy = _inputs(N, C, spatial, dtype, N * 1000 + C)
    assert ext_bf.hip_batch_norm_applies(x, w, b, rm, rv)
    rm0, rv0 = rm.clone(), rv.clone()
    y, mean, invstd, _ = ext_bf.cudnn_batch_norm(x, w, b, rm, rv, True, 0.1, 1e-5)
    yo, mean_o, invstd_o, rm_o, rv_o = o_bn.forward(
        x.double().cpu().numpy(), w.cpu().numpy(), b.cpu().numpy(), rm0.cpu().numpy(), rv0.cpu().numpy(), 0.1, 1e-5)
    assert y.dtype == dtype and y.shape == x.shape
    assert np.allclose(mean.cpu().numpy(), mean_o, rtol=1e-5, atol=1e-6)
    assert np.allclose(invstd.cpu().numpy(), invstd_o, rtol=2e-5)
    assert np.allclose(rm.cpu().numpy(), rm_o, rtol=1e-5, atol=1e-6)
    assert np.allclose(rv.cpu().numpy(), rv_o, rtol=2e-5)
    err = np.abs(y.double().cpu().numpy() - yo)
    assert (err <= RND[dtype] * (np.abs(yo) + 4.0)).all(), float(err.max())

    gi, gw, gb = ext_bf.cudnn_batch_norm_backward(x, dy, w, rm, rv, mean, invstd, 1e-5, None)
    gi_o, gw_o, gb_o = o_bn.backward(x.double().cpu().numpy(), dy.double().cpu().numpy(), w.cpu().numpy(), 1e-5)
    count = x.numel() / C
    scale = np.sqrt(count)                       # sums of `count` terms of order 1
    assert np.allclose(gb.cpu().numpy(), gb_o, rtol=1e-5, atol=2e-5 * scale)
    assert np.allclose(gw.cpu().numpy(), gw_o, rtol=1e-5, atol=4e-5 * scale)
    err = np.abs(gi.double().cpu().numpy() - gi_o)
    assert (err <= RND[dtype] * (np.abs(gi_o) + 4.0)).all(), float(err.max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_against_torch_batch_norm_and_autograd(dtype):
    x, w, b, rm, rv, dy = _inputs(16, 64, (28, 28), dtype, 5)
    rm_t, rv_t = rm.clone(), rv.clone()
    xt = x.clone().requires_grad_(True)
    wt, bt = w.clone().requires_grad_(True), b.clone().requires_grad_(True)
    yt = F.batch_norm(xt, rm_t, rv_t, wt, bt, True, 0.1, 1e-5)
    yt.backward(dy)
    y, mean, invstd, _ = ext_bf.cudnn_batch_norm(x, w, b, rm, rv, True, 0.1, 1e-5)
    gi, gw, gb = ext_bf.cudnn_batch_norm_backward(x, dy, w, rm, rv, mean, invstd, 1e-5, None)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    assert torch.allclose(y.float(), yt.float(), rtol=tol, atol=tol)
    assert torch.allclose(rm, rm_t, rtol=1e-5, atol=1e-6) and torch.allclose(rv, rv_t, rtol=1e-5)
    assert torch.allclose(gi.float(), xt.grad.float(), rtol=tol, atol=tol)
    assert torch.allclose(gw, wt.grad, rtol=1e-3, atol=1e-2) and torch.allclose(gb, bt.grad, rtol=1e-3, atol=1e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("N,C,spatial", [(8, 64, (56, 56)), (5, 256, (7, 7)), (9, 64, (14, 14)), (3, 8, (8, 4)),
                                         (40, 512, ()), (7, 256, ())])
def test_group_min_max_from_the_statistics_pass(N, C, spatial, dtype):
    x, w, b, rm, rv, _ = _inputs(N, C, spatial, dtype, 11)
    y0, m0, i0, _, _ = ext_bf.hip_batch_norm_forward(x, w, b, rm.clone(), rv.clone(), 0.1, 1e-5)
    y, m, i, mn, mx = ext_bf.hip_batch_norm_forward(x, w, b, rm.clone(), rv.clone(), 0.1, 1e-5, minmax=True)
    mn_ref, mx_ref = ext_minimax.minimax(x.view(-1, 256))
    assert torch.equal(mn, mn_ref.view(-1)) and torch.equal(mx, mx_ref.view(-1))
    assert torch.equal(y, y0) and torch.equal(m, m0) and torch.equal(i, i0)     # and nothing else changes


def test_results_do_not_depend_on_the_schedule():
    x, w, b, rm, rv, dy = _inputs(64, 128, (14, 14), torch.bfloat16, 3)
    first = None
    for _ in range(3):
        y, mean, invstd, _, _ = ext_bf.hip_batch_norm_forward(x, w, b, None, None, 0.1, 1e-5)
        gi, gw, gb = ext_bf.hip_batch_norm_backward(x, dy, w, mean, invstd)
        cur = (y, mean, invstd, gi, gw, gb)
        if first is None:
            first = cur
        else:
            assert all(torch.equal(a, c) for a, c in zip(first, cur))


def test_no_affine_no_running_stats_and_fallback_shapes():
    x, _, _, _, _, dy = _inputs(6, 16, (8, 8), torch.float32, 4)
    y, mean, invstd, _ = ext_bf.cudnn_batch_norm(x, None, None, None, None, True, 0.1, 1e-5)
    yo, mean_o, invstd_o, _, _ = o_bn.forward(x.double().cpu().numpy(), None, None, None, None, 0.1, 1e-5)
    assert np.allclose(y.cpu().numpy(), yo, rtol=1e-5, atol=1e-5)
    gi, gw, gb = ext_bf.cudnn_batch_norm_backward(x, dy, None, None, None, mean, invstd, 1e-5, None)
    gi_o, _, gb_o = o_bn.backward(x.double().cpu().numpy(), dy.double().cpu().numpy(), None, 1e-5)
    assert np.allclose(gi.cpu().numpy(), gi_o, rtol=1e-4, atol=1e-5)
    # every dense shape runs the library's kernels; tensors that are not dense go to ATen
    for shape in ((32, 10), (4, 3, 7, 7)):
        xs = torch.randn(*shape, device=DEV)
        assert ext_bf.hip_batch_norm_applies(xs, None, None, None, None)
    xs = torch.randn(8, 6, 5, 5, device=DEV)[:, ::2]
    assert not ext_bf.hip_batch_norm_applies(xs, None, None, None, None)
    # affine parameters that are not fp32: ATen's native kernels
    xh = torch.randn(8, 16, 4, 4, device=DEV, dtype=torch.float16)
    wh, bh = torch.ones(16, device=DEV, dtype=torch.float16), torch.zeros(16, device=DEV, dtype=torch.float16)
    assert not ext_bf.hip_batch_norm_applies(xh, wh, bh, None, None)
    ys = ext_bf.cudnn_batch_norm(xh, wh, bh, None, None, True, 0.1, 1e-5)[0]
    ref = o_bn.forward(xh.double().cpu().numpy(), None, None, None, None, 0.1, 1e-5)[0]
    assert np.allclose(ys.double().cpu().numpy(), ref, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("N,C,spatial,channels_last", [
    (8, 64, (28, 28), False), (8, 64, (28, 28), True), (5, 24, (7, 7), False), (5, 24, (7, 7), True),
    (4, 3, (7, 7), False), (4, 3, (7, 7), True), (32, 512, (), False), (33, 10, (), False)])
def test_evaluation_mode_against_float64_and_torch(N, C, spatial, dtype, channels_last):
    # training = False in the reference's batch_norm Function (ops.py:458-461, :495-499)
    x, w, b, rm, rv, dy = _inputs(N, C, spatial, dtype, 77 + C)
    if channels_last:
        x, dy = _cl(x), _cl(dy)
    rm0, rv0 = rm.clone(), rv.clone()
    y, mean, invstd = ext_bf.native_batch_norm(x, w, b, rm, rv, False, 0.1, 1e-5)
    assert torch.equal(rm, rm0) and torch.equal(rv, rv0)             # the running estimates are only read
    assert y.dtype == dtype and y.stride() == x.stride()
    yo, mean_o, invstd_o = o_bn.forward_eval(x.double().cpu().numpy(), w.cpu().numpy(), b.cpu().numpy(),
                                             rm.cpu().numpy(), rv.cpu().numpy(), 1e-5)
    assert np.allclose(mean.cpu().numpy(), mean_o, rtol=1e-6) and np.allclose(invstd.cpu().numpy(), invstd_o, rtol=1e-6)
    err = np.abs(y.double().cpu().numpy() - yo)
    assert (err <= RND[dtype] * (np.abs(yo) + 4.0)).all(), float(err.max())
    gi, gw, gb = ext_bf.native_batch_norm_backward(dy, x, w, rm, rv, mean, invstd, False, 1e-5, [True, True, True])
    gi_o, gw_o, gb_o = o_bn.backward_eval(x.double().cpu().numpy(), dy.double().cpu().numpy(), w.cpu().numpy(),
                                          rm.cpu().numpy(), rv.cpu().numpy(), 1e-5)
    scale = np.sqrt(x.numel() / C)
    assert np.allclose(gb.cpu().numpy(), gb_o, rtol=1e-5, atol=2e-5 * scale)
    assert np.allclose(gw.cpu().numpy(), gw_o, rtol=1e-5, atol=8e-5 * scale)
    err = np.abs(gi.double().cpu().numpy() - gi_o)
    assert (err <= RND[dtype] * (np.abs(gi_o) + 4.0)).all(), float(err.max())
    # the same through autograd against torch's own evaluation-mode batch norm; empty saved
    # statistics (what ATen's forward returns in this mode) are rebuilt from the running estimates
    gi2, gw2, gb2 = ext_bf.native_batch_norm_backward(dy, x, w, rm, rv, x.new_empty(0), x.new_empty(0), False, 1e-5,
                                                      [True, False, True])
    assert gw2 is None and torch.equal(gb2, gb)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    xt = x.detach().clone().requires_grad_(True)
    F.batch_norm(xt, rm, rv, w, b, False, 0.1, 1e-5).backward(dy)
    assert torch.allclose(gi2.float(), xt.grad.float(), rtol=tol, atol=tol)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("N,C,spatial", [(8, 64, (56, 56)), (16, 256, (7, 7)), (37, 64, (14, 14)),
                                         (9, 32, (4, 2)), (12, 128, (28, 28)), (70, 512, ()), (9, 256, ())])
def test_backward_from_the_packed_stream_equals_unpack_then_backward(N, C, spatial, dtype):
    """The fused pass rebuilds x exactly as unpack_mixed_precision does, so every output is
    bit-identical to the two-step path, for every width 1..8 in one batch."""
    import actnn_amd.cpp_extension.quantization as ext_q
    from _util import bits_tensor
    x, w, b, rm, rv, dy = _inputs(N, C, spatial, dtype, 21)
    G = x[0].numel() // 256
    groups = x.view(N, G, 256)
    mn, mx = ext_minimax.minimax(groups.view(-1, 256))
    mn, mx = mn.view(N, G, 1), mx.view(N, G, 1)
    bits_dev, _ = bits_tensor([1 + (3 * i + i // 8) % 8 for i in range(N)])
    torch.cuda.manual_seed(5)
    packed, scale = ext_q.pack_mixed_precision(groups, mn, mx, bits_dev, True)
    _, mean, invstd, _, _ = ext_bf.hip_batch_norm_forward(x, w, b, None, None, 0.1, 1e-5)
    xq = ext_q.unpack_mixed_precision(packed, bits_dev, scale, mn, N, G, 256).view_as(x)
    ref = ext_bf.hip_batch_norm_backward(xq, dy, w, mean, invstd)
    quantized = (packed, bits_dev, scale, mn)
    assert ext_bf.hip_batch_norm_backward_packed_applies(x.shape, quantized, dy, w, mean, invstd)
    got = ext_bf.hip_batch_norm_backward_packed(x.shape, quantized, dy, w, mean, invstd)
    for a, r in zip(got, ref):
        assert torch.equal(a, r)
    _check_sumsq(lambda: ext_bf.hip_batch_norm_backward_packed(x.shape, quantized, dy, w, mean, invstd, sumsq=True),
                 lambda: ext_bf.hip_batch_norm_backward(xq, dy, w, mean, invstd, sumsq=True), ref)


def test_backward_from_the_packed_stream_fp32_with_compact_scale_storage():
    """An fp32 activation keeps its scale and minimum as bf16 (ops.py:115-116); the packed backward
    widens them exactly as dequantize_activation does (ops.py:129-131)."""
    import actnn_amd.cpp_extension.quantization as ext_q
    from _util import bits_tensor
    N, C, spatial = 10, 64, (28, 28)
    x, w, b, rm, rv, dy = _inputs(N, C, spatial, torch.float32, 23)
    G = x[0].numel() // 256
    groups = x.view(N, G, 256)
    mn, mx = ext_minimax.minimax(groups.view(-1, 256))
    mn, mx = mn.view(N, G, 1), mx.view(N, G, 1)
    bits_dev, _ = bits_tensor([1 + (5 * i) % 8 for i in range(N)])
    packed, scale = ext_q.pack_mixed_precision(groups, mn, mx, bits_dev, True)
    scale16, mn16 = scale.bfloat16(), mn.bfloat16()
    _, mean, invstd, _, _ = ext_bf.hip_batch_norm_forward(x, w, b, None, None, 0.1, 1e-5)
    xq = ext_q.unpack_mixed_precision(packed, bits_dev, scale16.float(), mn16.float(), N, G, 256).view_as(x)
    ref = ext_bf.hip_batch_norm_backward(xq, dy, w, mean, invstd)
    quantized = (packed, bits_dev, scale16, mn16)
    assert ext_bf.hip_batch_norm_backward_packed_applies(x.shape, quantized, dy, w, mean, invstd)
    got = ext_bf.hip_batch_norm_backward_packed(x.shape, quantized, dy, w, mean, invstd)
    for a, r in zip(got, ref):
        assert torch.equal(a, r)


def _check_sumsq(*args):
    """Both backward passes, asked for it, leave sum(dx^2) of the dx they store (float64 sum of the
    stored values, rtol 1e-5: fp32 partial sums of at most a few thousand products each) and
    change nothing else; the statistic lapses when dx is written to afterwards."""
    *passes, ref = args
    for run in passes:
        got = run()
        for a, r in zip(got, ref):
            assert torch.equal(a, r)
        total = ext_bf.known_sumsq(got[0])
        want = got[0].double().square().sum()
        assert total is not None and total.dtype == torch.float32
        assert abs(total.double().item() - want.item()) <= 1e-5 * want.item() + 1e-30
        got[0].mul_(2.0)
        assert ext_bf.known_sumsq(got[0]) is None
    assert ext_bf.known_sumsq(ref[0]) is None


# ------------------------------------------------------------------------------------------
# channels-last tensors ([N, HW, C] in memory)
# ------------------------------------------------------------------------------------------
def _cl(t):
    return t.contiguous(memory_format=torch.channels_last if t.dim() == 4 else torch.channels_last_3d)


CL_SHAPES = [(8, 64, (56, 56)), (16, 256, (7, 7)), (5, 32, (28, 28)), (37, 24, (14, 14)),
             (4, 2048, (7, 7)), (3, 320, (5, 5)), (2, 16, (3, 4, 5)), (70, 8, (8, 8)), (2, 512, (28, 28)),
             (4, 12, (7, 7)), (3, 20, (4, 4)), (2, 3, (9, 5))]          # C not a whole chunk: element by element


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("N,C,spatial", CL_SHAPES)
def test_channels_last_forward_backward_against_float64(N, C, spatial, dtype):
    x, w, b, rm, rv, dy = _inputs(N, C, spatial, dtype, N * 1000 + C + 1)
    x, dy = _cl(x), _cl(dy)
    assert ext_bf.hip_batch_norm_applies(x, w, b, rm, rv)
    rm0, rv0 = rm.clone(), rv.clone()
    y, mean, invstd, _ = ext_bf.cudnn_batch_norm(x, w, b, rm, rv, True, 0.1, 1e-5)
    assert y.stride() == x.stride()
    yo, mean_o, invstd_o, rm_o, rv_o = o_bn.forward(
        x.double().cpu().numpy(), w.cpu().numpy(), b.cpu().numpy(), rm0.cpu().numpy(), rv0.cpu().numpy(), 0.1, 1e-5)
    assert np.allclose(mean.cpu().numpy(), mean_o, rtol=1e-5, atol=1e-6)
    assert np.allclose(invstd.cpu().numpy(), invstd_o, rtol=2e-5)
    assert np.allclose(rm.cpu().numpy(), rm_o, rtol=1e-5, atol=1e-6)
    assert np.allclose(rv.cpu().numpy(), rv_o, rtol=2e-5)
    err = np.abs(y.double().cpu().numpy() - yo)
    assert (err <= RND[dtype] * (np.abs(yo) + 4.0)).all(), float(err.max())
    gi, gw, gb = ext_bf.cudnn_batch_norm_backward(x, dy, w, rm, rv, mean, invstd, 1e-5, None)
    assert gi.stride() == x.stride()
    gi_o, gw_o, gb_o = o_bn.backward(x.double().cpu().numpy(), dy.double().cpu().numpy(), w.cpu().numpy(), 1e-5)
    scale = np.sqrt(x.numel() / C)
    assert np.allclose(gb.cpu().numpy(), gb_o, rtol=1e-5, atol=2e-5 * scale)
    assert np.allclose(gw.cpu().numpy(), gw_o, rtol=1e-5, atol=4e-5 * scale)
    err = np.abs(gi.double().cpu().numpy() - gi_o)
    assert (err <= RND[dtype] * (np.abs(gi_o) + 4.0)).all(), float(err.max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("N,C,spatial", [(8, 64, (56, 56)), (5, 256, (7, 7)), (9, 128, (14, 14)),
                                         (3, 8, (8, 4)), (2, 512, (6, 6)), (3, 2048, (7, 7))])
def test_channels_last_group_min_max(N, C, spatial, dtype):
    from actnn_amd.utils import memory_order
    x, w, b, rm, rv, _ = _inputs(N, C, spatial, dtype, 12)
    x = _cl(x)
    assert ext_bf.hip_batch_norm_minmax_applies(x, w, b, rm, rv)
    y0, m0, i0, _, _ = ext_bf.hip_batch_norm_forward(x, w, b, rm.clone(), rv.clone(), 0.1, 1e-5)
    y, m, i, mn, mx = ext_bf.hip_batch_norm_forward(x, w, b, rm.clone(), rv.clone(), 0.1, 1e-5, minmax=True)
    mn_ref, mx_ref = ext_minimax.minimax(memory_order(x).reshape(-1, 256))
    assert torch.equal(mn, mn_ref.view(-1)) and torch.equal(mx, mx_ref.view(-1))
    assert torch.equal(y, y0) and torch.equal(m, m0) and torch.equal(i, i0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("N,C,spatial", [(8, 64, (56, 56)), (16, 256, (7, 7)), (37, 128, (14, 14)),
                                         (9, 32, (4, 2)), (5, 1024, (6, 6))])
def test_channels_last_backward_from_the_packed_stream(N, C, spatial, dtype):
    import actnn_amd.cpp_extension.quantization as ext_q
    from actnn_amd.ops import _Quantized
    from actnn_amd.utils import logical_order, memory_order
    from _util import bits_tensor
    x, w, b, rm, rv, dy = _inputs(N, C, spatial, dtype, 22)
    x, dy = _cl(x), _cl(dy)
    G = x[0].numel() // 256
    groups = memory_order(x).reshape(N, G, 256)
    mn, mx = ext_minimax.minimax(groups.view(-1, 256))
    mn, mx = mn.view(N, G, 1), mx.view(N, G, 1)
    bits_dev, _ = bits_tensor([1 + (3 * i + i // 8) % 8 for i in range(N)])
    torch.cuda.manual_seed(5)
    packed, scale = ext_q.pack_mixed_precision(groups, mn, mx, bits_dev, True)
    _, mean, invstd, _, _ = ext_bf.hip_batch_norm_forward(x, w, b, None, None, 0.1, 1e-5)
    xq = ext_q.unpack_mixed_precision(packed, bits_dev, scale, mn, N, G, 256)
    xq = logical_order(xq.view(N, *spatial, C), torch.channels_last)
    ref = ext_bf.hip_batch_norm_backward(xq, dy, w, mean, invstd)
    quantized = _Quantized((packed, bits_dev, scale, mn))
    quantized.memory_format = torch.channels_last
    assert ext_bf.hip_batch_norm_backward_packed_applies(x.shape, quantized, dy, w, mean, invstd)
    got = ext_bf.hip_batch_norm_backward_packed(x.shape, quantized, dy, w, mean, invstd)
    assert got[0].stride() == x.stride()
    for a, r in zip(got, ref):
        assert torch.equal(a, r)
    _check_sumsq(lambda: ext_bf.hip_batch_norm_backward_packed(x.shape, quantized, dy, w, mean, invstd, sumsq=True),
                 lambda: ext_bf.hip_batch_norm_backward(xq, dy, w, mean, invstd, sumsq=True), ref)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("N,C,spatial,channels_last",
                         [(n, c, sp, cl) for (n, c, sp) in [(8, 64, (56, 56)), (16, 256, (7, 7)), (37, 128, (14, 14)),
                                                            (9, 32, (4, 2)), (5, 1024, (6, 6)), (70, 64, (8, 8))]
                          for cl in (False, True)] + [(70, 512, (), False), (9, 256, (), False)])
def test_forward_with_packed_copy_equals_forward_then_pack(N, C, spatial, dtype, channels_last):
    """The normalising pass that also packs its input: output equal to the plain forward pass,
    stream and scales equal to pack_mixed_precision with the same generator state (every width)."""
    import actnn_amd.cpp_extension.quantization as ext_q
    from actnn_amd.utils import memory_order
    from _util import bits_tensor
    x, w, b, rm, rv, _ = _inputs(N, C, spatial, dtype, 31)
    if channels_last:
        x = _cl(x)
    assert ext_bf.hip_batch_norm_pack_applies(x, w, b, rm, rv)
    G = x[0].numel() // 256
    bits_dev, _ = bits_tensor([1 + (5 * i + i // 8) % 8 for i in range(N)])
    y_ref, mean_ref, invstd_ref, mn_ref, mx_ref = ext_bf.hip_batch_norm_forward(
        x, w, b, rm.clone(), rv.clone(), 0.1, 1e-5, minmax=True)
    torch.cuda.manual_seed(9)
    packed_ref, scale_ref = ext_q.pack_mixed_precision(
        memory_order(x).reshape(N, G, 256), mn_ref.view(N, G, 1), mx_ref.view(N, G, 1), bits_dev, True)
    ws, mean, invstd, mn, mx = ext_bf.hip_batch_norm_forward_stats(x, w, b, rm.clone(), rv.clone(), 0.1, 1e-5)
    torch.cuda.manual_seed(9)
    y, packed, scale = ext_bf.hip_batch_norm_forward_apply(x, ws, bits_dev, mn.view(N, G, 1), mx.view(N, G, 1))
    assert torch.equal(y, y_ref) and y.stride() == x.stride()
    assert torch.equal(mean, mean_ref) and torch.equal(invstd, invstd_ref)
    assert torch.equal(mn, mn_ref) and torch.equal(mx, mx_ref)
    assert torch.equal(scale, scale_ref)
    assert torch.equal(packed, packed_ref)
    y2, none1, none2 = ext_bf.hip_batch_norm_forward_apply(x, ws)
    assert torch.equal(y2, y_ref) and none1 is None and none2 is None


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("N,C,H", [(8, 64, 8), (4, 256, 4), (32, 16, 4), (6, 128, 8), (6, 512, 4), (3, 1024, 4),
                                   (5, 2048, 4)])
def test_apply_with_the_relu_folded_in_equals_apply_then_relu(dtype, N, C, H):
    """actnn_batch_norm_forward_apply_relu against actnn_batch_norm_forward_apply followed by
    actnn_relu_forward_minmax on the stored result: output, mask words, group min / max, scale and
    the packed stream bit for bit, over several widths and a sample boundary inside a block."""
    from actnn_amd import _lib
    import actnn_amd.cpp_extension.backward_func as bf
    import actnn_amd.cpp_extension.quantization as ext_q
    lib = _lib.load()
    g = torch.Generator(device=DEV).manual_seed(N * C + H)
    x = (torch.randn(N, C, H, H, device=DEV, generator=g) * 1.5).to(dtype).contiguous(memory_format=torch.channels_last)
    w = torch.rand(C, device=DEV, generator=g) * 2 - 0.5
    b = torch.randn(C, device=DEV, generator=g)
    ws, mean, invstd, mn, mx = bf.hip_batch_norm_forward_stats(x, w, b, None, None, 0.1, 1e-5)
    widths = torch.randint(1, 9, (N,), generator=torch.Generator().manual_seed(1), dtype=torch.int32)
    bits = ext_q.attach_bits_host(widths.to(DEV), widths)
    torch.cuda.manual_seed(5)
    y, packed, scale = bf.hip_batch_norm_forward_apply(x, ws, bits, mn, mx)
    from actnn_amd.utils import memory_order
    z_ref, mask_ref, zmn_ref, zmx_ref = ext_q.relu_forward_minmax(memory_order(y).contiguous())
    total, prefix = ext_q._bits_info(bits)
    HW, n = H * H, x.numel()
    out = torch.empty_like(x)
    packed2, scale2 = torch.empty_like(packed), torch.empty_like(scale)
    mask = torch.empty(ext_q.mask_words(n), dtype=torch.int32, device=DEV)
    zmn, zmx = torch.empty(n // 256, dtype=dtype, device=DEV), torch.empty(n // 256, dtype=dtype, device=DEV)
    torch.cuda.manual_seed(5)
    seed, offset = ext_q.g.philox_args(x.device)
    rc = lib.actnn_batch_norm_forward_apply_relu(
        x.data_ptr(), out.data_ptr(), ws.data_ptr(), ws.numel() * 4, bits.data_ptr(), prefix.data_ptr(), mn.data_ptr(),
        mx.data_ptr(), scale2.data_ptr(), packed2.data_ptr(), seed, offset, mask.data_ptr(), zmn.data_ptr(),
        zmx.data_ptr(), None, N, C, HW, ext_q.g.DTYPE_CODE[dtype], 1, None)
    assert rc == 0
    assert torch.equal(memory_order(out), z_ref) and torch.equal(mask, mask_ref)
    assert torch.equal(zmn, zmn_ref) and torch.equal(zmx, zmx_ref)
    assert torch.equal(packed2, packed) and torch.equal(scale2, scale)
    # with a residual: relu(bn(x) + residual) as the addition of the stored bn(x) and the ReLU make it
    res = (torch.randn(N, C, H, H, device=DEV, generator=g) * 1.5).to(dtype).contiguous(memory_format=torch.channels_last)
    memory_order(res).reshape(-1)[::3] = -memory_order(y).reshape(-1)[::3]          # exact cancellation
    z_ref, mask_ref, zmn_ref, zmx_ref = ext_q.relu_forward_minmax(memory_order(y + res).contiguous())
    rc = lib.actnn_batch_norm_forward_apply_relu(
        x.data_ptr(), out.data_ptr(), ws.data_ptr(), ws.numel() * 4, bits.data_ptr(), prefix.data_ptr(), mn.data_ptr(),
        mx.data_ptr(), scale2.data_ptr(), packed2.data_ptr(), seed, offset, mask.data_ptr(), zmn.data_ptr(),
        zmx.data_ptr(), res.data_ptr(), N, C, HW, ext_q.g.DTYPE_CODE[dtype], 1, None)
    assert rc == 0
    assert torch.equal(memory_order(out), z_ref) and torch.equal(mask, mask_ref)
    assert torch.equal(zmn, zmn_ref) and torch.equal(zmx, zmx_ref)
    assert torch.equal(packed2, packed) and torch.equal(scale2, scale)
    # refused: default layout, fp32, C that does not divide 256, elements not a multiple of 2048
    args = lambda **k: (x.data_ptr(), out.data_ptr(), ws.data_ptr(), ws.numel() * 4, bits.data_ptr(), prefix.data_ptr(),
                        mn.data_ptr(), mx.data_ptr(), scale2.data_ptr(), packed2.data_ptr(), seed, offset,
                        k.get("mask", mask.data_ptr()), zmn.data_ptr(), zmx.data_ptr(), None, k.get("N", N), k.get("C", C), HW,
                        k.get("dtype", ext_q.g.DTYPE_CODE[dtype]), k.get("cl", 1), None)
    for bad in (dict(cl=0), dict(dtype=0), dict(mask=None), dict(C=C * 3)):
        assert lib.actnn_batch_norm_forward_apply_relu(*args(**bad)) != 0, bad
    torch.cuda.synchronize()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("N,C,H", [(8, 64, 8), (4, 256, 4), (32, 16, 4), (6, 128, 8), (40, 64, 4), (6, 512, 4),
                                   (3, 1024, 4), (5, 2048, 4), (9, 512, 8)])
def test_backward_with_the_relu_mask_equals_relu_backward_then_backward(dtype, N, C, H):
    """actnn_batch_norm_backward_packed_relu against actnn_relu_backward followed by
    actnn_batch_norm_backward_packed: gradients and the table of squared sums bit for bit (several
    widths, blocks of one to many steps, sample boundaries inside a block of the mask)."""
    import actnn_amd.cpp_extension.backward_func as bf
    import actnn_amd.cpp_extension.quantization as ext_q
    from actnn_amd.ops import _Quantized
    from actnn_amd.utils import memory_order
    g = torch.Generator(device=DEV).manual_seed(N + C + H)
    x = (torch.randn(N, C, H, H, device=DEV, generator=g) * 1.5).to(dtype).contiguous(memory_format=torch.channels_last)
    go = torch.randn(N, C, H, H, device=DEV, generator=g).to(dtype).contiguous(memory_format=torch.channels_last)
    keep = torch.rand(N, H, H, C, device=DEV, generator=g) > 0.4
    _, mask = ext_q.relu_forward(torch.where(keep, 1.0, -1.0).to(dtype))
    w = torch.rand(C, device=DEV, generator=g) * 2 - 0.5
    b = torch.randn(C, device=DEV, generator=g)
    ws, mean, invstd, mn, mx = bf.hip_batch_norm_forward_stats(x, w, b, None, None, 0.1, 1e-5)
    widths = torch.randint(1, 9, (N,), generator=torch.Generator().manual_seed(2), dtype=torch.int32)
    bits = ext_q.attach_bits_host(widths.to(DEV), widths)
    _, packed, scale = bf.hip_batch_norm_forward_apply(x, ws, bits, mn, mx)
    q = _Quantized((packed, bits, scale, mn.view(N, -1, 1)))
    q.native_bf16, q.memory_format = dtype == torch.bfloat16, torch.channels_last
    masked = ext_q.relu_backward(memory_order(go), mask).permute(0, 3, 1, 2)
    assert torch.equal(memory_order(masked), torch.where(keep, memory_order(go), torch.zeros_like(memory_order(go))))
    ref = bf.hip_batch_norm_backward_packed(x.shape, q, masked, w, mean, invstd, sumsq=True)
    got = bf.hip_batch_norm_backward_packed(x.shape, q, go, w, mean, invstd, sumsq=True, relu_mask=mask)
    for u, v in zip(ref, got):
        assert torch.equal(u, v)
    assert torch.equal(bf.known_sumsq(ref[0]), bf.known_sumsq(got[0]))
