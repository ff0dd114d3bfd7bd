"""The benchmark configurations at their full sizes, checked through properties that do not need a
CPU pass over the whole tensor: a sampled subset against the oracle bit for bit, the stream of the
whole batch equal to the concatenation of the streams of its parts, round trips inside one
quantisation step, gather(input, index) == output, and equality with torch's own operators.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import actnn_amd.cpp_extension.minimax as ext_minimax
import actnn_amd.cpp_extension.quantization as ext_q
from oracle import calc_precision as o_calc
from oracle import layouts, simulate
from _util import DEV, bits_tensor, minmax_dev, np_bits

pytestmark = pytest.mark.gpu


def _config2(dtype=torch.float32):
    """fp32 [256,256,56,56] = [256, 3136, 256] groups: ReLU(N(0,1)) with a per-channel LogNormal(0,1)
    scale, bits from the greedy allocation at an average of 2 (1..8 per sample)."""
    N, C, HW = 256, 256, 56 * 56
    g = torch.Generator(device=DEV).manual_seed(2)
    x = torch.relu(torch.randn(N, C, HW, generator=g, device=DEV))
    x *= torch.exp(torch.randn(1, C, 1, generator=g, device=DEV))
    x *= torch.exp(0.7 * torch.randn(N, 1, 1, generator=g, device=DEV))      # samples differ in range
    x = x.to(dtype).view(N, -1, 256)
    mn, mx = minmax_dev(x)
    rng = (mx.float() - mn.float()).view(N, -1)
    sens = (rng * rng).sum(1).cpu().numpy().astype(np.float32)               # C_n of the allocation
    b = o_calc.calc_precision(np.full(N, 8, np.int32), sens, np.full(N, x[0].numel(), np.int32),
                              2 * N * x[0].numel())
    return x, mn, mx, [int(v) for v in b]


def test_config2_full_size_deterministic_mode():
    x, mn, mx, bits = _config2()
    assert len(set(bits)) > 2
    _check_config2(x, mn, mx, bits)


def test_config2_full_size_on_the_benchmarks_own_tensor():
    """The tensor and widths `bench.py` measures (BASELINE's distribution: identically distributed
    samples, so the greedy allocation gives nearly every sample 2 bits), through the same checks."""
    import os
    import sys
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    import bench
    x, mn, mx, _, b = bench.make_config2(DEV)
    _check_config2(x, mn, mx, [int(v) for v in b])


def _check_config2(x, mn, mx, bits):
    N, G, gs = x.shape
    assert (N, G, gs) == (256, 3136, 256)
    assert min(bits) >= 1 and max(bits) <= 8 and abs(np.mean(bits) - 2.0) < 0.02
    bits_dev, bits_host = bits_tensor(bits)
    noise = torch.rand(x.shape, generator=torch.Generator(device=DEV).manual_seed(3), device=DEV) - 0.5
    packed, scale = ext_q.pack_mixed_precision(x, mn, mx, bits_dev, True, noise=noise)
    words_per_sample = np.array(bits, np.int64) * (G * gs // 32)
    starts = np.concatenate([[0], np.cumsum(words_per_sample)])
    assert packed.numel() == starts[-1]

    # (1) the stream of the batch is the concatenation of the streams of its parts (ragged cut)
    cut = 101
    for lo, hi in ((0, cut), (cut, N)):
        bd, _ = bits_tensor(bits[lo:hi])
        part, sc = ext_q.pack_mixed_precision(x[lo:hi].contiguous(), mn[lo:hi].contiguous(),
                                              mx[lo:hi].contiguous(), bd, True,
                                              noise=noise[lo:hi].contiguous())
        assert torch.equal(part, packed[starts[lo]:starts[hi]])
        assert torch.equal(sc, scale[lo:hi])

    # (2) sampled samples against the oracle, bit for bit (one of every bit width that occurs)
    picks = sorted({bits.index(b) for b in set(bits)} | {0, N - 1})
    for n in picks:
        xs, ns = x[n:n + 1].cpu(), noise[n:n + 1].cpu()
        mn_c, mx_c = xs.min(2, keepdim=True)[0], xs.max(2, keepdim=True)[0]
        assert torch.equal(mn[n:n + 1].cpu(), mn_c) and torch.equal(mx[n:n + 1].cpu(), mx_c)
        codes, scale_o = simulate.quantize_simulate(xs.clone(), bits_host[n:n + 1], mn_c, mx_c, ns)
        words = layouts.pack_mixed(codes.numpy(), bits_host[n:n + 1].numpy())
        assert np.array_equal(packed[starts[n]:starts[n + 1]].cpu().numpy(), words), n
        assert np.array_equal(np_bits(scale[n:n + 1]), np_bits(scale_o)), n

    # (3) round trip: every element comes back inside one quantisation step (plus rounding)
    out = ext_q.unpack_mixed_precision(packed, bits_dev, scale, mn, N, G, gs)
    step = 1.0 / scale
    err = (out - x).abs()
    assert bool((err <= step * 1.0001 + 1e-5).all())
    # ... and unpack of the parts equals the parts of the unpack
    bd, _ = bits_tensor(bits[cut:])
    out_hi = ext_q.unpack_mixed_precision(packed[starts[cut]:].contiguous(), bd, scale[cut:].contiguous(),
                                          mn[cut:].contiguous(), N - cut, G, gs)
    assert torch.equal(out_hi, out[cut:])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_config2_full_size_rng_mode_is_unbiased(dtype):
    """In-kernel Philox at full size: the mean error over the 2e8 elements is a tiny fraction of a
    step, errors stay inside one step, and two calls draw different noise."""
    x, mn, mx, bits = _config2(dtype)
    N, G, gs = x.shape
    bits_dev, _ = bits_tensor(bits)
    torch.cuda.manual_seed(77)
    packed, scale = ext_q.pack_mixed_precision(x, mn, mx, bits_dev, True)
    packed2, _ = ext_q.pack_mixed_precision(x, mn, mx, bits_dev, True)
    assert not torch.equal(packed, packed2)
    out = ext_q.unpack_mixed_precision(packed, bits_dev, scale, mn, N, G, gs)
    e = (out.float() - x.float()) * scale.float()                  # error in steps
    # one step, plus for bf16 the rounding of the output (2^-8 relative on values of up to 2^bits steps)
    levels = torch.tensor([float(2 ** b) for b in bits], device=DEV).view(N, 1, 1)
    tol_one = 1.0001 if dtype == torch.float32 else 1.0 + levels * 2.0 ** -7
    assert bool((e.abs() <= tol_one).all())
    # groups with a usable range only (constant groups have scale ~ 1e6 and no information)
    live = ((mx.float() - mn.float()) > 1e-3).expand_as(e)
    mean_err = float(e[live].mean())
    assert abs(mean_err) < (2e-4 if dtype == torch.float32 else 4e-3), mean_err


def test_config3_full_size_relu_and_max_pool():
    g = torch.Generator(device=DEV).manual_seed(5)
    x = torch.randn(256, 64, 112, 112, generator=g, device=DEV).half()
    go = torch.randn(256, 64, 112, 112, generator=g, device=DEV).half()
    # ReLU: values and gradient equal torch's, mask words follow the layout on a sampled range
    y, mask = ext_q.relu_forward(x)
    assert torch.equal(y, F.relu(x))
    gi = ext_q.relu_backward(go, mask)
    assert torch.equal(gi, torch.where(x > 0, go, torch.zeros_like(go)))
    flat = x.view(-1)
    for first_block in (0, 12345, flat.numel() // 512 - 3):
        seg = (flat[first_block * 512:(first_block + 3) * 512] > 0).cpu().numpy()
        exp = layouts.mask_words(seg)
        assert np.array_equal(mask[first_block * 16:(first_block + 3) * 16].cpu().numpy(), exp)
    assert int(mask.numel()) == flat.numel() // 32
    # max-pool 3x3 s2 p1: values equal torch's, the index points at the maximum, gradient equals torch's
    k, s, p = (3, 3), (2, 2), (1, 1)
    yp, idx = ext_q.max_pool2d_forward(x, k, s, p, (1, 1))
    ref, ref_idx = F.max_pool2d(x, k, s, p, return_indices=True)
    assert torch.equal(yp, ref)
    Ho, Wo = yp.shape[2:]
    hb = torch.arange(Ho, device=DEV).view(1, 1, Ho, 1) * 2 - 1
    wb = torch.arange(Wo, device=DEV).view(1, 1, 1, Wo) * 2 - 1
    ii = idx.long()
    flat_idx = (hb + ii // 3) * 112 + (wb + ii % 3)
    assert torch.equal(x.view(256, 64, -1).gather(2, flat_idx.view(256, 64, -1)).view_as(yp), yp)
    gp = torch.randn(yp.shape, generator=g, device=DEV).half()
    gin = ext_q.max_pool2d_backward(gp, idx, x.shape, k, s, p)
    # where torch's arg-max and ours agree (everywhere except ties) the gradients are the same sums
    xr = x.clone().requires_grad_(True)
    F.max_pool2d(xr, k, s, p).backward(gp)
    same = torch.isclose(gin.float(), xr.grad.float(), atol=2e-2, rtol=2e-2)
    assert float(same.float().mean()) > 0.9999
    assert abs(float(gin.float().sum()) - float(gp.float().sum())) < 1e-3 * gp.numel() ** 0.5 + 50.0


def test_minimax_full_size_against_torch():
    x, mn, mx, _ = _config2()
    assert torch.equal(mn, x.min(2, keepdim=True)[0]) and torch.equal(mx, x.max(2, keepdim=True)[0])
    xh = x.half()
    mnh, mxh = ext_minimax.minimax(xh.view(-1, 256))
    assert torch.equal(mnh.view(-1), xh.min(2)[0].view(-1)) and torch.equal(mxh.view(-1), xh.max(2)[0].view(-1))
