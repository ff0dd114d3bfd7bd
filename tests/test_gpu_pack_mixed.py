"""pack/unpack_mixed_precision parity.

Deterministic mode (explicit noise): packed words and scale must equal the oracle's
config.simulate restatement bit for bit; dequantised values within 1 ulp (fp32).
RNG mode: the kernel's codes must equal the oracle's model of the kernel (same Philox
stream), and the distribution must be unbiased with the exact closed-form variance.
"""
import numpy as np
import pytest
import torch

import actnn_amd.cpp_extension.quantization as ext_q
from oracle import kernel_mode, layouts, simulate
from _util import DEV, assert_rng_tier, bits_tensor, make_groups, minmax_dev, np_bits, ulp_diff_f32

pytestmark = pytest.mark.gpu


def _det_case(x, noise, bits_list):
    N, G, gs = x.shape
    xd, nd = x.to(DEV), noise.to(DEV)
    mn, mx = minmax_dev(xd)
    bits_dev, bits_host = bits_tensor(bits_list)
    packed, scale = ext_q.pack_mixed_precision(xd, mn, mx, bits_dev, True, noise=nd)
    torch.cuda.synchronize()
    # oracle on the same inputs (min/max recomputed on CPU: equality is checked too)
    mn_c = x.min(dim=2, keepdim=True)[0]
    mx_c = x.max(dim=2, keepdim=True)[0]
    assert torch.equal(mn.cpu(), mn_c) and torch.equal(mx.cpu(), mx_c)
    codes, scale_o = simulate.quantize_simulate(x.clone(), bits_host, mn_c, mx_c, noise)
    words = layouts.pack_mixed(codes.numpy(), bits_host.numpy())
    assert packed.dtype == torch.int32 and packed.numel() == words.size
    assert np.array_equal(np_bits(scale), np_bits(scale_o)), "scale differs"
    assert np.array_equal(packed.cpu().numpy(), words), "packed words differ"
    out = ext_q.unpack_mixed_precision(packed, bits_dev, scale, mn, N, G, gs)
    deq = simulate.dequantize_simulate(codes, scale_o, mn_c)
    return out, deq


def test_config1_fp32_uniform_2bit_bit_exact():
    # benchmark config 1: relu(randn(32,64,56,56)) -> [32,784,256], 2 bits, seeded noise
    torch.manual_seed(0)
    x = torch.relu(torch.randn(32, 64, 56, 56)).view(32, 784, 256)
    noise = torch.rand(32, 784, 256, generator=torch.Generator().manual_seed(1)) - 0.5
    out, deq = _det_case(x, noise, [2] * 32)
    assert ulp_diff_f32(out.cpu().numpy(), deq.numpy()).max() <= 1
    assert np.array_equal(np_bits(out), np_bits(deq))     # in fact identical


@pytest.mark.parametrize("kind", ["relu", "chan", "shift", "plain"])
@pytest.mark.parametrize("G", [1, 5, 32, 37, 70])
def test_mixed_bits_fp32(kind, G):
    bits = [1, 2, 3, 4, 5, 6, 7, 8, 2, 1, 8, 3]
    x, noise = make_groups(len(bits), G, 256, torch.float32, 10 + G, kind)
    out, deq = _det_case(x, noise, bits)
    assert ulp_diff_f32(out.cpu().numpy(), deq.numpy()).max() <= 1


def test_constant_and_tiny_groups():
    x, noise = make_groups(4, 6, 256, torch.float32, 3)
    x[0, 0] = 0.0          # all-zero group (post-ReLU dead channel): range 0
    x[1, 2] = 5.5          # constant group
    x[2, 3] = x[2, 3] * 1e-7
    out, deq = _det_case(x, noise, [2, 1, 8, 4])
    assert ulp_diff_f32(out.cpu().numpy(), deq.numpy()).max() <= 1


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_sixteen_bit_inputs(dtype):
    bits = [1, 2, 3, 4, 5, 6, 7, 8]
    x, noise = make_groups(len(bits), 9, 256, dtype, 21, "relu")
    out, deq = _det_case(x, noise, bits)
    assert out.dtype == dtype
    assert np.array_equal(np_bits(out), np_bits(deq))


@pytest.mark.parametrize("gs", [32, 64, 128, 512])
def test_other_group_sizes(gs):
    bits = [1, 2, 3, 4, 5, 6, 7, 8]
    x, noise = make_groups(len(bits), 3, gs, torch.float32, gs)
    out, deq = _det_case(x, noise, bits)
    assert ulp_diff_f32(out.cpu().numpy(), deq.numpy()).max() <= 1


def _rng_pack(x, bits_list, seed):
    N, G, gs = x.shape
    xd = x.to(DEV)
    mn, mx = minmax_dev(xd)
    bits_dev, bits_host = bits_tensor(bits_list)
    torch.cuda.manual_seed(seed)
    gen = torch.cuda.default_generators[0]
    offset = gen.get_offset()
    packed, scale = ext_q.pack_mixed_precision(xd, mn, mx, bits_dev, True)
    assert gen.get_offset() == offset + 4          # the generator advances like a torch op
    return xd, mn, mx, bits_dev, bits_host, packed, scale, seed, offset


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("gs", [256, 64])
def test_rng_mode_matches_kernel_model(dtype, gs):
    bits = [1, 2, 3, 4, 5, 6, 7, 8, 2, 2]
    x, _ = make_groups(len(bits), 33, gs, dtype, 5, "chan")
    xd, mn, mx, bits_dev, bits_host, packed, scale, seed, offset = _rng_pack(x, bits, 1234)
    scale_o = kernel_mode.kernel_scale(mn.cpu(), mx.cpu(), bits_host.numpy())
    assert np.array_equal(np_bits(scale), np_bits(scale_o))
    codes = kernel_mode.rng_codes(x, mn.cpu(), scale_o, bits_host.numpy(), seed, offset)
    assert np.array_equal(packed.cpu().numpy(), layouts.pack_mixed(codes, bits_host.numpy()))
    out = ext_q.unpack_mixed_precision(packed, bits_dev, scale, mn, *x.shape)
    deq = kernel_mode.kernel_dequant(codes, scale_o, mn.cpu())
    assert np.array_equal(np_bits(out), np_bits(deq))


@pytest.mark.parametrize("bits", [1, 2, 4])
def test_rng_mode_unbiased_with_closed_form_variance(bits):
    # 10^4 independent roundings of the same 4 groups: replicate them as 10^4 samples
    trials, G = 10_000, 4
    base, _ = make_groups(1, G, 256, torch.float32, 77, "chan")
    x = base.expand(trials, G, 256).contiguous()
    xd, mn, mx, bits_dev, bits_host, packed, scale, seed, offset = _rng_pack(x, [bits] * trials, 99)
    out = ext_q.unpack_mixed_precision(packed, bits_dev, scale, mn, trials, G, 256)
    out64 = out.double().cpu().numpy()
    x64 = base.double().numpy()[0]
    rng_ = (mx - mn)[0].double().cpu().numpy()                         # [G,1]
    sc = scale[0].double().cpu().numpy()
    # unbiasedness: group-mean error over all trials below 1e-3 of the range
    err = out64.mean(axis=0) - x64                                     # [G,256]
    assert (np.abs(err.mean(axis=1, keepdims=True)) < 1e-3 * rng_).all()
    # per element: within 5 sigma of zero using the exact variance
    var_code = kernel_mode.code_variance(base, mn[:1].cpu(), scale[:1].cpu(), bits)[0]   # [G,256]
    sigma = np.sqrt(var_code / trials) / sc
    exp_bias = kernel_mode.expected_code(base, mn[:1].cpu(), scale[:1].cpu(), bits)[0] / sc \
        + mn[0].double().cpu().numpy() - x64
    assert (np.abs(err - exp_bias) <= 5 * sigma + 1e-6 * rng_).all()
    assert (np.abs(exp_bias) <= 2.0 ** -16 / sc + 1e-6 * rng_).all()  # the model itself is unbiased
    # per-group variance against the closed form sum f(1-f)/scale^2, within 5 %
    var_emp = out64.var(axis=0, ddof=1).sum(axis=1)
    var_ref = (var_code / sc ** 2).sum(axis=1)
    assert (np.abs(var_emp - var_ref) <= 0.05 * var_ref).all()
    # ActNN's bound: per-element variance <= R^2 / (4 B^2)   (qscheme.py:84)
    B = 2 ** bits - 1
    assert (out64.var(axis=0) <= (rng_ ** 2) / (4 * B * B) * 1.1 + 1e-12).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5, 6, 7, 8])
def test_rng_mode_criterion_on_every_dtype_and_width(dtype, bits):
    # 10^4 roundings of the same 4 groups; the codes are read back with the unpack kernel itself
    # (scale 1, min 0 in fp32: code / 1 + 0 is the code)
    trials, G = 10_000, 4
    base, _ = make_groups(1, G, 256, dtype, 70 + bits, "chan")
    x = base.expand(trials, G, 256).contiguous()
    xd, mn, mx, bits_dev, bits_host, packed, scale, seed, offset = _rng_pack(x, [bits] * trials, 31 + bits)
    ones = torch.ones(trials, G, 1, device=DEV)
    codes = ext_q.unpack_mixed_precision(packed, bits_dev, ones, torch.zeros_like(ones), trials, G, 256)
    assert codes.dtype == torch.float32 and float(codes.max()) <= 2 ** bits - 1 and float(codes.min()) >= 0
    assert_rng_tier(base, bits, codes, mn, scale)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("bits", [1, 2, 4, 8])
def test_rng_mode_mean_code_of_16bit_tensors(dtype, bits):
    # 16-bit tensors round with an 8-bit draw: over 4096 independent roundings the mean code of every
    # element is the model's expectation (within 5 sigma of its exact variance), and that
    # expectation is the exact (x - min) * scale to within 2^-9 of a level
    trials, G = 4096, 2
    base, _ = make_groups(1, G, 256, dtype, 78, "chan")
    x = base.expand(trials, G, 256).contiguous()
    xd, mn, mx, bits_dev, bits_host, packed, scale, seed, offset = _rng_pack(x, [bits] * trials, 17)
    codes = layouts.unpack_mixed(packed.cpu().numpy(), bits_host.numpy(), trials, G, 256)
    mean = codes.astype(np.float64).mean(axis=0)
    expect = kernel_mode.expected_code(base, mn[:1].cpu(), scale[:1].cpu(), bits)[0]
    sigma = np.sqrt(kernel_mode.code_variance(base, mn[:1].cpu(), scale[:1].cpu(), bits)[0] / trials)
    assert (np.abs(mean - expect) <= 5 * sigma + 1e-9).all()
    exact = (base.double() - mn[:1].double().cpu()).numpy()[0] * scale[0].double().cpu().numpy()
    exact = np.minimum(exact, 2 ** bits - 1)
    assert (np.abs(expect - exact) <= 2.0 ** -9 + 2.0 ** -12).all()
    # the criterion of the RNG mode - mean error below 1e-3 of the range - per group, measured and
    # in expectation (one level is 1 / (2^bits - 1) of the range)
    B = 2 ** bits - 1
    assert (np.abs((mean - exact).mean(axis=1)) / B < 1e-3).all()
    assert (np.abs((expect - exact).mean(axis=1)) / B < 2e-4).all()


def test_streams_of_different_calls_differ():
    x, _ = make_groups(4, 8, 256, torch.float32, 1)
    a = _rng_pack(x, [2] * 4, 5)[5]
    xd = x.to(DEV)
    mn, mx = minmax_dev(xd)
    bits_dev, _ = bits_tensor([2] * 4)
    b, _ = ext_q.pack_mixed_precision(xd, mn, mx, bits_dev, True)     # offset advanced by the first call
    assert not torch.equal(a, b)


def test_argument_checks():
    x, _ = make_groups(2, 2, 256, torch.float32, 1)
    xd = x.to(DEV)
    mn, mx = minmax_dev(xd)
    bits_dev, _ = bits_tensor([2, 2])
    with pytest.raises(RuntimeError):
        ext_q.pack_mixed_precision(xd, mn, mx, bits_dev, False)              # stochastic must be true
    with pytest.raises(RuntimeError):
        ext_q.pack_mixed_precision(xd.view(4, 256), mn, mx, bits_dev, True)  # rank
    with pytest.raises(RuntimeError):
        ext_q.pack_mixed_precision(xd, mn, mx, bits_dev.float(), True)       # bits dtype
    with pytest.raises(RuntimeError):
        ext_q.pack_mixed_precision(x, mn, mx, bits_dev, True)                # host tensor
    with pytest.raises(RuntimeError):
        ext_q.pack_mixed_precision(xd, mn, mx, bits_tensor([2, 9])[0], True) # width out of range
    # bits without an attached host copy still work (one device->host sync)
    plain_bits = torch.tensor([3, 1], dtype=torch.int32, device=DEV)
    p, s = ext_q.pack_mixed_precision(xd, mn, mx, plain_bits, True)
    assert p.numel() == 4 * 2 * 256 // 32
