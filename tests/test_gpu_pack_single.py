"""pack/unpack_single_precision parity (fixed width 1/2/4/8, 8/bits samples per byte)."""
import numpy as np
import pytest
import torch

import actnn_amd.cpp_extension.quantization as ext_q
from oracle import kernel_mode, layouts, simulate
from _util import DEV, assert_rng_tier, make_groups, minmax_dev, np_bits, ulp_diff_f32

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
@pytest.mark.parametrize("N", [1, 5, 8, 33])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_deterministic_mode_bit_exact(bits, N, dtype):
    G, gs = 7, 256
    x, noise = make_groups(N, G, gs, dtype, 100 * bits + N, "chan")
    xd = x.to(DEV)
    mn, mx = minmax_dev(xd)
    packed, scale = ext_q.pack_single_precision(xd, mn, mx, bits, True, noise=noise.to(DEV))
    mn_c, mx_c = x.min(dim=2, keepdim=True)[0], x.max(dim=2, keepdim=True)[0]
    codes, scale_o = simulate.quantize_simulate(x.clone(), bits, mn_c, mx_c, noise)
    ref = layouts.pack_single(codes.numpy(), bits)
    assert packed.dtype == torch.int8 and packed.numel() == ref.size == layouts.single_total_bytes(N, G, gs, bits)
    assert np.array_equal(np_bits(scale), np_bits(scale_o))
    wpt = 8 // bits
    live = (N + wpt - 1) // wpt * G * gs           # the trailing "+8 bits" byte is never written
    assert np.array_equal(packed.cpu().numpy()[:live], ref[:live])
    out = ext_q.unpack_single_precision(packed, bits, scale, mn, N, G, gs)
    deq = simulate.dequantize_simulate(codes, scale_o, mn_c)
    assert out.dtype == dtype
    if dtype == torch.float32:
        assert ulp_diff_f32(out.cpu().numpy(), deq.numpy()).max() <= 1
    assert np.array_equal(np_bits(out), np_bits(deq))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("bits", [1, 2, 4, 8])
@pytest.mark.parametrize("gs", [256, 64, 24, 8])
def test_rng_mode_matches_kernel_model(bits, gs, dtype):
    # (16-bit tensors: lanes share Philox calls when a group has an even number of octets - 256, 64 -
    # and draw their own otherwise - 24, 8; 6 samples leave the last byte's samples partly unused)
    N, G = 6, 5
    x, _ = make_groups(N, G, gs, dtype, bits, "chan")
    xd = x.to(DEV)
    mn, mx = minmax_dev(xd)
    torch.cuda.manual_seed(4321)
    offset = torch.cuda.default_generators[0].get_offset()
    packed, scale = ext_q.pack_single_precision(xd, mn, mx, bits, True)
    scale_o = kernel_mode.kernel_scale(mn.cpu(), mx.cpu(), bits)
    assert np.array_equal(np_bits(scale), np_bits(scale_o))
    codes = kernel_mode.rng_codes(x, mn.cpu(), scale_o, bits, 4321, offset)
    ref = layouts.pack_single(codes, bits)
    live = (N + 8 // bits - 1) // (8 // bits) * G * gs
    assert np.array_equal(packed.cpu().numpy()[:live], ref[:live])
    out = ext_q.unpack_single_precision(packed, bits, scale, mn, N, G, gs)
    assert np.array_equal(np_bits(out), np_bits(kernel_mode.kernel_dequant(codes, scale_o, mn.cpu())))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("bits", [1, 2, 4, 8])
def test_rng_mode_criterion_on_every_dtype_and_width(dtype, bits):
    # 10^4 roundings of the same 4 groups, codes read back with the unpack kernel (scale 1, min 0)
    trials, G = 10_000, 4
    base, _ = make_groups(1, G, 256, dtype, 40 + bits, "chan")
    xd = base.expand(trials, G, 256).contiguous().to(DEV)
    mn, mx = minmax_dev(xd)
    packed, scale = ext_q.pack_single_precision(xd, mn, mx, bits, True)
    ones = torch.ones(trials, G, 1, device=DEV)
    codes = ext_q.unpack_single_precision(packed, bits, ones, torch.zeros_like(ones), trials, G, 256)
    assert codes.dtype == torch.float32
    assert_rng_tier(base, bits, codes, mn, scale)


def test_rng_mode_unbiased():
    trials, G, bits = 4096, 2, 2
    base, _ = make_groups(1, G, 256, torch.float32, 8, "chan")
    xd = base.expand(trials, G, 256).contiguous().to(DEV)
    mn, mx = minmax_dev(xd)
    packed, scale = ext_q.pack_single_precision(xd, mn, mx, bits, True)
    out = ext_q.unpack_single_precision(packed, bits, scale, mn, trials, G, 256).double().cpu().numpy()
    rng_ = (mx - mn)[0].double().cpu().numpy()
    err = out.mean(axis=0) - base[0].double().numpy()
    assert (np.abs(err.mean(axis=1, keepdims=True)) < 1e-3 * rng_).all()


def test_argument_checks():
    x, _ = make_groups(4, 2, 256, torch.float32, 1)
    xd = x.to(DEV)
    mn, mx = minmax_dev(xd)
    for bad in (3, 5, 0, 16):
        with pytest.raises(RuntimeError):
            ext_q.pack_single_precision(xd, mn, mx, bad, True)        # 8 % bits != 0
    with pytest.raises(RuntimeError):
        ext_q.pack_single_precision(xd, mn, mx, 2, False)
    p, s = ext_q.pack_single_precision(xd, mn, mx, 2, True)
    with pytest.raises(RuntimeError):
        ext_q.unpack_single_precision(p.int(), 2, s, mn, 4, 2, 256)    # packed dtype
