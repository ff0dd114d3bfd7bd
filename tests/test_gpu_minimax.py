"""minimax kernel vs torch.min/max(dim=1), exact (the reference's own check,
tests/test_minimax.py:9-30)."""
import pytest
import torch

import actnn_amd.cpp_extension.minimax as ext_minimax
from _util import DEV

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,D", [(1024, 256), (1000, 256), (3, 256), (257, 512), (130, 128),
                                 (77, 64), (50, 100), (19, 40), (33, 7), (5, 2048)])
def test_minimax_exact(dtype, M, D):
    torch.manual_seed(M * 1000 + D)
    x = (torch.randn(M, D) * 3).to(dtype).to(DEV)
    mn, mx = ext_minimax.minimax(x)
    assert mn.dtype == dtype and mn.shape == (M,)
    assert torch.equal(mn, x.min(dim=1)[0])
    assert torch.equal(mx, x.max(dim=1)[0])


def test_minimax_large_and_constant_rows():
    x = torch.randn(200_000, 256, device=DEV)
    x[123] = 7.0
    x[456] = -0.0
    mn, mx = ext_minimax.minimax(x)
    assert torch.equal(mn, x.min(dim=1)[0]) and torch.equal(mx, x.max(dim=1)[0])
    assert mn[123] == 7.0 and mx[123] == 7.0


def test_minimax_rejects_bad_arguments():
    with pytest.raises(RuntimeError):
        ext_minimax.minimax(torch.randn(4, 256))                      # not a device tensor
    with pytest.raises(RuntimeError):
        ext_minimax.minimax(torch.randn(4, 512, device=DEV)[:, ::2])  # not contiguous
    with pytest.raises(RuntimeError):
        ext_minimax.minimax(torch.zeros(4, 256, dtype=torch.int32, device=DEV))
    mn, mx = ext_minimax.minimax(torch.empty(0, 256, device=DEV))
    assert mn.numel() == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("N,G", [(1, 1), (3, 7), (16, 784), (5, 3136)])
def test_range_sqr_matches_the_oracle(dtype, N, G):
    """Fused sensitivity kernel vs the oracle (float64 sum of the dtype-rounded differences), with
    no multiplier, a device scalar and one value per sample; fp32 summation order differs: 1e-5."""
    import numpy as np
    from oracle import kernel_mode
    g = torch.Generator().manual_seed(N * 1000 + G)
    mn = torch.randn(N * G, generator=g).to(dtype)
    mx = (mn.float() + torch.rand(N * G, generator=g) * 4).to(dtype)
    per = torch.rand(N, generator=g) + 0.5
    for mult in (None, per[:1].clone().view(()), per):
        out = ext_minimax.range_sqr(mn.to(DEV), mx.to(DEV), N, 0.37,
                                    None if mult is None else mult.to(DEV))
        assert out.dtype == torch.float32 and out.shape == (N,)
        to_np = (lambda t: t.numpy()) if dtype != torch.bfloat16 else None
        if dtype == torch.bfloat16:        # numpy has no bf16: round the difference with torch instead
            d = (mx - mn).float().numpy().astype(np.float64).reshape(N, G)
            exp = (d ** 2).sum(1) * 0.37
            if mult is not None:
                exp = exp * mult.numpy().astype(np.float64)
        else:
            exp = kernel_mode.range_sqr(to_np(mn).reshape(N, G), to_np(mx).reshape(N, G), 0.37,
                                        None if mult is None else mult.numpy())
        assert np.allclose(out.cpu().numpy(), exp, rtol=1e-5, atol=0)


def test_range_sqr_rejects_bad_arguments():
    mn = torch.zeros(8, device=DEV)
    with pytest.raises(RuntimeError):
        ext_minimax.range_sqr(mn, torch.zeros(9, device=DEV), 2)
    with pytest.raises(RuntimeError):
        ext_minimax.range_sqr(mn, mn, 2, 1.0, torch.ones(3, device=DEV))
    with pytest.raises(RuntimeError):
        ext_minimax.range_sqr(mn.int(), mn.int(), 2)
    assert ext_minimax.range_sqr(mn[:0], mn[:0], 0).numel() == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(4, 64, 56, 56), (3, 8, 5, 7), (16, 4096), (2, 3, 5, 5), (1, 16, 300, 301), (5, 24, 14, 14)])
def test_sample_sqnorm(dtype, shape):
    """Per-sample sum of squares against a float64 sum (fp32 accumulation: 1e-5 relative), for the
    default and the channels-last layout, and the ATen fallback for shapes without whole vectors."""
    g = torch.Generator(device=DEV).manual_seed(sum(shape))
    x = (torch.randn(*shape, generator=g, device=DEV) * 3).to(dtype)
    ref = x.double().reshape(shape[0], -1).square().sum(1)
    got = ext_minimax.sample_sqnorm(x)
    assert got.dtype == torch.float32 and got.shape == (shape[0],)
    assert torch.allclose(got.double(), ref, rtol=1e-5)
    if len(shape) == 4:
        got_cl = ext_minimax.sample_sqnorm(x.contiguous(memory_format=torch.channels_last))
        assert torch.allclose(got_cl.double(), ref, rtol=1e-5)
