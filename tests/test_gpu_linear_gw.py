"""Fused 2-bit QLinear weight gradient vs torch's bf16 GEMM on the dequantised input
(benchmark config 4 tolerance: rtol 2e-2)."""
import pytest
import torch

import actnn_amd.cpp_extension.minimax as ext_minimax
import actnn_amd.cpp_extension.quantization as ext_q
from _util import DEV

pytestmark = pytest.mark.gpu


def _case(M, O, I, dtype, out_dtype, seed=0):
    g_ = torch.Generator(device=DEV).manual_seed(seed)
    # Student-t(3) heavy tails per feature, as in config 4
    z = torch.randn(M, I, generator=g_, device=DEV)
    chi = torch.randn(3, M, I, generator=g_, device=DEV).square().sum(0) / 3
    x = (z / chi.sqrt() * torch.rand(1, I, generator=g_, device=DEV)).to(dtype)
    go = torch.randn(M, O, generator=g_, device=DEV).to(dtype)
    G = I // 256
    xg = x.view(M, G, 256)
    mn, mx = ext_minimax.minimax(xg.view(-1, 256))
    mn, mx = mn.view(M, G, 1), mx.view(M, G, 1)
    packed, scale = ext_q.pack_single_precision(xg, mn, mx, 2, True)
    deq = ext_q.unpack_single_precision(packed, 2, scale, mn, M, G, 256).view(M, I)
    gw = ext_q.linear_grad_weight_q2(go, packed, scale, mn, I, out_dtype)
    ref = torch.mm(go.bfloat16().t(), deq.bfloat16()).float()
    return gw, ref


@pytest.mark.parametrize("M,O,I", [(256, 256, 256), (512, 512, 1024), (100, 264, 512), (36, 8, 256),
                                   (2048, 1000, 2048)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_matches_bf16_gemm(M, O, I, dtype):
    gw, ref = _case(M, O, I, dtype, dtype)
    assert gw.shape == (O, I) and gw.dtype == dtype
    # rtol 2e-2 plus an absolute term for results that cancel to near zero: the bf16 rounding noise of
    # a K-term dot product scales with the typical magnitude of the results, not with each result
    err = (gw.float() - ref).abs()
    rms = ref.square().mean().sqrt()
    tol = 2e-2 * ref.abs() + 4e-2 * rms
    assert (err <= tol).all(), float((err / (ref.abs() + 2 * rms)).max())
    # and tighter on the whole: relative Frobenius error
    # (bf16 scale/min make the reference's own dequantisation round twice in bf16)
    assert (gw.float() - ref).norm() / ref.norm() < (5e-3 if dtype == torch.float16 else 1e-2)


def test_fp32_output_and_config4_shape():
    gw, ref = _case(8192, 4096, 4096, torch.float16, torch.float32)
    assert gw.dtype == torch.float32
    assert (gw - ref).norm() / ref.norm() < 5e-3
    err = (gw - ref).abs()
    assert (err <= 2e-2 * ref.abs() + 4e-2 * ref.square().mean().sqrt()).all()


def test_argument_checks():
    go = torch.randn(8, 8, device=DEV, dtype=torch.float16)
    packed = torch.zeros(8 * 256 // 4 + 1, dtype=torch.int8, device=DEV)
    sc = torch.ones(8, 1, 1, device=DEV, dtype=torch.float16)
    with pytest.raises(RuntimeError):
        ext_q.linear_grad_weight_q2(go.float(), packed, sc, sc, 256)       # grad_output dtype
    with pytest.raises(RuntimeError):
        ext_q.linear_grad_weight_q2(go, packed, sc, sc, 128)               # in_features % 256
    with pytest.raises(RuntimeError):
        ext_q.linear_grad_weight_q2(go[:6], packed, sc[:6], sc[:6], 256)   # M % 4
    out = ext_q.linear_grad_weight_q2(go, packed, sc, sc, 256)
    assert out.shape == (8, 256)
