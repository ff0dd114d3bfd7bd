"""Fused 2-bit QLinear weight gradient vs torch's bf16 GEMM on the dequantised input
(benchmark config 4 tolerance: rtol 2e-2)."""
import pytest
import torch

import actnn_amd.cpp_extension.minimax as ext_minimax
import actnn_amd.cpp_extension.quantization as ext_q
from _util import DEV

pytestmark = pytest.mark.gpu


def _inputs(M, O, I, dtype, seed=0):
    g_ = torch.Generator(device=DEV).manual_seed(seed)
    # Student-t(3) heavy tails per feature, as in config 4
    z = torch.randn(M, I, generator=g_, device=DEV)
    chi = torch.randn(3, M, I, generator=g_, device=DEV).square().sum(0) / 3
    x = (z / chi.sqrt() * torch.rand(1, I, generator=g_, device=DEV)).to(dtype)
    go = torch.randn(M, O, generator=g_, device=DEV).to(dtype)
    G = I // 256
    xg = x.view(M, G, 256)
    mn, mx = ext_minimax.minimax(xg.view(-1, 256))
    return xg, go, mn.view(M, G, 1), mx.view(M, G, 1)


def _case(M, O, I, dtype, out_dtype, seed=0, bits=2):
    """-> (fused result, torch.mm(go.bf16().t(), dequantised.bf16())).  bits: an int (fixed-width
    stream) or a list of per-row widths (mixed-width stream)."""
    xg, go, mn, mx = _inputs(M, O, I, dtype, seed)
    G = I // 256
    if isinstance(bits, int):
        packed, scale = ext_q.pack_single_precision(xg, mn, mx, bits, True)
        deq = ext_q.unpack_single_precision(packed, bits, scale, mn, M, G, 256).view(M, I)
        gw = ext_q.linear_grad_weight(go, packed, bits, scale, mn, I, out_dtype)
    else:
        host = torch.tensor(bits, dtype=torch.int32)
        b = ext_q.attach_bits_host(host.to(DEV), host)
        packed, scale = ext_q.pack_mixed_precision(xg, mn, mx, b, True)
        deq = ext_q.unpack_mixed_precision(packed, b, scale, mn, M, G, 256).view(M, I)
        gw = ext_q.linear_grad_weight(go, packed, b, scale, mn, I, out_dtype)
    ref = torch.mm(go.bfloat16().t(), deq.bfloat16()).float()
    return gw, ref


def _check(gw, ref, dtype):
    # rtol 2e-2 (benchmark config 4) plus an absolute term for results that cancel to near zero: the
    # bf16 rounding noise of a K-term dot product scales with the typical magnitude of the results,
    # not with each result.  The reference operand is itself rounded to bf16 (2^-9 per term), so the
    # two sums differ by a few 1e-3 of the rms and the relative bound alone can only hold for results
    # above about a tenth of the rms: that is all but a Gaussian's central 10 % or so.
    err = (gw.float() - ref).abs()
    rms = ref.square().mean().sqrt()
    assert (err <= 2e-2 * ref.abs() + 4e-2 * rms).all(), float((err / (ref.abs() + 2 * rms)).max())
    assert float((err > 2e-2 * ref.abs()).float().mean()) < 0.15
    assert float(err.square().mean().sqrt() / rms) < 1e-2
    # and tighter on the whole: relative Frobenius error
    # (bf16 scale/min make the reference's own dequantisation round twice in bf16)
    assert (gw.float() - ref).norm() / ref.norm() < (5e-3 if dtype == torch.float16 else 1e-2)


@pytest.mark.parametrize("M,O,I", [(256, 256, 256), (512, 512, 1024), (100, 264, 512), (36, 8, 256),
                                   (2048, 1000, 2048), (512, 1000, 2048), (64, 256, 256), (130, 8, 256)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_matches_bf16_gemm(M, O, I, dtype):
    print(f"[linear_gw] fixed 2 bits M={M} O={O} I={I} {dtype}", flush=True)
    gw, ref = _case(M, O, I, dtype, dtype)
    assert gw.shape == (O, I) and gw.dtype == dtype
    _check(gw, ref, dtype)


@pytest.mark.parametrize("bits", [1, 4, 8])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_other_fixed_widths(bits, dtype):
    # levels L1 / L2 save 4 bits; rows that do not fill the last byte's samples (M % (8 / bits) != 0)
    for M, O, I in ((256, 256, 512), (37, 72, 256), (513, 1000, 2048)):
        print(f"[linear_gw] fixed {bits} bits M={M} O={O} I={I} {dtype}", flush=True)
        gw, ref = _case(M, O, I, dtype, dtype, seed=bits, bits=bits)
        _check(gw, ref, dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_mixed_width_stream(dtype):
    # what QScheme hands linear.backward at the default level: one width per row, here every
    # width from 1 to 8, the degenerate first-step allocation (8, ..., 8, 5, 1, ..., 1) and the
    # ResNet-50 classifier's shape at batch 512
    torch.manual_seed(0)
    for M, O, I in ((64, 256, 256), (200, 264, 768), (512, 1000, 2048)):
        bits = torch.randint(1, 9, (M,)).tolist()
        print(f"[linear_gw] mixed widths M={M} O={O} I={I} {dtype}", flush=True)
        gw, ref = _case(M, O, I, dtype, dtype, seed=M, bits=bits)
        _check(gw, ref, dtype)
    M = 256
    bits = [8] * 36 + [5] + [1] * 219
    gw, ref = _case(M, 512, 512, dtype, torch.float32, seed=3, bits=bits)
    assert gw.dtype == torch.float32
    _check(gw, ref, dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_few_tiles_and_many_rows_split_the_sum_over_blocks(dtype):
    # one to four output tiles and thousands of rows: the library asks for a workspace and splits
    # the sum over the rows (rows that do not fill the last split or the last 64-row step included)
    from actnn_amd import _lib
    lib = _lib.load()
    torch.manual_seed(1)
    for M, O, I, bits in ((8192, 256, 256, 2), (4096 + 37, 264, 512, 2), (6000, 128, 256, 4),
                          (5000, 256, 512, None), (3000, 72, 256, 1)):
        assert lib.actnn_linear_grad_weight_workspace_bytes(M, O, I) >= 2 * O * I * 4, (M, O, I)
        widths = bits if bits is not None else torch.randint(1, 9, (M,)).tolist()
        print(f"[linear_gw] split M={M} O={O} I={I} bits={bits} {dtype}", flush=True)
        gw, ref = _case(M, O, I, dtype, dtype, seed=M, bits=widths)
        _check(gw, ref, dtype)
    # shapes that fill the chip, or have too few rows to gain, stay unsplit
    assert lib.actnn_linear_grad_weight_workspace_bytes(8192, 4096, 4096) == 0
    assert lib.actnn_linear_grad_weight_workspace_bytes(512, 1000, 2048) == 0
    assert lib.actnn_linear_grad_weight_workspace_bytes(64, 256, 256) == 0


def test_split_sum_multiplies_the_same_values():
    # one-hot gradients over 4096 rows (split over blocks): every row of the dequantised input comes
    # out of the sum exactly, whichever block multiplied it
    from actnn_amd import _lib
    M, I = 4096, 256
    assert _lib.load().actnn_linear_grad_weight_workspace_bytes(M, 256, I) > 0
    xg, _, mn, mx = _inputs(M, 64, I, torch.bfloat16, seed=5)
    packed, scale = ext_q.pack_single_precision(xg, mn, mx, 2, True)
    deq = ext_q.unpack_single_precision(packed, 2, scale, mn, M, 1, 256).view(M, I)
    for first in (0, 1000, M - 256):
        go = torch.zeros(M, 256, device=DEV, dtype=torch.bfloat16)
        go[first:first + 256] = torch.eye(256, device=DEV, dtype=torch.bfloat16)
        gw = ext_q.linear_grad_weight(go, packed, 2, scale, mn, I, torch.float32)
        assert torch.equal(gw, deq[first:first + 256].float()), first


def test_fp32_output_and_config4_shape():
    gw, ref = _case(8192, 4096, 4096, torch.float16, torch.float32)
    assert gw.dtype == torch.float32
    assert (gw - ref).norm() / ref.norm() < 5e-3
    _check(gw, ref, torch.float16)


def test_activation_values_equal_the_unpack_kernel():
    # one-hot gradients pick single rows of the dequantised input out of the product: the values the
    # GEMM multiplies are bit for bit what unpack_single / unpack_mixed write (then exact in fp32)
    for dtype in (torch.float16, torch.bfloat16):
        for bits in (2, 4, [1, 2, 3, 4, 5, 6, 7, 8] * 8):
            M, I = 64, 512
            xg, _, mn, mx = _inputs(M, 64, I, dtype, seed=11)
            go = torch.eye(M, device=DEV, dtype=dtype)                      # O = M: grad_w[o] = row o of x
            if isinstance(bits, int):
                packed, scale = ext_q.pack_single_precision(xg, mn, mx, bits, True)
                deq = ext_q.unpack_single_precision(packed, bits, scale, mn, M, I // 256, 256).view(M, I)
                gw = ext_q.linear_grad_weight(go, packed, bits, scale, mn, I, torch.float32)
            else:
                host = torch.tensor(bits, dtype=torch.int32)
                b = ext_q.attach_bits_host(host.to(DEV), host)
                packed, scale = ext_q.pack_mixed_precision(xg, mn, mx, b, True)
                deq = ext_q.unpack_mixed_precision(packed, b, scale, mn, M, I // 256, 256).view(M, I)
                gw = ext_q.linear_grad_weight(go, packed, b, scale, mn, I, torch.float32)
            assert torch.equal(gw, deq.float()), (dtype, bits)


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
    with pytest.raises(RuntimeError):
        ext_q.linear_grad_weight(go, packed, 3, sc, sc, 256)               # 8 % bits
    with pytest.raises(RuntimeError):
        ext_q.linear_grad_weight(go, packed, torch.ones(8, dtype=torch.int32, device=DEV), sc, sc, 256)   # int8 stream, tensor bits
    out = ext_q.linear_grad_weight_q2(go, packed, sc, sc, 256)
    assert out.shape == (8, 256)
