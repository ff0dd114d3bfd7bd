"""Exhaustive check of the 16-bit dequantisation arithmetic: for EVERY f16 / bf16 scale bit
pattern and every 8-bit code, unpack must equal (scalar_t)code / scale + min computed with true
divisions on the host (one rounding per operation, quantization_cuda_kernel.cu:171)."""
import numpy as np
import pytest
import torch

import actnn_amd.cpp_extension.quantization as ext_q
from oracle import layouts
from _util import DEV, bits_tensor, np_bits

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("mn_value", [0.0, -1.3125, 117.0])
def test_every_scale_and_code(dtype, mn_value):
    N, G, gs = 256, 256, 256                       # 65536 groups: one per 16-bit pattern
    scale = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dtype).view(N, G, 1)
    mn = torch.full((N, G, 1), mn_value, dtype=dtype)
    codes = np.broadcast_to(np.arange(256, dtype=np.int32), (N, G, gs))      # element d carries code d
    words = layouts.pack_mixed(codes, [8] * N)
    bits_dev, _ = bits_tensor([8] * N)
    out = ext_q.unpack_mixed_precision(torch.from_numpy(words).to(DEV), bits_dev, scale.to(DEV), mn.to(DEV), N, G, gs)
    q = torch.arange(256, dtype=torch.float32).to(dtype).view(1, 1, gs)
    ref = (q / scale + mn).to(dtype)               # torch CPU: one rounding per operation
    got, exp = np_bits(out), np_bits(ref)
    nan = torch.isnan(ref).numpy()
    assert np.array_equal(np.isnan(out.float().cpu().numpy()), nan)
    assert np.array_equal(got[~nan], exp[~nan])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_single_precision_path_uses_the_same_arithmetic(dtype):
    N, G, gs = 8, 64, 256
    g_ = torch.Generator().manual_seed(3)
    scale = (torch.rand(N, G, 1, generator=g_) * 50 + 1e-3).to(dtype)
    mn = torch.randn(N, G, 1, generator=g_).to(dtype)
    codes = torch.randint(0, 256, (N, G, gs), generator=g_, dtype=torch.int32)
    packed = torch.from_numpy(layouts.pack_single(codes.numpy(), 8))
    out = ext_q.unpack_single_precision(packed.to(DEV), 8, scale.to(DEV), mn.to(DEV), N, G, gs)
    ref = (codes.to(dtype) / scale + mn).to(dtype)
    assert np.array_equal(np_bits(out), np_bits(ref))
