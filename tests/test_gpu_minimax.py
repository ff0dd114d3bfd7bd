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
