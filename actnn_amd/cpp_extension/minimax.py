"""``minimax(data) -> (min, max)``: row-wise min/max of a [M, D] device tensor
(reference: cpp_extension/minimax.cc:7-16)."""
import torch

from . import _glue as g
from .._lib import check
from ..utils import channels_last_format


def minimax(data):
    g.check_float(data, "data")                        # minimax.cc:8
    if data.dim() != 2:
        raise RuntimeError("The dimension of data is not correct!")
    M, D = data.shape
    mn = torch.empty(M, dtype=data.dtype, device=data.device)
    mx = torch.empty(M, dtype=data.dtype, device=data.device)
    with g.on_device(data.device):
        check(g.lib().actnn_minimax(data.data_ptr(), mn.data_ptr(), mx.data_ptr(), M, D,
                                    g.DTYPE_CODE[data.dtype], g.stream_ptr(data.device)), "minimax")
    return mn, mx


def range_sqr(mn, mx, N, factor=1.0, mult=None):
    """fp32 [N]: factor * mult * sum over the groups of sample n of (mx - mn)^2, in one kernel
    (reference: the tensor expression of qscheme.py:80-82).  mn / mx: the [N * G] outputs of
    ``minimax``; mult: None, a 0-dim fp32 device tensor or an fp32 device tensor of N values."""
    g.check_float(mn, "min")
    if mx.dtype != mn.dtype or mx.shape != mn.shape or mn.numel() % max(N, 1) != 0:
        raise RuntimeError("range_sqr: min and max do not match")
    mn = mn.contiguous()
    mx = mx.contiguous()
    G = mn.numel() // N if N else 0
    out = torch.empty(N, dtype=torch.float32, device=mn.device)
    mult_ptr, per_sample = None, 0
    if mult is not None:
        if mult.dtype != torch.float32 or mult.device != mn.device or mult.numel() not in (1, N):
            raise RuntimeError("range_sqr: mult must be fp32 on the same device with 1 or N values")
        mult = mult.contiguous()
        mult_ptr, per_sample = mult.data_ptr(), int(mult.numel() == N and N != 1)
    with g.on_device(mn.device):
        check(g.lib().actnn_range_sqr(mn.data_ptr(), mx.data_ptr(), out.data_ptr(), N, G, float(factor),
                                      mult_ptr, per_sample, g.DTYPE_CODE[mn.dtype], g.stream_ptr(mn.device)),
              "range_sqr")
    return out


def sample_sqnorm(x):
    """fp32 [N]: squared L2 norm of every sample of a dense tensor (any layout: the sum does not
    care about the order), one pass at memory speed."""
    N = x.shape[0]
    F = x.numel() // max(N, 1)
    elems = 16 // x.element_size()
    dense = x.is_contiguous() or channels_last_format(x) is not None
    if (N == 0 or N > 65535 or F % elems != 0 or x.dtype not in g.DTYPE_CODE or not x.is_cuda
            or not dense or x.data_ptr() % 16 != 0):
        return torch.linalg.vector_norm(x.reshape(N, -1), dim=1, dtype=torch.float32).square()
    slices = max(1, min(64, F // 8192))
    part = torch.empty(N, slices, dtype=torch.float32, device=x.device)
    with g.on_device(x.device):
        check(g.lib().actnn_sample_sqnorm(x.data_ptr(), part.data_ptr(), N, F, slices,
                                          g.DTYPE_CODE[x.dtype], g.stream_ptr(x.device)), "sample_sqnorm")
    return part.sum(1) if slices > 1 else part.view(N)
