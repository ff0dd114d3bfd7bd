"""``minimax(data) -> (min, max)``: row-wise min/max of a [M, D] device tensor
(reference: cpp_extension/minimax.cc:7-16)."""
import torch

from . import _glue as g
from .._lib import check


def minimax(data):
    g.check_float(data, "data")                        # minimax.cc:8
    if data.dim() != 2:
        raise RuntimeError("The dimension of data is not correct!")
    M, D = data.shape
    mn = torch.empty(M, dtype=data.dtype, device=data.device)
    mx = torch.empty(M, dtype=data.dtype, device=data.device)
    with torch.cuda.device(data.device):
        check(g.lib().actnn_minimax(data.data_ptr(), mn.data_ptr(), mx.data_ptr(), M, D,
                                    g.DTYPE_CODE[data.dtype], g.stream_ptr(data.device)), "minimax")
    return mn, mx
