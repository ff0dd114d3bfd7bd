"""``calc_precision(b, C, w, target) -> b``: greedy bit allocation on CPU tensors; ``b`` is
modified in place and returned (reference: cpp_extension/calc_precision.cc:9-50).
``calc_precision_dp`` of the reference has no Python caller and is not provided."""
import torch

from . import _glue as g
from .._lib import check


def calc_precision(b, C, w, target):
    for t, name in ((b, "b"), (C, "C"), (w, "w")):
        if not (isinstance(t, torch.Tensor) and t.device.type == "cpu"):
            raise RuntimeError(f"{name} must be a CPU tensor!")           # calc_precision.cc:10-15
        if not t.is_contiguous():
            raise RuntimeError(f"{name} must be contiguous!")
    if b.dtype != torch.int32 or w.dtype != torch.int32 or C.dtype != torch.float32:
        raise RuntimeError("calc_precision expects b:int32, C:float32, w:int32")
    if not (b.numel() == C.numel() == w.numel()):
        raise RuntimeError("calc_precision: b, C and w must have the same length")
    check(g.lib().actnn_calc_precision(b.data_ptr(), C.data_ptr(), w.data_ptr(), b.numel(),
                                       float(target)), "calc_precision")
    return b
