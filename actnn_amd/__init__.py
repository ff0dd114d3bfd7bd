"""actnn_amd: MI355X-native activation-compressed training layers.

Same public names as the reference package (actnn/actnn/__init__.py:1-10); the kernels live in
libactnn_hip.so (include/actnn_hip.h) and there is no CPU fallback.
"""
from . import dataloader, ops  # noqa: F401
from .conf import config, set_optimization_level
from .layers import (AddReLU, QAddReLU, QAvgPool2d, QBatchNorm1d, QBatchNorm2d, QBatchNorm3d, QConv1d, QConv2d, QConv3d,
                     QConvTranspose1d, QConvTranspose2d, QConvTranspose3d, QDropout, QLinear, QMaxPool2d,
                     QReLU, QSyncBatchNorm)
from .module import QModule
from .qbnscheme import QBNScheme
from .qscheme import QScheme
from .utils import compute_tensor_bytes, exp_recorder, get_memory_usage

__all__ = ["config", "set_optimization_level", "QModule", "QScheme", "QBNScheme", "QConv1d", "QConv2d",
           "QConv3d", "QConvTranspose1d", "QConvTranspose2d", "QConvTranspose3d", "QLinear", "QBatchNorm1d", "QBatchNorm2d", "QBatchNorm3d", "QSyncBatchNorm", "QReLU", "QDropout",
           "AddReLU", "QAddReLU",
           "QMaxPool2d", "QAvgPool2d", "get_memory_usage", "compute_tensor_bytes", "exp_recorder", "ops",
           "dataloader"]
