"""QModule: wrap a model and swap its layers for the compressed-activation ones
(behaviour of the reference's actnn/actnn/module.py:14-100)."""
from collections import OrderedDict

import torch
import torch.nn as nn

from .conf import config
from .layers import (AddReLU, QAddReLU, QAvgPool2d, QBatchNorm1d, QBatchNorm2d, QBatchNorm3d, QConv1d, QConv2d, QConv3d,
                     QConvTranspose1d, QConvTranspose2d, QConvTranspose3d, QDropout, QLinear, QMaxPool2d,
                     QReLU, QSyncBatchNorm)

_Q_TYPES = (QConv1d, QConv2d, QConv3d, QConvTranspose1d, QConvTranspose2d, QConvTranspose3d, QBatchNorm1d,
            QBatchNorm2d, QBatchNorm3d, QSyncBatchNorm, QReLU, QAddReLU, QDropout, QLinear, QMaxPool2d, QAvgPool2d)


def _convert(child):
    """The replacement for one child module, or None to recurse into it.  As in the reference the
    new layer is built from the child's hyper-parameters only (fresh parameters)."""
    for conv, qconv in ((nn.Conv1d, QConv1d), (nn.Conv2d, QConv2d), (nn.Conv3d, QConv3d)):
        if isinstance(child, conv):
            return qconv(child.in_channels, child.out_channels, child.kernel_size, child.stride,
                         child.padding, child.dilation, child.groups, child.bias is not None,
                         child.padding_mode)
    for conv, qconv in ((nn.ConvTranspose1d, QConvTranspose1d), (nn.ConvTranspose2d, QConvTranspose2d),
                        (nn.ConvTranspose3d, QConvTranspose3d)):
        if isinstance(child, conv):
            return qconv(child.in_channels, child.out_channels, child.kernel_size, child.stride,
                         child.padding, child.output_padding, child.groups, child.bias is not None,
                         child.dilation, child.padding_mode)
    if config.enable_quantized_bn:
        for bn, qbn in ((nn.BatchNorm1d, QBatchNorm1d), (nn.BatchNorm2d, QBatchNorm2d),
                        (nn.BatchNorm3d, QBatchNorm3d)):
            if isinstance(child, bn):
                return qbn(child.num_features, child.eps, child.momentum, child.affine,
                           child.track_running_stats)
    if isinstance(child, nn.Linear):
        return QLinear(child.in_features, child.out_features, child.bias is not None)
    if isinstance(child, nn.ReLU):
        return QReLU()
    if isinstance(child, AddReLU):
        return QAddReLU()
    if isinstance(child, nn.Dropout):
        return QDropout(child.p)
    if isinstance(child, nn.MaxPool2d):
        return QMaxPool2d(child.kernel_size, child.stride, child.padding, child.dilation,
                          child.return_indices, child.ceil_mode)
    if isinstance(child, nn.AvgPool2d):
        return QAvgPool2d(child.kernel_size, child.stride, child.padding, child.ceil_mode,
                          child.count_include_pad, child.divisor_override)
    return None


class QModule(nn.Module):
    def __init__(self, model, channels_last=False):
        """`channels_last=True` (an addition to the reference's signature) keeps 4-D parameters
        and inputs in the channels-last layout, the one this GPU's convolution kernels work in; the
        Q-layers then compress activations in memory order without transposes."""
        super().__init__()
        self.model = model
        self.channels_last = bool(channels_last)
        QModule.convert_layers(model)
        if self.channels_last:
            self.model.to(memory_format=torch.channels_last)

    @staticmethod
    def convert_layers(module):
        for name, child in module.named_children():
            if isinstance(child, _Q_TYPES):
                continue
            new = _convert(child)
            if new is None:
                QModule.convert_layers(child)
            else:
                setattr(module, name, new)

    def forward(self, *args, **kwargs):
        if self.channels_last:
            args = tuple(a.contiguous(memory_format=torch.channels_last)
                         if isinstance(a, torch.Tensor) and a.dim() == 4 else a for a in args)
        return self.model(*args, **kwargs)

    def _apply(self, fn, recurse=True):
        # .to(device) / .half() of the wrapper must not undo the layout of the parameters
        ret = super()._apply(fn, recurse)
        if getattr(self, "channels_last", False):
            for p in self.model.parameters():
                if p.dim() == 4 and not p.is_contiguous(memory_format=torch.channels_last):
                    p.data = p.data.contiguous(memory_format=torch.channels_last)
        return ret

    def train(self, mode=True):
        config.training = mode
        return super().train(mode)

    def eval(self):
        config.training = False
        return super().eval()

    def load_state_dict(self, state_dict, strict=True):
        # checkpoints interchange with the unwrapped model: add the wrapper's "model." prefix
        return super().load_state_dict(OrderedDict(("model." + k, v) for k, v in state_dict.items()), strict)

    def state_dict(self, destination=None, prefix="", keep_vars=False):
        ret = super().state_dict(destination=destination, prefix=prefix, keep_vars=keep_vars)
        return OrderedDict((k[len("model."):], v) for k, v in ret.items())
