"""Drop-in nn.Module layers that keep their saved activations compressed (behaviour of the
reference's actnn/actnn/layers.py; the sync-BN variant is not part of this build).

Under torch.autocast the custom autograd functions receive their floating-point arguments already
cast to the autocast dtype (autocast does not look inside custom Functions); the reference
predates autocast, this is the one addition here.
"""
import warnings

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch.nn.modules.pooling import _AvgPoolNd, _MaxPoolNd
from torch.nn.modules.utils import _pair, _single, _triple

from .conf import config
from .cpp_extension import quantization as ext_quantization
from .ops import (SkipGradient, batch_norm, batch_norm_add_relu, batch_norm_relu, batch_norm_relu_geometry, conv1d,
                  conv2d, conv3d, conv_transpose1d, conv_transpose2d, conv_transpose3d, linear)
from .ops import skip_connection as ops_skip_connection
from .qbnscheme import QBNScheme
from .qscheme import QScheme
from .utils import channels_last_format, logical_order, memory_order


def _autocast_apply(fn, *args):
    """Run fn.apply(*args); inside an autocast region cast float tensors to the autocast dtype
    first and switch autocast off for the call."""
    if torch.is_autocast_enabled("cuda"):
        dt = torch.get_autocast_dtype("cuda")
        args = tuple(a.to(dt) if isinstance(a, torch.Tensor) and a.is_floating_point() and a.is_cuda else a
                     for a in args)
        with torch.autocast(device_type="cuda", enabled=False):
            return fn.apply(*args)
    return fn.apply(*args)


def _relu_shares_min_max(x):
    return (config.share_relu_min_max and config.training and config.compress_activation and config.pergroup
            and not config.simulate and config.group_size == 256 and x.dim() >= 2
            and (x.numel() // max(x.shape[0], 1)) % 256 == 0 and ext_quantization.relu_minmax_applies(x))


def known_group_minmax(input):
    """(mn, mx) left on `input` by the layer that produced it, if they still describe it."""
    known = getattr(input, "_actnn_group_minmax", None)
    if known is None or known[2] != input._version or known[0].dtype != input.dtype \
            or known[0].numel() * 256 != input.numel():
        return None
    return known[0], known[1]


def _num_locations(kernel_size, dims):
    if isinstance(kernel_size, int):
        return kernel_size ** dims
    n = 1
    for k in kernel_size[:dims]:
        n *= k
    return n


class _QConvMixin:
    """Shared by QConv1d/2d/3d: scheme registration and the training-time dispatch."""
    _dims = 2
    _function = conv2d
    _zero_pad = staticmethod(_pair)

    def _init_scheme(self, kernel_size, groups, group):
        if config.adaptive_conv_scheme:
            self.scheme = QScheme(self, num_locations=_num_locations(kernel_size, self._dims), group=group,
                                  depthwise_groups=groups)
        else:
            self.scheme = None

    def forward(self, input):
        if not config.training:
            return super().forward(input)
        if self.padding_mode != "zeros":
            input = F.pad(input, self._reversed_padding_repeated_twice, mode=self.padding_mode)
            padding = self._zero_pad(0)
        elif isinstance(self.padding, str):
            # 'valid' / 'same': the backward operator wants integers.  nn.Conv*d has worked the
            # string out per side (last dimension first); a symmetric amount is passed on as the
            # convolution's own padding, an asymmetric one ('same' with an even extent) is applied
            # to the input beforehand, as torch's own convolution does.
            sides = self._reversed_padding_repeated_twice
            pairs = [(sides[2 * i], sides[2 * i + 1]) for i in range(self._dims)]
            if all(left == right for left, right in pairs):
                padding = tuple(left for left, _ in reversed(pairs))
            else:
                input = F.pad(input, sides)
                padding = self._zero_pad(0)
        else:
            padding = self.padding
        return _autocast_apply(self._function, input, self.weight, self.bias, self.stride, padding,
                               self.dilation, self.groups, self.scheme, known_group_minmax(input))


class QConv1d(_QConvMixin, nn.Conv1d):
    _dims, _function, _zero_pad = 1, conv1d, staticmethod(_single)

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1,
                 groups=1, bias=True, padding_mode="zeros", group=0):
        super().__init__(in_channels, out_channels, kernel_size, stride, padding, dilation, groups,
                         bias, padding_mode)
        self._init_scheme(kernel_size, groups, group)


class QConv2d(_QConvMixin, nn.Conv2d):
    _dims, _function, _zero_pad = 2, conv2d, staticmethod(_pair)

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1,
                 groups=1, bias=True, padding_mode="zeros", group=0):
        super().__init__(in_channels, out_channels, kernel_size, stride, padding, dilation, groups,
                         bias, padding_mode)
        self._init_scheme(kernel_size, groups, group)


class QConv3d(_QConvMixin, nn.Conv3d):
    _dims, _function, _zero_pad = 3, conv3d, staticmethod(_triple)

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1,
                 groups=1, bias=True, padding_mode="zeros", group=0):
        super().__init__(in_channels, out_channels, kernel_size, stride, padding, dilation, groups,
                         bias, padding_mode)
        self._init_scheme(kernel_size, groups, group)


class _QConvTransposeMixin:
    """Shared by QConvTranspose1d/2d/3d (layers.py:101-191)."""
    _dims = 2
    _function = conv_transpose2d

    def _init_scheme(self, kernel_size, groups, group):
        if config.adaptive_conv_scheme:
            self.scheme = QScheme(self, num_locations=_num_locations(kernel_size, self._dims), group=group,
                                  depthwise_groups=groups)
        else:
            self.scheme = None

    def forward(self, input, output_size=None):
        if not config.training:
            return super().forward(input, output_size)
        if self.padding_mode != "zeros":
            raise ValueError("Only `zeros` padding mode is supported for %s" % type(self).__name__)
        output_padding = self._output_padding(input, output_size, self.stride, self.padding, self.kernel_size,
                                              self._dims, self.dilation)
        return _autocast_apply(self._function, input, self.weight, self.bias, self.stride, self.padding,
                               output_padding, self.groups, self.dilation, self.scheme)


class QConvTranspose1d(_QConvTransposeMixin, nn.ConvTranspose1d):
    _dims, _function = 1, conv_transpose1d

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, output_padding=0,
                 groups=1, bias=True, dilation=1, padding_mode="zeros", group=0):
        super().__init__(in_channels, out_channels, kernel_size, stride, padding, output_padding, groups,
                         bias, dilation, padding_mode)
        self._init_scheme(kernel_size, groups, group)


class QConvTranspose2d(_QConvTransposeMixin, nn.ConvTranspose2d):
    _dims, _function = 2, conv_transpose2d

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, output_padding=0,
                 groups=1, bias=True, dilation=1, padding_mode="zeros", group=0):
        super().__init__(in_channels, out_channels, kernel_size, stride, padding, output_padding, groups,
                         bias, dilation, padding_mode)
        self._init_scheme(kernel_size, groups, group)


class QConvTranspose3d(_QConvTransposeMixin, nn.ConvTranspose3d):
    _dims, _function = 3, conv_transpose3d

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, output_padding=0,
                 groups=1, bias=True, dilation=1, padding_mode="zeros", group=0):
        super().__init__(in_channels, out_channels, kernel_size, stride, padding, output_padding, groups,
                         bias, dilation, padding_mode)
        self._init_scheme(kernel_size, groups, group)


class QLinear(nn.Linear):
    num_layers = 0

    def __init__(self, input_features, output_features, bias=True, group=0):
        super().__init__(input_features, output_features, bias)
        self.scheme = QScheme(self, group=group) if config.adaptive_conv_scheme else None

    def forward(self, input):
        if not config.training:
            return super().forward(input)
        return _autocast_apply(linear, input, self.weight, self.bias, self.scheme)


class _QBatchNormMixin:
    def _init_scheme(self, group):
        self.scheme = QBNScheme(group=group) if config.adaptive_bn_scheme else None

    def forward(self, input, relu=None, residual=None):
        """`relu`: the QReLU that follows this layer, when the caller hands the pair over together
        (bn_relu): where the shape allows, the ReLU is folded into the normalise + pack pass.
        `residual` with a QAddReLU as `relu` (bn_add_relu): relu(bn(input) + residual) likewise."""
        skip = getattr(residual, "_actnn_skip", None)
        if not config.training:
            out = super().forward(input)
            return out if relu is None else relu(out) if residual is None else relu(out, residual)
        self._check_input_dim(input)
        factor = 0.0 if self.momentum is None else self.momentum
        if self.training and self.track_running_stats and self.num_batches_tracked is not None:
            self.num_batches_tracked = self.num_batches_tracked + 1
            factor = 1.0 / float(self.num_batches_tracked) if self.momentum is None else self.momentum
        # batch statistics in training mode, and in eval mode when there are no running buffers
        bn_training = True if self.training else (self.running_mean is None and self.running_var is None)
        keep_buffers = (not self.training) or self.track_running_stats
        # statistics and affine parameters stay fp32 under autocast (mixed-precision batch norm)
        running_mean = self.running_mean if keep_buffers else None
        running_var = self.running_var if keep_buffers else None
        if relu is not None:
            geo = batch_norm_relu_geometry(input, running_mean, running_var, self.weight, self.bias, bn_training,
                                           self.scheme)
            if geo is not None and residual is not None and not (
                    config.fused_bn_add_relu and residual.shape == input.shape and residual.dtype == input.dtype and residual.device == input.device
                    and residual.is_contiguous(memory_format=torch.channels_last) and residual.data_ptr() % 16 == 0):
                geo = None
            if geo is not None:
                if residual is None:
                    out, mn, mx = batch_norm_relu.apply(input, running_mean, running_var, self.weight, self.bias,
                                                        bn_training, factor, self.eps, self.scheme, geo)
                else:
                    out, mn, mx = batch_norm_add_relu.apply(input, residual, running_mean, running_var, self.weight,
                                                            self.bias, bn_training, factor, self.eps, self.scheme, geo,
                                                            skip)
                if _relu_shares_min_max(memory_order(out)):
                    out._actnn_group_minmax = (mn, mx, out._version)
                return out
        if relu is None and config.fused_skip_gradient and input.is_cuda:
            # (should the output become the identity of a closing step, as a downsample branch's does)
            tie = SkipGradient()
            out = batch_norm.apply(input, running_mean, running_var, self.weight, self.bias, bn_training, factor,
                                   self.eps, self.scheme, tie)
            out._actnn_skip = tie
            return out
        out = batch_norm.apply(input, running_mean, running_var, self.weight, self.bias, bn_training, factor,
                               self.eps, self.scheme)
        return out if relu is None else relu(out) if residual is None else relu(out, residual)


class QBatchNorm1d(_QBatchNormMixin, nn.BatchNorm1d):
    def __init__(self, num_features, eps=1e-05, momentum=0.1, affine=True, track_running_stats=True, group=0):
        super().__init__(num_features, eps, momentum, affine, track_running_stats)
        self._init_scheme(group)


class QBatchNorm2d(_QBatchNormMixin, nn.BatchNorm2d):
    def __init__(self, num_features, eps=1e-05, momentum=0.1, affine=True, track_running_stats=True, group=0):
        super().__init__(num_features, eps, momentum, affine, track_running_stats)
        self._init_scheme(group)


class QBatchNorm3d(_QBatchNormMixin, nn.BatchNorm3d):
    def __init__(self, num_features, eps=1e-05, momentum=0.1, affine=True, track_running_stats=True, group=0):
        super().__init__(num_features, eps, momentum, affine, track_running_stats)
        self._init_scheme(group)


class QSyncBatchNorm(_QBatchNormMixin, nn.SyncBatchNorm):
    """nn.SyncBatchNorm with a compressed saved input (layers.py:383-462).  The statistics of one
    process need no exchange, and that is the case built here: without an initialised process
    group, or in a group of one rank, the layer is QBatchNorm on its own batch - the path the
    reference takes for world_size == 1 (layers.py:444-455).  Across ranks the reference gathers
    [mean, invstd, count] and reduces the two gradient sums (ops.py:519-526,585-588); this build
    runs on one GPU and raises instead of normalising with local statistics only."""

    def __init__(self, num_features, eps=1e-05, momentum=0.1, affine=True, track_running_stats=True,
                 process_group=None, group=0):
        super().__init__(num_features, eps, momentum, affine, track_running_stats, process_group)
        self._init_scheme(group)

    def forward(self, input):
        if not input.is_cuda:
            raise ValueError("SyncBatchNorm expected input tensor to be on GPU")
        uses_batch_statistics = self.training or (self.running_mean is None and self.running_var is None)
        if uses_batch_statistics and torch.distributed.is_available() and torch.distributed.is_initialized():
            group = self.process_group or torch.distributed.group.WORLD
            if torch.distributed.get_world_size(group) > 1:
                raise NotImplementedError("QSyncBatchNorm across ranks is not part of this single-GPU build")
        return super().forward(input)


class QReLU(nn.Module):
    """ReLU that saves a 1-bit mask; used in training and evaluation alike (layers.py:364-369)."""

    def __init__(self, inplace=False):
        super().__init__()

    def forward(self, input):
        # the mask follows memory order, so a channels-last activation needs no transposition
        fmt = channels_last_format(input)
        x = memory_order(input) if fmt is not None else input
        if _relu_shares_min_max(x):
            # the layer that compresses this output next (a convolution) finds the group min / max
            # on the tensor instead of reading it once more for them
            out, mn, mx = ext_quantization.ActQuantizedReLUMinMax.apply(x)
            out = logical_order(out, fmt) if fmt is not None else out
            out._actnn_group_minmax = (mn, mx, out._version)
            return out
        out = ext_quantization.act_quantized_relu(x)
        return logical_order(out, fmt) if fmt is not None else out


def bn_relu(bn, relu, input):
    """relu(bn(input)) for a model that knows the two layers follow each other: converted layers get
    the pair in one pass where the shape allows (the normalised tensor is then never written),
    everything else is the two calls."""
    if isinstance(bn, _QBatchNormMixin) and not isinstance(bn, QSyncBatchNorm) and type(relu) is QReLU:
        return bn(input, relu)
    return relu(bn(input))


def bn_add_relu(bn, add_relu, input, residual):
    """add_relu(bn(input), residual) = relu(bn(input) + residual), the closing step of a residual block,
    for a model that knows the layers follow each other: converted layers get the three in one pass
    where the shape allows, everything else is the two calls."""
    if isinstance(bn, _QBatchNormMixin) and not isinstance(bn, QSyncBatchNorm) and type(add_relu) is QAddReLU:
        return bn(input, add_relu, residual)
    return add_relu(bn(input), residual)


def skip_connection(add_relu, input):
    """(input for the block's layers, input for the skip connection) of a residual block that ends in
    bn_add_relu(bn, add_relu, ..., the second one).  With converted layers the two are tied so that the
    closing ReLU's backward and the addition of the two gradients of `input` become one pass; anything
    else gets `input` twice."""
    if (type(add_relu) is QAddReLU and config.training and config.fused_skip_gradient and input.is_cuda
            and input.requires_grad and torch.is_grad_enabled()):
        skip = SkipGradient()
        main, identity = ops_skip_connection.apply(input, skip)
        shared = getattr(input, "_actnn_group_minmax", None)
        if shared is not None and shared[2] == input._version:
            main._actnn_group_minmax = (shared[0], shared[1], main._version)
        identity._actnn_skip = skip
        return main, identity
    return input, input


class AddReLU(nn.Module):
    """relu(a + b): the closing step of a residual block as a module of its own, so that QModule can
    swap it for the fused layer below (plain torch here; the sum is a tensor of its own)."""

    def forward(self, a, b):
        return F.relu(a + b, inplace=True)


class QAddReLU(nn.Module):
    """relu(a + b) in one pass over the two operands, saving the 1-bit mask: the values and the mask
    of the addition followed by QReLU, without writing and re-reading the sum."""

    def __init__(self):
        super().__init__()
        self.relu = QReLU()

    def forward(self, a, b):
        fmt = channels_last_format(a)
        if fmt == channels_last_format(b):
            x, r = (memory_order(a), memory_order(b)) if fmt is not None else (a, b)
            if ext_quantization.add_relu_applies(x, r):
                if _relu_shares_min_max(x):
                    out, mn, mx = ext_quantization.ActQuantizedAddReLUMinMax.apply(x, r)
                    out = logical_order(out, fmt) if fmt is not None else out
                    out._actnn_group_minmax = (mn, mx, out._version)
                    return out
                out = ext_quantization.ActQuantizedAddReLU.apply(x, r)
                return logical_order(out, fmt) if fmt is not None else out
        return self.relu(a + b)


class QDropout(nn.Dropout):
    def __init__(self, p=0.5):
        super().__init__(p=p)

    def forward(self, input):
        if self.training:
            fmt = channels_last_format(input)
            if fmt is not None:
                return logical_order(ext_quantization.act_quantized_dropout(memory_order(input), self.p), fmt)
            return ext_quantization.act_quantized_dropout(input, self.p)
        return super().forward(input)


class QMaxPool2d(_MaxPoolNd):
    def __init__(self, kernel_size, stride=None, padding=0, dilation=1, return_indices=False, ceil_mode=False):
        super().__init__(kernel_size, stride, padding, dilation, return_indices, ceil_mode)
        self.kernel_size = _pair(kernel_size)
        self.stride = _pair(stride if stride is not None else kernel_size)
        self.padding = _pair(padding)
        self.dilation = _pair(dilation)

    def forward(self, input):
        if channels_last_format(input) is not None and not ext_quantization.pool_takes_channels_last(input):
            # channel counts the channels-last kernels do not take: transpose in and out so that
            # the model stays channels-last
            out = ext_quantization.act_quantized_max_pool2d(
                input.contiguous(), self.kernel_size, self.stride, self.padding, self.dilation,
                self.ceil_mode, self.return_indices, config.pool_index_nibbles)
            return out.contiguous(memory_format=torch.channels_last)
        return ext_quantization.act_quantized_max_pool2d(input, self.kernel_size, self.stride, self.padding,
                                                         self.dilation, self.ceil_mode, self.return_indices,
                                                         config.pool_index_nibbles)


class QAvgPool2d(_AvgPoolNd):
    """The reference has no average-pool kernel and silently runs max-pool instead
    (layers.py:506-515); that behaviour is kept, with its warning."""

    def __init__(self, kernel_size, stride=None, padding=0, ceil_mode=False, count_include_pad=True,
                 divisor_override=None):
        super().__init__()
        self.kernel_size = _pair(kernel_size)
        self.stride = _pair(stride if stride is not None else kernel_size)
        self.padding = _pair(padding)
        self.ceil_mode = ceil_mode
        self.count_include_pad = count_include_pad
        self.divisor_override = divisor_override

    def forward(self, input):
        warnings.warn("avg_pool2d is replaced by max_pool2d: no memory-saving average-pool kernel exists.")
        return ext_quantization.act_quantized_max_pool2d(input, self.kernel_size, self.stride, self.padding,
                                                         (1, 1), self.ceil_mode, False, config.pool_index_nibbles)
