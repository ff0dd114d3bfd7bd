"""Autograd functions that keep their input compressed between forward and backward, and the
quantise / dequantise glue around the kernels (behaviour of the reference's
actnn/actnn/ops.py:22-629; sync_batch_norm across ranks is not part of this build).
"""
import functools
import math

import torch
import torch.nn.functional as F
from torch.autograd.function import Function
from torch.nn.modules.utils import _pair, _single, _triple

from .conf import config
from .cpp_extension import backward_func as ext_backward_func
from .cpp_extension import quantization as ext_quantization
from .utils import (channels_last_format, compute_tensor_bytes, empty_cache, get_memory_usage,
                    logical_order, memory_order, swap_to_cpu, swap_to_device)


# ------------------------------------------------------------------------------------------
# quantise / dequantise
# ------------------------------------------------------------------------------------------
def quantize_and_pack(data, bits, mn, mx):
    """data [N,G,gs] -> (packed stream or simulated codes, scale [N,G,1])  (ops.py:22-52)."""
    if config.simulate:
        # the reference's pure-torch quantiser, run on the tensor's own device (ops.py:23-41)
        N = data.shape[0]
        if isinstance(bits, int):
            bits = torch.ones(N, dtype=torch.int32, device=data.device) * bits
        B = (2 ** bits - 1).view(N, 1, 1)
        mn = mn - 1e-6
        mx = mx + 1e-6
        scale = B / (mx - mn)
        output = (data - mn) * scale
        if config.stochastic:
            output.add_(output.new(output.shape).uniform_(-0.5, 0.5))
        output = F.relu(output)
        output = torch.min(output, B.float()).round_().int()
        return output, scale
    pack = ext_quantization.pack_single_precision if isinstance(bits, int) \
        else ext_quantization.pack_mixed_precision
    output, scale = pack(data, mn, mx, bits, config.stochastic)
    if config.swap:
        output = swap_to_cpu(output)
    return output, scale


def dequantize_and_unpack(data, shape, bits, scale, mn):
    """Inverse of quantize_and_pack; returns [N, G, gs] in the dtype of scale (ops.py:55-74)."""
    if config.simulate:
        return data / scale + mn
    if config.swap:
        data = swap_to_device(data)
    N = shape[0]
    gs = config.group_size
    features = math.prod(shape[1:])
    features = features + (gs - features % gs) % gs
    unpack = ext_quantization.unpack_single_precision if isinstance(bits, int) \
        else ext_quantization.unpack_mixed_precision
    return unpack(data, bits, scale, mn, N, features // gs, gs)


def no_scheme_compute_quantization_bits(input, known_minmax=None):
    """Fixed width for every sample when no scheme is attached (ops.py:77-96).  Always per-group
    ranges: `config.pergroup` is a rule of the schemes, this path of the reference never reads it."""
    from .qscheme import group_min_max
    N = input.shape[0]
    groups, mn, mx, _ = group_min_max(input, known_minmax, whole_tensor_range=False)
    return groups, config.activation_compression_bits[0], mn.view(N, -1, 1), mx.view(N, -1, 1)


def quantize_activation(input, scheme):
    """-> (q_input, q_bits, q_scale, q_min); for fp32 activations scale and min are kept as
    bfloat16 (ops.py:99-118)."""
    return finish_quantize(start_quantize(input, scheme))


def start_quantize(input, scheme, known_minmax=None):
    """First half of quantize_activation: everything up to the point where the per-sample widths
    are needed on the host.  The caller may launch other GPU work (the layer's forward) before
    calling finish_quantize, which hides the device->host round trip of the allocation.
    `known_minmax`: per-group (mn, mx) of `input` when another kernel has produced them already."""
    if not config.compress_activation:
        return ("raw", input)
    if scheme:
        return ("scheme", input.dtype, scheme, scheme.start_quantization_bits(input, known_minmax))
    return ("fixed", input.dtype, no_scheme_compute_quantization_bits(input, known_minmax))


def finish_quantize(started):
    if started[0] == "raw":
        input = started[1]
        return (swap_to_cpu(input) if config.swap else input), None, None, None
    if started[0] == "scheme":
        _, dtype, scheme, st = started
        groups, q_bits, q_min, mx = scheme.finish_quantization_bits(st)
    else:
        _, dtype, (groups, q_bits, q_min, mx) = started
    q_input, q_scale = quantize_and_pack(groups, q_bits, q_min, mx)
    if dtype == torch.float32:
        return q_input, q_bits, q_scale.to(torch.bfloat16), q_min.to(torch.bfloat16)
    return q_input, q_bits, q_scale, q_min


def dequantize_activation(quantized, q_input_shape):
    """Rebuild a tensor of shape q_input_shape (ops.py:121-139)."""
    if not config.compress_activation:
        ret = quantized[0]
        return swap_to_device(ret) if config.swap else ret
    q_input, q_bits, q_scale, q_min = quantized
    if q_scale.dtype == torch.bfloat16 and _stored_as_bf16(q_input_shape, quantized):
        q_scale = q_scale.to(torch.float32)
        q_min = q_min.to(torch.float32)
    out = dequantize_and_unpack(q_input, q_input_shape, q_bits, q_scale, q_min)
    N = q_input_shape[0]
    features = math.prod(q_input_shape[1:])
    out = out.view(N, -1)[:, :features]
    memory_format = getattr(quantized, "memory_format", None)
    if memory_format is not None:
        # saved in channels-last order: rebuild [N, ..., C] and hand out the channels-last view
        out = out.reshape(N, *q_input_shape[2:], q_input_shape[1])
        return logical_order(out.contiguous(), memory_format)
    return out.reshape(*q_input_shape).contiguous()


def _stored_as_bf16(shape, quantized):
    """True when bf16 scale/min are the compact storage of an fp32 activation (to be widened
    before unpacking, ops.py:129-131) rather than the native dtype of a bf16 activation - a case
    the reference, which knows f32/f16 only, never meets.  The saved tuple carries the marker."""
    return not getattr(quantized, "native_bf16", False)


class _Quantized(tuple):
    """(q_input, q_bits, q_scale, q_min) plus what the tuple cannot say: whether bf16 scale/min
    are the activation's own dtype, and the memory format the activation was compressed in."""
    native_bf16 = False
    memory_format = None


def quantize_saved(input, scheme):
    return finish_saved(start_quantize(input, scheme), input)


def quantize_on_device(input, scheme, known_minmax=None):
    """start_quantize + finish_saved behind one library call, for the case the layers meet at every
    step: a scheme whose widths are made on the device, whole groups of 256, per-group ranges,
    in-kernel stochastic rounding, nothing swapped.  -> the saved tuple, or None when the case is
    another one (the caller then takes the two halves; nothing has been launched).  Same kernels on
    the same generator state: the result is the two halves' bit for bit."""
    if not (scheme and config.fused_quantize and config.compress_activation and config.pergroup
            and config.stochastic and not config.simulate and not config.swap and config.group_size == 256):
        return None
    if not (input.is_cuda and input.dtype in ext_quantization.g.DTYPE_CODE and input.dim() >= 2):
        return None
    N = input.shape[0]
    fmt = channels_last_format(input)
    flat = (input.permute(0, *range(2, input.dim()), 1) if fmt is not None else input).reshape(N, -1)
    features = flat.shape[1]
    if N == 0 or features == 0 or features % 256 != 0 or not flat.is_contiguous():
        return None
    if known_minmax is not None:
        mn, mx = known_minmax
        if not (mn.dtype == input.dtype and mx.dtype == input.dtype and mn.numel() * 256 == input.numel()
                and mx.numel() == mn.numel() and mn.is_contiguous() and mx.is_contiguous()):
            known_minmax = None
    alloc = scheme.allocation_arguments(N, features // input.shape[1], input.device)
    if alloc is None:
        return None
    q_input, q_bits, q_scale, mn = ext_quantization.quantize_activation_device(
        flat.view(-1, 256), N, known_minmax, alloc)
    scheme.adopt_device_bits(q_bits, features, alloc)
    q_min = mn.view(N, -1, 1)
    if input.dtype == torch.float32:
        q_scale, q_min = q_scale.to(torch.bfloat16), q_min.to(torch.bfloat16)
    return _mark_saved(_Quantized((q_input, q_bits, q_scale, q_min)), input)


def _mark_saved(q, input):
    q.native_bf16 = input.dtype == torch.bfloat16
    q.memory_format = channels_last_format(input)
    return q


def finish_saved(started, input):
    return _mark_saved(_Quantized(finish_quantize(started)), input)


# ------------------------------------------------------------------------------------------
# convolution (1d / 2d / 3d share one implementation, ops.py:145-264)
# ------------------------------------------------------------------------------------------
conv_layer_ct = 0
bn_layer_ct = 0
total_act_mem = 0


def _conv_forward(ctx, forward_op, input, weight, bias, stride, padding, dilation, groups, scheme,
                  known_minmax=None):
    # min/max and sensitivities first, then the convolution itself, then the allocation and
    # the pack: the convolution runs while the sensitivities travel to the host
    if known_minmax is not None and (known_minmax[0].dtype != input.dtype
                                     or known_minmax[0].numel() * config.group_size != input.numel()):
        known_minmax = None                  # e.g. the input was cast on its way here
    quantized = quantize_on_device(input, scheme, known_minmax)
    if quantized is not None:
        output = forward_op(input, weight, bias, stride, padding, dilation, groups)
    else:
        started = start_quantize(input, scheme, known_minmax)
        output = forward_op(input, weight, bias, stride, padding, dilation, groups)
        quantized = finish_saved(started, input)
    ctx.scheme = scheme
    ctx.saved = quantized, weight, bias
    ctx.other_args = (input.shape, stride, padding, dilation, groups)
    empty_cache(config.empty_cache_threshold)
    if config.debug_memory_op_forward:
        global conv_layer_ct, total_act_mem
        print("========== conv forward %d ==========" % conv_layer_ct)
        get_memory_usage(True)
        conv_layer_ct += 1
        total_act_mem += compute_tensor_bytes(list(quantized))
        print("Act mem: %.2f MB" % (total_act_mem / 1024 ** 2))
    return output


def _conv_backward(ctx, grad_output, bias_reduce_dims, aug):
    if ctx.scheme:
        ctx.scheme.set_scale(grad_output)
    q_input_shape, stride, padding, dilation, groups = ctx.other_args
    padding, stride, dilation = aug(padding), aug(stride), aug(dilation)
    quantized, weight, bias = ctx.saved
    input = dequantize_activation(quantized, q_input_shape)
    memory_format = getattr(quantized, "memory_format", None) or torch.contiguous_format
    del quantized, ctx.saved
    empty_cache(config.empty_cache_threshold)
    grad_output = grad_output.contiguous(memory_format=memory_format)
    need = [ctx.needs_input_grad[0], ctx.needs_input_grad[1]]

    ws_mem = compute_tensor_bytes([grad_output, input, input]) if config.pipeline_threshold else 0
    if config.pipeline_threshold and ws_mem > config.pipeline_threshold and all(need):
        # micro-batched backward: grad_input overwrites the dequantised input chunk by chunk so
        # the transient working set stays bounded (ops.py:202-220)
        chunks = int((ws_mem + config.pipeline_threshold) // config.pipeline_threshold)
        grad_weight = None
        for x_i, g_i in zip(torch.chunk(input, chunks), torch.chunk(grad_output, chunks)):
            gi, gw = ext_backward_func.cudnn_convolution_backward(
                x_i, g_i, weight, padding, stride, dilation, groups,
                config.cudnn_benchmark_conv2d, False, False, need)
            x_i[:] = gi
            grad_weight = gw if grad_weight is None else grad_weight.add_(gw)
        grad_input = input
    else:
        grad_input, grad_weight = ext_backward_func.cudnn_convolution_backward(
            input, grad_output, weight, padding, stride, dilation, groups,
            config.cudnn_benchmark_conv2d, False, False, need)
    grad_bias = grad_output.sum(bias_reduce_dims) if bias is not None and ctx.needs_input_grad[2] else None
    if ctx.scheme:
        ctx.scheme.if_allocate_perlayer()
    return grad_input, grad_weight, grad_bias, None, None, None, None, None, None


class conv1d(Function):
    @staticmethod
    def forward(ctx, input, weight, bias=None, stride=1, padding=0, dilation=1, groups=1, scheme=None,
                known_minmax=None):
        return _conv_forward(ctx, F.conv1d, input, weight, bias, stride, padding, dilation, groups, scheme,
                             known_minmax)

    @staticmethod
    def backward(ctx, grad_output):
        return _conv_backward(ctx, grad_output, [0, 2], _single)


class conv2d(Function):
    @staticmethod
    def forward(ctx, input, weight, bias=None, stride=1, padding=0, dilation=1, groups=1, scheme=None,
                known_minmax=None):
        return _conv_forward(ctx, F.conv2d, input, weight, bias, stride, padding, dilation, groups, scheme,
                             known_minmax)

    @staticmethod
    def backward(ctx, grad_output):
        return _conv_backward(ctx, grad_output, [0, 2, 3], _pair)


class conv3d(Function):
    @staticmethod
    def forward(ctx, input, weight, bias=None, stride=1, padding=0, dilation=1, groups=1, scheme=None,
                known_minmax=None):
        return _conv_forward(ctx, F.conv3d, input, weight, bias, stride, padding, dilation, groups, scheme,
                             known_minmax)

    @staticmethod
    def backward(ctx, grad_output):
        return _conv_backward(ctx, grad_output, [0, 2, 3, 4], _triple)


# ------------------------------------------------------------------------------------------
# transposed convolution (ops.py:267-383): same saved-input handling, other backward call
# ------------------------------------------------------------------------------------------
def _conv_transpose_forward(ctx, forward_op, input, weight, bias, stride, padding, output_padding, groups,
                            dilation, scheme):
    started = start_quantize(input, scheme)
    output = forward_op(input, weight, bias, stride, padding, output_padding, groups, dilation)
    ctx.scheme = scheme
    ctx.saved = finish_saved(started, input), weight, bias
    ctx.other_args = (input.shape, stride, padding, output_padding, dilation, groups)
    empty_cache(config.empty_cache_threshold)
    return output


def _conv_transpose_backward(ctx, grad_output, bias_reduce_dims, aug):
    if ctx.scheme:
        ctx.scheme.set_scale(grad_output)
    q_input_shape, stride, padding, output_padding, dilation, groups = ctx.other_args
    padding, output_padding, stride, dilation = aug(padding), aug(output_padding), aug(stride), aug(dilation)
    quantized, weight, bias = ctx.saved
    input = dequantize_activation(quantized, q_input_shape)
    memory_format = getattr(quantized, "memory_format", None) or torch.contiguous_format
    del quantized, ctx.saved
    empty_cache(config.empty_cache_threshold)
    grad_output = grad_output.contiguous(memory_format=memory_format)
    grad_input, grad_weight = ext_backward_func.cudnn_convolution_transpose_backward(
        input, grad_output, weight, padding, output_padding, stride, dilation, groups,
        config.cudnn_benchmark_conv2d, False, False, [ctx.needs_input_grad[0], ctx.needs_input_grad[1]])
    grad_bias = grad_output.sum(bias_reduce_dims) if bias is not None and ctx.needs_input_grad[2] else None
    if ctx.scheme:
        ctx.scheme.if_allocate_perlayer()
    return grad_input, grad_weight, grad_bias, None, None, None, None, None, None


class conv_transpose1d(Function):
    @staticmethod
    def forward(ctx, input, weight, bias=None, stride=1, padding=0, output_padding=0, groups=1, dilation=1,
                scheme=None):
        return _conv_transpose_forward(ctx, F.conv_transpose1d, input, weight, bias, stride, padding,
                                       output_padding, groups, dilation, scheme)

    @staticmethod
    def backward(ctx, grad_output):
        return _conv_transpose_backward(ctx, grad_output, [0, 2], _single)


class conv_transpose2d(Function):
    @staticmethod
    def forward(ctx, input, weight, bias=None, stride=1, padding=0, output_padding=0, groups=1, dilation=1,
                scheme=None):
        return _conv_transpose_forward(ctx, F.conv_transpose2d, input, weight, bias, stride, padding,
                                       output_padding, groups, dilation, scheme)

    @staticmethod
    def backward(ctx, grad_output):
        return _conv_transpose_backward(ctx, grad_output, [0, 2, 3], _pair)


class conv_transpose3d(Function):
    @staticmethod
    def forward(ctx, input, weight, bias=None, stride=1, padding=0, output_padding=0, groups=1, dilation=1,
                scheme=None):
        return _conv_transpose_forward(ctx, F.conv_transpose3d, input, weight, bias, stride, padding,
                                       output_padding, groups, dilation, scheme)

    @staticmethod
    def backward(ctx, grad_output):
        return _conv_transpose_backward(ctx, grad_output, [0, 2, 3, 4], _triple)


# ------------------------------------------------------------------------------------------
# linear (ops.py:386-433)
# ------------------------------------------------------------------------------------------
def _fused_grad_weight_ok(quantized, shape, go):
    """The fused kernel takes a 2-D input saved in whole groups of 256 per row - as the fixed-width
    stream (levels L1 / L2, or any int width) or the per-sample stream of the schemes (L3 and up) -
    with 16-bit gradients (autocast, or a 16-bit model).  Every block of that kernel decodes the
    activation tile it multiplies, so a tile is decoded once per 256 output rows: that hides behind
    the matrix instructions for the 2-bit fixed-width stream (a table and byte permutes, 1.5
    instructions per value) and not for the others, which cost 2.8 - 3.5 times unpack + mm on
    [8192,4096]^T x [8192,4096].  By default only the former takes the fused kernel."""
    if not config.compress_activation or config.simulate or config.swap or not config.fused_linear_grad_weight:
        return False
    q_input, q_bits, q_scale, q_min = quantized
    every_stream = config.fused_linear_grad_weight == "always"
    if isinstance(q_bits, int):
        if q_bits not in (1, 2, 4, 8) or (q_bits != 2 and not every_stream):
            return False
    elif not (every_stream and isinstance(q_bits, torch.Tensor) and q_bits.dtype == torch.int32 and q_bits.is_cuda):
        return False
    return (len(shape) == 2 and shape[-1] % config.group_size == 0 and config.group_size == 256
            and go.shape[1] % 8 == 0 and go.dtype in (torch.float16, torch.bfloat16)
            and isinstance(q_input, torch.Tensor) and q_input.is_cuda)


class linear(Function):
    @staticmethod
    def forward(ctx, input, weight, bias=None, scheme=None):
        started = start_quantize(input, scheme)
        output = F.linear(input, weight, bias)
        quantized = finish_saved(started, input)
        empty_cache(config.empty_cache_threshold)
        ctx.scheme = scheme
        ctx.saved = quantized, weight, bias
        ctx.other_args = input.shape
        return output

    @staticmethod
    def backward(ctx, grad_output):
        if ctx.scheme:
            ctx.scheme.set_scale(grad_output)
        quantized, weight, bias = ctx.saved
        q_input_shape = ctx.other_args
        go = grad_output.reshape(-1, grad_output.shape[-1])
        if _fused_grad_weight_ok(quantized, q_input_shape, go):
            # the weight gradient is computed straight from the packed stream (dequantised tiles
            # only ever exist in LDS), nothing is materialised
            q_input, q_bits, q_scale, q_min = quantized
            if q_scale.dtype == torch.bfloat16 and _stored_as_bf16(q_input_shape, quantized):
                q_scale, q_min = q_scale.to(torch.float32), q_min.to(torch.float32)    # ops.py:129-131
            grad_weight = ext_quantization.linear_grad_weight(
                go, q_input, q_bits, q_scale, q_min, q_input_shape[-1], weight.dtype) \
                if ctx.needs_input_grad[1] else None
        else:
            input = dequantize_activation(quantized, q_input_shape)
            x = input.reshape(-1, input.shape[-1])
            grad_weight = go.t().mm(x) if ctx.needs_input_grad[1] else None
            del input, x
        del quantized, ctx.saved
        empty_cache(config.empty_cache_threshold)
        grad_input = go.mm(weight).view(*q_input_shape) if ctx.needs_input_grad[0] else None
        grad_bias = go.sum(0) if bias is not None and ctx.needs_input_grad[2] else None
        if ctx.scheme:
            ctx.scheme.if_allocate_perlayer()
        return grad_input, grad_weight, grad_bias, None


# ------------------------------------------------------------------------------------------
# batch norm (ops.py:436-502)
# ------------------------------------------------------------------------------------------
def _leaves_grad_sqnorm():
    """Batch-norm backward leaves the squared norm of its input gradient for the set_scale of the
    convolution before it (the statistic is one number per layer unless gradients are tracked per
    sample)."""
    from .qscheme import QScheme
    return config.share_grad_sqnorm and QScheme.update_scale and not config.use_gradient


def _bn_shares_min_max(input, weight, bias, running_mean, running_var, training):
    return (training and config.compress_activation and not config.simulate and config.group_size == 256
            and ext_backward_func.hip_batch_norm_minmax_applies(input, weight, bias, running_mean, running_var))


@functools.lru_cache(maxsize=64)
def _uniform_bits(N, bits, device):
    """int32 [N] on `device`, every sample `bits` wide, with its sum and prefix attached: the
    fixed-width schemes as a special case of the per-sample stream the fused kernels write."""
    q_bits = torch.full((N,), bits, dtype=torch.int32, device=device)
    ext_quantization.attach_bits_host(q_bits, torch.full((N,), bits, dtype=torch.int32))
    ext_quantization._bits_info(q_bits)
    return q_bits


def _bn_quantize_geometry(input, running_mean, running_var, weight, bias, training, scheme):
    """(N, C, HW, channels_last) when statistics -> widths -> normalise + pack can go through one
    library call for this input, else None."""
    if not (scheme and config.fused_quantize and config.fused_bn_pack and config.stochastic and training
            and config.compress_activation and config.pergroup and not config.simulate and not config.swap
            and config.group_size == 256):
        return None
    return ext_backward_func.hip_batch_norm_quantize_geometry(input, weight, bias, running_mean, running_var)


def batch_norm_relu_geometry(input, running_mean, running_var, weight, bias, training, scheme):
    """The geometry to hand to batch_norm_relu when the ReLU that follows the batch norm can be
    folded into its normalise + pack pass, else None (the caller then applies the two layers)."""
    from .qscheme import allocate_on_device
    if not config.fused_bn_relu:
        return None
    if not scheme:
        # one width for all (levels L1/L2): statistics, then normalise + pack with the ReLU folded in
        if not (_fixed_width() and config.fused_bn_pack and config.stochastic and not config.swap
                and _bn_shares_min_max(input, weight, bias, running_mean, running_var, training)):
            return None
        geo = ext_backward_func.hip_batch_norm_quantize_geometry(input, weight, bias, running_mean, running_var)
        return geo if geo is not None and ext_backward_func.hip_batch_norm_relu_applies(geo, input.dtype) else None
    geo = _bn_quantize_geometry(input, running_mean, running_var, weight, bias, training, scheme)
    if geo is None or not ext_backward_func.hip_batch_norm_relu_applies(geo, input.dtype):
        return None
    return geo if allocate_on_device(geo[0], scheme.initial_bits) else None


def _fixed_width():
    """True when activations are compressed at one configured width (no per-sample allocation)."""
    return (config.compress_activation and not config.simulate
            and isinstance(config.activation_compression_bits[0], int)
            and 1 <= config.activation_compression_bits[0] <= 8)


def _batch_norm_relu_forward(input, residual, running_mean, running_var, weight, bias, momentum, eps, scheme, geo):
    """-> (output, save_mean, save_invstd, saved tuple, mask, group min, group max of the output) of
    relu(bn(input) [+ residual]) for a `geo` of batch_norm_relu_geometry."""
    N = geo[0]
    if scheme:
        alloc = scheme.allocation_arguments(N, geo[2], input.device)
        (output, save_mean, save_var, mn, _mx, q_bits, q_input, q_scale, mask, out_mn,
         out_mx) = ext_backward_func.hip_batch_norm_forward_quantize(
            input, geo, weight, bias, running_mean, running_var, momentum, eps, alloc, relu=True, residual=residual)
        scheme.adopt_device_bits(q_bits, input.numel() // N, alloc)
    else:
        ws, save_mean, save_var, mn, mx = ext_backward_func.hip_batch_norm_forward_stats(
            input, weight, bias, running_mean, running_var, momentum, eps)
        q_bits = _uniform_bits(N, config.activation_compression_bits[0], input.device)
        output, q_input, q_scale, mask, out_mn, out_mx = ext_backward_func.hip_batch_norm_forward_apply(
            input, ws, q_bits, mn, mx, relu=True, residual=residual)
    quantized = _mark_saved(_Quantized((q_input, q_bits, q_scale, mn.view(N, -1, 1))), input)
    return output, save_mean, save_var, quantized, mask, out_mn, out_mx


class batch_norm(Function):
    @staticmethod
    def forward(ctx, input, running_mean, running_var, weight, bias, training,
                exponential_average_factor, eps, scheme, skip=None):
        """`skip` (a SkipGradient the caller also attaches to the output): when the output is the
        identity of a block's closing step, that step may leave its ReLU's mask and the gradient of
        its output there instead of returning the masked gradient."""
        ctx.skip = skip
        ctx.set_materialize_grads(False)
        fixed_width = not scheme and _fixed_width()
        # (the pass rounds stochastically, like pack_*; with config.stochastic off the unfused
        # sequence below is taken and pack_* refuses, as in the reference)
        fused = None
        # statistics -> widths -> normalise + pack behind one library call (the second branch below,
        # for a scheme whose widths are made on the device; same kernels, same generator state)
        geo = _bn_quantize_geometry(input, running_mean, running_var, weight, bias, training, scheme)
        alloc = scheme.allocation_arguments(geo[0], geo[2], input.device) if geo is not None else None
        if alloc is not None:
            fused = ext_backward_func.hip_batch_norm_forward_quantize(
                input, geo, weight, bias, running_mean, running_var, exponential_average_factor, eps, alloc)
        if fused is not None:
            output, save_mean, save_var, mn, mx, q_bits, q_input, q_scale = fused
            N = geo[0]
            scheme.adopt_device_bits(q_bits, input.numel() // N, alloc)
            q_min = mn.view(N, -1, 1)
            if input.dtype == torch.float32:
                q_scale, q_min = q_scale.to(torch.bfloat16), q_min.to(torch.bfloat16)
            reserve = None
            started = ("done", _mark_saved(_Quantized((q_input, q_bits, q_scale, q_min)), input))
        elif ((scheme or fixed_width) and config.fused_bn_pack and config.stochastic
                and _bn_shares_min_max(input, weight, bias, running_mean, running_var, training)
                and ext_backward_func.hip_batch_norm_pack_applies(input, weight, bias, running_mean, running_var)):
            # two reads of the input in total: the statistics pass also yields the quantiser's
            # per-group min/max, the widths are allocated from them, and the normalising pass
            # writes the packed copy of the input next to the output
            ws, save_mean, save_var, mn, mx = ext_backward_func.hip_batch_norm_forward_stats(
                input, weight, bias, running_mean, running_var, exponential_average_factor, eps)
            if scheme:
                _, q_bits, q_min, q_max = scheme.finish_quantization_bits(
                    scheme.start_quantization_bits(input, (mn, mx)))
            else:
                # no per-sample allocation (levels L1/L2): the same stream at one width for all
                N = input.shape[0]
                q_bits = _uniform_bits(N, config.activation_compression_bits[0], input.device)
                q_min, q_max = mn.view(N, -1, 1), mx.view(N, -1, 1)
            output, q_input, q_scale = ext_backward_func.hip_batch_norm_forward_apply(
                input, ws, q_bits, q_min, q_max)
            if input.dtype == torch.float32:
                # compact storage of an fp32 activation's scale and minimum (ops.py:115-116)
                q_scale, q_min = q_scale.to(torch.bfloat16), q_min.to(torch.bfloat16)
            if config.swap:
                q_input = swap_to_cpu(q_input)
            reserve = None
            started = ("done", _mark_saved(_Quantized((q_input, q_bits, q_scale, q_min)), input))
        elif _bn_shares_min_max(input, weight, bias, running_mean, running_var, training):
            # the statistics pass of the library's batch norm also yields the per-group min/max
            # the quantiser needs: one read of the input less
            output, save_mean, save_var, mn, mx = ext_backward_func.hip_batch_norm_forward(
                input, weight, bias, running_mean, running_var, exponential_average_factor, eps, minmax=True)
            reserve = None
            started = start_quantize(input, scheme, (mn, mx))
        elif training:
            started = start_quantize(input, scheme)
            output, save_mean, save_var, reserve = ext_backward_func.cudnn_batch_norm(
                input, weight, bias, running_mean, running_var, training, exponential_average_factor, eps)
        else:
            started = start_quantize(input, scheme)
            output, save_mean, save_var = ext_backward_func.native_batch_norm(
                input, weight, bias, running_mean, running_var, training, exponential_average_factor, eps)
            reserve = None
        quantized = started[1] if started[0] == "done" else finish_saved(started, input)
        empty_cache(config.empty_cache_threshold)
        if config.debug_memory_op_forward:
            global bn_layer_ct, total_act_mem
            print("========== bn forward %d ==========" % bn_layer_ct)
            get_memory_usage(True)
            bn_layer_ct += 1
            total_act_mem += compute_tensor_bytes(list(quantized))
            print("Act mem: %.2f MB" % (total_act_mem / 1024 ** 2))
        ctx.scheme = scheme
        ctx.other_args = input.shape
        ctx.saved = (quantized, weight, running_mean, running_var, save_mean, save_var, training, eps, reserve)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        skip, ctx.skip = ctx.skip, None
        grad, mask, fmt = skip.take() if skip is not None else (None, None, None)
        if grad is not None:
            if grad_output is None:
                # the output's only use was as that identity: the backward passes mask as they read
                return _batch_norm_backward(ctx, logical_order(grad, fmt), relu_mask=mask) + (None,)
            grad_output = grad_output + logical_order(ext_quantization.relu_backward(grad, mask), fmt)
        if grad_output is None:
            return (None,) * 10
        return _batch_norm_backward(ctx, grad_output) + (None,)


def _batch_norm_backward(ctx, grad_output, relu_mask=None):
    """`relu_mask`: the mask of a ReLU the batch norm's output went through (batch_norm_relu);
    `grad_output` is then the gradient of the ReLU's output, masked by the batch-norm passes as they
    read it where they can, else by the ReLU's own backward pass first."""
    quantized, weight, running_mean, running_var, save_mean, save_var, training, eps, reserve = ctx.saved

    def relu_backward_first(grad):
        fmt = getattr(quantized, "memory_format", None)
        grad = ext_quantization.relu_backward(memory_order(grad.contiguous(memory_format=fmt)), relu_mask)
        return logical_order(grad, fmt)

    if (training and config.compress_activation and not config.simulate
            and config.group_size == 256 and config.fused_bn_backward):
        if config.swap and isinstance(quantized[0], torch.Tensor) and not quantized[0].is_cuda:
            back = _Quantized((swap_to_device(quantized[0]),) + tuple(quantized[1:]))
            back.native_bf16, back.memory_format = quantized.native_bf16, quantized.memory_format
            quantized = back
        grad_output = grad_output.contiguous(
            memory_format=getattr(quantized, "memory_format", None) or torch.contiguous_format)
        if ext_backward_func.hip_batch_norm_backward_packed_applies(
                ctx.other_args, quantized, grad_output, weight, save_mean, save_var):
            # the kernels decode the saved input from its bit stream: no full-precision copy
            # (batch_norm_relu exists only for shapes whose passes take the mask)
            if relu_mask is not None and not config.fused_bn_relu_backward:
                grad_output, relu_mask = relu_backward_first(grad_output), None
            grads = ext_backward_func.hip_batch_norm_backward_packed(
                ctx.other_args, quantized, grad_output, weight, save_mean, save_var,
                sumsq=_leaves_grad_sqnorm(), relu_mask=relu_mask)
            del quantized, ctx.saved
            if ctx.scheme:
                ctx.scheme.if_allocate_perlayer()
            return grads[0], None, None, grads[1], grads[2], None, None, None, None
    if relu_mask is not None:
        grad_output = relu_backward_first(grad_output)
    input = dequantize_activation(quantized, ctx.other_args)
    memory_format = getattr(quantized, "memory_format", None) or torch.contiguous_format
    del quantized, ctx.saved
    empty_cache(config.empty_cache_threshold)
    if training:
        grad_input, grad_weight, grad_bias = ext_backward_func.cudnn_batch_norm_backward(
            input.contiguous(memory_format=memory_format),
            grad_output.contiguous(memory_format=memory_format), weight, running_mean, running_var,
            save_mean, save_var, eps, reserve, sumsq=_leaves_grad_sqnorm())
    else:
        grad_input, grad_weight, grad_bias = ext_backward_func.native_batch_norm_backward(
            grad_output, input, weight, running_mean, running_var, save_mean, save_var, training, eps,
            [ctx.needs_input_grad[0], ctx.needs_input_grad[3], ctx.needs_input_grad[4]])
    if ctx.scheme:
        ctx.scheme.if_allocate_perlayer()
    return grad_input, None, None, grad_weight, grad_bias, None, None, None, None


class batch_norm_relu(Function):
    """relu(batch_norm(input)) with the ReLU folded into the pass that normalises and packs: the
    normalised tensor is never written.  Saves what the two layers save - the compressed input and
    the ReLU's 1-bit mask - and returns the group min / max of the output beside it (not
    differentiable), as QReLU does.  Only for inputs batch_norm_relu_geometry accepts (`geo`)."""

    @staticmethod
    def forward(ctx, input, running_mean, running_var, weight, bias, training,
                exponential_average_factor, eps, scheme, geo):
        output, save_mean, save_var, quantized, mask, out_mn, out_mx = _batch_norm_relu_forward(
            input, None, running_mean, running_var, weight, bias, exponential_average_factor, eps, scheme, geo)
        empty_cache(config.empty_cache_threshold)
        ctx.scheme = scheme
        ctx.other_args = input.shape
        ctx.saved = (quantized, weight, running_mean, running_var, save_mean, save_var, training, eps, None)
        ctx.relu_mask = mask
        ctx.mark_non_differentiable(out_mn, out_mx)
        ctx.set_materialize_grads(False)
        return output, out_mn, out_mx

    @staticmethod
    def backward(ctx, grad_output, _grad_mn, _grad_mx):
        if grad_output is None:
            return (None,) * 10
        mask, ctx.relu_mask = ctx.relu_mask, None
        return _batch_norm_backward(ctx, grad_output, mask) + (None,)


class batch_norm_add_relu(Function):
    """relu(batch_norm(input) + residual) - the closing step of a residual block - in the batch norm's
    normalise + pack pass: neither the normalised tensor nor the sum is written.  Values, mask and
    gradients are those of the batch norm, the tensor addition and the ReLU one after the other.
    `residual` is laid out like `input` (same shape, dtype and memory format)."""

    @staticmethod
    def forward(ctx, input, residual, running_mean, running_var, weight, bias, training,
                exponential_average_factor, eps, scheme, geo, skip=None):
        ctx.skip = skip
        output, save_mean, save_var, quantized, mask, out_mn, out_mx = _batch_norm_relu_forward(
            input, residual, running_mean, running_var, weight, bias, exponential_average_factor, eps, scheme, geo)
        empty_cache(config.empty_cache_threshold)
        ctx.scheme = scheme
        ctx.other_args = input.shape
        ctx.saved = (quantized, weight, running_mean, running_var, save_mean, save_var, training, eps, None)
        ctx.relu_mask = mask
        ctx.mark_non_differentiable(out_mn, out_mx)
        ctx.set_materialize_grads(False)
        return output, out_mn, out_mx

    @staticmethod
    def backward(ctx, grad_output, _grad_mn, _grad_mx):
        if grad_output is None:
            return (None,) * 12
        fmt = ctx.saved[0].memory_format
        mask, ctx.relu_mask = ctx.relu_mask, None
        skip, ctx.skip = ctx.skip, None
        if (skip is not None and ctx.needs_input_grad[1] and config.fused_skip_gradient
                and skip.hand_over(memory_order(grad_output.contiguous(memory_format=fmt)), mask, fmt)):
            # the residual's producer takes it from there (skip_connection: the block's own input, whose
            # gradient - this one, masked - is added to the one from the block's first convolution in
            # one pass; batch_norm: the downsample branch, whose backward passes mask as they read),
            # and this batch norm masks what it reads itself
            grads = _batch_norm_backward(ctx, grad_output, relu_mask=mask)
            return (grads[0], None) + grads[1:] + (None, None)
        # the masked gradient is the residual's gradient, so it is written once and the batch norm reads it
        grad = logical_order(ext_quantization.relu_backward(
            memory_order(grad_output.contiguous(memory_format=fmt)), mask), fmt)
        grads = _batch_norm_backward(ctx, grad)
        return (grads[0], grad) + grads[1:] + (None, None)


class SkipGradient:
    """What the closing step of a residual block leaves for the block's input: the gradient of the
    block's output and the closing ReLU's mask.  Their product is the gradient that reaches the input
    over the skip connection."""

    __slots__ = ("grad", "mask", "memory_format")

    def __init__(self):
        self.grad = self.mask = self.memory_format = None

    def hand_over(self, grad, mask, memory_format):
        """False when something is already held (the tensor is the identity of two closing steps): the
        caller then returns its masked gradient the ordinary way."""
        if self.grad is not None:
            return False
        self.grad, self.mask, self.memory_format = grad, mask, memory_format
        return True

    def take(self):
        held = (self.grad, self.mask, self.memory_format)
        self.grad = self.mask = self.memory_format = None
        return held


class skip_connection(Function):
    """The input of a residual block, once for the block's layers and once for the skip connection.
    Autograd would add the two gradients that come back; here the closing step (batch_norm_add_relu)
    may leave the skip connection's gradient unmasked in `skip`, and masking and addition are one pass:
    the same values as relu_backward followed by the tensor addition."""

    @staticmethod
    def forward(ctx, input, skip):
        ctx.skip = skip
        ctx.set_materialize_grads(False)
        return input.view_as(input), input.view_as(input)

    @staticmethod
    def backward(ctx, grad_main, grad_skip):
        grad, mask, fmt = ctx.skip.take()
        total = grad_main
        if grad_skip is not None:
            total = grad_skip if total is None else total + grad_skip
        if grad is None:
            return total, None
        if total is None:
            return logical_order(ext_quantization.relu_backward(grad, mask), fmt), None
        other = memory_order(total.contiguous(memory_format=fmt))
        if other.dtype != grad.dtype or other.data_ptr() % 16:
            return total + logical_order(ext_quantization.relu_backward(grad, mask), fmt), None
        return logical_order(ext_quantization.relu_backward_add(grad, mask, other), fmt), None


class adaptive_avg_pool2d(Function):
    """Global average pool that keeps only the input's shape for the backward pass
    (ops.py:617-629); output size (1, 1) only, as there."""

    @staticmethod
    def forward(ctx, input, output_size):
        if tuple(output_size) != (1, 1):
            raise AssertionError("adaptive_avg_pool2d supports output_size (1, 1) only")
        ctx.saved = input.shape
        return torch.mean(input, dim=[2, 3], keepdim=True)

    @staticmethod
    def backward(ctx, grad_output):
        shape = ctx.saved
        return (grad_output / (shape[2] * shape[3])).expand(shape), None
