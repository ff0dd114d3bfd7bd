"""Backward ATen entry points the reference re-exports (cpp_extension/backward_func.cc:81-91),
mapped onto the ATen ops that exist on PyTorch-ROCm (MIOpen behind them).  No new kernels:
this module only keeps the reference's names and argument order.

The three layer-norm exports of the reference have no Python caller and are not provided.
"""
import torch

_aten = torch.ops.aten


def cudnn_convolution_backward(input, grad_output, weight, padding, stride, dilation, groups,
                               benchmark, deterministic, allow_tf32, output_mask):
    """-> (grad_input, grad_weight).  at::cudnn_convolution_backward (backward_func.cc:82);
    benchmark / deterministic / allow_tf32 are cuDNN knobs with no MIOpen counterpart here."""
    gi, gw, _ = _aten.convolution_backward(
        grad_output, input, weight, None, list(stride), list(padding), list(dilation), False,
        [0] * len(stride), groups, [bool(output_mask[0]), bool(output_mask[1]), False])
    return gi, gw


def cudnn_convolution_transpose_backward(input, grad_output, weight, padding, output_padding, stride,
                                         dilation, groups, benchmark, deterministic, allow_tf32,
                                         output_mask):
    """-> (grad_input, grad_weight).  at::cudnn_convolution_transpose_backward (backward_func.cc:83)."""
    gi, gw, _ = _aten.convolution_backward(
        grad_output, input, weight, None, list(stride), list(padding), list(dilation), True,
        list(output_padding), groups, [bool(output_mask[0]), bool(output_mask[1]), False])
    return gi, gw


def cudnn_batch_norm(input, weight, bias, running_mean, running_var, training,
                     exponential_average_factor, epsilon):
    """-> (output, save_mean, save_var, reserve).  at::native::cudnn_batch_norm
    (backward_func.cc:87) -> miopen_batch_norm; `reserve` is an empty placeholder."""
    out, save_mean, save_var = _aten.miopen_batch_norm(
        input, weight, bias, running_mean, running_var, training, exponential_average_factor, epsilon)
    return out, save_mean, save_var, input.new_empty(0, dtype=torch.uint8)


def cudnn_batch_norm_backward(input, grad_output, weight, running_mean, running_var, save_mean,
                              save_var, epsilon, reserve):
    """-> (grad_input, grad_weight, grad_bias).  at::native::cudnn_batch_norm_backward
    (backward_func.cc:88) -> miopen_batch_norm_backward."""
    return _aten.miopen_batch_norm_backward(input, grad_output, weight, running_mean, running_var,
                                            save_mean, save_var, epsilon)


def native_batch_norm(input, weight, bias, running_mean, running_var, training, momentum, eps):
    """at::native_batch_norm (backward_func.cc:89)."""
    return _aten.native_batch_norm(input, weight, bias, running_mean, running_var, training, momentum, eps)


def native_batch_norm_backward(grad_out, input, weight, running_mean, running_var, save_mean,
                               save_invstd, train, eps, output_mask):
    """at::native_batch_norm_backward (backward_func.cc:90)."""
    return _aten.native_batch_norm_backward(grad_out, input, weight, running_mean, running_var,
                                            save_mean, save_invstd, train, eps, list(output_mask))
