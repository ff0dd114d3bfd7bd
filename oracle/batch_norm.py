"""Training-mode batch normalisation, forward and backward, in float64 (test infrastructure).

The reference does not implement batch norm itself: `batch_norm.forward` / `.backward`
(actnn/actnn/ops.py:436-502) call cuDNN through at::cudnn_batch_norm and
at::cudnn_batch_norm_backward (cpp_extension/backward_func.cc:87-88; cuDNN is a third-party
library that is not part of the reference's tree and is unpinned by it).  This file restates the
published algorithm (Ioffe & Szegedy 2015, the spatial mode both libraries document): statistics
per channel over the batch and all positions, biased variance for normalisation, unbiased
variance into the running estimate, and the closed-form gradient.

Pinned by torch's own `F.batch_norm` and autograd on CPU (tests/test_oracle_batch_norm.py), which
is also what the reference's own test compares its layer with (tests/test_conv_layer.py and
test_bn_correctness against torch modules).
"""
import numpy as np


def _moments(x):
    x = np.asarray(x, np.float64)
    axes = (0,) + tuple(range(2, x.ndim))
    shape = (1, -1) + (1,) * (x.ndim - 2)
    mean = x.mean(axes)
    var = ((x - mean.reshape(shape)) ** 2).mean(axes)
    return x, axes, shape, mean, var


def forward(x, weight, bias, running_mean, running_var, momentum, eps):
    """-> (y, save_mean, save_invstd, new_running_mean, new_running_var), all float64."""
    x, axes, shape, mean, var = _moments(x)
    invstd = 1.0 / np.sqrt(var + eps)
    w = np.ones_like(mean) if weight is None else np.asarray(weight, np.float64)
    b = np.zeros_like(mean) if bias is None else np.asarray(bias, np.float64)
    y = (x - mean.reshape(shape)) * (invstd * w).reshape(shape) + b.reshape(shape)
    count = x.size / x.shape[1]
    new_rm = new_rv = None
    if running_mean is not None:
        new_rm = (1.0 - momentum) * np.asarray(running_mean, np.float64) + momentum * mean
    if running_var is not None:
        unbiased = var * (count / (count - 1.0)) if count > 1 else var
        new_rv = (1.0 - momentum) * np.asarray(running_var, np.float64) + momentum * unbiased
    return y, mean, invstd, new_rm, new_rv


def backward(x, grad_out, weight, eps):
    """-> (grad_input, grad_weight, grad_bias), float64: with xhat = (x - mean) * invstd,
    grad_bias = sum(dy), grad_weight = sum(dy * xhat),
    grad_input = weight * invstd * (dy - mean(dy) - xhat * mean(dy * xhat))."""
    x, axes, shape, mean, var = _moments(x)
    dy = np.asarray(grad_out, np.float64)
    invstd = 1.0 / np.sqrt(var + eps)
    w = np.ones_like(mean) if weight is None else np.asarray(weight, np.float64)
    xhat = (x - mean.reshape(shape)) * invstd.reshape(shape)
    grad_bias = dy.sum(axes)
    grad_weight = (dy * xhat).sum(axes)
    count = x.size / x.shape[1]
    grad_input = (w * invstd).reshape(shape) * (
        dy - (grad_bias / count).reshape(shape) - xhat * (grad_weight / count).reshape(shape))
    return grad_input, grad_weight, grad_bias


def forward_eval(x, weight, bias, running_mean, running_var, eps):
    """Evaluation mode -> (y, mean, invstd): the running estimates are the statistics
    (ops.py:458-461 hands this case to at::native_batch_norm with training = false)."""
    x = np.asarray(x, np.float64)
    shape = (1, -1) + (1,) * (x.ndim - 2)
    mean = np.asarray(running_mean, np.float64)
    invstd = 1.0 / np.sqrt(np.asarray(running_var, np.float64) + eps)
    w = np.ones_like(mean) if weight is None else np.asarray(weight, np.float64)
    b = np.zeros_like(mean) if bias is None else np.asarray(bias, np.float64)
    return (x - mean.reshape(shape)) * (invstd * w).reshape(shape) + b.reshape(shape), mean, invstd


def backward_eval(x, grad_out, weight, running_mean, running_var, eps):
    """Evaluation mode -> (grad_input, grad_weight, grad_bias): the statistics are constants, so
    grad_input = dy * weight * invstd, grad_weight = sum(dy * xhat), grad_bias = sum(dy)."""
    x = np.asarray(x, np.float64)
    dy = np.asarray(grad_out, np.float64)
    axes = (0,) + tuple(range(2, x.ndim))
    shape = (1, -1) + (1,) * (x.ndim - 2)
    mean = np.asarray(running_mean, np.float64)
    invstd = 1.0 / np.sqrt(np.asarray(running_var, np.float64) + eps)
    w = np.ones_like(mean) if weight is None else np.asarray(weight, np.float64)
    xhat = (x - mean.reshape(shape)) * invstd.reshape(shape)
    return dy * (w * invstd).reshape(shape), (dy * xhat).sum(axes), dy.sum(axes)
