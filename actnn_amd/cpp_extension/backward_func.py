"""Backward ATen entry points the reference re-exports (cpp_extension/backward_func.cc:81-91),
under the reference's names and argument order.  The convolutions map onto the ATen ops that
exist on PyTorch-ROCm (MIOpen behind them); batch norm - training and evaluation mode, any dense
shape in the default or the channels-last layout, [N, C] inputs included - runs this library's
own kernels (actnn_batch_norm_*) and falls back to ATen only for tensors that are not dense or
whose affine parameters are not fp32.

The three layer-norm exports of the reference have no Python caller and are not provided.
"""
import functools

import torch

from . import _glue
from ..utils import channels_last_format

_aten = torch.ops.aten


def _shape_geometry(shape, dtype, channels_last):
    """(N, C, HW) when the library's batch-norm kernels take a tensor of this shape, else None."""
    return _geometry_of(tuple(int(d) for d in shape), dtype, bool(channels_last))


@functools.lru_cache(maxsize=4096)
def _geometry_of(shape, dtype, channels_last):
    # asked several times per layer and step with the same few shapes: remembered
    if len(shape) < 2 or dtype not in _glue.DTYPE_CODE:
        return None
    N, C = shape[0], shape[1]
    HW = 1
    for d in shape[2:]:
        HW *= d
    if N * C * HW == 0 or _workspace_bytes(N, C, HW, _glue.DTYPE_CODE[dtype], int(channels_last)) < 0:
        return None
    return N, C, HW


@functools.lru_cache(maxsize=4096)
def _workspace_bytes(N, C, HW, code, channels_last):
    return _glue.lib().actnn_batch_norm_workspace_bytes(N, C, HW, code, channels_last)


@functools.lru_cache(maxsize=4096)
def _sumsq_entries(N, C, HW, code, channels_last):
    return _glue.lib().actnn_batch_norm_backward_sumsq_entries(N, C, HW, code, channels_last)


def _leave_sumsq(grad_input, table):
    """Attach the partial sums of grad_input^2 that the backward pass left, for the layer that
    receives this gradient next (QScheme.set_scale); the version pins them to these contents."""
    grad_input._actnn_sumsq = (table, grad_input._version)


def known_sumsq(grad):
    """Total of grad^2 as a 0-d fp32 tensor if the kernel that wrote `grad` left it, else None."""
    left = getattr(grad, "_actnn_sumsq", None)
    if left is None or left[1] != grad._version:
        return None
    return left[0].sum()


def _bn_geometry(input):
    """(N, C, HW, channels_last) of a dense tensor in the default or the channels-last layout."""
    if not (isinstance(input, torch.Tensor) and input.is_cuda):
        return None
    channels_last = channels_last_format(input) is not None
    if not channels_last and not input.is_contiguous():
        return None
    geo = _shape_geometry(input.shape, input.dtype, channels_last)
    return None if geo is None else geo + (channels_last,)


def _f32_or_none(t):
    return t is None or (t.dtype == torch.float32 and t.is_cuda and t.is_contiguous())


def hip_batch_norm_applies(input, weight, bias, running_mean, running_var):
    return (_bn_geometry(input) is not None and input.data_ptr() % 16 == 0
            and all(_f32_or_none(t) for t in (weight, bias, running_mean, running_var)))


@functools.lru_cache(maxsize=4096)
def _groups_align(N, C, HW, code, channels_last):
    """Groups of 256 elements (in memory order) coincide with runs of threads of the streaming
    kernels: the group min/max, the packed copy and the packed backward exist for the shape."""
    return bool(_glue.lib().actnn_batch_norm_groups_align(N, C, HW, code, int(channels_last)))


def hip_batch_norm_minmax_applies(input, weight, bias, running_mean, running_var):
    """True when the forward pass can also return the quantiser's per-group min/max."""
    if not hip_batch_norm_applies(input, weight, bias, running_mean, running_var):
        return False
    N, C, HW, channels_last = _bn_geometry(input)
    return _groups_align(N, C, HW, _glue.DTYPE_CODE[input.dtype], channels_last)


def _ptr(t):
    return None if t is None else t.data_ptr()


def hip_batch_norm_forward(input, weight, bias, running_mean, running_var, momentum, eps, minmax=False):
    """-> (output, save_mean, save_invstd, mn, mx): training-mode batch norm; with `minmax` the
    minimum and maximum of every group of 256 elements of a sample that are consecutive in memory
    come out of the same pass over the input (None, None otherwise)."""
    N, C, HW, channels_last = _bn_geometry(input)
    lib = _glue.lib()
    code = _glue.DTYPE_CODE[input.dtype]
    ws_bytes = _workspace_bytes(N, C, HW, code, int(channels_last))
    ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device=input.device)
    out = torch.empty_like(input)                       # same strides as the input
    save_mean = torch.empty(C, dtype=torch.float32, device=input.device)
    save_invstd = torch.empty(C, dtype=torch.float32, device=input.device)
    mn = mx = None
    if minmax:
        groups = N * C * HW // 256
        mn = torch.empty(groups, dtype=input.dtype, device=input.device)
        mx = torch.empty(groups, dtype=input.dtype, device=input.device)
    with _glue.on_device(input.device):
        _glue._lib.check(lib.actnn_batch_norm_forward(
            input.data_ptr(), _ptr(weight), _ptr(bias), _ptr(running_mean), _ptr(running_var),
            out.data_ptr(), save_mean.data_ptr(), save_invstd.data_ptr(), _ptr(mn), _ptr(mx),
            ws.data_ptr(), ws_bytes, N, C, HW, float(momentum), float(eps), code, int(channels_last),
            _glue.stream_ptr(input.device)), "batch_norm_forward")
    return out, save_mean, save_invstd, mn, mx


def hip_batch_norm_forward_stats(input, weight, bias, running_mean, running_var, momentum, eps, minmax=True):
    """First half of the forward pass -> (workspace, save_mean, save_invstd, mn, mx); the workspace
    carries the per-channel coefficients to hip_batch_norm_forward_apply."""
    N, C, HW, channels_last = _bn_geometry(input)
    lib = _glue.lib()
    code = _glue.DTYPE_CODE[input.dtype]
    ws_bytes = _workspace_bytes(N, C, HW, code, int(channels_last))
    ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device=input.device)
    save_mean = torch.empty(C, dtype=torch.float32, device=input.device)
    save_invstd = torch.empty(C, dtype=torch.float32, device=input.device)
    mn = mx = None
    if minmax:
        groups = N * C * HW // 256
        mn = torch.empty(groups, dtype=input.dtype, device=input.device)
        mx = torch.empty(groups, dtype=input.dtype, device=input.device)
    with _glue.on_device(input.device):
        _glue._lib.check(lib.actnn_batch_norm_forward_stats(
            input.data_ptr(), _ptr(weight), _ptr(bias), _ptr(running_mean), _ptr(running_var),
            save_mean.data_ptr(), save_invstd.data_ptr(), _ptr(mn), _ptr(mx), ws.data_ptr(), ws_bytes,
            N, C, HW, float(momentum), float(eps), code, int(channels_last),
            _glue.stream_ptr(input.device)), "batch_norm_forward_stats")
    return ws, save_mean, save_invstd, mn, mx


def hip_batch_norm_forward_apply(input, workspace, bits=None, mn=None, mx=None, relu=False, residual=None):
    """Second half -> (output, packed, scale).  With `bits` (int32 [N] on the device) and the group
    min/max, the pass also quantises the input: `packed` and `scale` are what
    pack_mixed_precision(groups of input, mn, mx, bits, True) returns for the same generator state.
    With `relu` (packing only, hip_batch_norm_relu_applies) the output is relu(bn(input)) -
    relu(bn(input) + residual) with a `residual` laid out like the input - and the tuple ends with
    the ReLU's mask and the group min / max of the output."""
    from .quantization import _bits_info, mask_words
    N, C, HW, channels_last = _bn_geometry(input)
    lib = _glue.lib()
    code = _glue.DTYPE_CODE[input.dtype]
    out = torch.empty_like(input)
    packed = scale = prefix = None
    seed = offset = 0
    if bits is not None:
        G = C * HW // 256
        total, prefix = _bits_info(bits)
        packed = torch.empty(total * G * 8, dtype=torch.int32, device=input.device)
        scale = torch.empty(N, G, 1, dtype=input.dtype, device=input.device)
        seed, offset = _glue.philox_args(input.device)
    if relu:
        if bits is None:
            raise RuntimeError("the ReLU is folded into the packing pass only")
        mask = torch.empty(mask_words(N * C * HW), dtype=torch.int32, device=input.device)
        zmn = torch.empty(N * G, dtype=input.dtype, device=input.device)
        zmx = torch.empty(N * G, dtype=input.dtype, device=input.device)
        with _glue.on_device(input.device):
            _glue._lib.check(lib.actnn_batch_norm_forward_apply_relu(
                input.data_ptr(), out.data_ptr(), workspace.data_ptr(), workspace.numel() * 4, _ptr(bits),
                _ptr(prefix), _ptr(mn), _ptr(mx), _ptr(scale), _ptr(packed), seed, offset, mask.data_ptr(),
                zmn.data_ptr(), zmx.data_ptr(), _ptr(residual), N, C, HW, code, int(channels_last),
                _glue.stream_ptr(input.device)), "batch_norm_forward_apply_relu")
        return out, packed, scale, mask, zmn, zmx
    with _glue.on_device(input.device):
        _glue._lib.check(lib.actnn_batch_norm_forward_apply(
            input.data_ptr(), out.data_ptr(), workspace.data_ptr(), workspace.numel() * 4, _ptr(bits),
            _ptr(prefix), _ptr(mn), _ptr(mx), _ptr(scale), _ptr(packed), seed, offset, N, C, HW, code,
            int(channels_last), _glue.stream_ptr(input.device)), "batch_norm_forward_apply")
    return out, packed, scale


def hip_batch_norm_quantize_geometry(input, weight, bias, running_mean, running_var):
    """(N, C, HW, channels_last) when statistics, group min/max and the packed copy can all come from
    the fused passes (what hip_batch_norm_minmax_applies and hip_batch_norm_pack_applies ask, looked
    up once), else None."""
    geo = _bn_geometry(input)
    if geo is None or input.data_ptr() % 16 != 0:
        return None
    if not (_f32_or_none(weight) and _f32_or_none(bias) and _f32_or_none(running_mean) and _f32_or_none(running_var)):
        return None
    N, C, HW, channels_last = geo
    if not _groups_align(N, C, HW, _glue.DTYPE_CODE[input.dtype], channels_last):
        return None
    if channels_last and N * HW >= 2 ** 31:
        return None
    return geo


def hip_batch_norm_relu_applies(geo, dtype):
    """True when the normalise + pack pass can also apply the ReLU that follows the batch norm:
    channels-last 16-bit tensors whose waves own whole 512-element blocks of the mask (rows of a
    divisor of 256 channels) or the same half of two (rows of a multiple of 512), in whole steps."""
    N, C, HW, channels_last = geo
    return (channels_last and dtype in (torch.float16, torch.bfloat16)
            and ((C <= 256 and 256 % C == 0) or C % 512 == 0) and (N * HW) % (2048 // min(C, 256)) == 0)


def hip_batch_norm_forward_quantize(input, geo, weight, bias, running_mean, running_var, momentum, eps, alloc,
                                    relu=False, residual=None):
    """Statistics + group min/max -> widths on the device -> normalise + pack, in one call:
    -> (output, save_mean, save_invstd, mn, mx, bits, packed, scale), what
    hip_batch_norm_forward_stats, allocate_bits_device and hip_batch_norm_forward_apply return one
    after the other.  `geo` from hip_batch_norm_quantize_geometry, `alloc` the scheme's
    AllocationArgs (factor, mult, initial, target, total, sens_out).  With `relu`
    (hip_batch_norm_relu_applies) the output is relu(bn(input)) - relu(bn(input) + residual) with a
    `residual` laid out like the input - and the tuple ends with the ReLU's mask and the group
    min / max of the output."""
    from .quantization import attach_bits_total, mask_words
    N, C, HW, channels_last = geo
    dev, dtype = input.device, input.dtype
    code = _glue.DTYPE_CODE[dtype]
    ws_bytes = _workspace_bytes(N, C, HW, code, int(channels_last))
    G = C * HW // 256
    f32, i32 = torch.float32, torch.int32
    ws = torch.empty(ws_bytes // 4, dtype=f32, device=dev)
    save_mean = torch.empty(C, dtype=f32, device=dev)
    save_invstd = torch.empty(C, dtype=f32, device=dev)
    mn = torch.empty(N * G, dtype=dtype, device=dev)
    mx = torch.empty(N * G, dtype=dtype, device=dev)
    out = torch.empty_like(input)
    sens = alloc.sens_out if alloc.sens_out is not None else torch.empty(N, dtype=f32, device=dev)
    bits = torch.empty(N, dtype=i32, device=dev)
    prefix = torch.empty(N + 1, dtype=i32, device=dev)
    packed = torch.empty(alloc.total * G * 8, dtype=i32, device=dev)
    scale = torch.empty(N, G, 1, dtype=dtype, device=dev)
    mask = zmn = zmx = None
    if relu:
        mask = torch.empty(mask_words(N * C * HW), dtype=i32, device=dev)
        zmn = torch.empty(N * G, dtype=dtype, device=dev)
        zmx = torch.empty(N * G, dtype=dtype, device=dev)
    mult, mult_ptr, per_sample = _mult_args(alloc.mult, N, dev)          # (`mult` held until the launch)
    seed, offset = _glue.philox_args(dev)
    with _glue.on_device(dev):
        _glue._lib.check(_glue.lib().actnn_batch_norm_forward_quantize(
            input.data_ptr(), _ptr(weight), _ptr(bias), _ptr(running_mean), _ptr(running_var), out.data_ptr(),
            save_mean.data_ptr(), save_invstd.data_ptr(), mn.data_ptr(), mx.data_ptr(), ws.data_ptr(), ws_bytes,
            alloc.factor, mult_ptr, per_sample, sens.data_ptr(), bits.data_ptr(), prefix.data_ptr(),
            alloc.initial, alloc.target, scale.data_ptr(), packed.data_ptr(), seed, offset, _ptr(mask), _ptr(zmn),
            _ptr(zmx), _ptr(residual), N, C, HW, float(momentum), float(eps), code, int(channels_last),
            _glue.stream_ptr(dev)),
            "batch_norm_forward_quantize")
    attach_bits_total(bits, alloc.total, prefix)
    if relu:
        return out, save_mean, save_invstd, mn, mx, bits, packed, scale, mask, zmn, zmx
    return out, save_mean, save_invstd, mn, mx, bits, packed, scale


def _mult_args(mult, N, dev):
    """(tensor, pointer, per-sample flag) of the sensitivity's multiplier: nothing, one device scalar
    or one value per sample (fp32 on `dev`), as allocate_bits_device takes it."""
    if mult is None:
        return None, None, 0
    if mult.dtype != torch.float32 or mult.device != dev or mult.numel() not in (1, N):
        raise RuntimeError("the sensitivity's multiplier must be fp32 on the same device with 1 or N values")
    if not mult.is_contiguous():
        mult = mult.contiguous()
    return mult, mult.data_ptr(), int(mult.numel() == N and N != 1)


def hip_batch_norm_pack_applies(input, weight, bias, running_mean, running_var):
    """True when the forward pass can also write the packed copy of its input."""
    if input.dtype not in (torch.float16, torch.bfloat16, torch.float32):
        return False
    if not hip_batch_norm_minmax_applies(input, weight, bias, running_mean, running_var):
        return False
    N, C, HW, channels_last = _bn_geometry(input)
    return not channels_last or N * HW < 2 ** 31


def hip_batch_norm_backward(input, grad_output, weight, save_mean, save_invstd, sumsq=False):
    """-> (grad_input, grad_weight, grad_bias) of training-mode batch norm; `grad_output` has the
    strides of `input`.  With `sumsq` the pass also leaves the partial sums of grad_input^2 on
    grad_input (see known_sumsq)."""
    N, C, HW, channels_last = _bn_geometry(input)
    lib = _glue.lib()
    code = _glue.DTYPE_CODE[input.dtype]
    ws_bytes = _workspace_bytes(N, C, HW, code, int(channels_last))
    entries = _sumsq_entries(N, C, HW, code, int(channels_last)) if sumsq else 0
    ws = torch.empty(ws_bytes // 4 + entries, dtype=torch.float32, device=input.device)
    grad_input = torch.empty_like(input)
    grad_weight = torch.empty(C, dtype=torch.float32, device=input.device)
    grad_bias = torch.empty(C, dtype=torch.float32, device=input.device)
    with _glue.on_device(input.device):
        _glue._lib.check(lib.actnn_batch_norm_backward(
            input.data_ptr(), grad_output.data_ptr(), _ptr(weight), save_mean.data_ptr(),
            save_invstd.data_ptr(), grad_input.data_ptr(), grad_weight.data_ptr(), grad_bias.data_ptr(),
            ws.data_ptr(), ws_bytes, ws.data_ptr() + ws_bytes if entries else None, entries,
            N, C, HW, code, int(channels_last), _glue.stream_ptr(input.device)), "batch_norm_backward")
    if entries:
        _leave_sumsq(grad_input, ws[ws_bytes // 4:])
    return grad_input, grad_weight, grad_bias


def hip_batch_norm_backward_packed_applies(shape, quantized, grad_output, weight, save_mean, save_invstd):
    """True when the batch-norm backward kernels can read the saved input straight from its
    mixed-precision stream: activation with scale/min in its own dtype (or, for an fp32
    activation, in their compact bf16 storage, ops.py:115-116), whole groups of 256, and a
    gradient laid out like the activation was when it was compressed."""
    q_input, q_bits, q_scale, q_min = quantized
    dtype = grad_output.dtype
    memory_format = getattr(quantized, "memory_format", None)
    channels_last = memory_format is not None
    geo = _shape_geometry(shape, dtype, channels_last)
    compact = (dtype == torch.float32 and q_scale.dtype == torch.bfloat16
               and not getattr(quantized, "native_bf16", False))
    return (geo is not None and dtype in (torch.float16, torch.bfloat16, torch.float32)
            and _groups_align(geo[0], geo[1], geo[2], _glue.DTYPE_CODE[dtype], channels_last)
            and isinstance(q_bits, torch.Tensor)
            and isinstance(q_input, torch.Tensor) and q_input.is_cuda and q_input.dtype == torch.int32
            and (q_scale.dtype == dtype or compact) and q_min.dtype == q_scale.dtype
            and q_scale.is_contiguous() and q_min.is_contiguous()
            and tuple(grad_output.shape) == tuple(shape)
            and grad_output.is_contiguous(memory_format=memory_format or torch.contiguous_format)
            and (not channels_last or geo[0] * geo[2] < 2 ** 31)
            and grad_output.data_ptr() % 16 == 0
            and all(_f32_or_none(t) for t in (weight, save_mean, save_invstd)))


def hip_batch_norm_backward_packed(shape, quantized, grad_output, weight, save_mean, save_invstd, sumsq=False,
                                   relu_mask=None):
    """-> (grad_input, grad_weight, grad_bias); the saved input is decoded inside the kernels.
    `sumsq` as in hip_batch_norm_backward.  `relu_mask`: `grad_output` is the gradient of a ReLU the
    batch norm's output went through, and the passes apply that ReLU's mask as they read it
    (shapes of hip_batch_norm_relu_applies)."""
    from .quantization import _bits_info
    q_input, q_bits, q_scale, q_min = quantized
    channels_last = getattr(quantized, "memory_format", None) is not None
    N, C, HW = _shape_geometry(shape, grad_output.dtype, channels_last)
    lib = _glue.lib()
    code = _glue.DTYPE_CODE[grad_output.dtype]
    total, prefix = _bits_info(q_bits)
    if q_input.numel() < total * (C * HW // 256) * 8:
        raise RuntimeError("batch_norm_backward_packed: packed stream is too short")
    if q_scale.dtype != grad_output.dtype:              # fp32 activation, bf16 storage: widened as
        q_scale = q_scale.to(grad_output.dtype)         # dequantize_activation widens it (ops.py:129-131)
        q_min = q_min.to(grad_output.dtype)
    ws_bytes = _workspace_bytes(N, C, HW, code, int(channels_last))
    dev = grad_output.device
    entries = _sumsq_entries(N, C, HW, code, int(channels_last)) if sumsq else 0
    ws = torch.empty(ws_bytes // 4 + entries, dtype=torch.float32, device=dev)
    grad_input = torch.empty_like(grad_output)
    grad_weight = torch.empty(C, dtype=torch.float32, device=dev)
    grad_bias = torch.empty(C, dtype=torch.float32, device=dev)
    with _glue.on_device(dev):
        if relu_mask is not None:
            _glue._lib.check(lib.actnn_batch_norm_backward_packed_relu(
                q_input.data_ptr(), q_bits.data_ptr(), prefix.data_ptr(), q_scale.data_ptr(), q_min.data_ptr(),
                grad_output.data_ptr(), relu_mask.data_ptr(), _ptr(weight), save_mean.data_ptr(),
                save_invstd.data_ptr(), grad_input.data_ptr(), grad_weight.data_ptr(), grad_bias.data_ptr(),
                ws.data_ptr(), ws_bytes, ws.data_ptr() + ws_bytes if entries else None, entries,
                N, C, HW, code, int(channels_last), _glue.stream_ptr(dev)), "batch_norm_backward_packed_relu")
        else:
            _glue._lib.check(lib.actnn_batch_norm_backward_packed(
                q_input.data_ptr(), q_bits.data_ptr(), prefix.data_ptr(), q_scale.data_ptr(), q_min.data_ptr(),
                grad_output.data_ptr(), _ptr(weight), save_mean.data_ptr(), save_invstd.data_ptr(),
                grad_input.data_ptr(), grad_weight.data_ptr(), grad_bias.data_ptr(), ws.data_ptr(), ws_bytes,
                ws.data_ptr() + ws_bytes if entries else None, entries,
                N, C, HW, code, int(channels_last), _glue.stream_ptr(dev)), "batch_norm_backward_packed")
    if entries:
        _leave_sumsq(grad_input, ws[ws_bytes // 4:])
    return grad_input, grad_weight, grad_bias


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


def _miopen_takes(input, weight, bias):
    """MIOpen's batch norm wants fp32 affine parameters (and wants them to exist); other
    combinations go to ATen's native kernels, which save the same (mean, invstd) pair."""
    return all(t is not None and t.dtype == torch.float32 for t in (weight, bias))


def cudnn_batch_norm(input, weight, bias, running_mean, running_var, training,
                     exponential_average_factor, epsilon):
    """-> (output, save_mean, save_var, reserve).  at::native::cudnn_batch_norm
    (backward_func.cc:87); save_var holds the inverse standard deviation, as cuDNN's and
    MIOpen's do; `reserve` is an empty placeholder."""
    if training and hip_batch_norm_applies(input, weight, bias, running_mean, running_var):
        out, save_mean, save_invstd, _, _ = hip_batch_norm_forward(
            input, weight, bias, running_mean, running_var, exponential_average_factor, epsilon)
        return out, save_mean, save_invstd, input.new_empty(0, dtype=torch.uint8)
    if not _miopen_takes(input, weight, bias):
        out, save_mean, save_var = _aten.native_batch_norm(
            input, weight, bias, running_mean, running_var, training, exponential_average_factor, epsilon)
        return out, save_mean, save_var, input.new_empty(0, dtype=torch.uint8)
    out, save_mean, save_var = _aten.miopen_batch_norm(
        input, weight, bias, running_mean, running_var, training, exponential_average_factor, epsilon)
    return out, save_mean, save_var, input.new_empty(0, dtype=torch.uint8)


def cudnn_batch_norm_backward(input, grad_output, weight, running_mean, running_var, save_mean,
                              save_var, epsilon, reserve, sumsq=False):
    """-> (grad_input, grad_weight, grad_bias).  at::native::cudnn_batch_norm_backward
    (backward_func.cc:88).  `sumsq` (an addition): see hip_batch_norm_backward."""
    if (hip_batch_norm_applies(input, weight, None, save_mean, save_var)
            and grad_output.dtype == input.dtype and grad_output.shape == input.shape
            and grad_output.stride() == input.stride() and grad_output.data_ptr() % 16 == 0):
        return hip_batch_norm_backward(input, grad_output, weight, save_mean, save_var, sumsq)
    if not _miopen_takes(input, weight, weight):
        return _aten.native_batch_norm_backward(grad_output, input, weight, running_mean, running_var,
                                                save_mean, save_var, True, epsilon, [True, True, True])
    return _aten.miopen_batch_norm_backward(input, grad_output, weight, running_mean, running_var,
                                            save_mean, save_var, epsilon)


def hip_batch_norm_forward_eval(input, weight, bias, running_mean, running_var, eps):
    """-> (output, mean, invstd): evaluation-mode batch norm with this library's kernels; mean and
    invstd are the running mean and 1 / sqrt(running_var + eps), kept for the backward pass."""
    N, C, HW, channels_last = _bn_geometry(input)
    lib = _glue.lib()
    code = _glue.DTYPE_CODE[input.dtype]
    ws_bytes = _workspace_bytes(N, C, HW, code, int(channels_last))
    ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device=input.device)
    out = torch.empty_like(input)
    mean = torch.empty(C, dtype=torch.float32, device=input.device)
    invstd = torch.empty(C, dtype=torch.float32, device=input.device)
    with _glue.on_device(input.device):
        _glue._lib.check(lib.actnn_batch_norm_forward_eval(
            input.data_ptr(), _ptr(weight), _ptr(bias), running_mean.data_ptr(), running_var.data_ptr(),
            out.data_ptr(), mean.data_ptr(), invstd.data_ptr(), ws.data_ptr(), ws_bytes, N, C, HW, float(eps),
            code, int(channels_last), _glue.stream_ptr(input.device)), "batch_norm_forward_eval")
    return out, mean, invstd


def hip_batch_norm_backward_eval(input, grad_output, weight, mean, invstd):
    """-> (grad_input, grad_weight, grad_bias) of evaluation-mode batch norm."""
    N, C, HW, channels_last = _bn_geometry(input)
    lib = _glue.lib()
    code = _glue.DTYPE_CODE[input.dtype]
    ws_bytes = _workspace_bytes(N, C, HW, code, int(channels_last))
    ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device=input.device)
    grad_input = torch.empty_like(input)
    grad_weight = torch.empty(C, dtype=torch.float32, device=input.device)
    grad_bias = torch.empty(C, dtype=torch.float32, device=input.device)
    with _glue.on_device(input.device):
        _glue._lib.check(lib.actnn_batch_norm_backward_eval(
            input.data_ptr(), grad_output.data_ptr(), _ptr(weight), mean.data_ptr(), invstd.data_ptr(),
            grad_input.data_ptr(), grad_weight.data_ptr(), grad_bias.data_ptr(), ws.data_ptr(), ws_bytes,
            N, C, HW, code, int(channels_last), _glue.stream_ptr(input.device)), "batch_norm_backward_eval")
    return grad_input, grad_weight, grad_bias


def native_batch_norm(input, weight, bias, running_mean, running_var, training, momentum, eps):
    """at::native_batch_norm (backward_func.cc:89).  In evaluation mode with running estimates - the
    case the reference's batch_norm Function calls it for (ops.py:458-461) - this library's kernels
    run whenever the tensors qualify; save_mean / save_invstd then hold the running mean and
    1 / sqrt(running_var + eps) where ATen returns empty tensors."""
    if (not training and running_mean is not None and running_var is not None
            and hip_batch_norm_applies(input, weight, bias, running_mean, running_var)):
        return hip_batch_norm_forward_eval(input, weight, bias, running_mean, running_var, eps)
    return _aten.native_batch_norm(input, weight, bias, running_mean, running_var, training, momentum, eps)


def native_batch_norm_backward(grad_out, input, weight, running_mean, running_var, save_mean,
                               save_invstd, train, eps, output_mask):
    """at::native_batch_norm_backward (backward_func.cc:90); evaluation mode as above."""
    if (not train and running_mean is not None and running_var is not None
            and hip_batch_norm_applies(input, weight, None, running_mean, running_var)
            and grad_out.dtype == input.dtype and grad_out.shape == input.shape
            and grad_out.stride() == input.stride() and grad_out.data_ptr() % 16 == 0):
        C = input.shape[1]
        if save_mean is None or save_mean.numel() != C or save_invstd is None or save_invstd.numel() != C:
            save_mean, save_invstd = running_mean, torch.rsqrt(running_var + eps)
        gi, gw, gb = hip_batch_norm_backward_eval(input, grad_out, weight, save_mean, save_invstd)
        mask = list(output_mask)
        return (gi if mask[0] else None, gw if mask[1] else None, gb if mask[2] else None)
    return _aten.native_batch_norm_backward(grad_out, input, weight, running_mean, running_var,
                                            save_mean, save_invstd, train, eps, list(output_mask))


def prepare_layer_norm_inputs(input, normalized_shape, weight, bias):
    """-> (X, gamma, beta, M, N): contiguous operands and the [M, N] geometry of a layer norm
    over the trailing `normalized_shape` (backward_func.cc:14-72, re-exported at :83; no caller
    in the reference's Python)."""
    normalized_shape = tuple(int(d) for d in normalized_shape)
    if len(normalized_shape) < 1:
        raise RuntimeError("Expected normalized_shape to be at least 1-dimensional")
    for t, name in ((weight, "weight"), (bias, "bias")):
        if t is not None and tuple(t.shape) != normalized_shape:
            raise RuntimeError(f"Expected {name} to be of same shape as normalized_shape, but got {name} of "
                               f"shape {tuple(t.shape)} and normalized_shape = {normalized_shape}")
    lead = input.dim() - len(normalized_shape)
    if lead < 0 or tuple(input.shape[lead:]) != normalized_shape:
        raise RuntimeError(f"Given normalized_shape={normalized_shape}, expected input with shape "
                           f"[*, {', '.join(map(str, normalized_shape))}], but got input of size {tuple(input.shape)}")
    M = 1
    for d in input.shape[:lead]:
        M *= d
    N = 1
    for d in normalized_shape:
        N *= d
    return (input.contiguous(), None if weight is None else weight.contiguous(),
            None if bias is None else bias.contiguous(), M, N)


def layer_norm_cuda(X, gamma, beta, M, N, eps):
    """-> (Y, mean [M], rstd [M]) of the [M, N] problem (at::native::layer_norm_cuda,
    backward_func.cc:84); ATen's kernel through its current name."""
    Y, mean, rstd = _aten.native_layer_norm(X.reshape(M, N), [N], None if gamma is None else gamma.reshape(N),
                                            None if beta is None else beta.reshape(N), eps)
    return Y.view_as(X), mean.reshape(M), rstd.reshape(M)


def layer_norm_backward_cuda(dY, X, mean, rstd, gamma, M, N, grad_input_mask):
    """-> (dX, dgamma, dbeta) (at::native::layer_norm_backward_cuda, backward_func.cc:85)."""
    flat = None if gamma is None else gamma.reshape(N)
    # ATen's current entry also takes the bias, of which only the shape matters: gamma stands in
    dX, dgamma, dbeta = _aten.native_layer_norm_backward(
        dY.reshape(M, N), X.reshape(M, N), [N], mean.reshape(M, 1), rstd.reshape(M, 1), flat, flat,
        list(grad_input_mask))
    shape = None if gamma is None else gamma.shape
    return (None if dX is None else dX.view_as(X), None if dgamma is None or shape is None else dgamma.view(shape),
            None if dbeta is None or shape is None else dbeta.view(shape))
