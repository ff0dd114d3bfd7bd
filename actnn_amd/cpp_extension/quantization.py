"""Operators of the reference's ``actnn.cpp_extension.quantization`` module
(cpp_extension/quantization.cc:198-206), same names and positional arguments, running the
gfx950 kernels through the C ABI.  Extras that the reference does not have are keyword-only:
``noise=`` (deterministic mode) on the two pack functions.
"""
import torch
from torch.autograd import Function

from . import _glue as g
from .._lib import check
from ..utils import channels_last_format

MASK_BLOCK = 512


# ------------------------------------------------------------------------------------------
# per-sample bit widths: host copy, total and device prefix sums travel with the tensor
# ------------------------------------------------------------------------------------------
def attach_bits_host(bits_dev, bits_host):
    """Remember the host copy of a device ``bits`` tensor so that pack/unpack need no
    device->host sync (the reference syncs twice per pack: .cu:92, :98).  The hand-off is tied to
    the tensor's version counter: after an in-place change of ``bits_dev`` it is ignored."""
    bits_dev._actnn_host = (bits_dev._version, bits_host)
    bits_dev._actnn_info = None
    return bits_dev


def attach_bits_total(bits_dev, total, prefix=None):
    """For widths computed on the device (no host copy): remember their sum, which the caller
    knows from the budget, so that the packed stream can be sized without a sync; `prefix` is the
    device exclusive prefix sum [N+1] when the caller has it already."""
    bits_dev._actnn_total = (bits_dev._version, int(total))
    bits_dev._actnn_info = None if prefix is None else (bits_dev._version, int(total), prefix)
    return bits_dev


def _fresh(bits, name):
    """Value attached to `bits` under `name`, or None when `bits` has been written since."""
    tagged = getattr(bits, name, None)
    if tagged is None or tagged[0] != bits._version:
        return None
    return tagged[1] if len(tagged) == 2 else tagged[1:]


def _bits_info(bits):
    """(sum(bits), device exclusive prefix [N+1]) of an int32 device tensor, cached on it together
    with the tensor's version counter: an in-place change of `bits` invalidates the cache (and the
    attached host copy / total), and the widths are then read back and range-checked again."""
    cached = _fresh(bits, "_actnn_info")
    if cached is not None:
        return cached
    total = _fresh(bits, "_actnn_total")               # widths made on the device: only their sum is known
    if total is None:
        host = _fresh(bits, "_actnn_host")
        if host is None:
            host = bits.cpu()                          # sync, like the reference's .item() calls
        if host.numel() and (int(host.min()) < 1 or int(host.max()) > 8):
            raise RuntimeError("pack_mixed_precision supports 1..8 bits per sample")
        total = int(host.sum())
    N = bits.numel()
    prefix = torch.empty(N + 1, dtype=torch.int32, device=bits.device)
    with g.on_device(bits.device):
        check(g.lib().actnn_bits_prefix(bits.data_ptr(), prefix.data_ptr(), N,
                                        g.stream_ptr(bits.device)), "bits_prefix")
    bits._actnn_info = (bits._version, total, prefix)
    return total, prefix


# ------------------------------------------------------------------------------------------
# pack / unpack, mixed precision  (quantization.cc:46-73)
# ------------------------------------------------------------------------------------------
def pack_mixed_precision(data, min, max, bits, stochastic, *, noise=None):
    g.check_float(data, "data", 3)
    g.check_float(min, "min", 3)
    g.check_float(max, "max", 3)
    g.check_typed(bits, "bits", torch.int32, 1)
    if not stochastic:
        raise RuntimeError("pack_mixed_precision: stochastic must be true")      # .cu:122
    N, G, gs = data.shape
    if gs % 32 != 0:
        raise RuntimeError("group_size must be a multiple of 32")                  # .cu:94
    if min.dtype != data.dtype or max.dtype != data.dtype:
        raise RuntimeError("The type of min/max is not correct!")
    if min.numel() != N * G or max.numel() != N * G or bits.numel() != N:
        raise RuntimeError("pack_mixed_precision: shape mismatch")
    if noise is not None:
        g.check_float(noise, "noise", 3)
        if noise.shape != data.shape or noise.dtype != data.dtype:
            raise RuntimeError("noise must match data in shape and dtype")
        noise = g.aligned(noise)
    data = g.aligned(data)
    total, prefix = _bits_info(bits)
    n_words = (total * G * gs + 31) // 32                                          # .cu:98-100
    packed = torch.empty(n_words, dtype=torch.int32, device=data.device)
    scale = torch.empty(N, G, 1, dtype=data.dtype, device=data.device)
    seed, offset = (0, 0) if noise is not None else g.philox_args(data.device)
    with g.on_device(data.device):
        check(g.lib().actnn_pack_mixed(
            data.data_ptr(), min.data_ptr(), max.data_ptr(), bits.data_ptr(), prefix.data_ptr(),
            scale.data_ptr(), packed.data_ptr(), noise.data_ptr() if noise is not None else None,
            seed, offset, N, G, gs, g.DTYPE_CODE[data.dtype], g.stream_ptr(data.device)),
            "pack_mixed_precision")
    return packed, scale


def quantize_activation_device(rows, N, known_minmax, alloc):
    """[min/max of every group] -> widths on the device -> pack, in one call: what minimax,
    allocate_bits_device and pack_mixed_precision do one after the other for `rows` (contiguous
    [N * G, 256] view of the activation).  `known_minmax`: (mn, mx) [N * G] in the rows' dtype when
    another kernel has produced them, else None.  `alloc`: the scheme's AllocationArgs.
    -> (packed, bits with sum and prefix attached, scale [N, G, 1], mn [N * G])."""
    from .backward_func import _mult_args
    dev, dtype = rows.device, rows.dtype
    G = rows.shape[0] // N
    rows = g.aligned(rows)
    if known_minmax is None:
        mn = torch.empty(N * G, dtype=dtype, device=dev)
        mx = torch.empty(N * G, dtype=dtype, device=dev)
    else:
        mn, mx = known_minmax
    sens = alloc.sens_out if alloc.sens_out is not None else torch.empty(N, dtype=torch.float32, device=dev)
    bits = torch.empty(N, dtype=torch.int32, device=dev)
    prefix = torch.empty(N + 1, dtype=torch.int32, device=dev)
    packed = torch.empty(alloc.total * G * 8, dtype=torch.int32, device=dev)
    scale = torch.empty(N, G, 1, dtype=dtype, device=dev)
    mult, mult_ptr, per_sample = _mult_args(alloc.mult, N, dev)           # (`mult` held until the launch)
    seed, offset = g.philox_args(dev)
    with g.on_device(dev):
        check(g.lib().actnn_quantize_activation(
            rows.data_ptr(), mn.data_ptr(), mx.data_ptr(), int(known_minmax is not None), alloc.factor, mult_ptr,
            per_sample, sens.data_ptr(), bits.data_ptr(), prefix.data_ptr(), alloc.initial, alloc.target,
            scale.data_ptr(), packed.data_ptr(), seed, offset, N, G, g.DTYPE_CODE[dtype], g.stream_ptr(dev)),
            "quantize_activation")
    attach_bits_total(bits, alloc.total, prefix)
    return packed, bits, scale, mn


def unpack_mixed_precision(data, bits, scale, min, N, num_groups, group_size):
    g.check_typed(data, "data", torch.int32, 1)
    g.check_typed(bits, "bits", torch.int32, 1)
    g.check_float(scale, "scale", 3)
    g.check_float(min, "min", 3)
    if group_size % 32 != 0:
        raise RuntimeError("group_size must be a multiple of 32")                  # .cu:186
    if min.dtype != scale.dtype:
        raise RuntimeError("The type of min is not correct!")
    if scale.numel() != N * num_groups or min.numel() != N * num_groups or bits.numel() != N:
        raise RuntimeError("unpack_mixed_precision: shape mismatch")
    total, prefix = _bits_info(bits)
    if data.numel() < (total * num_groups * group_size + 31) // 32:
        raise RuntimeError("unpack_mixed_precision: packed stream is too short")
    out = torch.empty(N, num_groups, group_size, dtype=scale.dtype, device=data.device)
    with g.on_device(data.device):
        check(g.lib().actnn_unpack_mixed(
            data.data_ptr(), bits.data_ptr(), prefix.data_ptr(), scale.data_ptr(), min.data_ptr(),
            out.data_ptr(), N, num_groups, group_size, g.DTYPE_CODE[scale.dtype],
            g.stream_ptr(data.device)), "unpack_mixed_precision")
    return out


# ------------------------------------------------------------------------------------------
# pack / unpack, single precision  (quantization.cc:77-102)
# ------------------------------------------------------------------------------------------
def single_packed_bytes(N, G, gs, bits):
    wpt = 8 // bits
    n_round = N + (wpt - N % wpt) % wpt                                            # .cu:274
    return (bits * n_round * G * gs + 8) // 8                                      # .cu:275-277


def pack_single_precision(data, min, max, bits, stochastic, *, noise=None):
    g.check_float(data, "data", 3)
    g.check_float(min, "min", 3)
    g.check_float(max, "max", 3)
    bits = int(bits)
    if bits < 1 or 8 % bits != 0:
        raise RuntimeError("pack_single_precision: 8 % bits must be 0")            # .cu:272
    if not stochastic:
        raise RuntimeError("pack_single_precision: stochastic must be true")     # .cu:298
    N, G, gs = data.shape
    if gs % 8 != 0:
        raise RuntimeError("group_size must be a multiple of 8")
    if min.dtype != data.dtype or max.dtype != data.dtype:
        raise RuntimeError("The type of min/max is not correct!")
    if min.numel() != N * G or max.numel() != N * G:
        raise RuntimeError("pack_single_precision: shape mismatch")
    if noise is not None:
        g.check_float(noise, "noise", 3)
        if noise.shape != data.shape or noise.dtype != data.dtype:
            raise RuntimeError("noise must match data in shape and dtype")
        noise = g.aligned(noise)
    data = g.aligned(data)
    packed = torch.empty(single_packed_bytes(N, G, gs, bits), dtype=torch.int8, device=data.device)
    scale = torch.empty(N, G, 1, dtype=data.dtype, device=data.device)
    wpt = 8 // bits
    seed, offset = (0, 0) if noise is not None else g.philox_args(data.device)
    with g.on_device(data.device):
        check(g.lib().actnn_pack_single(
            data.data_ptr(), min.data_ptr(), max.data_ptr(), bits, scale.data_ptr(),
            packed.data_ptr(), noise.data_ptr() if noise is not None else None, seed, offset,
            N, G, gs, g.DTYPE_CODE[data.dtype], g.stream_ptr(data.device)), "pack_single_precision")
    del wpt
    return packed, scale


def unpack_single_precision(data, bits, scale, min, N, num_groups, group_size):
    g.check_typed(data, "data", torch.int8, 1)
    g.check_float(scale, "scale", 3)
    g.check_float(min, "min", 3)
    bits = int(bits)
    if bits < 1 or 8 % bits != 0:
        raise RuntimeError("unpack_single_precision: 8 % bits must be 0")          # .cu:375
    if min.dtype != scale.dtype:
        raise RuntimeError("The type of min is not correct!")
    if scale.numel() != N * num_groups or min.numel() != N * num_groups:
        raise RuntimeError("unpack_single_precision: shape mismatch")
    if data.numel() < single_packed_bytes(N, num_groups, group_size, bits) - 1:
        raise RuntimeError("unpack_single_precision: packed stream is too short")
    out = torch.empty(N, num_groups, group_size, dtype=scale.dtype, device=data.device)
    with g.on_device(data.device):
        check(g.lib().actnn_unpack_single(
            data.data_ptr(), bits, scale.data_ptr(), min.data_ptr(), out.data_ptr(), N, num_groups,
            group_size, g.DTYPE_CODE[scale.dtype], g.stream_ptr(data.device)),
            "unpack_single_precision")
    return out


# ------------------------------------------------------------------------------------------
# fused QLinear weight gradient (no counterpart among the reference's operators: it replaces
# dequantize + grad_output.t().mm(input) of linear.backward, actnn/actnn/ops.py:407-421)
# ------------------------------------------------------------------------------------------
def linear_grad_weight(grad_output, packed, bits, scale, min, in_features, out_dtype=None):
    """grad_w[O, I] = grad_output[M, O]^T @ dequant(x)[M, I] with x given as it was saved: `bits`
    an int (the fixed-width stream of pack_single_precision, int8) or an int32 tensor [M] (the
    mixed-width stream of pack_mixed_precision, int32), scale/min [M, I/256, 1].  The dequantised
    tile only ever exists in LDS."""
    mixed = isinstance(bits, torch.Tensor)
    g.check_typed(packed, "packed", torch.int32 if mixed else torch.int8, 1)
    g.check_float(scale, "scale", 3)
    g.check_float(min, "min", 3)
    if not (isinstance(grad_output, torch.Tensor) and grad_output.is_cuda and grad_output.dim() == 2):
        raise RuntimeError("grad_output must be a 2-d CUDA tensor")
    if grad_output.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError("The type of grad_output is not correct!")
    grad_output = g.aligned(grad_output.contiguous())
    M, O = grad_output.shape
    I = int(in_features)
    if I % 256 != 0 or O % 8 != 0:
        raise RuntimeError("linear_grad_weight needs in_features % 256 == 0 and out_features % 8 == 0")
    G = I // 256
    if scale.numel() != M * G or min.numel() != scale.numel() or min.dtype != scale.dtype:
        raise RuntimeError("linear_grad_weight: scale/min do not match the packed input")
    if mixed:
        g.check_typed(bits, "bits", torch.int32, 1)
        if bits.numel() != M:
            raise RuntimeError("linear_grad_weight: one width per row expected")
        total, prefix = _bits_info(bits)
        if packed.numel() < (total * G * 256 + 31) // 32:
            raise RuntimeError("linear_grad_weight: packed stream is too short")
        bits_ptr, prefix_ptr, fixed = bits.data_ptr(), prefix.data_ptr(), 0
    else:
        fixed = int(bits)
        if fixed not in (1, 2, 4, 8):
            raise RuntimeError("linear_grad_weight: 8 % bits must be 0")
        if packed.numel() < single_packed_bytes(M, G, 256, fixed) - 1:
            raise RuntimeError("linear_grad_weight: packed stream is too short")
        bits_ptr = prefix_ptr = None
    out_dtype = out_dtype or grad_output.dtype
    gw = torch.empty(O, I, dtype=out_dtype, device=grad_output.device)
    # few output tiles and many rows: the sum over the rows is split over blocks (partial tiles in `ws`)
    ws_bytes = g.lib().actnn_linear_grad_weight_workspace_bytes(M, O, I)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=gw.device) if ws_bytes > 0 else None
    with g.on_device(gw.device):
        check(g.lib().actnn_linear_grad_weight_ws(
            grad_output.data_ptr(), packed.data_ptr(), bits_ptr, prefix_ptr, fixed, scale.data_ptr(),
            min.data_ptr(), gw.data_ptr(), M, O, I, g.DTYPE_CODE[grad_output.dtype], g.DTYPE_CODE[scale.dtype],
            g.DTYPE_CODE[out_dtype], ws.data_ptr() if ws is not None else None, ws_bytes,
            g.stream_ptr(gw.device)), "linear_grad_weight")
    return gw


def linear_grad_weight_q2(grad_output, packed, scale, min, in_features, out_dtype=None):
    """The 2-bit fixed-width case of linear_grad_weight (rows in whole groups of four)."""
    if grad_output.dim() == 2 and grad_output.shape[0] % 4 != 0:
        raise RuntimeError("linear_grad_weight_q2 needs M % 4 == 0")
    return linear_grad_weight(grad_output, packed, 2, scale, min, in_features, out_dtype)


# ------------------------------------------------------------------------------------------
# ReLU / Dropout with 1-bit masks  (quantization.cc:106-148)
# ------------------------------------------------------------------------------------------
def mask_words(n):
    """int32 words of the mask of ``n`` elements: 16 per block of 512 elements.  Equals the
    reference's ceil(n/32) when n % 512 == 0; its tail block writes 16 words regardless
    (.cu:441-443), so the whole block is allocated here."""
    return (n + MASK_BLOCK - 1) // MASK_BLOCK * 16


def relu_forward(x):
    x = g.aligned(x)
    n = x.numel()
    y = torch.empty_like(x)
    mask = torch.empty(mask_words(n), dtype=torch.int32, device=x.device)
    with g.on_device(x.device):
        check(g.lib().actnn_relu_forward(x.data_ptr(), y.data_ptr(), mask.data_ptr(), n,
                                         g.DTYPE_CODE[x.dtype], g.stream_ptr(x.device)), "relu_forward")
    return y, mask


def relu_forward_minmax(x):
    """-> (y, mask, mn, mx): ReLU whose pass also yields the min / max of every group of 256
    consecutive outputs (16-bit tensors of whole 2048-element tiles)."""
    n = x.numel()
    y = torch.empty_like(x)
    mask = torch.empty(mask_words(n), dtype=torch.int32, device=x.device)
    mn = torch.empty(n // 256, dtype=x.dtype, device=x.device)
    mx = torch.empty(n // 256, dtype=x.dtype, device=x.device)
    with g.on_device(x.device):
        check(g.lib().actnn_relu_forward_minmax(x.data_ptr(), y.data_ptr(), mask.data_ptr(), mn.data_ptr(),
                                                mx.data_ptr(), n, g.DTYPE_CODE[x.dtype],
                                                g.stream_ptr(x.device)), "relu_forward_minmax")
    return y, mask, mn, mx


def relu_minmax_applies(x):
    return (x.is_cuda and x.dtype in (torch.float16, torch.bfloat16) and x.is_contiguous()
            and x.numel() > 0 and x.numel() % 2048 == 0 and x.data_ptr() % 16 == 0)


def relu_backward(grad_output, mask):
    grad_output = g.aligned(grad_output.contiguous())
    gin = torch.empty_like(grad_output)
    with g.on_device(gin.device):
        check(g.lib().actnn_relu_backward(grad_output.data_ptr(), mask.data_ptr(), gin.data_ptr(),
                                          gin.numel(), g.DTYPE_CODE[gin.dtype],
                                          g.stream_ptr(gin.device)), "relu_backward")
    return gin


def relu_backward_add(grad_output, mask, other):
    """other + relu_backward(grad_output, mask) in one pass (rounded as the tensor addition rounds);
    the three tensors are dense in the same memory order."""
    gin = torch.empty_like(grad_output)
    with g.on_device(gin.device):
        check(g.lib().actnn_relu_backward_add(grad_output.data_ptr(), mask.data_ptr(), other.data_ptr(),
                                              gin.data_ptr(), gin.numel(), g.DTYPE_CODE[gin.dtype],
                                              g.stream_ptr(gin.device)), "relu_backward_add")
    return gin


class ActQuantizedReLU(Function):
    """quantization.cc:106-119: saves only the 1-bit mask."""

    @staticmethod
    def forward(ctx, input):
        output, mask = relu_forward(input)
        ctx.save_for_backward(mask)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        (mask,) = ctx.saved_tensors
        return relu_backward(grad_output, mask)


class ActQuantizedReLUMinMax(Function):
    """The same operator, additionally returning the group min / max of its output (not
    differentiable) for the layer that compresses this output next."""

    @staticmethod
    def forward(ctx, input):
        output, mask, mn, mx = relu_forward_minmax(input)
        ctx.save_for_backward(mask)
        ctx.mark_non_differentiable(mn, mx)
        ctx.set_materialize_grads(False)          # no zero tensors for the two statistics
        return output, mn, mx

    @staticmethod
    def backward(ctx, grad_output, _grad_mn, _grad_mx):
        if grad_output is None:
            return None
        (mask,) = ctx.saved_tensors
        return relu_backward(grad_output, mask)


def relu_add_forward(x, residual, minmax=False):
    """-> (y, mask[, mn, mx]) of relu(x + residual) in one pass; the sum is rounded to the tensors'
    dtype as the tensor addition rounds it."""
    n = x.numel()
    y = torch.empty_like(x)
    mask = torch.empty(mask_words(n), dtype=torch.int32, device=x.device)
    mn = mx = None
    if minmax:
        mn = torch.empty(n // 256, dtype=x.dtype, device=x.device)
        mx = torch.empty(n // 256, dtype=x.dtype, device=x.device)
    with g.on_device(x.device):
        check(g.lib().actnn_relu_add_forward(
            x.data_ptr(), residual.data_ptr(), y.data_ptr(), mask.data_ptr(),
            mn.data_ptr() if minmax else None, mx.data_ptr() if minmax else None, n,
            g.DTYPE_CODE[x.dtype], g.stream_ptr(x.device)), "relu_add_forward")
    return (y, mask, mn, mx) if minmax else (y, mask)


class ActQuantizedAddReLU(Function):
    """relu(input + residual) that saves only the 1-bit mask; both operands receive the masked
    gradient."""

    @staticmethod
    def forward(ctx, input, residual):
        output, mask = relu_add_forward(input, residual)
        ctx.save_for_backward(mask)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        (mask,) = ctx.saved_tensors
        grad = relu_backward(grad_output, mask)
        return grad, grad


class ActQuantizedAddReLUMinMax(Function):
    """The same, additionally returning the group min / max of the output (not differentiable)."""

    @staticmethod
    def forward(ctx, input, residual):
        output, mask, mn, mx = relu_add_forward(input, residual, minmax=True)
        ctx.save_for_backward(mask)
        ctx.mark_non_differentiable(mn, mx)
        ctx.set_materialize_grads(False)
        return output, mn, mx

    @staticmethod
    def backward(ctx, grad_output, _grad_mn, _grad_mx):
        if grad_output is None:
            return None, None
        (mask,) = ctx.saved_tensors
        grad = relu_backward(grad_output, mask)
        return grad, grad


def add_relu_applies(x, residual):
    """Same shape, dtype, device and dense memory order, 16-byte aligned."""
    return (x.is_cuda and residual.is_cuda and x.device == residual.device and x.dtype == residual.dtype
            and x.dtype in g.DTYPE_CODE and x.shape == residual.shape and x.is_contiguous()
            and residual.is_contiguous() and x.numel() > 0
            and x.data_ptr() % 16 == 0 and residual.data_ptr() % 16 == 0)


def act_quantized_relu(input):
    g.check_float(input, "input")                                                  # quantization.cc:122
    return ActQuantizedReLU.apply(input)


def dropout_forward(x, p):
    x = g.aligned(x)
    n = x.numel()
    y = torch.empty_like(x)
    mask = torch.empty(mask_words(n), dtype=torch.int32, device=x.device)
    seed, offset = g.philox_args(x.device)
    with g.on_device(x.device):
        check(g.lib().actnn_dropout_forward(x.data_ptr(), y.data_ptr(), mask.data_ptr(), n, float(p),
                                            seed, offset, g.DTYPE_CODE[x.dtype],
                                            g.stream_ptr(x.device)), "dropout_forward")
    return y, mask


def dropout_backward(grad_output, mask, p):
    grad_output = g.aligned(grad_output.contiguous())
    gin = torch.empty_like(grad_output)
    with g.on_device(gin.device):
        check(g.lib().actnn_dropout_backward(grad_output.data_ptr(), mask.data_ptr(), gin.data_ptr(),
                                             gin.numel(), float(p), g.DTYPE_CODE[gin.dtype],
                                             g.stream_ptr(gin.device)), "dropout_backward")
    return gin


class ActQuantizedDropout(Function):
    """quantization.cc:128-143."""

    @staticmethod
    def forward(ctx, input, dropout_p):
        output, mask = dropout_forward(input, dropout_p)
        ctx.save_for_backward(mask)
        ctx.dropout_p = float(dropout_p)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        (mask,) = ctx.saved_tensors
        return dropout_backward(grad_output, mask, ctx.dropout_p), None


def act_quantized_dropout(input, dropout_p):
    g.check_float(input, "input")                                                  # quantization.cc:146
    return ActQuantizedDropout.apply(input, dropout_p)


# ------------------------------------------------------------------------------------------
# MaxPool2d with int8 arg-max indices  (quantization.cc:152-196)
# ------------------------------------------------------------------------------------------
def _pair_check(v, name):
    v = [int(a) for a in v]
    if len(v) != 2:
        raise RuntimeError(f"{name} must have 2 elements")                        # quantization.cc:156-159
    return v


def pool_takes_channels_last(x):
    """True for a channels-last tensor the [N, H, W, C] kernels take (whole 16-byte chunks of channels)."""
    return (channels_last_format(x) is not None and x.shape[1] % (16 // x.element_size()) == 0
            and x.data_ptr() % 16 == 0)


def max_pool2d_forward(x, kernel_size, stride, padding, dilation, nibble_indices=False):
    """-> (y, idx) in the memory format of x (default or channels-last).  idx: int8 of y's shape as in
    the reference, or with nibble_indices a flat uint8 tensor holding two indices per byte
    ((y.numel() + 1) // 2 bytes, in the order of y's memory)."""
    N, C, H, W = x.shape
    KH, KW = kernel_size
    Ho = (H + 2 * padding[0] - dilation[0] * (KH - 1) - 1) // stride[0] + 1       # .cu:679
    Wo = (W + 2 * padding[1] - dilation[1] * (KW - 1) - 1) // stride[1] + 1       # .cu:680
    channels_last = pool_takes_channels_last(x)
    fmt = torch.channels_last if channels_last else torch.contiguous_format
    if not channels_last:
        x = x.contiguous()
    y = torch.empty((N, C, Ho, Wo), dtype=x.dtype, device=x.device, memory_format=fmt)
    if nibble_indices:
        idx = torch.empty(((N * C * Ho * Wo + 1) // 2,), dtype=torch.uint8, device=x.device)
        fn = g.lib().actnn_max_pool2d_forward_cl_nibble if channels_last else g.lib().actnn_max_pool2d_forward_nibble
    else:
        idx = torch.empty((N, C, Ho, Wo), dtype=torch.int8, device=x.device, memory_format=fmt)
        fn = g.lib().actnn_max_pool2d_forward_cl if channels_last else g.lib().actnn_max_pool2d_forward
    with g.on_device(x.device):
        check(fn(
            x.data_ptr(), y.data_ptr(), idx.data_ptr(), N, C, H, W, Ho, Wo, KH, KW, stride[0],
            stride[1], padding[0], padding[1], g.DTYPE_CODE[x.dtype], g.stream_ptr(x.device)),
            "max_pool2d_forward")
    return y, idx


def max_pool2d_backward(grad_output, idx, input_shape, kernel_size, stride, padding, channels_last=None):
    """The gradient comes back in the memory format of `idx` (the format of the forward input).
    A uint8 `idx` is the two-per-byte format, which carries no layout of its own: `channels_last`
    says which kernels wrote it (default: whatever layout grad_output has)."""
    nibble_indices = idx.dtype == torch.uint8
    if nibble_indices:
        if channels_last is None:
            channels_last = pool_takes_channels_last(grad_output)
    else:
        channels_last = channels_last_format(idx) is not None
    fmt = torch.channels_last if channels_last else torch.contiguous_format
    grad_output = grad_output.contiguous(memory_format=fmt)
    N, C, H, W = input_shape
    Ho, Wo = grad_output.shape[2], grad_output.shape[3]
    gin = torch.empty((N, C, H, W), dtype=grad_output.dtype, device=grad_output.device, memory_format=fmt)
    if nibble_indices:
        if idx.numel() != (grad_output.numel() + 1) // 2:
            raise RuntimeError("max_pool2d_backward: the index tensor does not match grad_output")
        fn = g.lib().actnn_max_pool2d_backward_cl_nibble if channels_last else g.lib().actnn_max_pool2d_backward_nibble
    else:
        fn = g.lib().actnn_max_pool2d_backward_cl if channels_last else g.lib().actnn_max_pool2d_backward
    with g.on_device(gin.device):
        check(fn(
            grad_output.data_ptr(), idx.data_ptr(), gin.data_ptr(), N, C, H, W, Ho, Wo,
            kernel_size[0], kernel_size[1], stride[0], stride[1], padding[0], padding[1],
            g.DTYPE_CODE[gin.dtype], g.stream_ptr(gin.device)), "max_pool2d_backward")
    return gin


class ActQuantizedMaxPool2d(Function):
    """quantization.cc:152-191."""

    @staticmethod
    def forward(ctx, input, kernel_size, stride, padding, dilation, ceil_mode, return_indices,
                nibble_indices=False):
        kernel_size = _pair_check(kernel_size, "kernel_size")
        stride = _pair_check(stride, "stride")
        padding = _pair_check(padding, "padding")
        dilation = _pair_check(dilation, "dilation")
        if ceil_mode:
            raise RuntimeError("Do not support ceil_mode")                         # .cu:684
        if return_indices:
            raise RuntimeError("Do not support return_indices")                    # .cu:685
        if kernel_size[0] * kernel_size[1] >= 16:
            raise RuntimeError("kernel_size[0] * kernel_size[1] must be < 16")    # quantization.cc:162
        if input.dim() != 4:
            raise RuntimeError("The dimension of input is not correct!")
        output, idx = max_pool2d_forward(input, kernel_size, stride, padding, dilation, nibble_indices)
        ctx.save_for_backward(idx)
        ctx.geom = (tuple(input.shape), kernel_size, stride, padding, pool_takes_channels_last(input))
        return output

    @staticmethod
    def backward(ctx, grad_output):
        (idx,) = ctx.saved_tensors
        shape, kernel_size, stride, padding, channels_last = ctx.geom
        gin = max_pool2d_backward(grad_output, idx, shape, kernel_size, stride, padding, channels_last)
        return gin, None, None, None, None, None, None, None


def act_quantized_max_pool2d(input, kernel_size, stride, padding, dilation, ceil_mode, return_indices,
                             nibble_indices=False):
    """The reference's operator (quantization.cc:193-196); nibble_indices keeps the saved indices two
    per byte instead of one int8 each."""
    if not (isinstance(input, torch.Tensor) and input.is_cuda and input.dim() == 4 and pool_takes_channels_last(input)):
        g.check_float(input, "input")                                              # quantization.cc:194
    return ActQuantizedMaxPool2d.apply(input, kernel_size, stride, padding, dilation, ceil_mode,
                                       return_indices, nibble_indices)
