"""``calc_precision(b, C, w, target) -> b``: greedy bit allocation on CPU tensors; ``b`` is
modified in place and returned (reference: cpp_extension/calc_precision.cc:9-50).
``calc_precision_dp(A, C, max_b, target, states) -> (b, p)``: the reference's second export
(calc_precision.cc:58-125, no caller in its Python), a dynamic programme over widths and keep
probabilities.
``calc_precision_device`` runs the same allocation on the GPU for uniform start widths and unit
weights (what every layer asks for at every step), so that no host round trip is needed."""
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


def calc_precision_dp(A, C, max_b, target, states):
    for t, name in ((A, "A"), (C, "C")):
        if not (isinstance(t, torch.Tensor) and t.device.type == "cpu"):
            raise RuntimeError(f"{name} must be a CPU tensor!")           # calc_precision.cc:61-64
        if not t.is_contiguous():
            raise RuntimeError(f"{name} must be contiguous!")
    if A.dtype != torch.float32 or C.dtype != torch.float32 or A.numel() != C.numel():
        raise RuntimeError("calc_precision_dp expects A and C as float32 of the same length")
    b_vec, p_vec = torch.zeros_like(A), torch.zeros_like(A)
    rc = g.lib().actnn_calc_precision_dp(A.data_ptr(), C.data_ptr(), A.numel(), int(max_b), int(target),
                                         int(states), b_vec.data_ptr(), p_vec.data_ptr())
    if rc != 0:
        raise RuntimeError("DP Failed: no path to initial state!" if A.numel() and 0 < int(max_b) <= 30
                           and 0 < int(states) and int(max_b) * int(states) <= 255 and int(target) >= 0
                           else "calc_precision_dp: argument out of range")
    return b_vec, p_vec


DEVICE_MAX_CANDIDATES = 8192


def device_allocation_fits(N, initial_bits):
    return 1 <= int(initial_bits) <= 8 and N * (int(initial_bits) - 1) <= DEVICE_MAX_CANDIDATES


def calc_precision_device(C, initial_bits, target):
    """int32 device tensor [N]: the widths ``calc_precision(ones(N) * initial_bits, C, ones(N),
    target)`` would return, computed on the device of ``C`` (fp32 [N])."""
    if not (isinstance(C, torch.Tensor) and C.is_cuda and C.dtype == torch.float32 and C.dim() == 1):
        raise RuntimeError("C must be a 1-D fp32 device tensor!")
    N = C.numel()
    if not device_allocation_fits(N, initial_bits):
        raise RuntimeError("calc_precision_device: N * (initial_bits - 1) must be <= %d, initial_bits in 1..8"
                           % DEVICE_MAX_CANDIDATES)
    C = C.contiguous()
    bits = torch.empty(N, dtype=torch.int32, device=C.device)
    with g.on_device(C.device):
        check(g.lib().actnn_calc_precision_device(C.data_ptr(), bits.data_ptr(), N, int(initial_bits),
                                                  int(target), g.stream_ptr(C.device)), "calc_precision_device")
    return bits


def allocate_bits_device(mn, mx, N, factor, mult, initial_bits, target, sens_out=None):
    """-> (sensitivity fp32 [N], bits int32 [N], prefix int32 [N + 1]) on the device of mn:
    ``range_sqr`` -> ``calc_precision_device`` -> exclusive prefix of the widths, in one call.
    `sens_out`: where to write the sensitivities (fp32 [N], contiguous, same device)."""
    G = mn.numel() // N
    dev = mn.device
    if sens_out is None:
        sens = torch.empty(N, dtype=torch.float32, device=dev)
    else:
        if sens_out.dtype != torch.float32 or sens_out.device != dev or sens_out.numel() != N or not sens_out.is_contiguous():
            raise RuntimeError("allocate_bits_device: sens_out must be contiguous fp32 [N] on the same device")
        sens = sens_out
    bits = torch.empty(N, dtype=torch.int32, device=dev)
    prefix = torch.empty(N + 1, dtype=torch.int32, device=dev)
    mult_ptr, per_sample = None, 0
    if mult is not None:
        if mult.dtype != torch.float32 or mult.device != dev or mult.numel() not in (1, N):
            raise RuntimeError("allocate_bits_device: mult must be fp32 on the same device with 1 or N values")
        mult = mult.contiguous()
        mult_ptr, per_sample = mult.data_ptr(), int(mult.numel() == N and N != 1)
    with g.on_device(dev):
        check(g.lib().actnn_allocate_bits_device(
            mn.data_ptr(), mx.data_ptr(), float(factor), mult_ptr, per_sample, sens.data_ptr(), bits.data_ptr(),
            prefix.data_ptr(), N, G, int(initial_bits), int(target), g.DTYPE_CODE[mn.dtype], g.stream_ptr(dev)),
            "allocate_bits_device")
    return sens, bits, prefix
