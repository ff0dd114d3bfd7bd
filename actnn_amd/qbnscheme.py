"""Bit allocation for batch-norm inputs (behaviour of actnn/actnn/qbnscheme.py:9-60): the
sensitivity is the range term alone and the per-layer budget follows the preceding conv/linear."""
from .conf import config
from .qscheme import (AllocationArgs, PendingBits, QScheme, allocate_bits_on_device, allocate_on_device,
                      greedy_bits, group_min_max, range_sqr)


class QBNScheme(QScheme):
    layers = []

    def __init__(self, group=0):
        self.initial_bits = config.initial_bits
        self.bits = config.activation_compression_bits[group]
        QBNScheme.layers.append(self)
        self.prev_linear = QScheme.layers[-1] if len(QScheme.layers) > 0 else None

    def start_quantization_bits(self, input, known_minmax=None):
        self.prev_linear = QScheme.prev_layer
        N = input.shape[0]
        groups, mn, mx, num_pixels = group_min_max(input, known_minmax)
        if allocate_on_device(N, self.initial_bits) and mn.is_contiguous() and mx.is_contiguous():
            _, bits_dev = allocate_bits_on_device(mn, mx, N, num_pixels, 1.0, None, self.initial_bits, self.bits)
            return groups, mn, mx, None, input.numel() // N, bits_dev
        C_dev = range_sqr(mn, mx, N, num_pixels)                           # qbnscheme.py:44-47
        return groups, mn, mx, PendingBits(C_dev), input.numel() // N, None

    def allocation_arguments(self, N, num_pixels, device):
        self.prev_linear = QScheme.prev_layer
        if not allocate_on_device(N, self.initial_bits):
            return None
        return AllocationArgs(N, config.group_size / num_pixels, None, self.initial_bits, self.bits)

    def adopt_device_bits(self, bits_dev, dim, args):
        pass

    def finish_quantization_bits(self, started):
        groups, mn, mx, pending, _, bits_dev = started
        N = groups.shape[0]
        if bits_dev is None:
            bits_dev, _ = greedy_bits(pending.wait().clone(), N, self.initial_bits, self.bits, groups.device)
        return groups, bits_dev, mn.view(N, -1, 1), mx.view(N, -1, 1)

    @staticmethod
    def allocate_perlayer():
        for layer in QBNScheme.layers:
            layer.bits = layer.prev_linear.bits if layer.prev_linear is not None else 8

    @staticmethod
    def reset():
        QBNScheme.layers = []
