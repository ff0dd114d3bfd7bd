"""Per-sample / per-layer bit allocation policy for conv and linear inputs
(behaviour of the reference's actnn/actnn/qscheme.py:9-147, restated for this build).

Sensitivity of sample n:  C_n = num_locations / 4 / depthwise_groups * Range_sqr_n * grad_scale
with Range_sqr_n = ||max - min||^2 over the sample's groups * (group_size / pixels per channel);
bits come from the greedy allocation `calc_precision` starting at `initial_bits` down to an
average of `bits` per sample.
"""
import torch

from .conf import config
from .cpp_extension import backward_func as ext_backward_func
from .cpp_extension import calc_precision as ext_calc_precision
from .cpp_extension import minimax as ext_minimax
from .cpp_extension.quantization import attach_bits_host, attach_bits_total
from .utils import memory_order


def group_min_max(input, known=None, whole_tensor_range=None):
    """Flatten to [N, -1], zero-pad the feature axis to a multiple of group_size, view as groups
    and reduce each group (qscheme.py:59-74).  Returns (groups [N,G,gs], mn [N*G], mx [N*G],
    pixels per channel).  `known` = (mn, mx) already produced by another pass over the same
    tensor (the batch-norm statistics kernel); only given when no padding is needed.
    `whole_tensor_range`: replace the group ranges by the tensor's (default: `not config.pergroup`,
    the scheme's rule, qscheme.py:75-77)."""
    N = input.shape[0]
    flat = memory_order(input).reshape(N, -1)            # a view for default and channels-last layouts
    features = flat.shape[1]
    num_pixels = features // input.shape[1]
    gs = config.group_size
    if features % gs != 0:
        padded = (features // gs + 1) * gs
        flat = torch.cat([flat, torch.zeros(N, padded - features, dtype=input.dtype, device=input.device)], 1)
    elif not flat.is_contiguous():
        flat = flat.contiguous()
    rows = flat.view(-1, gs)
    mn, mx = known if known is not None else ext_minimax.minimax(rows)
    if whole_tensor_range is None:
        whole_tensor_range = not config.pergroup
    if whole_tensor_range:                      # one range for the whole tensor (qscheme.py:75-77)
        mn = torch.ones_like(mn) * mn.min()
        mx = torch.ones_like(mx) * mx.max()
    return rows.view(N, -1, gs), mn, mx, num_pixels


def range_sqr(mn, mx, N, num_pixels, factor=1.0, mult=None):
    """fp32 [N]: factor * mult * G * ||R_n||^2 / I  (qscheme.py:80-82), one kernel per call."""
    return ext_minimax.range_sqr(mn, mx, N, factor * config.group_size / num_pixels, mult)


class PendingBits:
    """Per-sample widths whose sensitivities are still on their way to the host.

    The allocation needs the ranges of every group of a sample on the CPU (greedy heap), which
    costs one device->host round trip per layer.  `start` queues the copy into pinned memory and
    records an event; the caller then launches the layer's own forward computation, and `finish`
    waits for the event only - so the GPU keeps working during the round trip instead of idling
    as it does with the reference's blocking `.cpu()` (qscheme.py:83-85)."""

    def __init__(self, C_dev, previous=None):
        # `previous`: the same layer's object of the step before, whose pinned buffer and event are
        # taken over (its values were picked up at the end of that step, or never will be)
        if previous is not None and previous.host.shape == C_dev.shape:
            self.host, self.event = previous.host, previous.event
        else:
            self.host = torch.empty(C_dev.shape, dtype=torch.float32, pin_memory=True)
            self.event = torch.cuda.Event()
        self.host.copy_(C_dev if C_dev.dtype == torch.float32 else C_dev.to(torch.float32), non_blocking=True)
        self.event.record()

    def wait(self):
        self.event.synchronize()
        return self.host


class SensitivityPool:
    """One device buffer and one pinned host buffer for the sensitivities of every layer of a step.

    With the widths made on the device, the host needs the sensitivities only at the end of the step
    (per-layer re-balancing).  A copy per layer put a device->host transfer and an event between the
    kernels of every layer; here every layer's allocation kernel writes its row of one [layers, N]
    buffer, and the whole buffer goes to the host in a single transfer, queued when the first
    backward of the step starts (behind the forward's kernels, ahead of the backward's, so that it
    has long arrived when the last backward asks for it)."""

    def __init__(self, rows, N, device):
        self.dev = torch.empty((rows, N), dtype=torch.float32, device=device)
        self.host = torch.empty((rows, N), dtype=torch.float32, pin_memory=True)
        self.event = torch.cuda.Event()
        self.dirty = False           # rows written since the last transfer
        self.rows = [self.dev[i] for i in range(rows)]

    def fits(self, rows, N, device):
        return self.dev.shape[0] >= rows and self.dev.shape[1] == N and self.dev.device == device

    def flush(self):
        """Queue the transfer if any row has been written since the last one."""
        if self.dirty:
            self.host.copy_(self.dev, non_blocking=True)
            self.event.record()
            self.dirty = False

    def row_on_host(self, index):
        self.flush()
        self.event.synchronize()
        return self.host[index].clone()


class _PooledRow:
    """What a layer keeps of its row of the pool: `wait()` as PendingBits has it."""

    def __init__(self, pool, index):
        self.pool, self.index = pool, index

    def wait(self):
        return self.pool.row_on_host(self.index)


def greedy_bits(C_host, N, initial_bits, avg_bits, device):
    """Per-sample widths: calc_precision(b = initial_bits, C, w = 1, target = int(avg_bits * N)),
    returned on the device with the host copy attached (qscheme.py:86-94)."""
    b = torch.ones(N, dtype=torch.int32) * int(initial_bits)
    w = torch.ones(N, dtype=torch.int32)
    b = ext_calc_precision.calc_precision(b, C_host, w, int(avg_bits * N))
    return attach_bits_host(b.to(device, non_blocking=True), b), b


def greedy_bits_device(C_dev, N, initial_bits, avg_bits):
    """The same widths computed on the device (no round trip): only their sum - fixed by the
    budget - is known on the host, which is all pack / unpack need to size the stream."""
    initial = int(initial_bits)
    target = int(avg_bits * N)
    bits = ext_calc_precision.calc_precision_device(C_dev, initial, target)
    taken = min(max(N * initial - target, 0), N * (initial - 1))
    return attach_bits_total(bits, N * initial - taken)


def allocate_bits_on_device(mn, mx, N, num_pixels, factor, mult, initial_bits, avg_bits, sens_out=None):
    """Sensitivities, widths and the prefix of the widths in one call -> (C on the device, bits
    with their sum and prefix attached).  `sens_out`: fp32 [N] on the device to write C into."""
    args = AllocationArgs(N, factor * config.group_size / num_pixels, mult, initial_bits, avg_bits, sens_out)
    C_dev, bits, prefix = ext_calc_precision.allocate_bits_device(
        mn, mx, N, args.factor, mult, args.initial, args.target, sens_out)
    return C_dev, attach_bits_total(bits, args.total, prefix)


def allocate_on_device(N, initial_bits):
    return config.device_allocation and ext_calc_precision.device_allocation_fits(N, initial_bits)


class AllocationArgs:
    """What the allocation kernels need for one layer's input (allocate_bits_on_device's arguments,
    resolved): `factor` and `mult` of the sensitivity, start width and target sum of the widths,
    the sum the widths will have (fixed by the budget, so the stream can be sized without a look
    at them), where the sensitivities go (a row of the step's pool, or None) and what the scheme
    keeps to read them back."""
    __slots__ = ("factor", "mult", "initial", "target", "total", "sens_out", "pending")

    def __init__(self, N, factor, mult, initial_bits, avg_bits, sens_out=None, pending=None):
        self.factor = float(factor)
        self.mult = mult
        self.initial = int(initial_bits)
        self.target = int(avg_bits * N)
        taken = min(max(N * self.initial - self.target, 0), N * (self.initial - 1))
        self.total = N * self.initial - taken
        self.sens_out = sens_out
        self.pending = pending


class _LazyHost:
    """Attribute pair for values whose host copy may still be in flight: `C` (sensitivities, wanted
    by the per-layer re-balancing at the end of the step) and `b` (widths, wanted by tests)."""

    def _get_C(self):
        pending = getattr(self, "_pending_C", None)
        if pending is not None:
            self._C = pending.wait().clone()
            self._pending_C = None
        return getattr(self, "_C", None)

    def _set_C(self, value):
        self._pending_C = None
        self._C = value

    C = property(_get_C, _set_C)

    def _get_b(self):
        b = getattr(self, "_b", None)
        return b.cpu() if isinstance(b, torch.Tensor) and b.is_cuda else b

    def _set_b(self, value):
        self._b = value

    b = property(_get_b, _set_b)


class QScheme(_LazyHost):
    num_samples = 1        # dataset size, only used with config.use_gradient
    num_layers = 0
    batch = None           # dataset indices of the current batch (config.use_gradient)
    update_scale = True
    layers = []
    prev_layer = None
    sensitivity_pool = None

    @staticmethod
    def pool_row(index, N, device):
        """Row `index` of the step's sensitivity pool (made, or made anew, when the number of layers,
        the batch size or the device changes)."""
        pool = QScheme.sensitivity_pool
        if pool is None or not pool.fits(len(QScheme.layers), N, device):
            if pool is not None:
                pool.flush()
                pool.event.synchronize()         # rows handed out earlier keep their host values
            pool = QScheme.sensitivity_pool = SensitivityPool(len(QScheme.layers), N, device)
        pool.dirty = True
        return pool, pool.rows[index]

    def __init__(self, layer, group=0, num_locations=1, depthwise_groups=1):
        self.initial_bits = config.initial_bits
        self.bits = config.activation_compression_bits[group]
        if config.use_gradient:
            assert QScheme.num_samples > 1
            self.scales = torch.zeros(QScheme.num_samples)
        else:
            self.scales = torch.tensor([0.0])
        self.index = len(QScheme.layers)            # row of the sensitivity pool
        QScheme.layers.append(self)
        self.C = None
        self.b = None
        self.dim = None
        self.num_locations = num_locations          # kernel positions per output
        self.depthwise_groups = depthwise_groups
        self.layer = layer
        self.group = group
        self.name = "layer_{}".format(QScheme.num_layers)
        QScheme.num_layers += 1

    # -- gradient statistics ----------------------------------------------------------------
    _batch_index_cache = None

    @staticmethod
    def batch_index(device):
        """QScheme.batch as an int64 index tensor on `device`, converted once per batch and device
        (the list object is held, so a new batch is a new object)."""
        cached = QScheme._batch_index_cache
        if cached is None or cached[0] is not QScheme.batch or cached[1] != device:
            index = torch.as_tensor(QScheme.batch, dtype=torch.long).to(device)
            QScheme._batch_index_cache = cached = (QScheme.batch, device, index)
        return cached[2]

    def get_scale(self, device=None):
        """Gradient statistic of the current batch (qscheme.py:37-45).  With config.use_gradient the
        per-sample table moves to `device` on first use and stays there: looking up and updating a
        batch's entries are indexed device operations, without a host round trip per layer."""
        if config.use_gradient:
            assert QScheme.batch is not None
            if device is not None and self.scales.device != device:
                self.scales = self.scales.to(device)
            scale = self.scales[QScheme.batch_index(self.scales.device)]
            return torch.where(scale == 0, scale.mean() + 1e-9, scale)     # samples not seen yet
        return self.scales

    def set_scale(self, grad):
        """Squared gradient norm per sample, kept as a running value (qscheme.py:47-55)."""
        if QScheme.sensitivity_pool is not None:
            QScheme.sensitivity_pool.flush()        # (called from every backward: the first one queues the transfer)
        if not QScheme.update_scale:
            return
        if not config.use_gradient and config.share_grad_sqnorm:
            total = ext_backward_func.known_sumsq(grad)     # left by the kernel that wrote `grad`
            if total is not None:
                self.scales = total / grad.shape[0]
                return
        # squared L2 norm per sample, accumulated in fp32 in one pass over the gradient
        sq = ext_minimax.sample_sqnorm(grad)
        if config.use_gradient:
            assert QScheme.batch is not None
            if self.scales.device != sq.device:
                self.scales = self.scales.to(sq.device)
            index = QScheme.batch_index(sq.device)
            self.scales[index] = self.scales[index] * 0.5 + sq * 0.5
        else:
            self.scales = sq.mean()

    # -- forward-time allocation ------------------------------------------------------------
    def sensitivity(self, mn, mx, N, num_pixels):
        """C_n = num_locations / 4 / depthwise_groups * Range_sqr_n * grad_sum_n  (qscheme.py:80-82)."""
        grad_sum = self.get_scale(mn.device).to(device=mn.device, dtype=torch.float32)
        return range_sqr(mn, mx, N, num_pixels, self.num_locations / 4 / self.depthwise_groups, grad_sum)

    def compute_quantization_bits(self, input):
        """-> (groups [N,G,gs], bits on device, mn [N,G,1], mx [N,G,1])  (qscheme.py:57-94)."""
        return self.finish_quantization_bits(self.start_quantization_bits(input))

    def allocation_arguments(self, N, num_pixels, device):
        """The layer's AllocationArgs when its widths are made on the device, else None; with the
        bookkeeping of start_quantization_bits (this layer becomes the one a batch norm follows, its
        row of the sensitivity pool is claimed)."""
        QScheme.prev_layer = self
        if not allocate_on_device(N, self.initial_bits):
            return None
        grad_sum = self.get_scale(device).to(device=device, dtype=torch.float32)
        pool, row = QScheme.pool_row(self.index, N, device)
        return AllocationArgs(N, self.num_locations / 4 / self.depthwise_groups * config.group_size / num_pixels,
                              grad_sum, self.initial_bits, self.bits, row, _PooledRow(pool, self.index))

    def adopt_device_bits(self, bits_dev, dim, args):
        """What finish_quantization_bits records when the widths were made on the device."""
        self.dim = dim
        self._pending_C = args.pending
        self.b = bits_dev

    def start_quantization_bits(self, input, known_minmax=None):
        """First half: min/max kernel, sensitivities, asynchronous copy to the host."""
        QScheme.prev_layer = self
        N = input.shape[0]
        groups, mn, mx, num_pixels = group_min_max(input, known_minmax)
        bits_dev = None
        if allocate_on_device(N, self.initial_bits) and mn.is_contiguous() and mx.is_contiguous():
            grad_sum = self.get_scale(mn.device).to(device=mn.device, dtype=torch.float32)
            pool, row = QScheme.pool_row(self.index, N, mn.device)
            _, bits_dev = allocate_bits_on_device(
                mn, mx, N, num_pixels, self.num_locations / 4 / self.depthwise_groups, grad_sum,
                self.initial_bits, self.bits, row)
            pending = _PooledRow(pool, self.index)
        else:
            C_dev = self.sensitivity(mn, mx, N, num_pixels)
            pending = self._last_pending = PendingBits(C_dev, getattr(self, "_last_pending", None))
        return groups, mn, mx, pending, input.numel() // N, bits_dev

    def finish_quantization_bits(self, started):
        """Second half.  Widths made on the device: nothing to wait for (the host copy of the
        sensitivities is picked up when the per-layer re-balancing asks for it).  Otherwise: wait
        for the sensitivities, greedy allocation on the host, widths back to the device."""
        groups, mn, mx, pending, dim, bits_dev = started
        N = groups.shape[0]
        self.dim = dim
        if bits_dev is not None:
            self._pending_C = pending
            self.b = bits_dev
        else:
            C = pending.wait().clone()
            bits_dev, b = greedy_bits(C, N, self.initial_bits, self.bits, groups.device)
            self.C = C
            self.b = b
        return groups, bits_dev, mn.view(N, -1, 1), mx.view(N, -1, 1)

    # -- per-layer re-balancing -------------------------------------------------------------
    @staticmethod
    def allocate_perlayer():
        """One greedy pass over all layers of a group (qscheme.py:96-128): either one item per
        layer (when the group's budget equals initial_bits) or one item per (layer, sample)."""
        for g, avg in enumerate(config.activation_compression_bits):
            layers = [l for l in QScheme.layers if l.group == g]
            L = len(layers)
            if L == 0:
                continue
            if avg == config.initial_bits:
                C = torch.tensor([float(l.C.sum()) for l in layers])
                w = torch.tensor([l.dim for l in layers], dtype=torch.int32)
                b = ext_calc_precision.calc_precision(torch.ones(L, dtype=torch.int32) * 8, C, w,
                                                      float(w.sum() * avg))
                for i, l in enumerate(layers):
                    l.bits = l.initial_bits = b[i]
            else:
                N = layers[0].C.shape[0]
                C = torch.cat([l.C for l in layers], 0)
                # (every layer's dim N times, and every layer's mean width, each in one tensor operation:
                # 54 small ones per step cost more than the allocation itself)
                w = torch.tensor([l.dim for l in layers], dtype=torch.int32).repeat_interleave(N)
                b = torch.ones(N * L, dtype=torch.int32) * config.initial_bits
                b = ext_calc_precision.calc_precision(b, C, w, float(w.sum() * avg))
                means = b.view(L, N).float().mean(1)
                for i, l in enumerate(layers):
                    l.bits = means[i]

    def if_allocate_perlayer(self):
        """Called at the end of every layer's backward; the layer whose backward runs last (the
        first one with a trainable weight) triggers the re-balancing (qscheme.py:130-147)."""
        if not (config.perlayer and config.compress_activation and config.training):
            return
        first = next((l for l in QScheme.layers if l.layer.weight.requires_grad), None)
        if self is not first or any(l.C is None for l in QScheme.layers):
            return
        from .qbnscheme import QBNScheme
        QScheme.allocate_perlayer()
        QBNScheme.allocate_perlayer()

    @staticmethod
    def reset():
        """Forget every registered scheme (build-side helper for tests and repeated model builds)."""
        QScheme.layers = []
        QScheme.num_layers = 0
        QScheme.prev_layer = None
        QScheme.batch = None
        QScheme._batch_index_cache = None
        QScheme.sensitivity_pool = None
