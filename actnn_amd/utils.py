"""Memory accounting and small helpers (reference: actnn/actnn/utils.py:10-80)."""
import json
import weakref
from collections import OrderedDict

import numpy as np
import torch


class _SwapSpace:
    """Host parking for saved tensors (levels L4 / swap; the reference copies with
    `non_blocking=True` on the compute stream, utils.py:10-13, and copies back the same way,
    ops.py:59-60, so every transfer sits in the path of the kernels around it).

    Here a separate copy stream (default priority) carries both directions: a tensor is parked as
    soon as the compute stream has produced it, while the forward pass goes on; in the backward
    pass, asking for a tensor also starts the transfers of the `depth` tensors parked before it -
    the ones the backward pass will ask for next - so that they arrive while the current layer
    computes.  Events order the two streams; `record_stream` keeps every buffer alive until the
    other stream is done with it."""
    depth = 3

    def __init__(self):
        self.streams = {}
        self.parked = []                      # weak references to the host tensors, in parking order

    def _stream(self, device):
        key = torch.device(device).index or 0
        if key not in self.streams:
            self.streams[key] = torch.cuda.Stream(device=device)
        return self.streams[key]

    def park(self, tensor):
        device = tensor.device
        copy = self._stream(device)
        host = torch.empty(tensor.shape, dtype=tensor.dtype, device="cpu", pin_memory=True)
        copy.wait_stream(torch.cuda.current_stream(device))       # the tensor is complete by then
        with torch.cuda.stream(copy):
            host.copy_(tensor, non_blocking=True)
            done = torch.cuda.Event()
            done.record(copy)
        tensor.record_stream(copy)                                 # not reused before the copy has run
        host._actnn_swap = {"done": done, "device": device, "ahead": None}
        if len(self.parked) > 4096:                                # forward-only use: forget the dead ones
            self.parked = [r for r in self.parked if r() is not None]
        self.parked.append(weakref.ref(host))
        return host

    def _start(self, host):
        meta = host._actnn_swap
        if meta["ahead"] is None:
            copy = self._stream(meta["device"])
            with torch.cuda.stream(copy):                          # same stream as the parking copy: ordered
                dev = host.to(meta["device"], non_blocking=True)
                arrived = torch.cuda.Event()
                arrived.record(copy)
            meta["ahead"] = (dev, arrived)

    def fetch(self, host):
        meta = getattr(host, "_actnn_swap", None)
        if meta is None:                                           # not parked by this class
            return host.cuda(non_blocking=True)
        compute = torch.cuda.current_stream(meta["device"])
        self._start(host)
        dev, arrived = meta["ahead"]
        compute.wait_event(arrived)
        dev.record_stream(compute)
        # the backward pass walks the parked tensors last-in first-out: get the next ones moving
        i = next((k for k in range(len(self.parked) - 1, -1, -1) if self.parked[k]() is host), None)
        if i is not None:
            del self.parked[i:]                                    # later ones have been consumed or dropped
            for ref in self.parked[max(0, i - self.depth):i]:
                prev = ref()
                if prev is not None:
                    self._start(prev)
        return dev

    def reset(self):
        self.parked.clear()


swap_space = _SwapSpace()


def swap_to_cpu(tensor):
    """Park a device tensor in pinned host memory (utils.py:10-13); asynchronous, on the copy stream."""
    return swap_space.park(tensor)


def swap_to_device(host):
    """The device copy of a parked tensor, ordered after its transfer on the current stream."""
    return swap_space.fetch(host)


def channels_last_format(t):
    """torch.channels_last / channels_last_3d when `t` is dense in that order and not in the
    default one, else None.  Tensors whose two orders coincide (C == 1 or no spatial extent)
    count as default."""
    if t.dim() == 4 and not t.is_contiguous() and t.is_contiguous(memory_format=torch.channels_last):
        return torch.channels_last
    if t.dim() == 5 and not t.is_contiguous() and t.is_contiguous(memory_format=torch.channels_last_3d):
        return torch.channels_last_3d
    return None


def memory_order(t):
    """`t` with its axes arranged as they lie in memory: a channels-last tensor [N, C, ...]
    comes back as the contiguous view [N, ..., C], everything else unchanged.  On MI355X the
    convolution kernels are channels-last natively, so activations of a channels-last model are
    compressed in that order instead of being transposed first: groups of 256 elements that are
    consecutive in memory, whatever the logical axis order."""
    if channels_last_format(t) is None:
        return t
    return t.permute(0, *range(2, t.dim()), 1)


def logical_order(t_mem, memory_format):
    """Inverse of memory_order for a tensor laid out [N, ..., C] in memory."""
    if memory_format is None:
        return t_mem
    return t_mem.permute(0, t_mem.dim() - 1, *range(1, t_mem.dim() - 1))


def get_memory_usage(print_info=False):
    """Bytes currently allocated by torch's caching allocator on device 0 - the reference's
    memory metric (utils.py:16-23; explicitly not the driver's view)."""
    allocated = torch.cuda.memory_allocated(0)
    if print_info:
        print("allocated: %.2f MB" % (allocated / 1024 / 1024), flush=True)
        print("reserved:  %.2f MB" % (torch.cuda.memory_reserved(0) / 1024 / 1024), flush=True)
    return allocated


_BYTES = {torch.float32: 4, torch.int32: 4, torch.bfloat16: 2, torch.float16: 2, torch.int16: 2,
          torch.int8: 1}


def compute_tensor_bytes(tensors):
    """Bytes held by a tensor or list of tensors, counting exactly the dtypes the reference
    counts (utils.py:26-40); anything else (None, python ints) contributes 0."""
    if not isinstance(tensors, (list, tuple)):
        tensors = [tensors]
    total = 0
    for t in tensors:
        if isinstance(t, torch.Tensor):
            total += t.numel() * _BYTES.get(t.dtype, 0)
    return total


def empty_cache(ratio):
    """Release cached blocks when less than `ratio` of the reserved memory is in use (utils.py:43-49)."""
    if ratio is None:
        return
    allocated = torch.cuda.memory_allocated(0)
    reserved = torch.cuda.memory_reserved(0)
    if reserved > 0 and allocated / reserved < ratio:
        torch.cuda.empty_cache()


class GlobalExpRecorder:
    """Key/value recorder dumped as JSON lines (utils.py:60-80)."""

    def __init__(self):
        self.val_dict = OrderedDict()

    def record(self, key, value, float_round=6):
        if isinstance(value, (np.int32, np.int64)):
            value = int(value)
        if isinstance(value, (float, np.float32, np.float64)):
            value = round(float(value), float_round)
        self.val_dict[key] = value

    def dump(self, filename):
        with open(filename, "a") as f:
            f.write(json.dumps(self.val_dict) + "\n")
        print("Save exp results to %s" % filename)

    def clear(self):
        self.val_dict.clear()


exp_recorder = GlobalExpRecorder()
