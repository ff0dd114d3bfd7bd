"""Memory accounting and small helpers (reference: actnn/actnn/utils.py:10-80)."""
import json
from collections import OrderedDict

import numpy as np
import torch


def swap_to_cpu(tensor):
    """Asynchronous copy into freshly allocated pinned host memory (utils.py:10-13)."""
    host = torch.empty(tensor.shape, dtype=tensor.dtype, device="cpu", pin_memory=True)
    host.copy_(tensor, non_blocking=True)
    return host


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
            total += int(np.prod(t.size())) * _BYTES.get(t.dtype, 0)
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
