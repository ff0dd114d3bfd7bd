"""Plumbing between torch tensors and the C ABI: argument checks that mirror the reference's
CHECK_CUDA_TENSOR_* macros (cpp_extension/ext_common.h), dtype codes, the current HIP stream
and the Philox (seed, offset) taken from torch's default device generator."""
import torch

from .. import _lib

DTYPE_CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def lib():
    return _lib.load()


def _name_check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def check_float(t, name, dim=None):
    """CHECK_CUDA_TENSOR_FLOAT / CHECK_CUDA_TENSOR_DIM_FLOAT (ext_common.h:14-27);
    bf16 is accepted in addition to the reference's f32/f16."""
    _name_check(isinstance(t, torch.Tensor) and t.is_cuda, f"{name} must be a CUDA tensor!")
    _name_check(t.is_contiguous(), f"{name} must be contiguous!")
    if dim is not None:
        _name_check(t.dim() == dim, f"The dimension of {name} is not correct!")
    _name_check(t.dtype in DTYPE_CODE, f"The type of {name} is not correct!")


def check_typed(t, name, dtype, dim=None):
    """CHECK_CUDA_TENSOR_TYPE / CHECK_CUDA_TENSOR_DIM_TYPE (ext_common.h:1-12)."""
    _name_check(isinstance(t, torch.Tensor) and t.is_cuda, f"{name} must be a CUDA tensor!")
    _name_check(t.is_contiguous(), f"{name} must be contiguous!")
    if dim is not None:
        _name_check(t.dim() == dim, f"The dimension of {name} is not correct!")
    _name_check(t.dtype == dtype, f"The type of {name} is not correct!")


def stream_ptr(device):
    """The current HIP stream of `device` as an integer (one C call; the Stream object that
    torch.cuda.current_stream builds costs several microseconds per kernel launch)."""
    index = device.index
    if index is None:
        index = torch.cuda.current_device()
    return torch._C._cuda_getCurrentRawStream(index)


class on_device:
    """`with on_device(t.device):` - makes the tensor's device current for the launch, like
    torch.cuda.device, but does nothing at all in the usual case that it already is."""
    __slots__ = ("index", "previous")

    def __init__(self, device):
        self.index = device.index
        self.previous = -1

    def __enter__(self):
        if self.index is not None:
            current = torch._C._cuda_getDevice()
            if current != self.index:
                self.previous = current
                torch.cuda.set_device(self.index)
        return self

    def __exit__(self, *exc):
        if self.previous >= 0:
            torch.cuda.set_device(self.previous)
        return False


def aligned(t):
    """The kernels use 16-byte vector accesses; torch allocations are 256-byte aligned, only
    views with a storage offset can break this."""
    return t if t.data_ptr() % 16 == 0 else t.clone()


def philox_args(device, increment=4):
    """(seed, offset) of the device's default generator, advancing the offset - the
    counterpart of CUDAGeneratorImpl::philox_engine_inputs under the generator mutex
    (quantization_cuda_kernel.cu:115-121)."""
    gen = torch.cuda.default_generators[device.index if device.index is not None
                                        else torch.cuda.current_device()]
    seed = gen.initial_seed()
    offset = gen.get_offset()
    gen.set_offset(offset + increment)
    return seed & 0xFFFFFFFFFFFFFFFF, offset & 0xFFFFFFFFFFFFFFFF
