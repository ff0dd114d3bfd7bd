"""Shared helpers of the GPU parity tests."""
import numpy as np
import torch

import actnn_amd.cpp_extension.minimax as ext_minimax
import actnn_amd.cpp_extension.quantization as ext_q

DEV = "cuda:0"


def np_bits(t):
    """Raw bit pattern of a float tensor as a numpy integer array (exact comparisons)."""
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.float32:
        return t.numpy().view(np.uint32)
    return t.view(torch.int16).numpy().view(np.uint16)


def make_groups(N, G, gs, dtype, seed, kind="relu", scale=1.0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(N, G, gs, generator=g) * scale
    if kind == "relu":
        x = torch.relu(x)
    elif kind == "chan":       # per-group log-normal scale, like benchmark config 2
        x = torch.relu(x) * torch.exp(torch.randn(1, G, 1, generator=g))
    elif kind == "shift":      # large offset relative to the range
        x = x + 100.0
    x = x.to(dtype)
    noise = (torch.rand(N, G, gs, generator=g) - 0.5).to(dtype)
    return x, noise


def minmax_dev(x_dev):
    N, G, gs = x_dev.shape
    mn, mx = ext_minimax.minimax(x_dev.view(-1, gs))
    return mn.view(N, G, 1), mx.view(N, G, 1)


def bits_tensor(bits_list):
    host = torch.tensor(bits_list, dtype=torch.int32)
    return ext_q.attach_bits_host(host.to(DEV), host), host


def ulp_diff_f32(a, b):
    """|a - b| in units in the last place of fp32 (a, b float32 numpy arrays, same sign region)."""
    ai = a.view(np.int32).astype(np.int64)
    bi = b.view(np.int32).astype(np.int64)
    ai = np.where(ai < 0, np.int64(-2**31) - ai, ai)
    bi = np.where(bi < 0, np.int64(-2**31) - bi, bi)
    return np.abs(ai - bi)
