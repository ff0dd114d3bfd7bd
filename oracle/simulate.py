"""Restatement of the reference's ``config.simulate`` quantiser (test infrastructure).

Follows actnn/actnn/ops.py:22-41 (quantise) and :55-57 (dequantise).  The only change
is that the uniform noise is an explicit argument instead of being drawn in place
(ops.py:36-38 draws ``output.new(output.shape).uniform_(-0.5, 0.5)``).
"""
import numpy as np
import torch
import torch.nn.functional as F


def quantize_simulate(data, bits, mn, mx, noise=None):
    """ops.py:23-41.  data [N,G,gs]; bits int or int32 tensor [N]; mn/mx [N,G,1].

    Returns (codes int32 [N,G,gs], scale [N,G,1]) exactly as the reference would with
    ``config.simulate = True`` and the given noise tensor (``None`` = not stochastic).
    """
    N = data.shape[0]
    output = data
    if isinstance(bits, int):                       # ops.py:27-28 (device fixed to CPU here)
        bits = torch.ones(N, dtype=torch.int32) * bits
    B = (2 ** bits - 1).view(N, 1, 1)               # ops.py:30
    mn = mn - 1e-6                                  # ops.py:31
    mx = mx + 1e-6                                  # ops.py:32
    scale = B / (mx - mn)                           # ops.py:33
    output = (output - mn) * scale                  # ops.py:34
    if noise is not None:                           # ops.py:36-38
        output.add_(noise)
    output = F.relu(output)                         # ops.py:40
    output = torch.min(output, B.float()).round_().int()   # ops.py:41
    return output, scale


def dequantize_simulate(codes, scale, mn):
    """ops.py:56-57: ``data / scale + mn`` with the *original* (unshifted) minimum."""
    return codes / scale + mn


def quantize_simulate_np(data, bits, mn, mx, noise=None):
    """Independent float32 step-by-step version (numpy, one rounding per operation).

    Used to cross-check ``quantize_simulate``: every line is one IEEE binary32 operation.
    fp32 only.
    """
    x = np.asarray(data, dtype=np.float32)
    N = x.shape[0]
    bits = np.broadcast_to(np.asarray(bits, dtype=np.int64), (N,))
    Bf = ((1 << bits) - 1).astype(np.float32).reshape(N, 1, 1)
    eps = np.float32(1e-6)
    mn_s = (np.asarray(mn, np.float32) - eps).astype(np.float32)
    mx_s = (np.asarray(mx, np.float32) + eps).astype(np.float32)
    den = (mx_s - mn_s).astype(np.float32)
    scale = (Bf / den).astype(np.float32)
    t = (x - mn_s).astype(np.float32)
    t = (t * scale).astype(np.float32)
    if noise is not None:
        t = (t + np.asarray(noise, np.float32)).astype(np.float32)
    t = np.maximum(t, np.float32(0))
    t = np.minimum(t, Bf)
    q = np.rint(t).astype(np.int32)                 # half-to-even, like round_()
    return q, scale


def dequantize_simulate_np(codes, scale, mn):
    q = np.asarray(codes).astype(np.float32)
    return ((q / np.asarray(scale, np.float32)).astype(np.float32)
            + np.asarray(mn, np.float32)).astype(np.float32)


def group_view(x, group_size=256):
    """Grouping rule of ops.py:77-96 / qscheme.py:57-74: flatten [N,-1], zero-pad the
    feature axis to a multiple of ``group_size``, view as [N, G, group_size]."""
    N = x.shape[0]
    flat = x.reshape(N, -1)
    nf = flat.shape[1]
    if nf % group_size != 0:
        new_nf = (nf // group_size + 1) * group_size
        flat = torch.cat([flat, torch.zeros(N, new_nf - nf, dtype=x.dtype)], 1)
    return flat.view(N, -1, group_size)


def minimax(rows):
    """minimax_cuda_kernel.cu:23-67 reduces to row-wise min and max
    (tests/test_minimax.py:20-30 checks it against exactly these two calls)."""
    return torch.min(rows, 1)[0], torch.max(rows, 1)[0]
