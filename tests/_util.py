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


def assert_rng_tier(base, bits, codes, mn, scale):
    """The criterion the in-kernel-RNG mode is held to, on `codes` [trials, G, gs] (a device tensor
    of the codes the kernel drew for `trials` independent roundings of the groups `base` [1, G, gs])
    with the kernel's own `mn`, `scale` [1, G, 1]:
      * unbiased: the mean error of the dequantised value code / scale + min over all trials,
        per group, is below 1e-3 of the group's range;
      * per-group variance (summed over the group's elements) within 5 % of the closed form
        sum f (1 - f) / scale^2, f = frac((x - min) * scale)  (quantization_cuda_kernel.cu:63-65,253:
        rounding up with probability f), and within 5 % of the exact variance of the K-bit draw the
        kernels use (oracle.kernel_mode.code_variance; K = 16 for fp32 tensors, 8 for 16-bit ones)."""
    from oracle import kernel_mode
    trials = codes.shape[0]
    B = 2 ** bits - 1
    c = codes.double()
    mean_code = c.mean(dim=0).cpu().numpy()                        # [G, gs]
    var_code = c.var(dim=0, unbiased=True).cpu().numpy()
    sc = scale[0].double().cpu().numpy()                           # [G, 1]
    lo = mn[0].double().cpu().numpy()
    x = base[0].double().numpy()
    t = np.minimum((x - lo) * sc, B)                               # exact position in levels, clamped like the kernel
    rng_ = B / sc                                                  # the group's range as the kernel sees it
    err = (mean_code - t) / sc                                     # mean error of code / scale + min
    assert (np.abs(err.mean(axis=1, keepdims=True)) < 1e-3 * rng_).all()
    # every element: within 5 sigma of the model's expectation
    expect = kernel_mode.expected_code(base, mn[:1].cpu(), scale[:1].cpu(), bits)[0]
    model_var = kernel_mode.code_variance(base, mn[:1].cpu(), scale[:1].cpu(), bits)[0]
    assert (np.abs(mean_code - expect) <= 5 * np.sqrt(model_var / trials) + 1e-9).all()
    f = t - np.floor(t)
    closed = (f * (1 - f) / sc ** 2).sum(axis=1)
    model = (model_var / sc ** 2).sum(axis=1)
    emp = (var_code / sc ** 2).sum(axis=1)
    assert (closed > 0).all()
    assert (np.abs(emp - closed) <= 0.05 * closed).all(), (emp, closed)
    assert (np.abs(emp - model) <= 0.05 * model).all(), (emp, model)
    # ActNN's bound per element: variance <= R^2 / (4 B^2)   (qscheme.py:84)
    assert (var_code / sc ** 2 <= rng_ ** 2 / (4 * B * B) * 1.1 + 1e-30).all()
