"""Arithmetic of the reference's CUDA kernels (not of ``config.simulate``) and the CPU
model of the HIP kernels' in-kernel-RNG mode.  Test infrastructure.

Reference arithmetic (quantization_cuda_kernel.cu):
  scale  = (scalar_t)(2^b - 1) / (max - min + 2e-6)         :32, :220 (the literal is a
           double, so the sum and the quotient are evaluated in double, then narrowed)
  code   = rint(max((x - min) * scale + u - 0.5, 0)), u ~ U(0,1]   :65, :253
  dequant= (scalar_t)code / scale + min                      :171, :359

The HIP kernels draw ``u`` as a 16-bit Philox value and evaluate the equivalent
stochastic floor ``floor(t + u)`` in 16.16 fixed point (``rng_codes`` below).  Rounding up
with probability frac(t) is the same distribution as the reference's ``rint(t + u - 0.5)``;
the stream values themselves are not comparable with cuRAND's (parity unpinned) - the
distribution is pinned by ``expected_code`` / ``code_variance`` (exact closed forms).
"""
import numpy as np
import torch

from . import philox

_NP = {torch.float32: np.float32, torch.float16: np.float16}


def _to_f64(t):
    return t.detach().to(torch.float64).numpy()


def _round_to(t64, dtype):
    """Round a float64 array to ``dtype`` (f32/f16/bf16), return as float64."""
    return torch.from_numpy(np.ascontiguousarray(t64)).to(dtype).to(torch.float64).numpy()


def kernel_scale(mn, mx, bits):
    """.cu:32 / :220.  mn, mx tensors [N,G,1] (f32/f16/bf16), bits int or int tensor [N]."""
    dtype = mn.dtype
    N = mn.shape[0]
    b = np.broadcast_to(np.asarray(bits, dtype=np.int64), (N,)).reshape(N, 1, 1)
    B = ((1 << b) - 1).astype(np.float64)
    # max - min in scalar_t: c10::Half arithmetic widens to float, subtracts, narrows again
    rng = (mx.detach().to(torch.float32) - mn.detach().to(torch.float32)).to(dtype).to(torch.float64).numpy()
    s = B / (rng + 2e-6)                                        # double
    # narrowed on store: double -> float -> scalar_t (c10::Half is constructed from float)
    return torch.from_numpy(s).to(torch.float32).to(dtype)


def kernel_dequant(codes, scale, mn):
    """.cu:171 / :359: per-op rounding in the tensor dtype."""
    dtype = scale.dtype
    q = torch.as_tensor(codes).to(dtype)
    return (q / scale + mn).to(dtype)


def rng_fixed_point(data, mn, scale, bits):
    """16.16 fixed-point image of t = (x - min) * scale as the HIP kernels compute it:
    d = fl32(x - mn); f = fl32(fma(d, scale * 2^16, 0.5)); f = min(f, B * 2^16);
    fix = trunc(max(f, 0)).  Returns uint32 [N,G,gs]."""
    N = data.shape[0]
    b = np.broadcast_to(np.asarray(bits, dtype=np.int64), (N,)).reshape(N, 1, 1)
    B = ((1 << b) - 1).astype(np.float64)
    x = data.detach().to(torch.float32).numpy()
    m = mn.detach().to(torch.float32).numpy()
    d = (x - m).astype(np.float32)
    S = (scale.detach().to(torch.float32).numpy() * np.float32(65536.0)).astype(np.float32)
    f = (d.astype(np.float64) * S.astype(np.float64) + 0.5).astype(np.float32)   # exact fma
    f = np.minimum(f, (B * 65536.0).astype(np.float32))
    f = np.maximum(np.nan_to_num(f, nan=0.0), np.float32(0))
    return np.trunc(f).astype(np.uint32)


def rng_codes(data, mn, scale, bits, seed, offset):
    """Codes the HIP RNG-mode kernels must produce (given their Philox stream)."""
    fix = rng_fixed_point(data, mn, scale, bits)
    e = np.arange(fix.size, dtype=np.uint64).reshape(fix.shape)
    r = philox.noise16(e, seed, offset)
    return ((fix.astype(np.uint64) + r.astype(np.uint64)) >> np.uint64(16)).astype(np.int32)


def expected_code(data, mn, scale, bits):
    """E[code] under the 16-bit stochastic floor = fix / 2^16 (exact)."""
    return rng_fixed_point(data, mn, scale, bits).astype(np.float64) / 65536.0


def code_variance(data, mn, scale, bits):
    """Var[code] = f (1 - f), f = fractional part of fix / 2^16 (exact closed form;
    ActNN's bound R^2/(4 B^2) per element is its maximum, qscheme.py:84)."""
    f = (rng_fixed_point(data, mn, scale, bits) & np.uint32(0xFFFF)).astype(np.float64) / 65536.0
    return f * (1.0 - f)


def range_sqr(mn, mx, factor=1.0, mult=None):
    """Per-sample sensitivity term: factor * mult * sum_g (mx - mn)^2 for mn, mx of shape [N, G]
    (numpy arrays of the activation dtype's values).  Follows actnn/actnn/qscheme.py:80-82
    (``torch.norm((mx - mn).view(N, -1), dim=1).float().square() * (group_size / num_pixels)``,
    then ``num_locations / 4 / depthwise_groups * Range_sqr * grad_sum``): the subtraction rounds
    to the tensor dtype; the square root and re-squaring of the reference are the identity up to
    rounding and are not repeated, the sum is taken in float64 here.  Pinned by the closed form for
    constant ranges (tests/test_oracle_simulate.py) and by torch's own expression on random data."""
    import numpy as np
    d = (np.asarray(mx) - np.asarray(mn)).astype(np.asarray(mn).dtype)      # rounds like the tensor op
    v = (d.astype(np.float64) ** 2).sum(axis=1) * float(factor)
    if mult is not None:
        v = v * np.asarray(mult, dtype=np.float64)
    return v
