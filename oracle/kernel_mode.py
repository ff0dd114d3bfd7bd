"""Arithmetic of the reference's CUDA kernels (not of ``config.simulate``) and the CPU
model of the HIP kernels' in-kernel-RNG mode.  Test infrastructure.

Reference arithmetic (quantization_cuda_kernel.cu):
  scale  = (scalar_t)(2^b - 1) / (max - min + 2e-6)         :32, :220 (the literal is a
           double, so the sum and the quotient are evaluated in double, then narrowed)
  code   = rint(max((x - min) * scale + u - 0.5, 0)), u ~ U(0,1]   :65, :253
  dequant= (scalar_t)code / scale + min                      :171, :359

The HIP kernels draw ``u`` as a K-bit Philox value (K = 16 for fp32 tensors, 8 for fp16 / bf16
tensors) and evaluate the equivalent stochastic floor ``floor(t + u)`` in a 32-bit fixed point
whose top b bits are the code (``rng_codes`` below).  Rounding up with probability frac(t) (to
within 2^-(K+1), centred) is the same distribution as the reference's ``rint(t + u - 0.5)``;
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


def fma32(a, b, c):
    """Correctly rounded float32 fma(a, b, c) of float32 arrays.  The product is exact in float64;
    the float64 sum is turned into round-to-odd with the error term of the addition, after which
    the narrowing to float32 rounds once (Boldo & Melquiond, "Emulation of FMA and correctly
    rounded sums", 2008).  Pinned in tests/test_oracle_kernel_mode.py against exact rational
    arithmetic."""
    a = np.asarray(a, dtype=np.float32).astype(np.float64)
    b = np.asarray(b, dtype=np.float32).astype(np.float64)
    c = np.asarray(c, dtype=np.float32).astype(np.float64)
    a, b, c = np.broadcast_arrays(a, b, c)
    with np.errstate(invalid="ignore", over="ignore"):
        p = a * b
        s = p + c
        bb = s - p
        err = (p - (s - bb)) + (c - bb)                      # TwoSum: p + c = s + err exactly
        inexact = np.isfinite(s) & np.isfinite(err) & (err != 0)
        bits = s.view(np.int64) if s.flags["C_CONTIGUOUS"] else np.ascontiguousarray(s).view(np.int64)
        even = (bits & 1) == 0
        # an inexact sum with an even last bit moves one step towards the true value (then odd)
        toward = np.where((err > 0) == (s > 0), 1, -1)       # the magnitude grows when err has the sign of s
        toward = np.where(s == 0, 0, toward)
        adj = np.where(inexact & even, toward, 0).astype(np.int64)
        s = (bits + adj).view(np.float64)
        return s.astype(np.float32)


def noise_bits(dtype):
    """Bits of the uniform draw per element: 16 for fp32 tensors, 8 for fp16 / bf16 tensors."""
    return 16 if dtype == torch.float32 else 8


def _rng_t(data, mn, scale, bits):
    """The noise-free part t of the HIP kernels' fixed point (one level = 2^(32 - b), one noise
    step U = 2^(32 - b - K)) and U.  fp32 tensors: t = fma(x - mn, scale * 2^(32-b), U/2);
    16-bit tensors: t = fma(x, scale * 2^(32-b), fma(-mn, scale * 2^(32-b), U/2))."""
    N = data.shape[0]
    K = noise_bits(data.dtype)
    b = np.broadcast_to(np.asarray(bits, dtype=np.int64), (N,)).reshape(N, 1, 1)
    x = data.detach().to(torch.float32).numpy()
    m = mn.detach().to(torch.float32).numpy()
    with np.errstate(over="ignore", invalid="ignore"):
        S = (scale.detach().to(torch.float32).numpy() * np.exp2(32 - b).astype(np.float32)).astype(np.float32)
        U = np.exp2(32 - b - K).astype(np.float32)
        if K == 16:
            t = fma32((x - m).astype(np.float32), S, np.float32(0.5) * U)
        else:
            t = fma32(x, S, fma32(-m, S, np.float32(0.5) * U))
    return t, U, b


def _sat_u32(w):
    """v_cvt_u32_f32: truncation, saturating at 0 and 2^32 - 1, NaN -> 0."""
    w = np.nan_to_num(np.asarray(w, dtype=np.float64), nan=0.0, posinf=2.0 ** 32, neginf=0.0)
    return np.clip(np.trunc(w), 0, 2.0 ** 32 - 1).astype(np.uint64)


def _codes_for(t, U, b, r):
    with np.errstate(over="ignore", invalid="ignore"):
        w = fma32(np.asarray(r, dtype=np.float32), U, t)
    return (_sat_u32(w) >> (32 - b).astype(np.uint64)).astype(np.int32)


def rng_codes(data, mn, scale, bits, seed, offset):
    """Codes the HIP RNG-mode kernels must produce (given their Philox stream):
    word = sat_u32(fma(r, U, t)), code = word >> (32 - b)."""
    t, U, b = _rng_t(data, mn, scale, bits)
    e = np.arange(t.size, dtype=np.uint64).reshape(t.shape)
    r = philox.noise16(e, seed, offset) if noise_bits(data.dtype) == 16 else philox.noise8(e, seed, offset)
    return _codes_for(t, U, b, r)


def _round_up_count(data, mn, scale, bits):
    """(code at draw 0, number of draws r in [0, 2^K) that give the next code, K).  The code is
    non-decreasing in r and the draws span less than one level, so the count is found by bisection."""
    t, U, b = _rng_t(data, mn, scale, bits)
    K = noise_bits(data.dtype)
    c0 = _codes_for(t, U, b, np.zeros(t.shape, np.float32))
    lo = np.zeros(t.shape, np.int64)            # invariant: code(lo - 1) == c0 (or lo == 0)
    hi = np.full(t.shape, 1 << K, np.int64)     # invariant: code(hi) > c0 (or hi == 2^K)
    for _ in range(K + 1):
        mid = (lo + hi) // 2
        up = _codes_for(t, U, b, np.minimum(mid, (1 << K) - 1).astype(np.float32)) > c0
        up &= mid < (1 << K)
        hi = np.where(up, mid, hi)
        lo = np.where(up, lo, np.minimum(mid + 1, hi))
    return c0, (1 << K) - hi, K


def expected_code(data, mn, scale, bits):
    """E[code] under the K-bit uniform draw (exact: code(0) + P(next code))."""
    c0, ups, K = _round_up_count(data, mn, scale, bits)
    return c0.astype(np.float64) + ups.astype(np.float64) / (1 << K)


def code_variance(data, mn, scale, bits):
    """Var[code] = p (1 - p), p = P(next code) (exact; ActNN's bound R^2/(4 B^2) per element is its
    maximum, qscheme.py:84)."""
    _, ups, K = _round_up_count(data, mn, scale, bits)
    p = ups.astype(np.float64) / (1 << K)
    return p * (1.0 - p)


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
