"""Pins oracle/kernel_mode.py::kernel_scale and ::kernel_dequant - the restatement of the
reference CUDA kernels' scale and dequantisation arithmetic (quantization_cuda_kernel.cu:32, :220
scale; :171, :359 dequantise) - on the CPU, without the HIP kernels:

* hand-checked known answers, found by a search over every positive fp16 range, where a plausible
  mistake gives another stored value: evaluating B / (range + 2e-6) in float instead of double
  (the literal 2e-6 is a double, so the sum and the quotient are doubles), or narrowing the double
  straight to half instead of double -> float -> half (c10::Half is only constructible from float);
* an exact rational-arithmetic model (fractions.Fraction with explicit round-to-nearest-even into
  each binary format) of the same chain, compared over random inputs for f32 / f16 / bf16;
* the special cases: a constant group (range 0) gives B / 2e-6, which is +inf in fp16 and finite
  in f32 / bf16; dequantising with an infinite scale returns the minimum; B = 255.
For bf16 no positive range and no width 1..8 exists where float and double evaluation differ (full
scan), so the double claim is not observable there; the chain is still checked against the model.
"""
import struct
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import kernel_mode as km

FORMATS = {"f64": (53, -1022, 1023), "f32": (24, -126, 127), "f16": (11, -14, 15), "bf16": (8, -126, 127)}


def rn(x, fmt):
    """Round the rational x to the nearest value of a binary format (ties to even), as a Fraction;
    float('inf') on overflow.  Written from the definition, independent of numpy / torch casts."""
    p, emin, emax = FORMATS[fmt]
    if x == 0:
        return Fraction(0)
    sign = -1 if x < 0 else 1
    a = abs(Fraction(x))
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    e = max(e, emin)
    quantum = Fraction(2) ** (e - p + 1)
    q = a / quantum
    n = q.numerator // q.denominator
    rem = q - n
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and n % 2 == 1):
        n += 1
    r = n * quantum
    if r >= Fraction(2) ** (emax + 1):
        return float("inf") * sign
    return sign * r


def model_scale(mn_fr, mx_fr, B, fmt):
    """.cu:32: scalar_t range; double sum with the double literal 2e-6; double quotient; stored
    through float into scalar_t."""
    rng = rn(mx_fr - mn_fr, fmt)
    den = rn(rng + Fraction(2e-6), "f64")
    q = rn(Fraction(B) / den, "f64")
    f = rn(q, "f32")
    return f if isinstance(f, float) else rn(f, fmt)


def f16_from_bits(b):
    return torch.tensor([b], dtype=torch.int16).view(torch.float16)


def bits_of(t):
    if t.dtype == torch.float32:
        return int(t.view(torch.int32).item()) & 0xFFFFFFFF
    return int(t.view(torch.int16).item()) & 0xFFFF


# (bits, fp16 bit pattern of the range, stored scale, what the mistake would store)
F16_FLOAT_EVALUATION_DIFFERS = [(1, 16460, 14194, 14195), (2, 1877, 30319, 30318), (4, 3282, 31278, 31279),
                                (5, 17178, 18525, 18526), (6, 12335, 24455, 24456), (8, 12984, 25790, 25791)]
F16_DIRECT_NARROWING_DIFFERS = [(3, 2963, 30548, 30549), (4, 7515, 27034, 27033), (5, 7015, 28720, 28719),
                                (5, 17380, 18396, 18395)]
# fp32: (bits, bit pattern of the range, stored scale, the all-float result)
F32_FLOAT_EVALUATION_DIFFERS = [(2, 1115606168, 1027663780, 1027663779), (2, 1079480562, 1063519083, 1063519084),
                                (2, 1109989653, 1032934907, 1032934906)]


@pytest.mark.parametrize("bits,range_bits,want,mistake",
                         F16_FLOAT_EVALUATION_DIFFERS + F16_DIRECT_NARROWING_DIFFERS)
def test_fp16_scale_known_answers(bits, range_bits, want, mistake):
    rng = f16_from_bits(range_bits)
    mn = torch.zeros(1, 1, 1, dtype=torch.float16)
    got = bits_of(km.kernel_scale(mn, rng.view(1, 1, 1), bits))
    assert got == want != mistake
    # the exact model agrees with the literal
    B = (1 << bits) - 1
    m = model_scale(Fraction(0), Fraction(float(rng)), B, "f16")
    assert bits_of(torch.tensor([float(m)], dtype=torch.float16)) == want


@pytest.mark.parametrize("bits,range_bits,want,mistake", F32_FLOAT_EVALUATION_DIFFERS)
def test_fp32_scale_known_answers(bits, range_bits, want, mistake):
    rng = torch.tensor([range_bits], dtype=torch.int32).view(torch.float32)
    mn = torch.zeros(1, 1, 1)
    assert bits_of(km.kernel_scale(mn, rng.view(1, 1, 1), bits)) == want != mistake
    # a shifted minimum leaves max - min (one float subtraction) and so the scale unchanged when exact
    assert bits_of(km.kernel_scale(mn + 2.0, (rng + 2.0).view(1, 1, 1), bits)) == \
        bits_of(km.kernel_scale(mn, ((rng + 2.0) - 2.0).view(1, 1, 1), bits))


@pytest.mark.parametrize("dtype,fmt", [(torch.float32, "f32"), (torch.float16, "f16"), (torch.bfloat16, "bf16")])
def test_scale_matches_the_exact_model(dtype, fmt):
    g = torch.Generator().manual_seed(3)
    N, G = 8, 40
    mn = (torch.randn(N, G, 1, generator=g) * 3).to(dtype)
    mx = (mn.float() + torch.rand(N, G, 1, generator=g) * torch.exp(2 * torch.randn(N, G, 1, generator=g))).to(dtype)
    bits = torch.tensor([1, 2, 3, 4, 5, 6, 7, 8], dtype=torch.int32)
    got = km.kernel_scale(mn, mx, bits.numpy())
    for n in range(N):
        B = (1 << int(bits[n])) - 1
        for j in range(G):
            m = model_scale(Fraction(float(mn[n, j, 0])), Fraction(float(mx[n, j, 0])), B, fmt)
            assert float(got[n, j, 0]) == float(m), (n, j)


def test_constant_group_and_widest_code():
    # range 0: B / 2e-6.  fp16 cannot hold it (max 65504) -> +inf; f32 / bf16 can
    z16 = torch.full((1, 1, 1), 0.75, dtype=torch.float16)
    assert torch.isinf(km.kernel_scale(z16, z16, 2)).all()
    z32 = torch.full((1, 1, 1), 0.75)
    assert float(km.kernel_scale(z32, z32, 2)) == 1500000.0            # 3 / 2e-6 rounds to 1.5e6 in f32
    assert float(km.kernel_scale(z32, z32, 8)) == 127500000.0          # 255 / 2e-6
    zb = torch.full((1, 1, 1), 0.75, dtype=torch.bfloat16)
    assert bits_of(km.kernel_scale(zb, zb, 2)) == 0x49B7                # 1.5e6 = 0x49B71B00 -> bf16 0x49B7
    # dequantising with an infinite scale gives the minimum for every code (code / inf = 0)
    codes = torch.tensor([[[0, 1, 2, 3]]])
    out = km.kernel_dequant(codes, km.kernel_scale(z16, z16, 2), z16)
    assert out.dtype == torch.float16 and bool((out == 0.75).all())


@pytest.mark.parametrize("dtype,fmt", [(torch.float32, "f32"), (torch.float16, "f16"), (torch.bfloat16, "bf16")])
def test_dequant_rounds_once_per_operation(dtype, fmt):
    # (scalar_t)code / scale + min: the quotient is rounded to scalar_t before the sum (.cu:171, :359)
    g = torch.Generator().manual_seed(5)
    scale = (torch.rand(6, 5, 1, generator=g) * 40 + 0.3).to(dtype)
    mn = (torch.randn(6, 5, 1, generator=g)).to(dtype)
    codes = torch.randint(0, 256, (6, 5, 7), generator=g)
    got = km.kernel_dequant(codes, scale, mn)
    fused_differs = 0
    for n in range(6):
        for j in range(5):
            s, m = Fraction(float(scale[n, j, 0])), Fraction(float(mn[n, j, 0]))
            for k in range(7):
                c = Fraction(int(codes[n, j, k]))
                want = rn(rn(c / s, fmt) + m, fmt)
                assert float(got[n, j, k]) == float(want)
                fused_differs += float(rn(c / s + m, fmt)) != float(want)
    if fmt != "f32":
        assert fused_differs > 0        # the test would notice a single-rounding implementation


def test_fma32_rounds_once():
    # against exact rational arithmetic, with cancelling addends (where a product rounded first, or a
    # float64 sum rounded a second time, gives another answer)
    rng = np.random.default_rng(0)
    n = 3000
    a = (rng.standard_normal(n) * 10.0 ** rng.integers(-3, 6, n)).astype(np.float32)
    b = (rng.standard_normal(n) * 10.0 ** rng.integers(-3, 6, n)).astype(np.float32)
    c = (rng.standard_normal(n) * 10.0 ** rng.integers(-3, 9, n)).astype(np.float32)
    c[: n // 3] = (-a[: n // 3].astype(np.float64) * b[: n // 3]).astype(np.float32)
    got = km.fma32(a, b, c)
    product_first_differs = 0
    for i in range(n):
        exact = Fraction(float(a[i])) * Fraction(float(b[i])) + Fraction(float(c[i]))
        assert float(got[i]) == float(rn(exact, "f32")), i
        product_first_differs += float(np.float32(a[i] * b[i]) + c[i]) != float(got[i])
    assert product_first_differs > 0
    # ties of the float64 sum that a second rounding would resolve the wrong way
    one, eps = np.float32(1.0), np.float32(2.0 ** -24)
    assert float(km.fma32(one, one + np.float32(2.0 ** -23), -one)) == 2.0 ** -23
    assert float(km.fma32(np.float32(1 + 2.0 ** -23), np.float32(1 + 2.0 ** -23), eps * eps)) == \
        float(rn(Fraction(1 + 2.0 ** -23) ** 2 + Fraction(2.0 ** -48), "f32"))


@pytest.mark.parametrize("dtype,K", [(torch.float32, 16), (torch.float16, 8), (torch.bfloat16, 8)])
def test_rng_model_rounds_up_with_probability_of_the_fraction(dtype, K):
    # brute force over every draw on a small case: the mean code is the exact t to within half a
    # step of the draw (plus, for 16-bit tensors, the rounding of the folded constant), for each width
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(8, 2, 256, generator=g) * 3 + 1).to(dtype)
    mn, mx = x.min(2, keepdim=True)[0], x.max(2, keepdim=True)[0]
    bits = torch.arange(1, 9, dtype=torch.int32)
    scale = km.kernel_scale(mn, mx, bits)
    t, U, b = km._rng_t(x, mn, scale, bits)
    draws = np.arange(1 << K, dtype=np.float32) if K == 8 else np.arange(0, 1 << K, 97, dtype=np.float32)
    mean = np.mean([km._codes_for(t, U, b, np.full(t.shape, r, np.float32)) for r in draws], axis=0)
    exact = (x.double() - mn.double()).numpy() * scale.double().numpy()
    # a scale rounded up in the tensor dtype can put the group maximum above B: the kernels clamp
    exact = np.minimum(exact, (2.0 ** bits.numpy() - 1).reshape(-1, 1, 1))
    tol = 2.0 ** -(K + 1) + (97 / 2.0 ** K if K == 16 else 0) + 2.0 ** -12
    assert np.abs(mean - exact).max() <= tol
    if K == 8:
        assert np.allclose(km.expected_code(x, mn, scale, bits), mean, atol=1e-12)
        p = mean - np.floor(mean + 1e-12)
        assert np.allclose(km.code_variance(x, mn, scale, bits), p * (1 - p), atol=1e-9)
    assert km._codes_for(t, U, b, np.full(t.shape, (1 << K) - 1, np.float32)).max() == 255
    assert (km._codes_for(t, U, b, np.zeros(t.shape, np.float32)).reshape(8, -1).max(1) <= 2 ** np.arange(1, 9) - 1).all()
