// Per-group quantisation parameters and per-element code arithmetic, shared by the mixed
// and single precision pack kernels.
//
// Two arithmetics exist because the reference has two:
//  * DET (explicit noise tensor): the reference's config.simulate quantiser,
//    actnn/actnn/ops.py:30-41 - min/max shifted by 1e-6 (rounded to the tensor dtype), one
//    rounding per tensor op in the tensor dtype, clamp to [0, B], round half to even.
//  * RNG (in-kernel Philox): the reference's CUDA kernel, quantization_cuda_kernel.cu:32,:65
//    - scale = B / (max - min + 2e-6) evaluated in double, code = stochastic rounding of
//    (x - min) * scale.  The rounding is done as floor(t + u) in 16.16 fixed point with a
//    16-bit uniform u, which rounds up with probability frac(t) like rint(t + u - 0.5).
//
// This file must be compiled with -ffp-contract=off: every operation below is meant to
// round on its own unless it is written as an explicit fmaf.
#pragma once

#include "device_utils.h"

namespace actnn {

template <typename T, bool DET> struct GroupQuant {
  // Returns the scale to store (already rounded to T, as float) and sets the two values
  // the per-element code needs: `mul` (scale, times 2^16 in RNG mode) and `sub` (the
  // minimum to subtract: shifted in DET mode, original in RNG mode).
  static ACTNN_DEV float prepare(float mn, float mx, int bits, float& mul, float& sub) {
    const float Bf = (float)((1 << bits) - 1);
    if (DET) {
      const float eps = Conv<T>::round(1e-6f);                  // scalar takes the tensor dtype
      const float mn_s = Conv<T>::round(mn - eps);              // ops.py:31
      const float mx_s = Conv<T>::round(mx + eps);              // ops.py:32
      const float den = Conv<T>::round(mx_s - mn_s);
      const float sc = Conv<T>::round(Bf / den);                // ops.py:33
      mul = sc;
      sub = mn_s;
      return sc;
    } else {
      const float range = Conv<T>::round(mx - mn);              // max - min in scalar_t
      const double q = (double)Bf / ((double)range + 2e-6);     // .cu:32 (double literal)
      const float sc = Conv<T>::round((float)q);
      mul = sc * 65536.0f;
      sub = mn;
      return sc;
    }
  }
};

// DET code: ops.py:34-41 with the noise as an operand.
template <typename T> ACTNN_DEV uint32_t det_code(float x, float noise, float mul, float sub, float Bf) {
  float t = Conv<T>::round(x - sub);
  t = Conv<T>::round(t * mul);
  t = Conv<T>::round(t + noise);
  t = fmaxf(t, 0.0f);
  t = fminf(t, Bf);
  return (uint32_t)(int)rintf(t);
}

// Dequantisation (scalar_t)code / scale + min with one rounding per operation (.cu:171, :359).
// For fp32 the quotient is the IEEE division.  For 16-bit types the quotient only has to be right
// after rounding to 8 or 11 significant bits, so it is computed as code * (1/scale) with one
// Newton step on the reciprocal and one residual correction (Markstein's sequence), which costs 3
// operations per element instead of ~12; tests/test_gpu_unpack_exhaustive.py checks it against
// the true division for every 16-bit scale value and every code.  Scales that are not ordinary
// positive numbers (inf for constant groups in fp16, 0, NaN) take the IEEE path.
template <typename T> struct Dequant {
  float sc, m, r;
  bool fast;
  ACTNN_DEV Dequant(float scale, float mn) : sc(scale), m(mn), r(0.0f), fast(false) {
    if (sizeof(T) == 2) {
      const float a = fabsf(scale);
      fast = a > 1e-30f && a < 1e30f;           // false for NaN too
      if (fast) {
        const float r0 = __builtin_amdgcn_rcpf(scale);
        r = fmaf(fmaf(-scale, r0, 1.0f), r0, r0);
      }
    }
  }
  ACTNN_DEV float operator()(uint32_t code) const {
    const float c = (float)code;
    float q;
    if (sizeof(T) == 2 && fast) {
      const float q0 = c * r;
      q = fmaf(fmaf(-sc, q0, c), r, q0);
    } else {
      q = c / sc;
    }
    return Conv<T>::round(Conv<T>::round(q) + m);
  }
};

// RNG code: fix = trunc(clamp(fma(x - min, scale * 2^16, 0.5), 0, B * 2^16)); (fix + r16) >> 16.
ACTNN_DEV uint32_t rng_code(float x, uint32_t r16, float mul, float sub, float Bfix) {
  const float d = x - sub;
  const float f = __builtin_amdgcn_fmed3f(fmaf(d, mul, 0.5f), 0.0f, Bfix);
  return ((uint32_t)f + r16) >> 16;
}

}  // namespace actnn
