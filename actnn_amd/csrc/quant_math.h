// Per-group quantisation parameters and per-element code arithmetic, shared by the mixed
// and single precision pack kernels.
//
// Two arithmetics exist because the reference has two:
//  * DET (explicit noise tensor): the reference's config.simulate quantiser,
//    actnn/actnn/ops.py:30-41 - min/max shifted by 1e-6 (rounded to the tensor dtype), one
//    rounding per tensor op in the tensor dtype, clamp to [0, B], round half to even.
//  * RNG (in-kernel Philox): the reference's CUDA kernel, quantization_cuda_kernel.cu:32,:65
//    - scale = B / (max - min + 2e-6) evaluated in double, code = stochastic rounding of
//    (x - min) * scale.  The rounding is done as floor(t + u) with a uniform integer draw of
//    K = Noise<T>::kBits bits (16 for fp32 tensors, 8 for 16-bit tensors), which rounds up with
//    probability frac(t) like rint(t + u - 0.5).  It is evaluated in a 32-bit fixed point whose
//    top `bits` bits are the code (see RngFixed below), so that the conversion to an integer is
//    also the clamp and the code can be shifted into the output word with one instruction.
//
// This file must be compiled with -ffp-contract=off: every operation below is meant to
// round on its own unless it is written as an explicit fmaf.
#pragma once

#include "device_utils.h"

namespace actnn {

// RNG mode arithmetic.  One code level is 2^(32 - bits) and one step of the K-bit draw r is
// U = 2^(32 - bits - K):
//   t = fma(x - min, scale * 2^(32 - bits), U / 2)                        fp32 tensors
//   t = fma(x, scale * 2^(32 - bits), U / 2 - min * scale * 2^(32 - bits)) 16-bit tensors
//   word = sat_u32(fma(r, U, t));  code = word >> (32 - bits)
// The conversion saturates (below 0 and NaN give 0, 2^32 and above give 2^32 - 1), which is the
// clamp to [0, B].  16-bit tensors fold the subtraction of the minimum into the constant: their
// values cannot resolve a group range below 2^-11 (2^-8 for bf16) of |min|, so the rounding of the
// constant moves t by at most 2^-13 * B / 2^bits of a level (bf16: 2^-16); for fp32 tensors
// |min| / range is unbounded and x - min (exact for nearby values) is kept.
template <typename T> struct RngFixed {
  static constexpr bool kFold = sizeof(T) == 2;
  static ACTNN_DEV float unit(int bits) { return ldexpf(1.0f, 32 - bits - Noise<T>::kBits); }
  // (mul, sub) for `word` from the stored scale (a value of T) and the group minimum
  static ACTNN_DEV void params(float sc, float mn, int bits, float& mul, float& sub) {
    mul = sc * ldexpf(1.0f, 32 - bits);
    sub = kFold ? fmaf(-mn, mul, 0.5f * unit(bits)) : mn;
  }
  static ACTNN_DEV uint32_t word(float x, uint32_t r, float mul, float sub, float u) {
    const float t = kFold ? fmaf(x, mul, sub) : fmaf(x - sub, mul, 0.5f * u);
    const float w = fmaf((float)r, u, t);
    uint32_t out;
    asm("v_cvt_u32_f32_e32 %0, %1" : "=v"(out) : "v"(w));     // the instruction saturates
    return out;
  }
};

// Shift register that collects codes from the top of RngFixed words: push() moves the register up
// by BITS and takes the code of `word` in at the bottom, so elements are pushed last-first.
template <int BITS, bool TWO> struct CodeShifter {
  uint32_t lo = 0, hi = 0;
  ACTNN_DEV void push(uint32_t word) {
    if (TWO) hi = __builtin_amdgcn_alignbit(hi, lo, 32 - BITS);
    lo = __builtin_amdgcn_alignbit(lo, word, 32 - BITS);
  }
};

template <typename T, bool DET> struct GroupQuant {
  // Returns the scale to store (already rounded to T, as float) and sets the two values
  // the per-element code needs.  DET mode: `mul` = scale, `sub` = the shifted minimum.
  // RNG mode: the (mul, sub) of RngFixed<T>::params.
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
      RngFixed<T>::params(sc, mn, bits, mul, sub);
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

}  // namespace actnn
