// Device-side helpers shared by the gfx950 kernels: typed 128-bit loads/stores,
// cross-lane exchange (DPP / ds_swizzle), the 32x32 bit transpose that turns per-lane code
// bits into the reference's ballot-style words, and Philox4x32-10.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "../../include/actnn_hip.h"

namespace actnn {

struct bf16_t { uint16_t bits; };   // raw bfloat16 storage

#define ACTNN_DEV __device__ __forceinline__

// ------------------------------------------------------------------ scalar conversions
// Bit casts go through by-value helpers: __builtin_bit_cast applied directly to a vector
// element expression (v.y, v[i]) reads element 0 with this compiler.
ACTNN_DEV float as_float(uint32_t u) { return __builtin_bit_cast(float, u); }
ACTNN_DEV uint32_t as_uint(float f) { return __builtin_bit_cast(uint32_t, f); }
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
ACTNN_DEV float bf16_bits_to_float(uint32_t b) { return __builtin_bit_cast(float, b << 16); }
// two floats -> two bf16 in one word, round to nearest even (one v_cvt_pk_bf16_f32 on gfx950)
ACTNN_DEV uint32_t pack_bf16x2(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2_t){lo, hi}, bf16x2_t));
}
ACTNN_DEV uint32_t float_to_bf16_bits(float f) { return pack_bf16x2(f, 0.0f) & 0xffffu; }
ACTNN_DEV float half_bits_to_float(uint32_t b) {
  return __half2float(__builtin_bit_cast(__half, (uint16_t)b));
}
ACTNN_DEV uint32_t float_to_half_bits(float f) {
  return __builtin_bit_cast(uint16_t, __float2half_rn(f));
}

template <typename T> struct Conv;
template <> struct Conv<float> {
  static constexpr int kBytes = 4;
  static ACTNN_DEV float load(const float* p, int64_t i) { return p[i]; }
  static ACTNN_DEV void store(float* p, int64_t i, float v) { p[i] = v; }
  static ACTNN_DEV float round(float v) { return v; }
};
template <> struct Conv<__half> {
  static constexpr int kBytes = 2;
  static ACTNN_DEV float load(const __half* p, int64_t i) { return __half2float(p[i]); }
  static ACTNN_DEV void store(__half* p, int64_t i, float v) { p[i] = __float2half_rn(v); }
  static ACTNN_DEV float round(float v) { return __half2float(__float2half_rn(v)); }
};
template <> struct Conv<bf16_t> {
  static constexpr int kBytes = 2;
  static ACTNN_DEV float load(const bf16_t* p, int64_t i) { return bf16_bits_to_float(p[i].bits); }
  static ACTNN_DEV void store(bf16_t* p, int64_t i, float v) { p[i].bits = (uint16_t)float_to_bf16_bits(v); }
  static ACTNN_DEV float round(float v) { return bf16_bits_to_float(float_to_bf16_bits(v)); }
};

// Two values rounded to T and back (what storing and reloading them would give): one packed
// conversion for bf16.
template <typename T> ACTNN_DEV void round_pair(float& a, float& b) {
  a = Conv<T>::round(a);
  b = Conv<T>::round(b);
}
template <> ACTNN_DEV void round_pair<bf16_t>(float& a, float& b) {
  const uint32_t w = pack_bf16x2(a, b);
  a = as_float(w << 16);
  b = as_float(w & 0xffff0000u);
}

// ------------------------------------------------------------------ 16-byte vector access
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// 16-byte non-temporal load: for data that the kernel reads exactly once AND whose cache
// lines are consumed whole by one load instruction of the wave (measured: 7.0 vs 6.4 TB/s on
// a pure read).  Lanes that come back to the same line with a second instruction (the
// 32-byte-per-lane pattern of fp32 pack) must use the plain load or they fetch the line twice.
ACTNN_DEV u32x4 load16_nt(const void* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}
ACTNN_DEV u32x4 load16(const void* p) { return *reinterpret_cast<const u32x4*>(p); }
ACTNN_DEV void store16(void* p, u32x4 v) { *reinterpret_cast<u32x4*>(p) = v; }
ACTNN_DEV void store16_nt(void* p, u32x4 v) { __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p)); }

// 16 bytes per lane from global memory straight into LDS: lane l's data lands at lds_base + 16 * l
// (lds_base uniform in the wave).  Written as an instruction sequence of its own: the load is
// asynchronous and the code that issues it waits for it explicitly (vmcnt) before the data is read; issued through the compiler's builtin, every LDS read that follows - also of
// another buffer - would first wait for all loads in flight.
// The statements write m0 and say so in their clobber lists, so that the compiler never assumes a
// value of its own survives them (it keeps m0 to itself - "reserved" - and warns about any clobber
// of it; the warning is switched off for these two functions only).
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
ACTNN_DEV void load_to_lds16(const void* src, const uint8_t* lds_base) {
  const uint32_t base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const uint8_t*)lds_base;
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
               :
               : "s"(__builtin_amdgcn_readfirstlane(base)), "v"(src)
               : "memory", "m0");
}
// The same with the non-temporal hint, for data that is read once.
ACTNN_DEV void load_to_lds16_nt(const void* src, const uint8_t* lds_base) {
  const uint32_t base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const uint8_t*)lds_base;
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off nt"
               :
               : "s"(__builtin_amdgcn_readfirstlane(base)), "v"(src)
               : "memory", "m0");
}
// The same with the source given as a base that is the same for the whole wave (it travels in
// scalar registers) plus a 32-bit byte offset per lane: no 64-bit address arithmetic per lane.
ACTNN_DEV void load_to_lds16_base(const void* wave_base, uint32_t lane_bytes, const uint8_t* lds_base) {
  const uint32_t base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const uint8_t*)lds_base;
  const uint64_t b = (uint64_t)(uintptr_t)wave_base;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)b), hi = __builtin_amdgcn_readfirstlane((uint32_t)(b >> 32));
  const uint64_t sb = ((uint64_t)hi << 32) | lo;
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(__builtin_amdgcn_readfirstlane(base)), "v"(lane_bytes), "s"(sb)
               : "memory", "m0");
}
#pragma clang diagnostic pop

// ------------------------------------------------------------------ 8 / 16 contiguous elements
// load8: 8 consecutive elements starting at p (32-byte aligned for f32, 16 for 16-bit types).
ACTNN_DEV void load8(const float* p, float (&v)[8]) {
  const u32x4 a = load16(p);
  const u32x4 b = load16(p + 4);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[i] = as_float(a[i]);
    v[4 + i] = as_float(b[i]);
  }
}
ACTNN_DEV void load8(const __half* p, float (&v)[8]) {
  const u32x4 a = load16(p);
  const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = half_bits_to_float(w[i] & 0xffffu);
    v[2 * i + 1] = half_bits_to_float(w[i] >> 16);
  }
}
ACTNN_DEV void load8(const bf16_t* p, float (&v)[8]) {
  const u32x4 a = load16(p);
  const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = as_float(w[i] << 16);
    v[2 * i + 1] = as_float(w[i] & 0xffff0000u);
  }
}
// The same 8 elements kept as loaded (4 registers for 16-bit types instead of 8 floats) until
// they are needed: raw8_load_nt / raw8_widen.
template <typename T> struct Raw8 { u32x4 a; };
template <> struct Raw8<float> { u32x4 a, b; };
ACTNN_DEV void raw8_load_nt(const float* p, Raw8<float>& r) { r.a = load16(p); r.b = load16(p + 4); }
ACTNN_DEV void raw8_load_nt(const __half* p, Raw8<__half>& r) { r.a = load16_nt(p); }
ACTNN_DEV void raw8_load_nt(const bf16_t* p, Raw8<bf16_t>& r) { r.a = load16_nt(p); }
template <typename T> ACTNN_DEV void raw8_zero(Raw8<T>& r) {
  r.a = (u32x4){0, 0, 0, 0};
  if constexpr (sizeof(T) == 4) r.b = (u32x4){0, 0, 0, 0};
}
ACTNN_DEV void raw8_widen(const Raw8<float>& r, float (&v)[8]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) { v[i] = as_float(r.a[i]); v[4 + i] = as_float(r.b[i]); }
}
ACTNN_DEV void raw8_widen(const Raw8<__half>& r, float (&v)[8]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = half_bits_to_float(r.a[i] & 0xffffu);
    v[2 * i + 1] = half_bits_to_float(r.a[i] >> 16);
  }
}
ACTNN_DEV void raw8_widen(const Raw8<bf16_t>& r, float (&v)[8]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = as_float(r.a[i] << 16);
    v[2 * i + 1] = as_float(r.a[i] & 0xffff0000u);
  }
}
// Non-temporal variants for streams that are touched once and whose cache lines are covered whole
// by one instruction of the wave (16 bytes per lane, lanes contiguous).
ACTNN_DEV void load8_nt(const float* p, float (&v)[8]) { load8(p, v); }   // fp32: 32 bytes per lane, plain
ACTNN_DEV void load8_nt(const __half* p, float (&v)[8]) {
  const u32x4 a = load16_nt(p);
  const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = half_bits_to_float(w[i] & 0xffffu);
    v[2 * i + 1] = half_bits_to_float(w[i] >> 16);
  }
}
ACTNN_DEV void load8_nt(const bf16_t* p, float (&v)[8]) {
  const u32x4 a = load16_nt(p);
  const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = as_float(w[i] << 16);
    v[2 * i + 1] = as_float(w[i] & 0xffff0000u);
  }
}
ACTNN_DEV void store8(float* p, const float (&v)[8]) {
  u32x4 a, b;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a[i] = as_uint(v[i]);
    b[i] = as_uint(v[4 + i]);
  }
  store16(p, a);
  store16(p + 4, b);
}
ACTNN_DEV void store8(__half* p, const float (&v)[8]) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] = float_to_half_bits(v[2 * i]) | (float_to_half_bits(v[2 * i + 1]) << 16);
  store16(p, (u32x4){w[0], w[1], w[2], w[3]});
}
ACTNN_DEV void store8(bf16_t* p, const float (&v)[8]) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] = pack_bf16x2(v[2 * i], v[2 * i + 1]);
  store16(p, (u32x4){w[0], w[1], w[2], w[3]});
}

ACTNN_DEV void store8_nt(float* p, const float (&v)[8]) { store8(p, v); }  // fp32: 32 bytes per lane, plain
ACTNN_DEV void store8_nt(__half* p, const float (&v)[8]) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] = float_to_half_bits(v[2 * i]) | (float_to_half_bits(v[2 * i + 1]) << 16);
  store16_nt(p, (u32x4){w[0], w[1], w[2], w[3]});
}
ACTNN_DEV void store8_nt(bf16_t* p, const float (&v)[8]) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] = pack_bf16x2(v[2 * i], v[2 * i + 1]);
  store16_nt(p, (u32x4){w[0], w[1], w[2], w[3]});
}

// ------------------------------------------------------------------ cross-lane exchange
// Value held by lane (lane ^ D), D in {1, 2, 4, 8, 16}.  1/2/8 are DPP moves, 4/16 go
// through ds_swizzle (LDS crossbar, no memory), so they do not take a VALU slot.
// Workgroups are dealt to the 8 XCDs round-robin by their index, and every XCD has its own L2.  A
// kernel whose neighbouring blocks read the same lines (overlapping windows) renumbers its blocks so
// that a run of consecutive logical blocks stays on one XCD: launch xcd_grid(n) blocks, work on block
// xcd_block(); logical blocks >= n have nothing to do.
constexpr int kXcds = 8;
constexpr int kCUs = 256;          // compute units of the chip, 32 per XCD
inline unsigned xcd_grid(int64_t n) { return (unsigned)((n + kXcds - 1) / kXcds * kXcds); }
ACTNN_DEV int64_t xcd_block() {
  return (int64_t)(blockIdx.x % kXcds) * (gridDim.x / kXcds) + blockIdx.x / kXcds;
}

// Division of a 32-bit unsigned number by a divisor that is fixed at launch: one multiply-high, two
// shifts and two additions (Granlund & Montgomery, "Division by invariant integers using
// multiplication", 1994, figure 4.1), exact for every numerator.  Built on the host, passed by value.
struct FastDiv {
  uint32_t d, m;
  int s1, s2;
  FastDiv() = default;
  explicit FastDiv(uint32_t divisor) : d(divisor) {
    int l = 0;
    while ((uint64_t(1) << l) < divisor) ++l;
    m = (uint32_t)(((uint64_t(1) << 32) * ((uint64_t(1) << l) - divisor)) / divisor + 1);
    s1 = l < 1 ? l : 1;
    s2 = l > 0 ? l - 1 : 0;
  }
  ACTNN_DEV uint32_t div(uint32_t n) const {
    const uint32_t t = __umulhi(n, m);
    return (t + ((n - t) >> s1)) >> s2;
  }
};

template <int D> ACTNN_DEV uint32_t lane_xor(uint32_t x);
template <> ACTNN_DEV uint32_t lane_xor<1>(uint32_t x) {
  return (uint32_t)__builtin_amdgcn_update_dpp((int)x, (int)x, 0xB1, 0xF, 0xF, true);   // quad_perm [1,0,3,2]
}
template <> ACTNN_DEV uint32_t lane_xor<2>(uint32_t x) {
  return (uint32_t)__builtin_amdgcn_update_dpp((int)x, (int)x, 0x4E, 0xF, 0xF, true);   // quad_perm [2,3,0,1]
}
template <> ACTNN_DEV uint32_t lane_xor<4>(uint32_t x) {
  return (uint32_t)__builtin_amdgcn_ds_swizzle((int)x, 0x101F);                      // xor 4
}
template <> ACTNN_DEV uint32_t lane_xor<8>(uint32_t x) {
  return (uint32_t)__builtin_amdgcn_update_dpp((int)x, (int)x, 0x128, 0xF, 0xF, true);  // row_ror:8
}
template <> ACTNN_DEV uint32_t lane_xor<16>(uint32_t x) {
  return (uint32_t)__builtin_amdgcn_ds_swizzle((int)x, 0x401F);                      // xor 16
}

template <int S> ACTNN_DEV uint32_t transpose_stage(uint32_t x, uint32_t lane) {
  constexpr uint32_t M = S == 16 ? 0xFFFF0000u : S == 8 ? 0xFF00FF00u : S == 4 ? 0xF0F0F0F0u
                       : S == 2 ? 0xCCCCCCCCu : 0xAAAAAAAAu;
  const uint32_t p = lane_xor<S>(x);
  const bool hi = (lane & S) != 0;
  const uint32_t u = __builtin_amdgcn_alignbit(p, p, hi ? S : 32 - S);   // hi: p >> S, lo: p << S (rotations)
  const uint32_t sel = hi ? M : ~M;
  return (x & sel) | (u & ~sel);
}

// 32x32 bit transpose inside each 32-lane half of the wave: afterwards bit j of lane p is
// what bit p of lane j was.  `lane` is the lane index (any value congruent mod 32).
ACTNN_DEV uint32_t transpose32(uint32_t x, uint32_t lane) {
  x = transpose_stage<16>(x, lane);
  x = transpose_stage<8>(x, lane);
  x = transpose_stage<4>(x, lane);
  x = transpose_stage<2>(x, lane);
  x = transpose_stage<1>(x, lane);
  return x;
}

// Two interleaved 32x32 bit transposes over the whole wave: the even lanes hold the 32 rows of
// one matrix (row j in lane 2j), the odd lanes those of another (row j in lane 2j+1).  Afterwards
// bit j of lane 2p+h is what bit p of lane 2j+h was.  Partner lanes are lane ^ 32, 16, 8, 4, 2.
template <int S> ACTNN_DEV uint32_t transpose_stage_x2(uint32_t x, uint32_t lane) {
  constexpr uint32_t M = S == 16 ? 0xFFFF0000u : S == 8 ? 0xFF00FF00u : S == 4 ? 0xF0F0F0F0u
                       : S == 2 ? 0xCCCCCCCCu : 0xAAAAAAAAu;
  uint32_t p;
  if constexpr (S == 16) p = (uint32_t)__builtin_amdgcn_ds_bpermute((int)((lane ^ 32u) << 2), (int)x);   // lane ^ 32
  else p = lane_xor<2 * S>(x);
  const bool hi = (lane & (2 * S)) != 0;
  const uint32_t u = __builtin_amdgcn_alignbit(p, p, hi ? S : 32 - S);
  const uint32_t sel = hi ? M : ~M;
  return (x & sel) | (u & ~sel);
}
ACTNN_DEV uint32_t transpose32_x2(uint32_t x, uint32_t lane) {
  x = transpose_stage_x2<16>(x, lane);
  x = transpose_stage_x2<8>(x, lane);
  x = transpose_stage_x2<4>(x, lane);
  x = transpose_stage_x2<2>(x, lane);
  x = transpose_stage_x2<1>(x, lane);
  return x;
}

// Minimum / maximum as single instructions.  fminf / fmaxf compile to the same instruction plus one
// more per operand that quiets signalling NaNs (the loops that use these are bound by
// instruction issue, and the extra instructions were a quarter of them); here a quiet NaN operand is
// ignored as in fminf / fmaxf, a signalling NaN is returned quieted.
ACTNN_DEV float min_f32(float a, float b) {
  float r;
  asm("v_min_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
ACTNN_DEV float max_f32(float a, float b) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
ACTNN_DEV float min3_f32(float a, float b, float c) {
  float r;
  asm("v_min3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
ACTNN_DEV float max3_f32(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
// minimum and maximum of N values (N = 4 or 8) in N / 2 instructions each
template <int N> ACTNN_DEV void minmax_of(const float (&v)[N], float& lo, float& hi) {
  lo = min3_f32(v[0], v[1], v[2]);
  hi = max3_f32(v[0], v[1], v[2]);
  if constexpr (N == 8) {
    lo = min3_f32(lo, v[3], v[4]);
    hi = max3_f32(hi, v[3], v[4]);
    lo = min3_f32(lo, v[5], v[6]);
    hi = max3_f32(hi, v[5], v[6]);
    lo = min_f32(lo, v[7]);
    hi = max_f32(hi, v[7]);
  } else {
    static_assert(N == 4, "4 or 8 values");
    lo = min_f32(lo, v[3]);
    hi = max_f32(hi, v[3]);
  }
}

// Minimum of lo and maximum of hi over groups of 16 * ROWS consecutive lanes (ROWS = 1, 2 or 4), both
// at once, with the lane exchange inside the arithmetic instruction (one instruction per step and
// value; through the exchange builtins it took three).  ROWS == 1: every lane ends with the result
// of its row of 16; ROWS == 2: the last row of each 32-lane half holds the half's result; ROWS == 4:
// the last row of the wave holds the wave's result.  All lanes of the groups must be active.  The
// s_nop's are the wait states the hardware asks for between a vector write and a cross-lane read
// of the same register (2) and after a vector write of EXEC (5); the compiler does not see into the
// block.
template <int ROWS> ACTNN_DEV void lanes_minmax(float& lo, float& hi) {
  asm("s_nop 4\n\t"
      "v_min_f32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32_dpp %1, %1, %1 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 0\n\t"
      "v_min_f32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32_dpp %1, %1, %1 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 0\n\t"
      "v_min_f32_dpp %0, %0, %0 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32_dpp %1, %1, %1 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 0\n\t"
      "v_min_f32_dpp %0, %0, %0 row_mirror row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32_dpp %1, %1, %1 row_mirror row_mask:0xf bank_mask:0xf"
      : "+v"(lo), "+v"(hi));
  if constexpr (ROWS >= 2)     // the last lane of rows 0 and 2 into rows 1 and 3
    asm("s_nop 1\n\t"
        "v_min_f32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
        "v_max_f32_dpp %1, %1, %1 row_bcast:15 row_mask:0xa bank_mask:0xf"
        : "+v"(lo), "+v"(hi));
  if constexpr (ROWS >= 4)     // the last lane of row 1 into rows 2 and 3
    asm("s_nop 1\n\t"
        "v_min_f32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
        "v_max_f32_dpp %1, %1, %1 row_bcast:31 row_mask:0xc bank_mask:0xf"
        : "+v"(lo), "+v"(hi));
}

// ------------------------------------------------------------------ Philox4x32-10
struct Philox4 { uint32_t x, y, z, w; };

ACTNN_DEV Philox4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3,
                                uint32_t k0, uint32_t k1) {
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0;
    const uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    // three-input xor in one instruction (v_bitop3_b32, truth table 0x96)
    const uint32_t n0 = __builtin_amdgcn_bitop3_b32((uint32_t)(p1 >> 32), c1, k0, 0x96);
    const uint32_t n2 = __builtin_amdgcn_bitop3_b32((uint32_t)(p0 >> 32), c3, k1, 0x96);
    c1 = (uint32_t)p1;
    c3 = (uint32_t)p0;
    c0 = n0;
    c2 = n2;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  return Philox4{c0, c1, c2, c3};
}

// ------------------------------------------------------------------ 1-bit masks of 16-bit tensors
// A wave that holds four 512-element blocks of a tensor, lane l elements 8l..8l+7 of each, and the
// blocks' 64 mask words (element 16j + k of a block is bit j of its word k), lane 2p + h the word
// p % 16 of block 2h + p / 16: lane pairs swap their 8-bit halves (one DPP move) so that the even
// lanes hold the rows of blocks A|B and the odd lanes those of C|D, and two interleaved 32x32 bit
// transposes turn rows into words or back.
// rows (per lane: 8 keep bits for each of the 4 blocks) -> this lane's mask word
ACTNN_DEV uint32_t rows_to_word(const uint32_t (&m)[4], uint32_t lane) {
  const bool odd = lane & 1u;
  const uint32_t ab = m[0] | (m[1] << 16), cd = m[2] | (m[3] << 16);
  const uint32_t recv = lane_xor<1>(odd ? ab : cd);           // the half-row the partner computed for me
  const uint32_t mine = odd ? cd : ab;
  const uint32_t row = odd ? (recv | (mine << 8)) : (mine | (recv << 8));
  return transpose32_x2(row, lane);
}
// inverse: this lane's mask word -> 8 keep bits for each of the 4 blocks
ACTNN_DEV void word_to_rows(uint32_t w, uint32_t lane, uint32_t (&m)[4]) {
  const bool odd = lane & 1u;
  const uint32_t row = transpose32_x2(w, lane);                // even: row of A|B, odd: row of C|D
  const uint32_t other = lane_xor<1>(row);
  const uint32_t ab = odd ? other : row, cd = odd ? row : other;
  const int sh = odd ? 8 : 0;
  m[0] = (ab >> sh) & 0xffu;
  m[1] = (ab >> (16 + sh)) & 0xffu;
  m[2] = (cd >> sh) & 0xffu;
  m[3] = (cd >> (16 + sh)) & 0xffu;
}


// ------------------------------------------------------------------ rounding noise
// The stochastic rounding draws one uniform integer per element; elements are numbered as they lie
// in memory and taken in octets (8 consecutive elements).  How many bits an element gets follows
// the resolution of the data: 16 for fp32 tensors, 8 for fp16 / bf16 tensors (whose own spacing
// near the top of a group's range is 2^-11 / 2^-8 of the value; an 8-bit draw rounds up with a
// probability within 2^-9 of the fractional part, centred).
//  * 16 bits: one Philox call per octet, counter = the octet's index; element k takes the
//    (k & 1)-th half (low first) of output word k >> 1.
//  * 8 bits: one Philox call per two consecutive octets, counter = octet index >> 1; octet h = index
//    & 1 takes output words 2h and 2h + 1, element k byte k & 3 of word 2h + (k >> 2).
// Dropout always uses the 16-bit form.
ACTNN_DEV Philox4 philox_at(uint64_t counter, uint64_t seed, uint64_t offset) {
  return philox4x32_10((uint32_t)counter, (uint32_t)(counter >> 32), (uint32_t)offset,
                       (uint32_t)(offset >> 32), (uint32_t)seed, (uint32_t)(seed >> 32));
}

ACTNN_DEV void philox_octet(uint64_t octet, uint64_t seed, uint64_t offset, uint32_t (&r16)[8]) {
  const Philox4 r = philox_at(octet, seed, offset);
  r16[0] = r.x & 0xffffu; r16[1] = r.x >> 16;
  r16[2] = r.y & 0xffffu; r16[3] = r.y >> 16;
  r16[4] = r.z & 0xffffu; r16[5] = r.z >> 16;
  r16[6] = r.w & 0xffffu; r16[7] = r.w >> 16;
}

template <typename T> struct Noise {
  static constexpr int kBits = sizeof(T) == 2 ? 8 : 16;
  static constexpr int kWords = 8 * kBits / 32;                 // words of noise per octet
  // the draw of element k of an octet whose words are w
  static ACTNN_DEV uint32_t at(const uint32_t (&w)[kWords], int k) {
    constexpr int per = 32 / kBits;
    return (w[k / per] >> (kBits * (k % per))) & ((1u << kBits) - 1u);
  }
  // Noise words of one octet, whatever the lanes around hold.
  static ACTNN_DEV void octet(uint64_t o, uint64_t seed, uint64_t offset, uint32_t (&w)[kWords]) {
    if constexpr (kBits == 16) {
      const Philox4 r = philox_at(o, seed, offset);
      w[0] = r.x; w[1] = r.y; w[2] = r.z; w[3] = r.w;
    } else {
      const Philox4 r = philox_at(o >> 1, seed, offset);
      const bool h = o & 1;
      w[0] = h ? r.z : r.x;
      w[1] = h ? r.w : r.y;
    }
  }
  // Noise words of two octets oa, ob of this lane when lane ^ 1 holds oa ^ 1 and ob ^ 1 and is
  // active, and the parity of the lane is the parity of both octets.  With 8-bit noise the two
  // lanes then need two Philox calls between them instead of four: the even lane evaluates the
  // pair of oa, the odd lane the pair of ob, and they hand each other the half they do not use.
  static ACTNN_DEV void octets(uint64_t oa, uint64_t ob, uint64_t seed, uint64_t offset,
                               uint32_t (&wa)[kWords], uint32_t (&wb)[kWords]) {
    if constexpr (kBits == 16) {
      octet(oa, seed, offset, wa);
      octet(ob, seed, offset, wb);
    } else {
      const bool odd = oa & 1;
      const Philox4 r = philox_at((odd ? ob : oa) >> 1, seed, offset);
      // even lane: r = pair(oa): (x, y) are mine for oa, (z, w) the neighbour's for oa ^ 1
      // odd lane:  r = pair(ob): (z, w) are mine for ob, (x, y) the neighbour's for ob ^ 1
      const uint32_t nx = lane_xor<1>(r.x), ny = lane_xor<1>(r.y);
      const uint32_t nz = lane_xor<1>(r.z), nw = lane_xor<1>(r.w);
      wa[0] = odd ? nz : r.x;
      wa[1] = odd ? nw : r.y;
      wb[0] = odd ? r.z : nx;
      wb[1] = odd ? r.w : ny;
    }
  }
};

// ------------------------------------------------------------------ host-side helpers
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

#define ACTNN_RETURN_LAUNCH_STATUS()                       \
  do {                                                     \
    hipError_t e_ = hipGetLastError();                     \
    return e_ == hipSuccess ? ACTNN_OK : (int)e_;          \
  } while (0)

}  // namespace actnn
