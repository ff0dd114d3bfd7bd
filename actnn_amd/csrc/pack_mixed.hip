// Mixed-precision pack / unpack (replaces quantization_cuda_kernel.cu:22-205).
//
// Stream layout (kept from the reference): sample n with b = bits[n] owns
// b * G * gs / 32 consecutive int32 words starting at prefix[n] * G * gs / 32; inside a group
// of gs = 32 * E elements, bit i of the code of element d = E * j + k is bit j of word
// k * b + i.  So a word is a 32-lane "ballot" over j, where lane j owns the E consecutive
// elements E*j .. E*j+E-1.
//
// gs == 256 fast path: a 32-lane half-wave owns a group; lane j loads its 8 contiguous
// elements (one 16-byte load for 16-bit types, two for f32), quantises them and
// concatenates the 8 codes into 8*b bits of a register (several groups share a register
// when 8*b <= 16).  One 32x32 bit transpose per register (5 exchange stages) then leaves
// word p in lane p, which is stored coalesced.  A 256-thread block handles 16 groups of one
// sample (2 per half-wave); the element loads are issued first, the block's scales are
// computed by the first threads and shared through LDS while the loads are in flight.
// unpack mirrors this; its fp32 stores go through LDS so that each store instruction of a
// wave writes one whole 1 KiB group.
//
// Other group sizes (multiples of 32 up to 1024) take a simple LDS-staged kernel.
#include "quant_math.h"

namespace actnn {
namespace {

// Groups per half-wave and block.  fp32: 2 measured best (16 KiB of input per block).
// 16-bit types: a block with 8 KiB of data is dominated by its own latency chain (widths ->
// scales -> data), so they take 4.
template <typename T> struct Gph {
  static constexpr int kPack = sizeof(T) == 2 ? 4 : 2;
  static constexpr int kUnpack = sizeof(T) == 2 ? 4 : 2;
};

constexpr int kThreads = 256;
constexpr int kHalfWaves = kThreads / 32;
constexpr int kGs = 256;

template <int BITS, int GPH> struct Tile {
  static constexpr int kWordsPerGroup = 8 * BITS;
  // consecutive groups that share one register (one transpose): as many as fit in 32 bits
  static constexpr int kFit = BITS == 1 ? 4 : BITS == 2 ? 2 : 1;
  static constexpr int kGroupsPerReg = kFit < GPH ? kFit : GPH;
  static constexpr bool kTwoRegs = BITS > 4;                                  // 8*BITS > 32
  // Group (within the block) that half-wave hw handles in its q-th slot: GPH consecutive groups
  // per half-wave, whatever the bit width, so that loads can be issued before the width is known.
  static __device__ __forceinline__ int group_of(int hw, int q) { return hw * GPH + q; }
};

// fp32 output of unpack: a lane owns 32 contiguous bytes, which as direct stores would be two
// half-used 16-byte accesses per cache line.  Instead lanes park their 8 values in the wave's
// private LDS slab and the wave stores whole 1 KiB groups with one non-temporal instruction each
// (measured 6.9 instead of 5.3 TB/s, and no dirty lines are left for the next kernel to wait on).
// Only lanes of one wave exchange data, so no block barrier is needed: LDS operations of a wave
// complete in order.  (The same staging for the fp32 loads of pack was measured slower.)
template <int GPH, typename TL>
ACTNN_DEV void stage_out_f32(float* __restrict__ out, int64_t elem_base, int groups_valid,
                             u32x4* __restrict__ slab, const float (&v)[GPH][8]) {
  const int wl = threadIdx.x & 63;
  const int w = threadIdx.x >> 6;
  const int h = (threadIdx.x >> 5) & 1;
  const uint32_t lane = threadIdx.x & 31;
#pragma unroll
  for (int q = 0; q < GPH; ++q) {
    u32x4 a, b;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      a[k] = as_uint(v[q][k]);
      b[k] = as_uint(v[q][4 + k]);
    }
    slab[(h * GPH + q) * 64 + 2 * lane] = a;
    slab[(h * GPH + q) * 64 + 2 * lane + 1] = b;
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
  for (int i = 0; i < 2 * GPH; ++i) {
    const int gl = TL::group_of(2 * w + i / GPH, i % GPH);
    if (gl < groups_valid) {
      store16_nt(out + elem_base + (int64_t)gl * kGs + wl * 4, slab[i * 64 + wl]);
    }
  }
}

template <typename T> struct IsF32 { static constexpr bool value = false; };
template <> struct IsF32<float> { static constexpr bool value = true; };
template <typename T> struct IsBf16 { static constexpr bool value = false; };
template <> struct IsBf16<bf16_t> { static constexpr bool value = true; };

// ---------------------------------------------------------------------------- pack (gs = 256)
// Issue the loads of this lane's elements (and noise in deterministic mode) for its GPH groups.
// The elements stay as loaded until their group is packed (16-bit types: 4 registers per group
// rather than 8), which keeps the kernel within the registers of 8 waves per SIMD.
template <typename T, bool DET, int GPH>
ACTNN_DEV void load_groups(const T* __restrict__ data, const T* __restrict__ noise, int64_t elem_base,
                           int groups_valid, Raw8<T> (&v)[GPH], Raw8<T> (&nz)[DET ? GPH : 1]) {
  using TL = Tile<1, GPH>;
  const uint32_t lane = threadIdx.x & 31;
  const int hw = threadIdx.x >> 5;
#pragma unroll
  for (int q = 0; q < GPH; ++q) {
    const int gl = TL::group_of(hw, q);
    if (gl < groups_valid) {
      const int64_t e = elem_base + (int64_t)gl * kGs + lane * 8;
      raw8_load_nt(data + e, v[q]);      // non-temporal for 16-bit types only (one instruction per line)
      if (DET) raw8_load_nt(noise + e, nz[DET ? q : 0]);
    } else {
      raw8_zero(v[q]);
      if (DET) raw8_zero(nz[DET ? q : 0]);
    }
  }
}

template <typename T, int BITS, bool DET>
ACTNN_DEV void pack_groups(const Raw8<T> (&raw)[Gph<T>::kPack], const Raw8<T> (&nzraw)[DET ? Gph<T>::kPack : 1],
                           int32_t* __restrict__ packed, int64_t elem_base, int64_t word_base,
                           int groups_valid, const float* s_mul, const float* s_sub,
                           uint64_t seed, uint64_t offset) {
  constexpr int kGroupsPerHalf = Gph<T>::kPack;
  using TL = Tile<BITS, kGroupsPerHalf>;
  constexpr int R = TL::kGroupsPerReg;
  constexpr int WPG = TL::kWordsPerGroup;
  constexpr float Bf = (float)((1 << BITS) - 1);
  const uint32_t lane = threadIdx.x & 31;
  const int hw = threadIdx.x >> 5;
  static_assert(kGroupsPerHalf % 2 == 0, "the noise of the groups is drawn in pairs");
  constexpr int NB = R > 2 ? R : 2;                    // groups whose noise is drawn together
  constexpr float kUnit = (float)(1u << (32 - BITS - Noise<T>::kBits));
  uint32_t rw[NB][Noise<T>::kWords];

#pragma unroll
  for (int q0 = 0; q0 < kGroupsPerHalf; q0 += R) {
    uint64_t acc = 0;                                  // DET
    CodeShifter<BITS, TL::kTwoRegs> sh;                // RNG
    if (!DET && q0 % NB == 0) {
      // noise of NB groups, two at a time: the octets of lane ^ 1 in the same two groups are
      // their neighbours (elem_base is a multiple of 256, so octet and lane parity agree)
#pragma unroll
      for (int p = 0; p < NB; p += 2) {
        const uint64_t o = (uint64_t)(elem_base >> 3) + (uint64_t)TL::group_of(hw, q0 + p) * 32 + lane;
        Noise<T>::octets(o, o + 32, seed, offset, rw[p], rw[p + 1]);
      }
    }
#pragma unroll
    for (int r = R - 1; r >= 0; --r) {                 // last group first: see CodeShifter
      const int q = q0 + r;
      const int gl = TL::group_of(hw, q);
      const float mul = s_mul[gl];
      const float sub = s_sub[gl];
      float v[8], nz[8];
      raw8_widen(raw[q], v);
      if (DET) raw8_widen(nzraw[DET ? q : 0], nz);
#pragma unroll
      for (int k = 7; k >= 0; --k) {
        if (DET) acc |= (uint64_t)det_code<T>(v[k], nz[k], mul, sub, Bf) << (r * WPG + k * BITS);
        else sh.push(RngFixed<T>::word(v[k], Noise<T>::at(rw[q % NB], k), mul, sub, kUnit));
      }
    }
    if (!DET) acc = ((uint64_t)sh.hi << 32) | sh.lo;
    const int glt = TL::group_of(hw, q0);            // first group of this register tile
    const int64_t tile_words = word_base + (int64_t)glt * WPG;
    const uint32_t lo = transpose32((uint32_t)acc, lane);
    // each half-wave stores its own 4-byte words (whole 128-byte lines), non-temporally: 3 % faster
    // than plain stores, and no dirty lines are left behind for the next kernel
    int32_t* dst = packed + tile_words;
    if (TL::kTwoRegs) {
      const uint32_t hi = transpose32((uint32_t)(acc >> 32), lane);
      if (glt < groups_valid) {
        __builtin_nontemporal_store((int32_t)lo, dst + lane);
        if ((int)lane < WPG - 32) __builtin_nontemporal_store((int32_t)hi, dst + 32 + lane);
      }
    } else {
      if ((int)lane < R * WPG && glt + (int)lane / WPG < groups_valid)
        __builtin_nontemporal_store((int32_t)lo, dst + lane);
    }
  }
}

template <typename T, bool DET>
__global__ __launch_bounds__(kThreads, DET ? 1 : 8) void pack_mixed_kernel(
    const T* __restrict__ data, const T* __restrict__ mn, const T* __restrict__ mx,
    const int32_t* __restrict__ bits, const int32_t* __restrict__ prefix, T* __restrict__ scale,
    int32_t* __restrict__ packed, const T* __restrict__ noise, uint64_t seed, uint64_t offset,
    int64_t G, int blocks_per_sample) {
  constexpr int GPH = Gph<T>::kPack;
  constexpr int kGroupsPerBlock = kHalfWaves * GPH;
  __shared__ float s_mul[kGroupsPerBlock];
  __shared__ float s_sub[kGroupsPerBlock];
  const int64_t n = blockIdx.x / blocks_per_sample;
  const int64_t gb = (int64_t)(blockIdx.x % blocks_per_sample) * kGroupsPerBlock;
  const int groups_valid = (int)((G - gb) < kGroupsPerBlock ? (G - gb) : kGroupsPerBlock);
  const int64_t elem_base = (n * G + gb) * kGs;

  // The element loads do not depend on the bit width or the scales: get them in flight first,
  // then compute the block's scales while they travel.
  Raw8<T> v[GPH];
  Raw8<T> nz[DET ? GPH : 1];
  // fp32 in RNG mode: a lane's 8 elements are 32 bytes, so a direct load would touch every cache
  // line with two instructions of the wave.  The wave's groups (4 KiB, contiguous) instead travel
  // straight into LDS, one whole 1 KiB group per instruction and no registers, and each lane then
  // picks its 32 bytes out of LDS.
  constexpr bool kViaLds = sizeof(T) == 4 && !DET;
  __shared__ __align__(16) uint8_t s_stage[kViaLds ? kGroupsPerBlock * kGs * 4 : 16];
  if constexpr (kViaLds) {
    const int wave = threadIdx.x >> 6;
    const uint32_t wl = threadIdx.x & 63;
#pragma unroll
    for (int i = 0; i < 2 * GPH; ++i) {
      const int gl = wave * 2 * GPH + i;                       // the wave's two half-waves own these groups
      if (gl < groups_valid)
        load_to_lds16_nt(data + elem_base + (int64_t)gl * kGs + wl * 4, s_stage + gl * (kGs * 4));
    }
  } else {
    load_groups<T, DET, GPH>(data, noise, elem_base, groups_valid, v, nz);
  }

  const int b = bits[n];
  if (threadIdx.x < kGroupsPerBlock) {
    float mul = 0.0f, sub = 0.0f;
    if ((int)threadIdx.x < groups_valid) {
      const int64_t gi = n * G + gb + threadIdx.x;
      const float sc = GroupQuant<T, DET>::prepare(Conv<T>::load(mn, gi), Conv<T>::load(mx, gi), b, mul, sub);
      Conv<T>::store(scale, gi, sc);
    }
    s_mul[threadIdx.x] = mul;
    s_sub[threadIdx.x] = sub;
  }
  __syncthreads();
  if constexpr (kViaLds) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");             // this wave's own groups have landed
    const uint32_t lane = threadIdx.x & 31;
    const int hw = threadIdx.x >> 5;
#pragma unroll
    for (int q = 0; q < GPH; ++q) {
      const int gl = Tile<1, GPH>::group_of(hw, q);
      raw8_zero(v[q]);
      if (gl < groups_valid) {
        const u32x4* src = reinterpret_cast<const u32x4*>(s_stage + gl * (kGs * 4) + lane * 32);
        v[q].a = src[0];
        v[q].b = src[1];
      }
    }
  }

  const int64_t word_base = (int64_t)prefix[n] * G * 8 + gb * 8 * b;
  switch (b) {
#define ACTNN_CASE(B_)                                                                          \
  case B_:                                                                                      \
    pack_groups<T, B_, DET>(v, nz, packed, elem_base, word_base, groups_valid, s_mul, s_sub,    \
                            seed, offset);                                                      \
    break;
    ACTNN_CASE(1) ACTNN_CASE(2) ACTNN_CASE(3) ACTNN_CASE(4)
    ACTNN_CASE(5) ACTNN_CASE(6) ACTNN_CASE(7) ACTNN_CASE(8)
#undef ACTNN_CASE
    default: break;   // bits outside 1..8 are rejected on the host when known; nothing is written
  }
}

// ---------------------------------------------------------------------------- unpack (gs = 256)
template <typename T, int BITS>
ACTNN_DEV void unpack_groups(const int32_t* __restrict__ packed, T* __restrict__ out,
                             int64_t elem_base, int64_t word_base, int groups_valid,
                             float* s_scale, float* s_min, float my_scale, float my_min, u32x4* slab) {
  constexpr int kGroupsPerHalf = Gph<T>::kUnpack;
  constexpr bool kStage = IsF32<T>::value;
  float vs[kStage ? kGroupsPerHalf : 1][8];
  using TL = Tile<BITS, kGroupsPerHalf>;
  constexpr int R = TL::kGroupsPerReg;
  constexpr int WPG = TL::kWordsPerGroup;
  constexpr uint32_t kMask = (1u << BITS) - 1u;
  const uint32_t lane = threadIdx.x & 31;
  const int hw = threadIdx.x >> 5;

  uint32_t wlo[kGroupsPerHalf / R], whi[kGroupsPerHalf / R];
#pragma unroll
  for (int t = 0; t < kGroupsPerHalf / R; ++t) {
    const int glt = TL::group_of(hw, t * R);
    const int64_t tile_words = word_base + (int64_t)glt * WPG;
    wlo[t] = 0;
    whi[t] = 0;
    if (TL::kTwoRegs) {
      if (glt < groups_valid) {
        wlo[t] = (uint32_t)packed[tile_words + lane];
        if ((int)lane < WPG - 32) whi[t] = (uint32_t)packed[tile_words + 32 + lane];
      }
    } else {
      if ((int)lane < R * WPG && glt + (int)lane / WPG < groups_valid)
        wlo[t] = (uint32_t)packed[tile_words + lane];
    }
  }
  // the block's scales and minima go to LDS only now, after the word loads have been issued, so
  // that the two global round trips overlap
  if ((int)threadIdx.x < groups_valid) {
    s_scale[threadIdx.x] = my_scale;
    s_min[threadIdx.x] = my_min;
  }
  __syncthreads();
#pragma unroll
  for (int t = 0; t < kGroupsPerHalf / R; ++t) {
    const int q0 = t * R;
    uint64_t acc = transpose32(wlo[t], lane);
    if (TL::kTwoRegs) acc |= (uint64_t)transpose32(whi[t], lane) << 32;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int gl = TL::group_of(hw, q0 + r);
      if (gl < groups_valid) {
        const Dequant<T> dq(s_scale[gl], s_min[gl]);
        if constexpr (sizeof(T) == 2 && BITS <= 2) {
          // A group at 1 or 2 bits has at most four distinct values.  Lane l evaluates level l & 3
          // (once instead of once per element), the four lanes of a quad exchange them (DPP
          // quad_perm broadcasts) into an 8-byte table, and every pair of elements is one byte
          // permute of that table.  Same arithmetic per level, hence the same bits.
          const float mine = dq(lane & 3u);
          const int h = (int)(sizeof(T) == 2 && IsBf16<T>::value ? float_to_bf16_bits(mine) : float_to_half_bits(mine));
          const uint32_t l0 = (uint32_t)__builtin_amdgcn_update_dpp(0, h, 0x00, 0xF, 0xF, true);   // quad_perm [0,0,0,0]
          const uint32_t l1 = (uint32_t)__builtin_amdgcn_update_dpp(0, h, 0x55, 0xF, 0xF, true);   // [1,1,1,1]
          const uint32_t l2 = (uint32_t)__builtin_amdgcn_update_dpp(0, h, 0xAA, 0xF, 0xF, true);   // [2,2,2,2]
          const uint32_t l3 = (uint32_t)__builtin_amdgcn_update_dpp(0, h, 0xFF, 0xF, 0xF, true);   // [3,3,3,3]
          const uint32_t lut_lo = l0 | (l1 << 16), lut_hi = l2 | (l3 << 16);
          const uint32_t a = (uint32_t)(acc >> (r * WPG));
          u32x4 outw;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const uint32_t c0 = (a >> (2 * j * BITS)) & kMask;
            const uint32_t c1 = (a >> ((2 * j + 1) * BITS)) & kMask;
            // bytes 2c, 2c+1 of the table for each of the two elements
            const uint32_t sel = (c0 * 0x0202u + 0x0100u) | ((c1 * 0x0202u + 0x0100u) << 16);
            outw[j] = __builtin_amdgcn_perm(lut_hi, lut_lo, sel);
          }
          store16_nt(out + elem_base + (int64_t)gl * kGs + lane * 8, outw);
          continue;
        }
        float v[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) v[k] = dq((uint32_t)(acc >> (r * WPG + k * BITS)) & kMask);
        if constexpr (kStage) {
#pragma unroll
          for (int k = 0; k < 8; ++k) vs[kStage ? q0 + r : 0][k] = v[k];
        } else {
          store8_nt(out + elem_base + (int64_t)gl * kGs + lane * 8, v);
        }
      }
    }
  }
  if constexpr (kStage)
    stage_out_f32<kGroupsPerHalf, TL>(reinterpret_cast<float*>(out), elem_base, groups_valid, slab, vs);
}

template <typename T>
__global__ __launch_bounds__(kThreads) void unpack_mixed_kernel(
    const int32_t* __restrict__ packed, const int32_t* __restrict__ bits,
    const int32_t* __restrict__ prefix, const T* __restrict__ scale, const T* __restrict__ mn,
    T* __restrict__ out, int64_t G, int blocks_per_sample) {
  constexpr int kGroupsPerBlock = kHalfWaves * Gph<T>::kUnpack;
  __shared__ float s_scale[kGroupsPerBlock];
  __shared__ float s_min[kGroupsPerBlock];
  constexpr bool kStage = IsF32<T>::value;
  __shared__ u32x4 s_slab[kStage ? kGroupsPerBlock * 64 : 1];
  u32x4* slab = s_slab + (kStage ? (threadIdx.x >> 6) * (2 * Gph<T>::kUnpack * 64) : 0);
  const int64_t n = blockIdx.x / blocks_per_sample;
  const int64_t gb = (int64_t)(blockIdx.x % blocks_per_sample) * kGroupsPerBlock;
  const int b = bits[n];
  const int groups_valid = (int)((G - gb) < kGroupsPerBlock ? (G - gb) : kGroupsPerBlock);
  float my_scale = 0.0f, my_min = 0.0f;
  if ((int)threadIdx.x < groups_valid) {
    const int64_t gi = n * G + gb + threadIdx.x;
    my_scale = Conv<T>::load(scale, gi);
    my_min = Conv<T>::load(mn, gi);
  }
  const int64_t elem_base = (n * G + gb) * kGs;
  const int64_t word_base = (int64_t)prefix[n] * G * 8 + gb * 8 * b;
  switch (b) {
#define ACTNN_CASE(B_)                                                                          \
  case B_:                                                                                      \
    unpack_groups<T, B_>(packed, out, elem_base, word_base, groups_valid, s_scale, s_min,       \
                         my_scale, my_min, slab);                                               \
    break;
    ACTNN_CASE(1) ACTNN_CASE(2) ACTNN_CASE(3) ACTNN_CASE(4)
    ACTNN_CASE(5) ACTNN_CASE(6) ACTNN_CASE(7) ACTNN_CASE(8)
#undef ACTNN_CASE
    default: break;
  }
}

// ---------------------------------------------------------------------------- generic group size
// One block per (sample, group); codes staged as bytes in LDS, then thread w assembles word w.
template <typename T, bool DET>
__global__ __launch_bounds__(kThreads) void pack_mixed_generic_kernel(
    const T* __restrict__ data, const T* __restrict__ mn, const T* __restrict__ mx,
    const int32_t* __restrict__ bits, const int32_t* __restrict__ prefix, T* __restrict__ scale,
    int32_t* __restrict__ packed, const T* __restrict__ noise, uint64_t seed, uint64_t offset,
    int64_t G, int gs) {
  __shared__ uint8_t s_code[1024];
  __shared__ float s_par[2];
  const int64_t n = blockIdx.x / G;
  const int64_t g = blockIdx.x % G;
  const int b = bits[n];
  if (b < 1 || b > 8) return;
  const int64_t gi = n * G + g;
  if (threadIdx.x == 0) {
    float mul, sub;
    const float sc = GroupQuant<T, DET>::prepare(Conv<T>::load(mn, gi), Conv<T>::load(mx, gi), b, mul, sub);
    Conv<T>::store(scale, gi, sc);
    s_par[0] = mul;
    s_par[1] = sub;
  }
  __syncthreads();
  const float mul = s_par[0], sub = s_par[1];
  const float Bf = (float)((1 << b) - 1);
  for (int d = threadIdx.x; d < gs; d += kThreads) {
    const int64_t e = gi * gs + d;
    const float x = Conv<T>::load(data, e);
    uint32_t c;
    if (DET) {
      c = det_code<T>(x, Conv<T>::load(noise, e), mul, sub, Bf);
    } else {
      uint32_t w[Noise<T>::kWords];
      Noise<T>::octet((uint64_t)e >> 3, seed, offset, w);
      uint32_t r = Noise<T>::at(w, 0);
#pragma unroll
      for (int k = 1; k < 8; ++k) r = ((int)(e & 7) == k) ? Noise<T>::at(w, k) : r;
      c = RngFixed<T>::word(x, r, mul, sub, RngFixed<T>::unit(b)) >> (32 - b);
    }
    s_code[d] = (uint8_t)c;
  }
  __syncthreads();
  const int E = gs / 32;
  const int L = E * b;
  const int64_t word_base = ((int64_t)prefix[n] * G + (int64_t)b * g) * E;
  for (int w = threadIdx.x; w < L; w += kThreads) {
    const int k = w / b, i = w % b;
    uint32_t word = 0;
    for (int j = 0; j < 32; ++j) word |= ((uint32_t)(s_code[E * j + k] >> i) & 1u) << j;
    packed[word_base + w] = (int32_t)word;
  }
}

template <typename T>
__global__ __launch_bounds__(kThreads) void unpack_mixed_generic_kernel(
    const int32_t* __restrict__ packed, const int32_t* __restrict__ bits,
    const int32_t* __restrict__ prefix, const T* __restrict__ scale, const T* __restrict__ mn,
    T* __restrict__ out, int64_t G, int gs) {
  __shared__ uint32_t s_word[256];   // E * b <= 32 * 8
  const int64_t n = blockIdx.x / G;
  const int64_t g = blockIdx.x % G;
  const int b = bits[n];
  if (b < 1 || b > 8) return;
  const int E = gs / 32;
  const int L = E * b;
  const int64_t word_base = ((int64_t)prefix[n] * G + (int64_t)b * g) * E;
  for (int w = threadIdx.x; w < L; w += kThreads) s_word[w] = (uint32_t)packed[word_base + w];
  __syncthreads();
  const int64_t gi = n * G + g;
  const Dequant<T> dq(Conv<T>::load(scale, gi), Conv<T>::load(mn, gi));
  for (int d = threadIdx.x; d < gs; d += kThreads) {
    const int j = d / E, k = d % E;
    uint32_t c = 0;
    for (int i = 0; i < b; ++i) c |= ((s_word[k * b + i] >> j) & 1u) << i;
    Conv<T>::store(out, gi * gs + d, dq(c));
  }
}

// ---------------------------------------------------------------------------- prefix sum
__global__ __launch_bounds__(1024) void bits_prefix_kernel(const int32_t* __restrict__ bits,
                                                           int32_t* __restrict__ prefix, int64_t N) {
  __shared__ int32_t s_part[1024];
  // thread t owns the contiguous chunk [t * per, (t + 1) * per)
  const int64_t per = (N + 1023) / 1024;
  const int64_t lo = (int64_t)threadIdx.x * per;
  const int64_t hi = lo + per < N ? lo + per : N;
  int32_t sum = 0;
  for (int64_t i = lo; i < hi; ++i) sum += bits[i];
  s_part[threadIdx.x] = sum;
  __syncthreads();
  for (int off = 1; off < 1024; off <<= 1) {           // inclusive Hillis-Steele scan
    int32_t add = threadIdx.x >= (unsigned)off ? s_part[threadIdx.x - off] : 0;
    __syncthreads();
    s_part[threadIdx.x] += add;
    __syncthreads();
  }
  int32_t run = threadIdx.x == 0 ? 0 : s_part[threadIdx.x - 1];
  if (threadIdx.x == 0) prefix[0] = 0;
  for (int64_t i = lo; i < hi; ++i) {
    run += bits[i];
    prefix[i + 1] = run;
  }
}

template <typename T>
int launch_pack(const void* data, const void* mn, const void* mx, const int32_t* bits,
                const int32_t* prefix, void* scale, int32_t* packed, const void* noise,
                uint64_t seed, uint64_t offset, int64_t N, int64_t G, int64_t gs, hipStream_t s) {
  const T* d = static_cast<const T*>(data);
  const T* nz = static_cast<const T*>(noise);
  if (gs == kGs) {
    constexpr int kGroupsPerBlock = kHalfWaves * Gph<T>::kPack;
    const int64_t bps = (G + kGroupsPerBlock - 1) / kGroupsPerBlock;
    if (N * bps > 0x7fffffffLL) return ACTNN_EINVAL;
    const dim3 grid((unsigned)(N * bps));
    if (noise)
      pack_mixed_kernel<T, true><<<grid, dim3(kThreads), 0, s>>>(
          d, static_cast<const T*>(mn), static_cast<const T*>(mx), bits, prefix,
          static_cast<T*>(scale), packed, nz, seed, offset, G, (int)bps);
    else
      pack_mixed_kernel<T, false><<<grid, dim3(kThreads), 0, s>>>(
          d, static_cast<const T*>(mn), static_cast<const T*>(mx), bits, prefix,
          static_cast<T*>(scale), packed, nz, seed, offset, G, (int)bps);
  } else {
    if (N * G > 0x7fffffffLL) return ACTNN_EINVAL;
    const dim3 grid((unsigned)(N * G));
    if (noise)
      pack_mixed_generic_kernel<T, true><<<grid, dim3(kThreads), 0, s>>>(
          d, static_cast<const T*>(mn), static_cast<const T*>(mx), bits, prefix,
          static_cast<T*>(scale), packed, nz, seed, offset, G, (int)gs);
    else
      pack_mixed_generic_kernel<T, false><<<grid, dim3(kThreads), 0, s>>>(
          d, static_cast<const T*>(mn), static_cast<const T*>(mx), bits, prefix,
          static_cast<T*>(scale), packed, nz, seed, offset, G, (int)gs);
  }
  ACTNN_RETURN_LAUNCH_STATUS();
}

template <typename T>
int launch_unpack(const int32_t* packed, const int32_t* bits, const int32_t* prefix,
                  const void* scale, const void* mn, void* out, int64_t N, int64_t G, int64_t gs,
                  hipStream_t s) {
  if (gs == kGs) {
    constexpr int kGroupsPerBlock = kHalfWaves * Gph<T>::kUnpack;
    const int64_t bps = (G + kGroupsPerBlock - 1) / kGroupsPerBlock;
    if (N * bps > 0x7fffffffLL) return ACTNN_EINVAL;
    unpack_mixed_kernel<T><<<dim3((unsigned)(N * bps)), dim3(kThreads), 0, s>>>(
        packed, bits, prefix, static_cast<const T*>(scale), static_cast<const T*>(mn),
        static_cast<T*>(out), G, (int)bps);
  } else {
    if (N * G > 0x7fffffffLL) return ACTNN_EINVAL;
    unpack_mixed_generic_kernel<T><<<dim3((unsigned)(N * G)), dim3(kThreads), 0, s>>>(
        packed, bits, prefix, static_cast<const T*>(scale), static_cast<const T*>(mn),
        static_cast<T*>(out), G, (int)gs);
  }
  ACTNN_RETURN_LAUNCH_STATUS();
}

}  // namespace
}  // namespace actnn

extern "C" int actnn_bits_prefix(const int32_t* bits, int32_t* prefix, int64_t N, void* stream) {
  using namespace actnn;
  if (N < 0 || !prefix || (N > 0 && !bits)) return ACTNN_EINVAL;
  bits_prefix_kernel<<<dim3(1), dim3(1024), 0, static_cast<hipStream_t>(stream)>>>(bits, prefix, N);
  ACTNN_RETURN_LAUNCH_STATUS();
}

extern "C" int actnn_pack_mixed(const void* data, const void* mn, const void* mx,
                                const int32_t* bits, const int32_t* prefix, void* scale,
                                int32_t* packed, const void* noise, uint64_t seed, uint64_t offset,
                                int64_t N, int64_t G, int64_t gs, int dtype, void* stream) {
  using namespace actnn;
  if (N < 0 || G < 0 || gs < 32 || gs > 1024 || gs % 32 != 0) return ACTNN_EINVAL;
  if (N == 0 || G == 0) return ACTNN_OK;
  if (!data || !mn || !mx || !bits || !prefix || !scale || !packed) return ACTNN_EINVAL;
  if (!aligned16(data) || (noise && !aligned16(noise))) return ACTNN_EALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case ACTNN_F32: return launch_pack<float>(data, mn, mx, bits, prefix, scale, packed, noise, seed, offset, N, G, gs, s);
    case ACTNN_F16: return launch_pack<__half>(data, mn, mx, bits, prefix, scale, packed, noise, seed, offset, N, G, gs, s);
    case ACTNN_BF16: return launch_pack<bf16_t>(data, mn, mx, bits, prefix, scale, packed, noise, seed, offset, N, G, gs, s);
    default: return ACTNN_EDTYPE;
  }
}

extern "C" int actnn_unpack_mixed(const int32_t* packed, const int32_t* bits, const int32_t* prefix,
                                  const void* scale, const void* mn, void* out, int64_t N,
                                  int64_t G, int64_t gs, int dtype, void* stream) {
  using namespace actnn;
  if (N < 0 || G < 0 || gs < 32 || gs > 1024 || gs % 32 != 0) return ACTNN_EINVAL;
  if (N == 0 || G == 0) return ACTNN_OK;
  if (!packed || !bits || !prefix || !scale || !mn || !out) return ACTNN_EINVAL;
  if (!aligned16(out)) return ACTNN_EALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case ACTNN_F32: return launch_unpack<float>(packed, bits, prefix, scale, mn, out, N, G, gs, s);
    case ACTNN_F16: return launch_unpack<__half>(packed, bits, prefix, scale, mn, out, N, G, gs, s);
    case ACTNN_BF16: return launch_unpack<bf16_t>(packed, bits, prefix, scale, mn, out, N, G, gs, s);
    default: return ACTNN_EDTYPE;
  }
}
