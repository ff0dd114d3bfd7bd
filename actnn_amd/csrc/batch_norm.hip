// Training-mode batch normalisation over contiguous [N, C, HW] tensors, forward and backward
// (the work the reference hands to cuDNN through cudnn_batch_norm / cudnn_batch_norm_backward,
// cpp_extension/backward_func.cc:87-88, called from ops.py:448-449 and ops.py:479-481).
//
// All four passes are HBM-bound streams and share one thread-to-data mapping.  A sample is a row
// of F = C*HW elements; a block owns a span of kThreads 16-byte chunks of that row and walks down
// the batch, so a thread meets the same offsets - hence the same one or two channels - in every
// sample.  Everything that depends on the channel (accumulators, coefficients, the position of a
// channel boundary inside the chunk) lives in registers for the whole loop, the loads are
// 16 bytes wide and contiguous across the block, and no per-element division or table lookup is
// needed.  Reductions finish once per block: lanes of one channel are combined with a segmented
// shuffle reduction, the per-wave results are added in a fixed order and written to a table of
// partial sums that a small second kernel folds per channel in double precision (no atomics: the
// result does not depend on the schedule).
//
// The statistics pass can also produce the per-group minimum and maximum of the activation
// quantiser (groups of 256 consecutive elements of the row) from the registers it already holds,
// which saves the quantiser's own read of the tensor.
#include <mutex>

#include "device_utils.h"
#include "quant_math.h"

namespace actnn {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;
// last-use operands are loaded, and results stored, non-temporally (both measured 3-5 % faster)
ACTNN_DEV u32x4 load_last(const void* p) { return load16_nt(p); }
ACTNN_DEV void store_out(void* p, u32x4 v) { store16_nt(p, v); }

typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));

// Arithmetic on the dwords of a 16-byte chunk.  16-bit types use the two-element dot product
// instructions, whose products are exact in fp32.
template <typename T> struct Chunk;
template <> struct Chunk<float> {
  static constexpr int kElems = 4, kPerDword = 1;
  static ACTNN_DEV void add(uint32_t a, float& s) { s += as_float(a); }
  static ACTNN_DEV void dot(uint32_t a, uint32_t b, float& s) { s = fmaf(as_float(a), as_float(b), s); }
  static ACTNN_DEV void widen(uint32_t a, float* v) { v[0] = as_float(a); }
  static ACTNN_DEV uint32_t narrow(const float* v) { return as_uint(v[0]); }
};
template <> struct Chunk<__half> {
  static constexpr int kElems = 8, kPerDword = 2;
  static ACTNN_DEV void add(uint32_t a, float& s) {
    s = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, a), __builtin_bit_cast(f16x2_t, 0x3c003c00u), s, false);
  }
  static ACTNN_DEV void dot(uint32_t a, uint32_t b, float& s) {
    s = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, a), __builtin_bit_cast(f16x2_t, b), s, false);
  }
  static ACTNN_DEV void widen(uint32_t a, float* v) {
    v[0] = half_bits_to_float(a & 0xffffu);
    v[1] = half_bits_to_float(a >> 16);
  }
  static ACTNN_DEV uint32_t narrow(const float* v) {
    return float_to_half_bits(v[0]) | (float_to_half_bits(v[1]) << 16);
  }
};
template <> struct Chunk<bf16_t> {
  static constexpr int kElems = 8, kPerDword = 2;
  static ACTNN_DEV void add(uint32_t a, float& s) {
    s = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, 0x3f803f80u), s, false);
  }
  static ACTNN_DEV void dot(uint32_t a, uint32_t b, float& s) {
    s = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), s, false);
  }
  static ACTNN_DEV void widen(uint32_t a, float* v) {
    v[0] = as_float(a << 16);
    v[1] = as_float(a & 0xffff0000u);
  }
  static ACTNN_DEV uint32_t narrow(const float* v) { return pack_bf16x2(v[0], v[1]); }
};

// Where a thread's chunk lies: the channel of its first element, how many of its elements belong
// to that channel (>= kElems when the chunk does not cross a boundary; the rest belong to the
// next channel - HW >= kElems is a precondition), and whether the chunk exists at all.
struct Place {
  int64_t elem;        // offset of the chunk in the row
  int64_t channel;     // channel of the first element
  int head;            // elements of the chunk in `channel`, clamped to kElems
  bool active;
};
template <int E> ACTNN_DEV Place place_of(int64_t F, int64_t HW) {
  Place p;
  p.elem = ((int64_t)blockIdx.x * kThreads + threadIdx.x) * E;
  p.active = p.elem < F;
  if (!p.active) p.elem = (int64_t)blockIdx.x * kThreads * E;       // a valid address; results dropped
  p.channel = p.elem / HW;
  const int64_t left = (p.channel + 1) * HW - p.elem;
  p.head = left >= E ? E : (int)left;
  return p;
}

// Dword masks that keep the elements of the chunk's first channel.
template <typename T> ACTNN_DEV void head_masks(int head, uint32_t (&m)[4]) {
  constexpr int PD = Chunk<T>::kPerDword;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int k = head - j * PD;
    m[j] = k <= 0 ? 0u : (PD == 2 && k == 1) ? 0x0000ffffu : 0xffffffffu;
  }
}

// Sum over the lanes of a run of equal keys (runs are contiguous); the first lane of a run
// ends with the run's total.
ACTNN_DEV void run_sums(int key, float& a, float& b) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int k2 = __shfl_down(key, d);
    const float a2 = __shfl_down(a, d), b2 = __shfl_down(b, d);
    if (lane + d < 64 && k2 == key) { a += a2; b += b2; }
  }
}

// Adds the block's per-thread sums into the table of partial sums.  (head0, head1) belong to the
// chunk's first channel, (tail0, tail1) to the next one (chunks that cross a boundary only).
// `s_acc` holds kWaves * (slots + 1) pairs; slot `slots` absorbs the chunks that do not exist.
// Within one instruction the lanes that write touch distinct slots (one lane per run of equal
// channels, one lane per channel boundary), and a wave's instructions reach LDS in order, so
// plain read-modify-write is enough and the order of the additions is fixed.
template <int E>
ACTNN_DEV void fold_block(float* s_acc, int slots, const Place& p, int64_t first_channel,
                          float head0, float head1, float tail0, float tail1,
                          float* __restrict__ part) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float* acc = s_acc + (size_t)wave * (slots + 1) * 2;
  for (int i = threadIdx.x; i < kWaves * (slots + 1) * 2; i += kThreads) s_acc[i] = 0.0f;
  __syncthreads();
  const int key = p.active ? (int)(p.channel - first_channel) : slots;
  if (!p.active) { head0 = 0.0f; head1 = 0.0f; }
  run_sums(key, head0, head1);
  const int prev = __shfl_up(key, 1);
  if (lane == 0 || prev != key) {
    acc[2 * key] += head0;
    acc[2 * key + 1] += head1;
  }
  if (p.active && p.head < E) {
    acc[2 * (key + 1)] += tail0;
    acc[2 * (key + 1) + 1] += tail1;
  }
  __syncthreads();
  const int64_t base = ((int64_t)blockIdx.x * gridDim.y + blockIdx.y) * slots * 2;
  for (int i = threadIdx.x; i < slots * 2; i += kThreads) {
    float v = 0.0f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) v += s_acc[(size_t)w * (slots + 1) * 2 + i];
    part[base + i] = v;
  }
}

// Where the input x of the backward passes comes from.  Both sources hand out the chunk of this
// thread for sample n in two steps, so that the loads of several samples can be in flight before
// the first one is used.
template <typename T> struct PlainInput {
  static constexpr bool kRows = false;
  static constexpr int kInFlight = 4;      // samples whose loads are issued before the first is used
  const T* p;            // already offset to the thread's chunk of sample 0
  int64_t F;
  struct Raw { u32x4 v; };
  ACTNN_DEV Raw fetch(int64_t n) const { return Raw{load16(p + n * F)}; }
  ACTNN_DEV u32x4 decode(const Raw& r) const { return r.v; }
};

// x kept as the mixed-precision bit stream of the activation quantiser (pack_mixed layout: sample
// n owns bits[n] * G * 8 words from prefix[n] * G * 8 on; in a group of 256 elements bit i of the
// code of element 8j + k is bit j of word k * bits + i).  The 32 lanes that own a group here are
// the 32 lanes of that layout - lane j holds elements 8j .. 8j+7 - so a half-wave loads the group's
// words, transposes them (32x32 bits) and every lane finds its 8 codes in its own register.
// Values are rebuilt exactly as actnn_unpack_mixed rebuilds them.
// fp32: a lane's 16-byte chunk is 4 elements, so the 64 lanes of a wave own a group and lanes 2j and
// 2j+1 share stream lane j.  Lane l loads word l (up to 64 words at 8 bits), each half of the wave
// transposes its 32 words, and lane l collects the two 32-bit halves of stream lane l >> 1 from
// lanes l >> 1 and 32 + (l >> 1) (ds_bpermute) before it takes its four codes out of them.
template <typename T> struct PackedInput {
  static constexpr bool kRows = false;
  static constexpr int kLanes = 256 / Chunk<T>::kElems;     // lanes that own a group: 32, or 64 for fp32
  static constexpr int kInFlight = 2;      // the decode needs registers: 2 measured faster than 1 and 4
  const int32_t* words;
  const int32_t* bits;
  const int32_t* prefix;
  const T* scale;
  const T* mn;
  int64_t G, g;          // groups per sample, this thread's group
  uint32_t lane32;       // lane within the group's kLanes lanes
  bool active;
  struct Raw { uint32_t lo, hi; float sc, m; int b; };
  // group `grp` of sample n, whose width b and first word (prefix[n] * G * 8) the caller knows
  ACTNN_DEV Raw fetch_known(int64_t n, int64_t grp, int b, int64_t first_word) const {
    Raw r{0u, 0u, 1.0f, 0.0f, b};
    if (active) {
      const int32_t* w = words + first_word + grp * b * 8;
      if ((int)lane32 < 8 * b) r.lo = (uint32_t)w[lane32];
      if (kLanes == 32 && (int)lane32 + 32 < 8 * b) r.hi = (uint32_t)w[lane32 + 32];
      r.sc = Conv<T>::load(scale, n * G + grp);
      r.m = Conv<T>::load(mn, n * G + grp);
    }
    return r;
  }
  ACTNN_DEV Raw fetch(int64_t n) const {
    return fetch_known(n, g, active ? bits[n] : 1, active ? (int64_t)prefix[n] * G * 8 : 0);
  }
  template <int BITS> ACTNN_DEV u32x4 decode_bits(const Raw& r) const {
    uint64_t acc = transpose32(r.lo, lane32);
    if (BITS > 4) acc |= (uint64_t)transpose32(r.hi, lane32) << 32;
    const Dequant<T> dq(r.sc, r.m);
    if constexpr (BITS <= 2) {
      // A group at 1 or 2 bits has at most four distinct values.  Lane l evaluates level l & 3
      // (11 operations once instead of once per element), the four lanes of a quad exchange them
      // (DPP quad_perm broadcasts) into an 8-byte table, and every pair of elements is one byte
      // permute of that table.  Same arithmetic per level, hence the same bits.
      const float mine = dq(lane32 & 3u);
      const float pair[2] = {mine, mine};
      const int h = (int)(Chunk<T>::narrow(pair) & 0xffffu);
      const uint32_t l0 = (uint32_t)__builtin_amdgcn_update_dpp(0, h, 0x00, 0xF, 0xF, true);   // quad_perm [0,0,0,0]
      const uint32_t l1 = (uint32_t)__builtin_amdgcn_update_dpp(0, h, 0x55, 0xF, 0xF, true);   // [1,1,1,1]
      const uint32_t l2 = (uint32_t)__builtin_amdgcn_update_dpp(0, h, 0xAA, 0xF, 0xF, true);   // [2,2,2,2]
      const uint32_t l3 = (uint32_t)__builtin_amdgcn_update_dpp(0, h, 0xFF, 0xF, 0xF, true);   // [3,3,3,3]
      const uint32_t lut_lo = l0 | (l1 << 16), lut_hi = l2 | (l3 << 16);
      // a copy of the codes moved up by 16 - BITS puts the second code of every pair 16 bits above the
      // first: one shift and one mask then give both (c0 | c1 << 16), and a multiply-add turns them into
      // the byte selectors 2c, 2c + 1 of the two elements
      constexpr uint32_t kPair = ((1u << BITS) - 1u) * 0x00010001u;
      const uint32_t a = (uint32_t)acc & 0xffffu;
      const uint32_t both = a | (a << (16 - BITS));
      uint32_t out[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t sel = __umul24((both >> (2 * j * BITS)) & kPair, 0x0202u) + 0x01000100u;
        out[j] = __builtin_amdgcn_perm(lut_hi, lut_lo, sel);
      }
      return u32x4{out[0], out[1], out[2], out[3]};
    }
    float v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = dq((uint32_t)(acc >> (k * BITS)) & ((1u << BITS) - 1u));
    return u32x4{Chunk<T>::narrow(v), Chunk<T>::narrow(v + 2), Chunk<T>::narrow(v + 4), Chunk<T>::narrow(v + 6)};
  }
  ACTNN_DEV u32x4 decode_f32(const Raw& r) const {
    const uint32_t t = transpose32(r.lo, lane32 & 31u);       // lanes 0..31: words 0..31, lanes 32..63: words 32..63
    const int j = (int)(lane32 >> 1);
    const uint32_t lo = (uint32_t)__builtin_amdgcn_ds_bpermute(j << 2, (int)t);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_ds_bpermute((32 + j) << 2, (int)t);
    const uint64_t acc = (uint64_t)lo | ((uint64_t)hi << 32);  // the 8 codes of stream lane j
    const uint32_t mine = (uint32_t)(acc >> (4 * r.b * (int)(lane32 & 1u)));   // elements 4 (l & 1) .. + 3
    const uint32_t mask = (1u << r.b) - 1u;
    const Dequant<T> dq(r.sc, r.m);
    u32x4 out;
#pragma unroll
    for (int m = 0; m < 4; ++m) out[m] = as_uint(dq((mine >> (m * r.b)) & mask));
    return out;
  }
  ACTNN_DEV u32x4 decode(const Raw& r) const {
    if constexpr (sizeof(T) == 4) {
      return decode_f32(r);
    } else {
      switch (r.b) {                     // uniform over the block: one sample, one width
        case 1: return decode_bits<1>(r);
        case 2: return decode_bits<2>(r);
        case 3: return decode_bits<3>(r);
        case 4: return decode_bits<4>(r);
        case 5: return decode_bits<5>(r);
        case 6: return decode_bits<6>(r);
        case 7: return decode_bits<7>(r);
        default: return decode_bits<8>(r);
      }
    }
  }
};

// Where the forward apply pass can leave the activation quantiser's output: the chunk a lane holds
// is its share of one quantisation group (32 lanes per group, 16-bit types), so the codes are made
// from the registers the normalisation reads anyway - same arithmetic, same Philox counters (the
// index of the 8-element chunk in the tensor as it lies in memory) and same stream layout as
// actnn_pack_mixed, hence the same bits.
struct PackSink {
  const int32_t* bits;
  const int32_t* prefix;
  const void* mn;
  const void* mx;
  void* scale;
  int32_t* packed;
  uint64_t seed, offset;
  int64_t G;             // groups per sample
  // backward apply only: when set, every wave leaves the sum of the squares of the gradient values
  // it wrote (as stored, i.e. rounded to T) in sumsq[(blockIdx.y * gridDim.x + blockIdx.x) * kWaves +
  // wave] - the gradient-norm statistic of the layer that receives this gradient, for free
  float* sumsq;
  // forward apply with the ReLU folded in: the 1-bit mask (layout of the ReLU operator: 16 words per
  // block of 512 elements) and the min / max of every group of 256 outputs
  int32_t* relu_mask;
  void* relu_mn;
  void* relu_mx;
  // ... and a residual added before the ReLU: y = relu(bn(x) + residual), laid out like x
  const void* relu_add;
};

// ReLU on a word of two 16-bit values (already rounded to T, so the rule sees what a separate pass
// over the stored tensor would see): -> the word with the non-positive halves zeroed; their keep
// flags in bits 0 and 1 of `keep`; the two results as floats.
template <typename T> ACTNN_DEV uint32_t relu_word(uint32_t w, uint32_t& keep, float& z0, float& z1) {
  float v[2];
  Chunk<T>::widen(w, v);
  const bool k0 = v[0] > 0.0f, k1 = v[1] > 0.0f;
  z0 = k0 ? v[0] : 0.0f;
  z1 = k1 ? v[1] : 0.0f;
  keep = (k0 ? 1u : 0u) | (k1 ? 2u : 0u);
  return (k0 ? w & 0x0000ffffu : 0u) | (k1 ? w & 0xffff0000u : 0u);
}
// The other direction: a backward pass whose incoming gradient is that of a ReLU's output takes the
// ReLU's mask along and zeroes what the ReLU's own backward pass would have zeroed, instead of reading
// a masked copy.  Keep bits of the wave's next four steps (a step of a block is 2048 elements: the
// wave's blocks are 4 apart), one word per lane and two bit transposes for the four.
// Where the 64 mask words of a wave's four steps lie.  Rows of up to 256 channels: a step of the wave
// is one whole 512-element block of the mask, and the blocks of consecutive steps are 4 apart.  Rows of
// a multiple of 512 channels: the wave's lanes 0-31 and 32-63 hold the same 256 columns of two
// consecutive rows, i.e. the same half (the column tile's parity) of two blocks C / 512 apart - the
// 16 low bits of each of the wave's words belong to the first block's words, the 16 high bits to the
// second's, and they are stored and loaded as halfwords.
struct MaskPlace {
  uint32_t first, second;  // word index (narrow rows) / halfword indices (wide rows) of the lane's word
  bool wide;               // (32-bit: the launcher takes tensors of up to 2^27 blocks)
};
ACTNN_DEV MaskPlace mask_place(int64_t ru_first, int64_t C, int R, int tile) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t slot = 2u * (lane & 1u) + (lane >> 5);            // which of the four steps the lane's word is of
  const uint32_t k = (lane >> 1) & 15u;
  const uint32_t wave = threadIdx.x >> 6;
  MaskPlace at;
  at.wide = C > 256;
  if (!at.wide) {
    const uint32_t block0 = (uint32_t)((ru_first * C) >> 9);      // the same for the whole block of threads
    at.first = (block0 + wave + 4u * slot) * 16u + k;
    at.second = 0u;
  } else {
    const uint32_t per_row = (uint32_t)(C >> 9);
    const uint32_t block0 = (uint32_t)ru_first * per_row + ((uint32_t)tile >> 1);
    const uint32_t block = block0 + (slot * (uint32_t)R + 2u * wave) * per_row;
    at.first = (block * 16u + k) * 2u + ((uint32_t)tile & 1u);
    at.second = at.first + per_row * 32u;
  }
  return at;
}
struct ReluRows {
  const int32_t* words;
  int64_t blocks;          // 512-element blocks of the tensor
  ACTNN_DEV void load(int64_t rb, int64_t C, int R, int tile, uint32_t (&m)[4]) const {
    const MaskPlace at = mask_place(rb, C, R, tile);
    const uint32_t end = (uint32_t)blocks * 16u;
    uint32_t w = 0u;
    if (!at.wide) {
      if (at.first < end) w = (uint32_t)words[at.first];
    } else {
      const uint16_t* half = reinterpret_cast<const uint16_t*>(words);
      if (at.first < 2u * end) w = half[at.first];
      if (at.second < 2u * end) w |= (uint32_t)half[at.second] << 16;
    }
    word_to_rows(w, threadIdx.x & 63u, m);
  }
};
// the chunk's eight 16-bit values with those zeroed whose keep bit (bit i of `row` for value i) is 0
ACTNN_DEV u32x4 keep_chunk(const u32x4& d, uint32_t row) {
  uint32_t w[4] = {d.x, d.y, d.z, d.w};
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const uint32_t a = 0u - ((row >> (2 * q)) & 1u), b = 0u - ((row >> (2 * q + 1)) & 1u);
    w[q] &= (a & 0x0000ffffu) | (b << 16);
  }
  return u32x4{w[0], w[1], w[2], w[3]};
}

ACTNN_DEV void leave_wave_sum(float* table, float v) {
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) v += __shfl_xor(v, d);
  if ((threadIdx.x & 63) == 0)
    table[((int64_t)blockIdx.y * gridDim.x + blockIdx.x) * kWaves + (threadIdx.x >> 6)] = v;
}

template <typename T, int BITS>
ACTNN_DEV void pack_chunk_bits(const float (&v)[8], const uint32_t (&rw)[Noise<T>::kWords], float mul, float sub,
                               uint32_t lane32, int32_t* __restrict__ dst) {
  constexpr float kUnit = (float)(1u << (32 - BITS - Noise<T>::kBits));
  CodeShifter<BITS, (BITS > 4)> sh;
#pragma unroll
  for (int k = 7; k >= 0; --k) sh.push(RngFixed<T>::word(v[k], Noise<T>::at(rw, k), mul, sub, kUnit));
  const uint64_t acc = ((uint64_t)sh.hi << 32) | sh.lo;
  const uint32_t lo = transpose32((uint32_t)acc, lane32);
  if ((int)lane32 < 8 * BITS) __builtin_nontemporal_store((int32_t)lo, dst + lane32);
  if (BITS > 4) {
    const uint32_t hi = transpose32((uint32_t)(acc >> 32), lane32);
    if ((int)lane32 < 8 * BITS - 32) __builtin_nontemporal_store((int32_t)hi, dst + 32 + lane32);
  }
}

// Quantisation parameters of the next 32 chunks a half-wave will pack (its 32 lanes own one group in
// every chunk): lane j works out the scale of chunk j - one evaluation of the double-precision
// quotient per group instead of one per lane and group - stores it, and hands (mul, sub) to the
// other lanes when chunk j's turn comes.
template <typename T> struct ParamQueue {
  float mul = 0.0f, sub = 0.0f;
  // lane j: gi = index of the group of chunk j (n * G + group within the sample), b = its width;
  // live = chunk j exists
  ACTNN_DEV void fill(const PackSink& ps, int64_t gi, int b, bool live) {
    mul = 0.0f;
    sub = 0.0f;
    if (live) {
      const float sc = GroupQuant<T, false>::prepare(Conv<T>::load(static_cast<const T*>(ps.mn), gi),
                                                     Conv<T>::load(static_cast<const T*>(ps.mx), gi), b, mul, sub);
      Conv<T>::store(static_cast<T*>(ps.scale), gi, sc);
    }
  }
  // (the lanes that own a group: a half-wave, or the whole wave for fp32)
  ACTNN_DEV void get(int j, float& m, float& sb) const {
    constexpr int kLanes = 256 / Chunk<T>::kElems;
    m = __shfl(mul, j, kLanes);
    sb = __shfl(sub, j, kLanes);
  }
};

// fp32: one group spans the wave - lane l holds elements 4l .. 4l+3, i.e. lanes 2j and 2j+1 share
// stream lane j and octet j.  Two chunks A and B of a lane (two samples, or two rows) are packed
// together: the even lane evaluates A's Philox call and the odd lane B's (each hands the other the
// two words it does not use), both quantise their four elements of A and of B, then the even lane
// collects A's eight codes and the odd lane B's (one exchange), and two interleaved 32x32 bit
// transposes leave word p of A in lane 2p and of B in lane 2p+1.  The widths of A and B may differ
// (different samples): everything here takes the width at run time.  Same arithmetic, counters
// and layout as actnn_pack_mixed, hence the same bits.
struct ChunkParams {
  float mul, sub;
  int b;
  int32_t* dst;            // first word of the chunk's group in the stream
  uint64_t octet;          // index of the lane pair's octet
};
ACTNN_DEV void pack_chunk_pair_f32(const PackSink& ps, const u32x4& xa, const ChunkParams& A, const u32x4& xb,
                                   const ChunkParams& B, bool has_b) {
  const uint32_t l = threadIdx.x & 63u;
  const bool odd = l & 1u;
  const uint32_t j = l >> 1;
  const Philox4 r = philox_at(odd ? B.octet : A.octet, ps.seed, ps.offset);
  const uint32_t nx = lane_xor<1>(r.x), ny = lane_xor<1>(r.y), nz = lane_xor<1>(r.z), nw = lane_xor<1>(r.w);
  // even lane: elements 0..3 of both octets (words 0, 1); odd lane: elements 4..7 (words 2, 3)
  const uint32_t na[2] = {odd ? nz : r.x, odd ? nw : r.y};
  const uint32_t nb[2] = {odd ? r.z : nx, odd ? r.w : ny};
  auto codes = [](const u32x4& x, const uint32_t (&n)[2], const ChunkParams& q) -> uint32_t {
    const float unit = as_float((uint32_t)(127 + 16 - q.b) << 23);          // 2^(32 - b - 16)
    uint32_t c = 0;
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const uint32_t r16 = (n[m >> 1] >> (16 * (m & 1))) & 0xffffu;
      c |= (RngFixed<float>::word(as_float(x[m]), r16, q.mul, q.sub, unit) >> (32 - q.b)) << (m * q.b);
    }
    return c;
  };
  const uint32_t ca = codes(xa, na, A), cb = codes(xb, nb, B);
  // the even lane keeps A and takes the odd lane's A codes (elements 4..7); the odd lane keeps B
  // and takes the even lane's B codes (elements 0..3)
  const uint32_t got = lane_xor<1>(odd ? ca : cb);
  const int b = odd ? B.b : A.b;
  const uint64_t acc = (uint64_t)(odd ? got : ca) | ((uint64_t)(odd ? cb : got) << (4 * b));
  int32_t* dst = odd ? B.dst : A.dst;
  const bool live = !odd || has_b;
  const uint32_t lo = transpose32_x2((uint32_t)acc, l);
  if (live && (int)j < 8 * b) __builtin_nontemporal_store((int32_t)lo, dst + j);
  if (A.b > 4 || B.b > 4) {                                                  // uniform over the wave
    const uint32_t hi = transpose32_x2((uint32_t)(acc >> 32), l);
    if (live && (int)j + 32 < 8 * b) __builtin_nontemporal_store((int32_t)hi, dst + 32 + j);
  }
}

// Noise words of two octets of this lane whose neighbours (index ^ 1) lane ^ 1 holds: the two lanes
// share their Philox calls when octet and lane parity agree (they do wherever a block starts on an
// even octet; the test is the same for every lane of a block).
template <typename T>
ACTNN_DEV void noise_pair(const PackSink& ps, uint64_t oa, uint64_t ob, uint32_t (&wa)[Noise<T>::kWords],
                          uint32_t (&wb)[Noise<T>::kWords], bool together) {
  // together: lane ^ 1 is known to make this call in the same step
  if (together && (((uint32_t)oa ^ threadIdx.x) & 1u) == 0 && (((uint32_t)ob ^ threadIdx.x) & 1u) == 0) {
    Noise<T>::octets(oa, ob, ps.seed, ps.offset, wa, wb);
  } else {
    Noise<T>::octet(oa, ps.seed, ps.offset, wa);
    Noise<T>::octet(ob, ps.seed, ps.offset, wb);
  }
}

// b: the sample's width, dst: first word of the chunk's group in the stream (both looked up by the
// caller, who knows how often the sample changes); (mul, sub): the group's parameters from the queue;
// rw: the noise words of the chunk's octet.  SCALAR_B: b is known to be one number for the wave (the
// sample comes from the block's index); otherwise the wave checks, and takes one scalar branch when
// its lanes agree - as they do except where a wave spans two samples of different widths.
template <typename T>
ACTNN_DEV void pack_chunk_width(const float (&v)[8], const uint32_t (&rw)[Noise<T>::kWords], float mul, float sub,
                                uint32_t lane32, int32_t* __restrict__ dst, int b) {
  switch (b) {
    case 1: pack_chunk_bits<T, 1>(v, rw, mul, sub, lane32, dst); break;
    case 2: pack_chunk_bits<T, 2>(v, rw, mul, sub, lane32, dst); break;
    case 3: pack_chunk_bits<T, 3>(v, rw, mul, sub, lane32, dst); break;
    case 4: pack_chunk_bits<T, 4>(v, rw, mul, sub, lane32, dst); break;
    case 5: pack_chunk_bits<T, 5>(v, rw, mul, sub, lane32, dst); break;
    case 6: pack_chunk_bits<T, 6>(v, rw, mul, sub, lane32, dst); break;
    case 7: pack_chunk_bits<T, 7>(v, rw, mul, sub, lane32, dst); break;
    case 8: pack_chunk_bits<T, 8>(v, rw, mul, sub, lane32, dst); break;
    default: break;
  }
}
template <typename T, bool SCALAR_B>
ACTNN_DEV void pack_chunk(const u32x4& ux, const uint32_t (&rw)[Noise<T>::kWords], float mul, float sub,
                          int32_t* __restrict__ dst, int b) {
  constexpr int PD = Chunk<T>::kPerDword;
  static_assert(Chunk<T>::kElems == 8, "16-bit types only");
  const uint32_t lane32 = threadIdx.x & 31;
  const uint32_t w[4] = {ux.x, ux.y, ux.z, ux.w};
  float v[8];
#pragma unroll
  for (int k = 0; k < 4; ++k) Chunk<T>::widen(w[k], v + k * PD);
  if constexpr (SCALAR_B) {
    pack_chunk_width<T>(v, rw, mul, sub, lane32, dst, b);
  } else {
    const int b0 = __builtin_amdgcn_readfirstlane(b);
    if (__builtin_amdgcn_ballot_w64(b != b0) == 0) pack_chunk_width<T>(v, rw, mul, sub, lane32, dst, b0);
    else pack_chunk_width<T>(v, rw, mul, sub, lane32, dst, b);
  }
}

template <typename T> ACTNN_DEV void bind_input(PlainInput<T>& xs, const Place& p) { xs.p += p.elem; }
template <typename T> ACTNN_DEV void bind_input(PackedInput<T>& xs, const Place& p) {
  xs.g = p.elem >> 8;
  xs.lane32 = threadIdx.x & (PackedInput<T>::kLanes - 1);
  xs.active = p.active;
}

// Pass 1 of either direction.  Forward: per-channel sum(x) and sum(x*x) (+ per-group min/max of
// x when MINMAX).  Backward: per-channel sum(dy) and sum(x*dy).
template <typename T, bool SPLIT, bool BWD, bool MINMAX, typename XS>
__global__ __launch_bounds__(kThreads, 6) void bn_reduce_kernel(
    XS xs, const T* __restrict__ dy, float* __restrict__ part,
    T* __restrict__ mn, T* __restrict__ mx, int64_t N, int64_t F, int64_t HW, int per_block, int slots) {
  constexpr int E = Chunk<T>::kElems;
  constexpr int kUnroll = XS::kInFlight;
  extern __shared__ float s_acc[];
  const Place p = place_of<E>(F, HW);
  bind_input(xs, p);
  uint32_t m[4];
  head_masks<T>(p.head, m);
  const int64_t n0 = (int64_t)blockIdx.y * per_block;
  const int64_t n1 = n0 + per_block < N ? n0 + per_block : N;
  float t0 = 0.0f, t1 = 0.0f, h0 = 0.0f, h1 = 0.0f;

  auto accumulate = [&](const u32x4& ux, const u32x4& ud, int64_t n) {
    const uint32_t w[4] = {ux.x, ux.y, ux.z, ux.w};
    const uint32_t d[4] = {ud.x, ud.y, ud.z, ud.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t a = BWD ? d[j] : w[j];
      Chunk<T>::add(a, t0);
      Chunk<T>::dot(w[j], a, t1);
      if (SPLIT) {
        const uint32_t am = a & m[j];
        Chunk<T>::add(am, h0);
        Chunk<T>::dot(w[j], am, h1);
      }
    }
    if (MINMAX) {
      constexpr int PD = Chunk<T>::kPerDword;
      constexpr int LPG = 256 / E;                      // lanes per quantisation group
      float v[E];
#pragma unroll
      for (int j = 0; j < 4; ++j) Chunk<T>::widen(w[j], v + j * PD);
      float lo, hi;
      minmax_of<E>(v, lo, hi);
      lanes_minmax<LPG / 16>(lo, hi);
      if ((threadIdx.x & (LPG - 1)) == LPG - 1 && p.active) {
        const int64_t g = n * (F >> 8) + (p.elem >> 8);
        Conv<T>::store(mn, g, lo);
        Conv<T>::store(mx, g, hi);
      }
    }
  };

  const T* pd = BWD ? dy + p.elem : nullptr;
  int64_t n = n0;
  for (; n + kUnroll <= n1; n += kUnroll) {
    typename XS::Raw rx[kUnroll];
    u32x4 ud[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      rx[u] = xs.fetch(n + u);
      if (BWD) ud[u] = load16(pd + (n + u) * F);
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const u32x4 ux = xs.decode(rx[u]);
      accumulate(ux, BWD ? ud[u] : ux, n + u);
    }
  }
  for (; n < n1; ++n) {
    const typename XS::Raw rx = xs.fetch(n);
    const u32x4 ux = xs.decode(rx);
    accumulate(ux, BWD ? load16(pd + n * F) : ux, n);
  }
  const int64_t first_channel = ((int64_t)blockIdx.x * kThreads * E) / HW;
  fold_block<E>(s_acc, slots, p, first_channel, SPLIT ? h0 : t0, SPLIT ? h1 : t1,
                SPLIT ? t0 - h0 : 0.0f, SPLIT ? t1 - h1 : 0.0f, part);
}

// Folds the table of partial sums of channel c in double precision: the wave's lanes take the
// (span, batch split) entries of the channel in a fixed assignment and are combined by a butterfly,
// so every lane ends with the same totals and the order of the additions is fixed.
// (channels-last tables, slots == 0, hold nsplit consecutive values per channel and sum.)
ACTNN_DEV void channel_totals(const float* __restrict__ part, int64_t c, int64_t HW, int64_t L,
                              int nsplit, int slots, double& s0, double& s1) {
  const int lane = threadIdx.x & 63;
  s0 = 0.0;
  s1 = 0.0;
  if (slots == 0) {
    const float* q0 = part + (c * 2) * (int64_t)nsplit;
    const float* q1 = q0 + nsplit;
#pragma unroll 8
    for (int i = lane; i < nsplit; i += 64) {
      s0 += (double)q0[i];
      s1 += (double)q1[i];
    }
  } else {
    const int64_t j0 = (c * HW) / L, j1 = ((c + 1) * HW - 1) / L;
    const int64_t count = (j1 - j0 + 1) * nsplit;
    for (int64_t i = lane; i < count; i += 64) {
      const int64_t j = j0 + i / nsplit, y = i % nsplit;
      const int64_t slot = c - (j * L) / HW;
      const float* q = part + ((j * nsplit + y) * slots + slot) * 2;
      s0 += (double)q[0];
      s1 += (double)q[1];
    }
  }
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) {
    s0 += __shfl_xor(s0, d);
    s1 += __shfl_xor(s1, d);
  }
}

// mean / inverse standard deviation of the batch, the running estimates (unbiased variance, as
// torch's batch norm keeps them) and the per-channel coefficients of y = a*x + b.
__global__ __launch_bounds__(kThreads) void bn_forward_finalize_kernel(
    const float* __restrict__ part, const float* __restrict__ weight, const float* __restrict__ bias,
    float* __restrict__ running_mean, float* __restrict__ running_var, float* __restrict__ save_mean,
    float* __restrict__ save_invstd, float* __restrict__ coef, int64_t N, int64_t C, int64_t HW,
    int64_t L, int nsplit, int slots, double momentum, double eps) {
  const int64_t c = (int64_t)blockIdx.x * kWaves + (threadIdx.x >> 6);     // one wave per channel
  if (c >= C) return;
  double S, Q;
  channel_totals(part, c, HW, L, nsplit, slots, S, Q);
  if ((threadIdx.x & 63) != 0) return;
  const double M = (double)N * (double)HW;
  const double mean = S / M;
  double var = Q / M - mean * mean;
  if (!(var > 0.0)) var = 0.0;
  const double invstd = 1.0 / sqrt(var + eps);
  save_mean[c] = (float)mean;
  save_invstd[c] = (float)invstd;
  if (running_mean) running_mean[c] = (float)((1.0 - momentum) * running_mean[c] + momentum * mean);
  if (running_var) {
    const double unbiased = M > 1.0 ? var * (M / (M - 1.0)) : var;
    running_var[c] = (float)((1.0 - momentum) * running_var[c] + momentum * unbiased);
  }
  const double a = (weight ? (double)weight[c] : 1.0) * invstd;
  coef[2 * c] = (float)a;
  coef[2 * c + 1] = (float)((bias ? (double)bias[c] : 0.0) - mean * a);
}

// grad_weight, grad_bias and the per-channel coefficients of dx = A*dy + B*x + K, from
// dx = w*r*(dy - mean(dy) - xhat*mean(dy*xhat)) with xhat = (x - mean)*r.
__global__ __launch_bounds__(kThreads) void bn_backward_finalize_kernel(
    const float* __restrict__ part, const float* __restrict__ weight, const float* __restrict__ save_mean,
    const float* __restrict__ save_invstd, float* __restrict__ dweight, float* __restrict__ dbias,
    float* __restrict__ coef, int64_t N, int64_t C, int64_t HW, int64_t L, int nsplit, int slots, bool eval) {
  const int64_t c = (int64_t)blockIdx.x * kWaves + (threadIdx.x >> 6);     // one wave per channel
  if (c >= C) return;
  double S, Q;                                   // sum(dy), sum(x*dy)
  channel_totals(part, c, HW, L, nsplit, slots, S, Q);
  if ((threadIdx.x & 63) != 0) return;
  const double M = (double)N * (double)HW;
  const double mean = save_mean[c], r = save_invstd[c];
  const double w = weight ? (double)weight[c] : 1.0;
  const double dot = (Q - mean * S) * r;         // sum(dy * xhat)
  if (dweight) dweight[c] = (float)dot;
  if (dbias) dbias[c] = (float)S;
  // evaluation mode: mean and r are constants (the running estimates), so dx = w * r * dy
  const double A = w * r;
  const double B = eval ? 0.0 : -w * r * r * (dot / M);
  coef[3 * c] = (float)A;
  coef[3 * c + 1] = (float)B;
  coef[3 * c + 2] = eval ? 0.0f : (float)(-A * (S / M) - B * mean);
}

// Evaluation mode: mean and variance are the running estimates; leaves them (as mean and inverse
// standard deviation) for the backward pass and the coefficients of y = a*x + b for the apply pass.
__global__ __launch_bounds__(kThreads) void bn_eval_coefficients_kernel(
    const float* __restrict__ weight, const float* __restrict__ bias, const float* __restrict__ running_mean,
    const float* __restrict__ running_var, float* __restrict__ save_mean, float* __restrict__ save_invstd,
    float* __restrict__ coef, int64_t C, double eps) {
  const int64_t c = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (c >= C) return;
  const double mean = running_mean[c];
  const double invstd = 1.0 / sqrt((double)running_var[c] + eps);
  if (save_mean) save_mean[c] = (float)mean;
  if (save_invstd) save_invstd[c] = (float)invstd;
  const double a = (weight ? (double)weight[c] : 1.0) * invstd;
  coef[2 * c] = (float)a;
  coef[2 * c + 1] = (float)((bias ? (double)bias[c] : 0.0) - mean * a);
}

// ------------------------------------------------------------------ any shape
// Shapes the chunked kernels do not take - a row of C*HW elements that is not a whole number of
// 16-byte chunks, planes shorter than a chunk, channels-last tensors whose C is not a multiple of
// the chunk - go element by element: a block per channel and slice of the batch for the sums (table
// layout of the channels-last passes: [channel][sum][slice]), a thread per element for the second
// pass.  Same arithmetic (fp32 sums folded in double, y = fma(x, a, b)), a fraction of the speed;
// such shapes are rare.
template <typename T, bool BWD, bool CL>
__global__ __launch_bounds__(kThreads) void bn_any_reduce_kernel(
    const T* __restrict__ x, const T* __restrict__ dy, float* __restrict__ part, int64_t N, int64_t C,
    int64_t HW, int64_t per_block) {
  __shared__ float s_wave[2 * kWaves];
  const int64_t c = blockIdx.x;
  const int64_t n0 = (int64_t)blockIdx.y * per_block;
  const int64_t n1 = n0 + per_block < N ? n0 + per_block : N;
  float s = 0.0f, q = 0.0f;
  for (int64_t n = n0; n < n1; ++n) {
    for (int64_t hw = threadIdx.x; hw < HW; hw += kThreads) {
      const int64_t at = CL ? (n * HW + hw) * C + c : (n * C + c) * HW + hw;
      const float xv = Conv<T>::load(x, at);
      const float a = BWD ? Conv<T>::load(dy, at) : xv;
      s += a;
      q = fmaf(xv, a, q);
    }
  }
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) {
    s += __shfl_xor(s, d);
    q += __shfl_xor(q, d);
  }
  if ((threadIdx.x & 63) == 0) {
    s_wave[2 * (threadIdx.x >> 6)] = s;
    s_wave[2 * (threadIdx.x >> 6) + 1] = q;
  }
  __syncthreads();
  if (threadIdx.x < 2) {
    float v = 0.0f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) v += s_wave[2 * w + threadIdx.x];
    part[(c * 2 + threadIdx.x) * gridDim.y + blockIdx.y] = v;
  }
}

template <typename T, bool BWD, bool CL>
__global__ __launch_bounds__(kThreads) void bn_any_apply_kernel(
    const T* __restrict__ x, const T* __restrict__ dy, const float* __restrict__ coef, T* __restrict__ out,
    int64_t total, int64_t C, int64_t HW) {
  constexpr int NC = BWD ? 3 : 2;
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < total; i += (int64_t)gridDim.x * kThreads) {
    const int64_t c = CL ? i % C : (i / HW) % C;
    const float xv = Conv<T>::load(x, i);
    const float v = BWD ? fmaf(Conv<T>::load(dy, i), coef[NC * c], fmaf(xv, coef[NC * c + 1], coef[NC * c + 2]))
                        : fmaf(xv, coef[NC * c], coef[NC * c + 1]);
    Conv<T>::store(out, i, v);
  }
}


// Pass 2 of either direction.  Forward: y = a*x + b.  Backward: dx = A*dy + B*x + K.
template <typename T, bool SPLIT, bool BWD, bool PACK, typename XS>
__global__ __launch_bounds__(kThreads) void bn_apply_kernel(
    XS xs, const T* __restrict__ dy, const float* __restrict__ coef,
    T* __restrict__ out, int64_t N, int64_t F, int64_t HW, int per_block, PackSink ps) {
  constexpr int E = Chunk<T>::kElems;
  constexpr int PD = Chunk<T>::kPerDword;
  constexpr int NC = BWD ? 3 : 2;
  constexpr int kUnroll = XS::kInFlight;
  static_assert(!(PACK && BWD), "the packed copy is made by the forward pass");
  const Place p = place_of<E>(F, HW);
  float sumsq = 0.0f;
  if (!BWD && !p.active) return;       // whole quantisation groups (32 lanes) leave together
  if (p.active) {                      // (backward: the lanes meet again for the wave's sum below)
  bind_input(xs, p);
  float k0[NC], k1[NC];
#pragma unroll
  for (int i = 0; i < NC; ++i) {
    k0[i] = coef[NC * p.channel + i];
    k1[i] = (SPLIT && p.head < E) ? coef[NC * (p.channel + 1) + i] : k0[i];
  }
  float ka[E], kb[E], kc[E];
#pragma unroll
  for (int i = 0; i < E; ++i) {
    const bool first = !SPLIT || i < p.head;
    ka[i] = first ? k0[0] : k1[0];
    kb[i] = first ? k0[1] : k1[1];
    kc[i] = BWD ? (first ? k0[NC - 1] : k1[NC - 1]) : 0.0f;
  }
  const int64_t n0 = (int64_t)blockIdx.y * per_block;
  const int64_t n1 = n0 + per_block < N ? n0 + per_block : N;

  auto apply = [&](const u32x4& ux, const u32x4& ud) -> u32x4 {
    const uint32_t w[4] = {ux.x, ux.y, ux.z, ux.w};
    const uint32_t d[4] = {ud.x, ud.y, ud.z, ud.w};
    uint32_t r[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float v[PD], g[PD], o[PD];
      Chunk<T>::widen(w[j], v);
      if (BWD) Chunk<T>::widen(d[j], g);
#pragma unroll
      for (int i = 0; i < PD; ++i) {
        const int e = j * PD + i;
        o[i] = BWD ? fmaf(g[i], ka[e], fmaf(v[i], kb[e], kc[e])) : fmaf(v[i], ka[e], kb[e]);
      }
      r[j] = Chunk<T>::narrow(o);
      if (BWD) Chunk<T>::dot(r[j], r[j], sumsq);
    }
    return u32x4{r[0], r[1], r[2], r[3]};
  };

  const T* pd = BWD ? dy + p.elem : nullptr;
  T* po = out + p.elem;
  if constexpr (PACK && sizeof(T) == 4) {
    // fp32: 64 samples at a time (the wave's 64 lanes own the group), packed two by two
    const int lane = threadIdx.x & 63;
    const int64_t grp = p.elem >> 8;
    ParamQueue<T> queue;
    auto params = [&](int64_t n, int jq) {
      ChunkParams q;
      queue.get(jq, q.mul, q.sub);
      q.b = ps.bits[n];
      q.dst = ps.packed + (int64_t)ps.prefix[n] * ps.G * 8 + grp * q.b * 8;
      q.octet = (uint64_t)((n * F + p.elem) >> 3);
      return q;
    };
    for (int64_t nb = n0; nb < n1; nb += 64) {
      const int64_t ne = nb + 64 < n1 ? nb + 64 : n1;
      {
        const int64_t nj = nb + lane;
        const bool live = nj < ne;
        queue.fill(ps, nj * ps.G + grp, live ? ps.bits[nj] : 1, live);
      }
      int64_t n = nb;
      for (; n + 2 <= ne; n += 2) {
        const typename XS::Raw rx0 = xs.fetch(n), rx1 = xs.fetch(n + 1);
        const u32x4 ux0 = xs.decode(rx0), ux1 = xs.decode(rx1);
        store_out(po + n * F, apply(ux0, ux0));
        store_out(po + (n + 1) * F, apply(ux1, ux1));
        pack_chunk_pair_f32(ps, ux0, params(n, (int)(n - nb)), ux1, params(n + 1, (int)(n + 1 - nb)), true);
      }
      if (n < ne) {
        const u32x4 ux = xs.decode(xs.fetch(n));
        store_out(po + n * F, apply(ux, ux));
        const ChunkParams q = params(n, (int)(n - nb));
        pack_chunk_pair_f32(ps, ux, q, ux, q, false);
      }
    }
  } else if constexpr (PACK) {
    // 32 samples at a time: lane j prepares the group's parameters for sample nb + j, then the
    // half-wave packs the samples two by two (the two chunks of a lane and those of lane ^ 1 are
    // neighbouring octets of the same two groups, and whole groups are present or absent together)
    const int lane32 = threadIdx.x & 31;
    const int64_t grp = p.elem >> 8;
    ParamQueue<T> queue;
    for (int64_t nb = n0; nb < n1; nb += 32) {
      const int64_t ne = nb + 32 < n1 ? nb + 32 : n1;
      {
        const int64_t nj = nb + lane32;
        const bool live = nj < ne;
        queue.fill(ps, nj * ps.G + grp, live ? ps.bits[nj] : 1, live);
      }
      int64_t n = nb;
      for (; n + 2 <= ne; n += 2) {
        typename XS::Raw rx[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) rx[u] = xs.fetch(n + u);
        uint32_t rw[2][Noise<T>::kWords];
        const uint64_t o = (uint64_t)((n * F + p.elem) >> 3);
        noise_pair<T>(ps, o, o + (uint64_t)(F >> 3), rw[0], rw[1], true);
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const u32x4 ux = xs.decode(rx[u]);
          store_out(po + (n + u) * F, apply(ux, ux));
          float mul, sub;
          queue.get((int)(n + u - nb), mul, sub);
          const int b = ps.bits[n + u];
          pack_chunk<T, true>(ux, rw[u], mul, sub, ps.packed + (int64_t)ps.prefix[n + u] * ps.G * 8 + grp * b * 8, b);
        }
      }
      for (; n < ne; ++n) {
        const typename XS::Raw rx = xs.fetch(n);
        const u32x4 ux = xs.decode(rx);
        store_out(po + n * F, apply(ux, ux));
        uint32_t rw[Noise<T>::kWords];
        Noise<T>::octet((uint64_t)((n * F + p.elem) >> 3), ps.seed, ps.offset, rw);
        float mul, sub;
        queue.get((int)(n - nb), mul, sub);
        const int b = ps.bits[n];
        pack_chunk<T, true>(ux, rw, mul, sub, ps.packed + (int64_t)ps.prefix[n] * ps.G * 8 + grp * b * 8, b);
      }
    }
  } else {
  int64_t n = n0;
  for (; n + kUnroll <= n1; n += kUnroll) {
    typename XS::Raw rx[kUnroll];
    u32x4 ud[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      rx[u] = xs.fetch(n + u);
      if (BWD) ud[u] = load_last(pd + (n + u) * F);
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const u32x4 ux = xs.decode(rx[u]);
      store_out(po + (n + u) * F, apply(ux, BWD ? ud[u] : ux));
    }
  }
  for (; n < n1; ++n) {
    const typename XS::Raw rx = xs.fetch(n);
    const u32x4 ux = xs.decode(rx);
    store_out(po + n * F, apply(ux, BWD ? load_last(pd + n * F) : ux));
  }
  }
  }
  if (BWD && ps.sumsq) leave_wave_sum(ps.sumsq, sumsq);
}

// ------------------------------------------------------------------ channels-last tensors
// [N, HW, C] in memory: a matrix of P = N * HW rows (pixels) by C columns (channels), the layout
// the convolution kernels of this GPU work in.  A block owns a tile of up to 256 columns and a run
// of consecutive rows; its threads form R rows of `tpr` chunks, thread (r, j) keeps the same E
// channels for the whole run, so the per-channel sums and coefficients again live in registers.
// For C <= 256 a block reads one contiguous stretch of memory; for wider tensors a row segment is
// 512 bytes.  With C % 256 == 0 or 256 % C == 0 a quantisation group (256 consecutive elements)
// is an aligned run of 256 / E threads, as in the default layout, so the group min/max and the
// decoding of a packed input carry over unchanged.
// A thread's row is `rb + r`: rb is the same for the whole block (a scalar: the loads then take a
// scalar base and a lane offset that never changes, so no per-load address arithmetic and no address
// registers), r is the thread's row inside one iteration.
template <typename T, bool NT = false> struct PlainRows {
  static constexpr bool kRows = true;
  static constexpr int kInFlight = 4;
  const T* p;
  int64_t C;
  uint32_t lane_bytes;   // (r * C + col) * sizeof(T) once bound
  struct Raw { u32x4 v; };
  ACTNN_DEV void bind(int64_t col, int r) { lane_bytes = (uint32_t)(((int64_t)r * C + col) * (int64_t)sizeof(T)); }
  ACTNN_DEV Raw fetch(int64_t rb) const {
    const char* q = reinterpret_cast<const char*>(p) + rb * C * (int64_t)sizeof(T) + lane_bytes;
    return Raw{NT ? load16_nt(q) : load16(q)};
  }
  ACTNN_DEV u32x4 decode(const Raw& r) const { return r.v; }
};
template <typename T> struct PackedRows {
  static constexpr bool kRows = true;
  static constexpr int kInFlight = 2;
  PackedInput<T> in;     // G = groups per sample
  int64_t C;
  uint32_t HW;
  FastDiv by_hw;
  using Raw = typename PackedInput<T>::Raw;
  // Per lane, fixed at bind(): its row inside one iteration and what it adds to the block's (scalar)
  // group position.  A thread stays inside one sample for many rows: the sample's width, its first
  // word and its first group are kept in registers and looked up again only when the row moves on to
  // the next sample, and everything else is 32-bit arithmetic on top of them (rows, groups and the
  // words of one sample stay below 2^31, which the launcher checks) - the fetch is a handful of
  // instructions where 64-bit index arithmetic per row took forty.
  uint32_t r, lane_group;
  uint32_t cur_row0, cur_group0;     // first row / first group of the sample of the last fetch
  int cur_b;
  const int32_t* cur_words;          // the sample's first word
  ACTNN_DEV void bind(int64_t column, int row_in_iteration) {
    r = (uint32_t)row_in_iteration;
    lane_group = (uint32_t)(((int64_t)row_in_iteration * C + column) >> 8);
    in.lane32 = threadIdx.x & (PackedInput<T>::kLanes - 1);
    in.active = true;
    cur_row0 = 0x80000000u;          // no row is inside: the first fetch looks up (rows < 2^31)
    cur_group0 = 0;
    cur_b = 1;
    cur_words = in.words;
  }
  ACTNN_DEV Raw fetch(int64_t rb) {
    const uint32_t row = (uint32_t)rb + r;
    if (row - cur_row0 >= HW) {                            // left the sample (or the first fetch)
      const uint32_t n = by_hw.div(row);
      cur_row0 = n * HW;
      cur_group0 = n * (uint32_t)in.G;
      cur_b = in.bits[n];
      cur_words = in.words + (int64_t)in.prefix[n] * in.G * 8;
    }
    // rb * C is a multiple of 256 (rb a multiple of R, and R * C of 256, wherever groups align)
    const int64_t block_group = (rb * C) >> 8;             // the same for the whole block
    const uint32_t group = (uint32_t)block_group + lane_group;
    const uint32_t at = __umul24(group - cur_group0, (uint32_t)(8 * cur_b)) + in.lane32;
    Raw raw{0u, 0u, 1.0f, 0.0f, cur_b};
    if ((int)in.lane32 < 8 * cur_b) raw.lo = (uint32_t)cur_words[at];
    if (PackedInput<T>::kLanes == 32 && (int)in.lane32 + 32 < 8 * cur_b) raw.hi = (uint32_t)cur_words[at + 32];
    raw.sc = Conv<T>::load(in.scale + block_group, lane_group);
    raw.m = Conv<T>::load(in.mn + block_group, lane_group);
    return raw;
  }
  ACTNN_DEV u32x4 decode(const Raw& r) const {
    // a wave holds a few consecutive rows, nearly always of one sample: then the width is one number
    // and the choice of the decoder a scalar branch, not a walk through eight masked ones
    const int b0 = __builtin_amdgcn_readfirstlane(r.b);
    if (__builtin_amdgcn_ballot_w64(r.b != b0) == 0) {
      Raw u = r;
      u.b = b0;
      return in.decode(u);
    }
    return in.decode(r);
  }
};

struct RowTile {
  int64_t col;           // first channel of the thread's chunk
  int r;                 // row of the thread inside one iteration
  bool active;
};
template <int E> ACTNN_DEV RowTile row_tile(int64_t C, int tpr, int R, int tile) {
  RowTile t;
  const int j = threadIdx.x % tpr;
  t.r = threadIdx.x / tpr;
  t.col = (int64_t)tile * 256 + (int64_t)j * E;
  t.active = t.r < R && t.col < C && j * E < 256;
  if (!t.active) t.col = 0;
  return t;
}

// Waves per SIMD the reduce pass is compiled for: the plain statistics pass fits 8 (64 registers),
// with the group min/max or the gradient 7, with the decoder of a packed input 5.
template <bool BWD, bool MINMAX, typename XS, bool MASKED = false> constexpr int cl_reduce_waves() {
  // (with the ReLU's mask rows 4: three measured 5 % slower, five spills and is 35 % slower)
  return MASKED ? 4 : XS::kInFlight == 2 ? 5 : (BWD || MINMAX) ? 7 : 8;
}
template <typename T, bool BWD, bool MINMAX, bool NT, typename XS, bool MASKED = false>
__global__ __launch_bounds__(kThreads, (cl_reduce_waves<BWD, MINMAX, XS, MASKED>())) void bn_cl_reduce_kernel(
    XS xs, const T* __restrict__ dy, float* __restrict__ part, T* __restrict__ mn, T* __restrict__ mx,
    int64_t P, int64_t C, int tpr, int R, int64_t ppb, int tiles, int nsplit, ReluRows relu = ReluRows{}) {
  constexpr int E = Chunk<T>::kElems;
  constexpr int PD = Chunk<T>::kPerDword;
  constexpr int U = XS::kInFlight;
  static_assert(!MASKED || (BWD && U == 2 && sizeof(T) == 2), "the ReLU mask goes with a 16-bit gradient, two loads in flight");
  __shared__ float s_part[kThreads * 2 * E];
  // Blocks are numbered so that consecutive block rows of a column tile run on one XCD.  A line of the
  // table of partial sums holds the values of 16 consecutive block rows; dealt round-robin, those rows
  // sat on different XCDs, each L2 sent its 4 bytes of the line to memory on its own, and the write
  // counter read eight times the table's size (26 MB on a pass that reads a 51 MB tensor).
  const int64_t block = xcd_block();
  if (block >= (int64_t)tiles * nsplit) return;
  const int tile = (int)(block % tiles), brow = (int)(block / tiles);
  const RowTile t = row_tile<E>(C, tpr, R, tile);
  xs.bind(t.col, t.r);
  const int64_t p0 = (int64_t)brow * ppb;
  const int64_t p1 = p0 + ppb < P ? p0 + ppb : P;
  // everything a lane adds to the block's (scalar) position: bytes into dy, groups into mn / mx
  const uint32_t lane_bytes = (uint32_t)(((int64_t)t.r * C + t.col) * (int64_t)sizeof(T));
  const uint32_t lane_group = (uint32_t)(((int64_t)t.r * C + t.col) >> 8);
  auto dy_at = [&](int64_t rb) -> u32x4 {
    const char* q = reinterpret_cast<const char*>(dy) + rb * C * (int64_t)sizeof(T) + lane_bytes;
    return NT ? load16_nt(q) : load16(q);
  };
  float s[E], q[E];
#pragma unroll
  for (int i = 0; i < E; ++i) { s[i] = 0.0f; q[i] = 0.0f; }

  auto accumulate = [&](const u32x4& ux, const u32x4& ud, int64_t rb) {
    const uint32_t w[4] = {ux.x, ux.y, ux.z, ux.w};
    const uint32_t d[4] = {ud.x, ud.y, ud.z, ud.w};
    float v[E], g[E];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      Chunk<T>::widen(w[k], v + k * PD);
      if (BWD) Chunk<T>::widen(d[k], g + k * PD);
    }
#pragma unroll
    for (int i = 0; i < E; ++i) {
      const float a = BWD ? g[i] : v[i];
      s[i] += a;
      q[i] = fmaf(v[i], a, q[i]);
    }
    if (MINMAX) {
      constexpr int LPG = 256 / E;
      float lo, hi;
      minmax_of<E>(v, lo, hi);
      lanes_minmax<LPG / 16>(lo, hi);
      if ((threadIdx.x & (LPG - 1)) == LPG - 1) {
        // rb * C is a multiple of 256 (rb a multiple of R, and R * C of 256, wherever groups align)
        T* lo_at = mn + ((rb * C) >> 8) + lane_group;
        T* hi_at = mx + ((rb * C) >> 8) + lane_group;
        Conv<T>::store(lo_at, 0, lo);
        Conv<T>::store(hi_at, 0, hi);
      }
    }
  };

  if constexpr (MASKED) {
    // (every step of a block is whole here - the launcher sees to it - and all lanes are active)
    auto two = [&](int64_t rb, uint32_t row0, uint32_t row1) __attribute__((always_inline)) {
      const typename XS::Raw rx0 = xs.fetch(rb), rx1 = xs.fetch(rb + R);
      const u32x4 ud0 = dy_at(rb), ud1 = dy_at(rb + R);
      accumulate(xs.decode(rx0), keep_chunk(ud0, row0), rb);
      accumulate(xs.decode(rx1), keep_chunk(ud1, row1), rb + R);
    };
    auto one = [&](int64_t rb, uint32_t row) __attribute__((always_inline)) {
      const typename XS::Raw rx = xs.fetch(rb);
      accumulate(xs.decode(rx), keep_chunk(dy_at(rb), row), rb);
    };
    int64_t rb = p0;
    uint32_t m[4];
    for (; rb + (int64_t)4 * R <= p1; rb += (int64_t)4 * R) {
      relu.load(rb, C, R, tile, m);
      two(rb, m[0], m[1]);
      two(rb + (int64_t)2 * R, m[2], m[3]);
    }
    if (rb < p1) {
      relu.load(rb, C, R, tile, m);
      one(rb, m[0]);
      if (rb + R < p1) one(rb + R, m[1]);
      if (rb + (int64_t)2 * R < p1) one(rb + (int64_t)2 * R, m[2]);
    }
  } else if (t.active) {
    int64_t rb = p0;
    // whole iterations: every row rb + u * R + r of the U loads lies below p1
    for (; rb + (int64_t)U * R <= p1; rb += (int64_t)U * R) {
      typename XS::Raw rx[U];
      u32x4 ud[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        rx[u] = xs.fetch(rb + (int64_t)u * R);
        if (BWD) ud[u] = dy_at(rb + (int64_t)u * R);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const u32x4 ux = xs.decode(rx[u]);
        accumulate(ux, BWD ? ud[u] : ux, rb + (int64_t)u * R);
      }
    }
    for (; rb < p1; rb += R) {
      if (rb + t.r < p1) {
        const typename XS::Raw rx = xs.fetch(rb);
        const u32x4 ux = xs.decode(rx);
        accumulate(ux, BWD ? dy_at(rb) : ux, rb);
      }
    }
  }
  // rows of the tile are folded in a fixed order; table: [channel][sum][block row]
#pragma unroll
  for (int i = 0; i < E; ++i) {
    s_part[threadIdx.x * 2 * E + i] = t.active ? s[i] : 0.0f;
    s_part[threadIdx.x * 2 * E + E + i] = t.active ? q[i] : 0.0f;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < tpr * 2 * E; i += kThreads) {
    const int j = i / (2 * E), k = i % (2 * E);
    const int64_t channel = (int64_t)tile * 256 + j * E + k % E;
    if (j * E < 256 && channel < C) {
      float v = 0.0f;
      for (int rr = 0; rr < R; ++rr) v += s_part[(rr * tpr + j) * 2 * E + k];
      part[(channel * 2 + k / E) * nsplit + brow] = v;
    }
  }
}

// RELU: 0 - none; 1 - the ReLU after the batch norm is applied by the pass (forward) / its mask to
// the incoming gradient (backward); 2 - forward only: relu(bn(x) + residual).
// (the passes that also apply a ReLU or its mask are held to 128 registers, four waves per SIMD: left
// alone the backward one takes 140 and runs 9 % slower)
template <typename T, bool BWD, bool PACK, typename XS, int RELU = 0>
__global__ __launch_bounds__(kThreads, (RELU ? 4 : 1)) void bn_cl_apply_kernel(
    XS xs, const T* __restrict__ dy, const float* __restrict__ coef, T* __restrict__ out,
    int64_t P, int64_t C, int tpr, int R, int64_t ppb, PackSink ps, FastDiv by_hw, ReluRows relu = ReluRows{}) {
  // (RELU with BWD: the gradient that comes in is masked by `relu` as it is read)
  static_assert(!(RELU && BWD) || (XS::kInFlight == 2 && sizeof(T) == 2), "the ReLU mask goes with a 16-bit gradient, two loads in flight");
  constexpr int E = Chunk<T>::kElems;
  constexpr int PD = Chunk<T>::kPerDword;
  constexpr int NC = BWD ? 3 : 2;
  constexpr int U = XS::kInFlight;
  static_assert(!(PACK && BWD), "the packed copy is made by the forward pass");
  static_assert(!RELU || BWD || (PACK && sizeof(T) == 2), "the ReLU is folded into the packing pass of 16-bit tensors");
  static_assert(RELU != 2 || !BWD, "the residual is added by the forward pass");
  // The sample that holds the row of the last pack: its width, its first word in the stream and its
  // first row / group.  A thread stays inside one sample for many rows, so these are looked up only
  // when a row leaves it, and a chunk's place in the stream is 32-bit arithmetic on top of them (rows,
  // groups and the words of one sample stay below 2^31, which the launcher checks).
  const uint32_t HW = by_hw.d;
  uint32_t cur_row0 = 0x80000000u, cur_group0 = 0;       // no row is inside: the first pack looks up
  int cur_b = 1;
  int32_t* cur_words = ps.packed;
  auto locate = [&](uint32_t row) {
    if (row - cur_row0 >= HW) {
      const uint32_t n = by_hw.div(row);
      cur_row0 = n * HW;
      cur_group0 = n * (uint32_t)ps.G;
      cur_b = ps.bits[n];
      cur_words = ps.packed + (int64_t)ps.prefix[n] * ps.G * 8;
    }
  };
  // first word of group `group` (counted over the tensor) of the located sample
  auto group_words = [&](uint32_t group) -> int32_t* { return cur_words + __umul24(group - cur_group0, (uint32_t)(8 * cur_b)); };
  const RowTile t = row_tile<E>(C, tpr, R, blockIdx.x);
  float sumsq = 0.0f;
  if (!BWD && !t.active) return;       // whole quantisation groups leave together
  if (t.active) {                      // (backward: the lanes meet again for the wave's sum below)
  xs.bind(t.col, t.r);
  float ka[E], kb[E], kc[E];
#pragma unroll
  for (int i = 0; i < E; ++i) {
    ka[i] = coef[NC * (t.col + i)];
    kb[i] = coef[NC * (t.col + i) + 1];
    kc[i] = BWD ? coef[NC * (t.col + i) + 2] : 0.0f;
  }
  const int64_t p0 = (int64_t)blockIdx.y * ppb;
  const int64_t p1 = p0 + ppb < P ? p0 + ppb : P;

  auto apply = [&](const u32x4& ux, const u32x4& ud) -> u32x4 {
    const uint32_t w[4] = {ux.x, ux.y, ux.z, ux.w};
    const uint32_t d[4] = {ud.x, ud.y, ud.z, ud.w};
    uint32_t r[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      float v[PD], g[PD], o[PD];
      Chunk<T>::widen(w[k], v);
      if (BWD) Chunk<T>::widen(d[k], g);
#pragma unroll
      for (int i = 0; i < PD; ++i) {
        const int e = k * PD + i;
        o[i] = BWD ? fmaf(g[i], ka[e], fmaf(v[i], kb[e], kc[e])) : fmaf(v[i], ka[e], kb[e]);
      }
      r[k] = Chunk<T>::narrow(o);
      if (BWD) Chunk<T>::dot(r[k], r[k], sumsq);
    }
    return u32x4{r[0], r[1], r[2], r[3]};
  };

  // row rb + t.r of dy / out: a scalar base (rb is the same for the whole block) plus the lane's bytes
  const uint32_t lane_bytes = (uint32_t)(((int64_t)t.r * C + t.col) * (int64_t)sizeof(T));
  auto dy_at = [&](int64_t rb) -> u32x4 {
    return load_last(reinterpret_cast<const char*>(dy) + rb * C * (int64_t)sizeof(T) + lane_bytes);
  };
  auto out_at = [&](int64_t rb) -> void* {
    return reinterpret_cast<char*>(out) + rb * C * (int64_t)sizeof(T) + lane_bytes;
  };
  // Position of the lane's chunk of row ru + t.r (ru the same for the whole block) in elements:
  // ru * C + lane_elems.  ru is a multiple of R and R * C of 256 wherever groups align, so the
  // octet and the group of the chunk are a scalar part plus a part that never changes.
  const uint32_t lane_elems = (uint32_t)((int64_t)t.r * C + t.col);
  if constexpr (PACK && sizeof(T) == 4) {
    // fp32: 64 steps at a time (the wave's 64 lanes own the group), rows packed two by two
    const int lane = threadIdx.x & 63;
    ParamQueue<T> queue;
    auto params = [&](int64_t ru, int jq) {
      locate((uint32_t)ru + (uint32_t)t.r);
      ChunkParams q;
      queue.get(jq, q.mul, q.sub);
      q.b = cur_b;
      q.dst = group_words((uint32_t)((ru * C) >> 8) + (lane_elems >> 8));
      q.octet = (uint64_t)((ru * C) >> 3) + (lane_elems >> 3);
      return q;
    };
    for (int64_t rb0 = p0; rb0 + t.r < p1; rb0 += (int64_t)64 * R) {
      const int64_t rb = rb0 + t.r;
      {
        const int64_t rj = rb + (int64_t)lane * R;
        const bool live = rj < p1;
        const uint32_t nj = live ? by_hw.div((uint32_t)rj) : 0;
        queue.fill(ps, (rj * C + t.col) >> 8, live ? ps.bits[nj] : 1, live);
      }
      int j = 0;
      for (; j + 2 <= 64 && rb + (int64_t)(j + 1) * R < p1; j += 2) {
        const int64_t ru0 = rb0 + (int64_t)j * R, ru1 = ru0 + R;
        const typename XS::Raw rx0 = xs.fetch(ru0), rx1 = xs.fetch(ru1);
        const u32x4 ux0 = xs.decode(rx0), ux1 = xs.decode(rx1);
        store_out(out_at(ru0), apply(ux0, ux0));
        store_out(out_at(ru1), apply(ux1, ux1));
        const ChunkParams qa = params(ru0, j);
        const ChunkParams qb = params(ru1, j + 1);
        pack_chunk_pair_f32(ps, ux0, qa, ux1, qb, true);
      }
      if (j < 64 && rb + (int64_t)j * R < p1) {
        const int64_t ru0 = rb0 + (int64_t)j * R;
        const u32x4 ux = xs.decode(xs.fetch(ru0));
        store_out(out_at(ru0), apply(ux, ux));
        const ChunkParams q = params(ru0, j);
        pack_chunk_pair_f32(ps, ux, q, ux, q, false);
      }
    }
  } else if constexpr (PACK) {
    // 32 steps (rows r0, r0 + R, ...) at a time: lane j prepares the parameters of the group the
    // half-wave meets in step j, then the rows are packed two by two so that lane pairs can share
    // their noise
    const int lane32 = threadIdx.x & 31;
    ParamQueue<T> queue;
    auto pack_one = [&](const u32x4& ux, const uint32_t (&rw)[Noise<T>::kWords], int64_t ru, int j) __attribute__((always_inline)) {
      locate((uint32_t)ru + (uint32_t)t.r);
      float mul, sub;
      queue.get(j, mul, sub);
      pack_chunk<T, false>(ux, rw, mul, sub, group_words((uint32_t)((ru * C) >> 8) + (lane_elems >> 8)), cur_b);
    };
    // RELU: the wave's 64 chunks of a step are 512 consecutive elements - one block of the mask - or,
    // in rows of a multiple of 512 channels, the same half of two blocks (mask_place), and a half-wave's
    // 32 chunks one group of 256 outputs (the launcher takes this path only when that holds and every
    // step of a block is whole).  emit() applies the rule to the normalised chunk,
    // stores it, leaves the group's min / max and the lane's 8 keep bits in `row`; four steps' rows
    // make the wave's 64 mask words (blocks 4 apart: a step of the block is 2048 elements).
    const uint32_t lane = threadIdx.x & 63u;
    auto emit = [&](int64_t ru, const u32x4& y, uint32_t& row, const u32x4& res) __attribute__((always_inline)) {
      if constexpr (RELU != 0) {
        uint32_t w[4] = {y.x, y.y, y.z, y.w};
        if constexpr (RELU == 2) {
          // bn(x), rounded to T as its store would round it, plus the residual, rounded as the tensor
          // addition rounds it
          const uint32_t a[4] = {res.x, res.y, res.z, res.w};
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            float u[2], v[2];
            Chunk<T>::widen(w[k], u);
            Chunk<T>::widen(a[k], v);
            u[0] += v[0];
            u[1] += v[1];
            w[k] = Chunk<T>::narrow(u);
          }
        }
        float z[8];
        row = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          uint32_t keep;
          w[k] = relu_word<T>(w[k], keep, z[2 * k], z[2 * k + 1]);
          row |= keep << (2 * k);
        }
        store_out(out_at(ru), u32x4{w[0], w[1], w[2], w[3]});
        float lo, hi;
        minmax_of<8>(z, lo, hi);
        lanes_minmax<2>(lo, hi);
        if ((lane & 31u) == 31u) {
          const uint32_t g = (uint32_t)((ru * C) >> 8) + (lane_elems >> 8);
          Conv<T>::store(static_cast<T*>(ps.relu_mn), g, lo);
          Conv<T>::store(static_cast<T*>(ps.relu_mx), g, hi);
        }
      } else {
        store_out(out_at(ru), y);
      }
    };
    auto leave_mask = [&](int64_t ru_first, const uint32_t (&rows)[4], int count) __attribute__((always_inline)) {
      const uint32_t word = rows_to_word(rows, lane);
      const int slot = 2 * (int)(lane & 1u) + (int)(lane >> 5);
      const MaskPlace at = mask_place(ru_first, C, R, blockIdx.x);
      if (slot < count) {
        if (!at.wide) {
          ps.relu_mask[at.first] = (int32_t)word;
        } else {
          uint16_t* half = reinterpret_cast<uint16_t*>(ps.relu_mask);
          half[at.first] = (uint16_t)word;
          half[at.second] = (uint16_t)(word >> 16);
        }
      }
    };
    auto res_at = [&](int64_t rb) __attribute__((always_inline)) -> u32x4 {
      if constexpr (RELU == 2)
        return load16_nt(reinterpret_cast<const char*>(ps.relu_add) + rb * C * (int64_t)sizeof(T) + lane_bytes);
      else
        return u32x4{0u, 0u, 0u, 0u};
    };
    auto pair = [&](int64_t rb0, int j, uint32_t& row0, uint32_t& row1) __attribute__((always_inline)) {
      const int64_t ru0 = rb0 + (int64_t)j * R, ru1 = ru0 + R;
      const typename XS::Raw rx0 = xs.fetch(ru0), rx1 = xs.fetch(ru1);
      const u32x4 res0 = res_at(ru0), res1 = res_at(ru1);
      uint32_t rw[2][Noise<T>::kWords];
      noise_pair<T>(ps, (uint64_t)((ru0 * C) >> 3) + (lane_elems >> 3), (uint64_t)((ru1 * C) >> 3) + (lane_elems >> 3),
                    rw[0], rw[1], (tpr & 1) == 0);      // lane ^ 1 is in the same row, hence in the same steps
      const u32x4 ux0 = xs.decode(rx0);
      emit(ru0, apply(ux0, ux0), row0, res0);
      pack_one(ux0, rw[0], ru0, j);
      const u32x4 ux1 = xs.decode(rx1);
      emit(ru1, apply(ux1, ux1), row1, res1);
      pack_one(ux1, rw[1], ru1, j + 1);
    };
    auto single = [&](int64_t rb0, int j, uint32_t& row) __attribute__((always_inline)) {
      const int64_t ru0 = rb0 + (int64_t)j * R;
      const u32x4 res = res_at(ru0);
      const u32x4 ux = xs.decode(xs.fetch(ru0));
      emit(ru0, apply(ux, ux), row, res);
      uint32_t rw[Noise<T>::kWords];
      Noise<T>::octet((uint64_t)((ru0 * C) >> 3) + (lane_elems >> 3), ps.seed, ps.offset, rw);
      pack_one(ux, rw, ru0, j);
    };
    for (int64_t rb0 = p0; rb0 + t.r < p1; rb0 += (int64_t)32 * R) {
      const int64_t rb = rb0 + t.r;
      {
        const int64_t rj = rb + (int64_t)lane32 * R;
        const bool live = rj < p1;
        const uint32_t nj = live ? by_hw.div((uint32_t)rj) : 0;
        queue.fill(ps, (rj * C + t.col) >> 8, live ? ps.bits[nj] : 1, live);
      }
      int j = 0;
      if constexpr (RELU != 0) {
        uint32_t rows[4] = {0u, 0u, 0u, 0u};
        for (; j + 4 <= 32 && rb + (int64_t)(j + 3) * R < p1; j += 4) {
          pair(rb0, j, rows[0], rows[1]);
          pair(rb0, j + 2, rows[2], rows[3]);
          leave_mask(rb0 + (int64_t)j * R, rows, 4);
        }
        // what is left of the block's rows: up to three steps
        const int64_t ru_first = rb0 + (int64_t)j * R;
        int left = 0;
        if (j < 32 && rb + (int64_t)j * R < p1) { single(rb0, j, rows[0]); ++j; ++left; }
        if (j < 32 && rb + (int64_t)j * R < p1) { single(rb0, j, rows[1]); ++j; ++left; }
        if (j < 32 && rb + (int64_t)j * R < p1) { single(rb0, j, rows[2]); ++j; ++left; }
        if (left) leave_mask(ru_first, rows, left);
      } else {
        for (; j + 2 <= 32 && rb + (int64_t)(j + 1) * R < p1; j += 2) {
          const int64_t ru0 = rb0 + (int64_t)j * R, ru1 = ru0 + R;
          const typename XS::Raw rx0 = xs.fetch(ru0), rx1 = xs.fetch(ru1);
          uint32_t rw[2][Noise<T>::kWords];
          noise_pair<T>(ps, (uint64_t)((ru0 * C) >> 3) + (lane_elems >> 3), (uint64_t)((ru1 * C) >> 3) + (lane_elems >> 3),
                        rw[0], rw[1], (tpr & 1) == 0);      // lane ^ 1 is in the same row, hence in the same steps
          const u32x4 ux0 = xs.decode(rx0);
          store_out(out_at(ru0), apply(ux0, ux0));
          pack_one(ux0, rw[0], ru0, j);
          const u32x4 ux1 = xs.decode(rx1);
          store_out(out_at(ru1), apply(ux1, ux1));
          pack_one(ux1, rw[1], ru1, j + 1);
        }
        for (; j < 32 && rb + (int64_t)j * R < p1; ++j) {
          const int64_t ru0 = rb0 + (int64_t)j * R;
          const u32x4 ux = xs.decode(xs.fetch(ru0));
          store_out(out_at(ru0), apply(ux, ux));
          uint32_t rw[Noise<T>::kWords];
          Noise<T>::octet((uint64_t)((ru0 * C) >> 3) + (lane_elems >> 3), ps.seed, ps.offset, rw);
          pack_one(ux, rw, ru0, j);
        }
      }
    }
  } else if constexpr (RELU && BWD) {
    auto two = [&](int64_t rb, uint32_t row0, uint32_t row1) __attribute__((always_inline)) {
      const typename XS::Raw rx0 = xs.fetch(rb), rx1 = xs.fetch(rb + R);
      const u32x4 ud0 = dy_at(rb), ud1 = dy_at(rb + R);
      store_out(out_at(rb), apply(xs.decode(rx0), keep_chunk(ud0, row0)));
      store_out(out_at(rb + R), apply(xs.decode(rx1), keep_chunk(ud1, row1)));
    };
    auto one = [&](int64_t rb, uint32_t row) __attribute__((always_inline)) {
      const typename XS::Raw rx = xs.fetch(rb);
      store_out(out_at(rb), apply(xs.decode(rx), keep_chunk(dy_at(rb), row)));
    };
    int64_t rb = p0;
    uint32_t m[4];
    for (; rb + (int64_t)4 * R <= p1; rb += (int64_t)4 * R) {
      relu.load(rb, C, R, (int)blockIdx.x, m);
      two(rb, m[0], m[1]);
      two(rb + (int64_t)2 * R, m[2], m[3]);
    }
    if (rb < p1) {
      relu.load(rb, C, R, (int)blockIdx.x, m);
      one(rb, m[0]);
      if (rb + R < p1) one(rb + R, m[1]);
      if (rb + (int64_t)2 * R < p1) one(rb + (int64_t)2 * R, m[2]);
    }
  } else {
  int64_t rb = p0;
  for (; rb + (int64_t)U * R <= p1; rb += (int64_t)U * R) {
    typename XS::Raw rx[U];
    u32x4 ud[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      rx[u] = xs.fetch(rb + (int64_t)u * R);
      if (BWD) ud[u] = dy_at(rb + (int64_t)u * R);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const u32x4 ux = xs.decode(rx[u]);
      store_out(out_at(rb + (int64_t)u * R), apply(ux, BWD ? ud[u] : ux));
    }
  }
  for (; rb < p1; rb += R) {
    if (rb + t.r < p1) {
      const typename XS::Raw rx = xs.fetch(rb);
      const u32x4 ux = xs.decode(rx);
      store_out(out_at(rb), apply(ux, BWD ? dy_at(rb) : ux));
    }
  }
  }
  }
  if (BWD && ps.sumsq) leave_wave_sum(ps.sumsq, sumsq);
}

// Launch geometry shared by the passes of one call.
struct Plan {
  int elems;           // elements per 16-byte chunk
  int64_t F, L, spans;
  int per_block, nsplit, slots;
  bool split;
  int64_t part_floats;
  // channels-last: P rows, column tiles of 256, tpr threads per row, R rows per iteration,
  // ppb rows per block, nsplit blocks along the rows (slots == 0 marks this table layout)
  bool channels_last;
  int64_t P, ppb, ppb_apply;   // rows per block in the reduce passes and in the apply passes
  int nsplit_apply;
  int tiles, tpr, R;
  bool groups_align;   // quantisation groups are aligned runs of threads
  bool big;            // the tensor does not fit the last-level cache: a pass finds nothing of it there
  bool any_shape;      // not a whole number of chunks per row / per pixel: the element-by-element kernels
  int64_t any_per_block;   // samples per block of their reduce pass
};
// The memory-side cache holds 256 MiB.  A tensor above that is gone from it by the time the next pass
// starts, so the passes that only read may use non-temporal loads (7.0 against 6.1 TB/s on a plain
// read); a smaller one is found there by the next pass, and non-temporal loads would lose that.
constexpr int64_t kLastLevelCacheBytes = (int64_t)256 << 20;
bool make_plan_cl(int64_t N, int64_t C, int64_t HW, int dtype, Plan& pl) {
  if (N <= 0 || C <= 0 || HW <= 0 || dtype < 0 || dtype > 2) return false;
  pl.channels_last = true;
  pl.elems = dtype == ACTNN_F32 ? 4 : 8;
  if (C % pl.elems != 0 || C > 0x7fffffffLL || HW > 0x7fffffffLL || N > ((int64_t)1 << 62) / (C * HW)) return false;
  pl.F = C * HW;
  pl.P = N * HW;
  pl.tiles = (int)((C + 255) / 256);
  pl.tpr = (int)((C < 256 ? C : 256) / pl.elems);
  pl.R = kThreads / pl.tpr;
  // About one round of blocks (7 or 8 of them fit a CU): what a block leaves in the table of partial
  // sums is still in the caches when the kernel ends and is written back then, at a fraction of the
  // streaming rate (measured on a plain read of 822 MB with such an epilogue: 4 MB of partial sums
  // cost 7 us, 8 MB 11 us, 16 MB 18 us), so fewer, longer blocks win: 2048 blocks measured 4 % faster
  // than 4096 over ResNet-50's shapes.  At least 64 rows per block.
  constexpr int64_t target = 2048, min_ppb = 64;
  const int64_t want = (target + pl.tiles - 1) / pl.tiles;
  int64_t ppb = (pl.P + want - 1) / want;
  if (ppb < min_ppb) ppb = min_ppb;
  if (ppb < (pl.P + 65534) / 65535) ppb = (pl.P + 65534) / 65535;
  ppb = (ppb + pl.R - 1) / pl.R * pl.R;
  pl.ppb = ppb;
  pl.nsplit = (int)((pl.P + ppb - 1) / ppb);
  // The apply passes have no block epilogue and no table: many short blocks even out the tail
  // (16384 and 32768 blocks measured alike, 8 % faster than the 4096 of the reduce passes; 8192 in between).
  constexpr int64_t apply_target = 16384;
  const int64_t want_a = (apply_target + pl.tiles - 1) / pl.tiles;
  int64_t ppa = (pl.P + want_a - 1) / want_a;
  if (ppa < 8 * pl.R) ppa = 8 * pl.R;
  if (ppa < (pl.P + 65534) / 65535) ppa = (pl.P + 65534) / 65535;
  ppa = (ppa + pl.R - 1) / pl.R * pl.R;
  pl.ppb_apply = ppa;
  pl.nsplit_apply = (int)((pl.P + ppa - 1) / ppa);
  pl.slots = 0;
  pl.split = false;
  pl.part_floats = C * 2 * pl.nsplit;
  pl.groups_align = pl.F % 256 == 0 && (C % 256 == 0 || 256 % C == 0);
  pl.big = N * pl.F * (dtype == ACTNN_F32 ? 4 : 2) > kLastLevelCacheBytes;
  pl.L = 0; pl.spans = 0; pl.per_block = 0;
  return true;
}
bool make_plan(int64_t N, int64_t C, int64_t HW, int dtype, Plan& pl) {
  if (N <= 0 || C <= 0 || HW <= 0 || dtype < 0 || dtype > 2) return false;
  pl.channels_last = false;
  pl.elems = dtype == ACTNN_F32 ? 4 : 8;
  if (HW < pl.elems || C > 0x7fffffffLL || C > ((int64_t)1 << 40) / HW) return false;
  pl.F = C * HW;
  if (pl.F % pl.elems != 0 || N > ((int64_t)1 << 62) / pl.F) return false;
  pl.L = (int64_t)kThreads * pl.elems;
  pl.spans = (pl.F + pl.L - 1) / pl.L;
  if (pl.spans > 0x7fffffffLL) return false;
  // Many more blocks than the 2048 the chip holds at once, so that the last round of blocks
  // does not leave most of it idle (2352 blocks measured 13 % slower than 15680), but at least 8
  // samples per block to pay for the block's final reduction.
  constexpr int64_t target = 32768, min_pb = 8;
  int64_t want = (target + pl.spans - 1) / pl.spans;
  if (want > 65535) want = 65535;
  int64_t per_block = (N + want - 1) / want;
  if (per_block < min_pb) per_block = min_pb;
  if (per_block > N) per_block = N;
  const int64_t nsplit = (N + per_block - 1) / per_block;
  if (nsplit > 65535 || per_block > 0x7fffffffLL) return false;
  pl.per_block = (int)per_block;
  pl.nsplit = (int)nsplit;
  int64_t slots = (pl.L - 1) / HW + 2;                    // channels one span can touch
  if (slots > C) slots = C;
  pl.slots = (int)slots;
  pl.split = HW % pl.elems != 0;
  pl.part_floats = pl.spans * nsplit * slots * 2;
  pl.groups_align = pl.F % 256 == 0;
  pl.big = N * pl.F * (dtype == ACTNN_F32 ? 4 : 2) > kLastLevelCacheBytes;
  return true;
}
// The plan of the element-by-element kernels: grid (C, nsplit) for the sums.
bool make_plan_any(int64_t N, int64_t C, int64_t HW, int dtype, bool channels_last, Plan& pl) {
  if (N <= 0 || C <= 0 || HW <= 0 || dtype < 0 || dtype > 2) return false;
  if (C > 0x7fffffffLL || HW > 0x7fffffffLL || C > ((int64_t)1 << 40) / HW || N > ((int64_t)1 << 62) / (C * HW)) return false;
  pl = Plan{};
  pl.any_shape = true;
  pl.channels_last = channels_last;
  pl.elems = dtype == ACTNN_F32 ? 4 : 8;
  pl.F = C * HW;
  pl.P = N * HW;
  // about 4096 blocks in all, each at least one sample
  int64_t want = (4096 + C - 1) / C;
  if (want > 65535) want = 65535;
  int64_t per_block = (N + want - 1) / want;
  if (per_block < 1) per_block = 1;
  pl.any_per_block = per_block;
  pl.nsplit = (int)((N + per_block - 1) / per_block);
  pl.slots = 0;                                  // the table layout of the channels-last passes
  pl.part_floats = C * 2 * pl.nsplit;
  pl.groups_align = false;
  pl.big = false;
  return true;
}
bool make_plan(int64_t N, int64_t C, int64_t HW, int dtype, int channels_last, Plan& pl) {
  if (N <= 0 || C <= 0 || HW <= 0 || dtype < 0 || dtype > 2) return false;
  const int elems = dtype == ACTNN_F32 ? 4 : 8;
  // [N, C] (one position per channel) is the channels-last layout with a single pixel per sample
  const bool cl = channels_last || HW == 1;
  pl.any_shape = false;
  pl.any_per_block = 0;
  if (cl ? C % elems != 0 : (HW < elems || (C * HW) % elems != 0)) return make_plan_any(N, C, HW, dtype, cl, pl);
  return cl ? make_plan_cl(N, C, HW, dtype, pl) : make_plan(N, C, HW, dtype, pl);
}
int64_t workspace_floats(const Plan& pl, int64_t C) { return pl.part_floats + 3 * C; }
// Shapes whose channels-last passes can make or apply a ReLU's mask (MaskPlace): every thread of a block
// active, whole steps only.
bool relu_mask_shape(const Plan& pl, int64_t C) {
  return pl.channels_last && !pl.any_shape && ((C <= 256 && 256 % C == 0) || C % 512 == 0) && pl.P % pl.R == 0 &&
         ((pl.P * C) >> 9) < ((int64_t)1 << 27);
}
int64_t apply_waves(const Plan& pl) {      // entries of the sum-of-squares table of the backward apply pass
  if (pl.any_shape) return 0;              // (the element-by-element kernels leave none)
  return (pl.channels_last ? (int64_t)pl.tiles * pl.nsplit_apply : pl.spans * pl.nsplit) * kWaves;
}

template <typename T, bool BWD, bool MINMAX, typename XS>
void launch_reduce(const Plan& pl, const XS& xs, const void* dy, float* part, void* mn, void* mx,
                   int64_t N, int64_t HW, hipStream_t s) {
  const dim3 grid((unsigned)pl.spans, (unsigned)pl.nsplit), blk(kThreads);
  const size_t lds = (size_t)kWaves * (pl.slots + 1) * 2 * sizeof(float);
  const T* pd = static_cast<const T*>(dy);
  T* lo = static_cast<T*>(mn);
  T* hi = static_cast<T*>(mx);
  if (pl.split)
    bn_reduce_kernel<T, true, BWD, MINMAX, XS><<<grid, blk, lds, s>>>(xs, pd, part, lo, hi, N, pl.F, HW, pl.per_block, pl.slots);
  else
    bn_reduce_kernel<T, false, BWD, MINMAX, XS><<<grid, blk, lds, s>>>(xs, pd, part, lo, hi, N, pl.F, HW, pl.per_block, pl.slots);
}

template <typename T, bool BWD, bool PACK, typename XS>
void launch_apply(const Plan& pl, const XS& xs, const void* dy, const float* coef, void* out,
                  int64_t N, int64_t HW, const PackSink& ps, hipStream_t s) {
  const dim3 grid((unsigned)pl.spans, (unsigned)pl.nsplit), blk(kThreads);
  const T* pd = static_cast<const T*>(dy);
  T* po = static_cast<T*>(out);
  if (pl.split)
    bn_apply_kernel<T, true, BWD, PACK, XS><<<grid, blk, 0, s>>>(xs, pd, coef, po, N, pl.F, HW, pl.per_block, ps);
  else
    bn_apply_kernel<T, false, BWD, PACK, XS><<<grid, blk, 0, s>>>(xs, pd, coef, po, N, pl.F, HW, pl.per_block, ps);
}

// Rows per block and block rows of a channels-last reduce pass whose kernel holds `waves` waves per
// SIMD: as many blocks as the chip holds at once (a block is one wave on each SIMD of its CU), so that
// the pass is one round of blocks that end together.  With the plan's 8 blocks per CU a kernel that
// holds 7 or 5 ran the rest as a second round on a chip that was mostly idle.  Never more block rows
// than the plan's, which sizes the table.
struct ClRows { int64_t ppb; int nsplit; };
ClRows cl_reduce_rows(const Plan& pl, int waves) {
  int64_t want = (int64_t)kCUs * waves / pl.tiles;
  if (want < 1) want = 1;
  int64_t ppb = (pl.P + want - 1) / want;
  if (ppb < pl.ppb) ppb = pl.ppb;
  ppb = (ppb + pl.R - 1) / pl.R * pl.R;
  return ClRows{ppb, (int)((pl.P + ppb - 1) / ppb)};
}
// -> the block rows of the table it leaves
template <typename T, bool BWD, bool MINMAX, bool NT, typename XS, bool MASKED = false>
int launch_cl_reduce(const Plan& pl, const XS& xs, const void* dy, float* part, void* mn, void* mx,
                     int64_t C, hipStream_t s, const ReluRows& relu = ReluRows{}) {
  const ClRows rows = cl_reduce_rows(pl, cl_reduce_waves<BWD, MINMAX, XS, MASKED>());
  const dim3 grid(xcd_grid((int64_t)pl.tiles * rows.nsplit)), blk(kThreads);
  bn_cl_reduce_kernel<T, BWD, MINMAX, NT, XS, MASKED><<<grid, blk, 0, s>>>(
      xs, static_cast<const T*>(dy), part, static_cast<T*>(mn), static_cast<T*>(mx), pl.P, C, pl.tpr, pl.R, rows.ppb,
      pl.tiles, rows.nsplit, relu);
  return rows.nsplit;
}
template <typename T, bool BWD, bool PACK, typename XS, int RELU = 0>
void launch_cl_apply(const Plan& pl, const XS& xs, const void* dy, const float* coef, void* out, int64_t C,
                     const PackSink& ps, hipStream_t s, const ReluRows& relu = ReluRows{}) {
  const dim3 grid((unsigned)pl.tiles, (unsigned)pl.nsplit_apply), blk(kThreads);
  bn_cl_apply_kernel<T, BWD, PACK, XS, RELU><<<grid, blk, 0, s>>>(
      xs, static_cast<const T*>(dy), coef, static_cast<T*>(out), pl.P, C, pl.tpr, pl.R, pl.ppb_apply, ps,
      FastDiv((uint32_t)(pl.F / C)), relu);
}

template <typename T>
int forward_stats_t(const Plan& pl, const void* x, const float* weight, const float* bias, float* running_mean,
                    float* running_var, float* save_mean, float* save_invstd, void* mn, void* mx, float* ws,
                    int64_t N, int64_t C, int64_t HW, double momentum, double eps, hipStream_t s) {
  float* part = ws;
  float* coef = ws + pl.part_floats;
  int nsplit = pl.nsplit;
  if (pl.any_shape) {
    const dim3 grid((unsigned)C, (unsigned)pl.nsplit), blk(kThreads);
    if (pl.channels_last)
      bn_any_reduce_kernel<T, false, true><<<grid, blk, 0, s>>>(static_cast<const T*>(x), nullptr, part, N, C, HW, pl.any_per_block);
    else
      bn_any_reduce_kernel<T, false, false><<<grid, blk, 0, s>>>(static_cast<const T*>(x), nullptr, part, N, C, HW, pl.any_per_block);
  } else if (pl.channels_last) {
    if (pl.big) {
      const PlainRows<T, true> xs{static_cast<const T*>(x), C};
      if (mn) nsplit = launch_cl_reduce<T, false, true, true>(pl, xs, nullptr, part, mn, mx, C, s);
      else nsplit = launch_cl_reduce<T, false, false, true>(pl, xs, nullptr, part, nullptr, nullptr, C, s);
    } else {
      const PlainRows<T> xs{static_cast<const T*>(x), C};
      if (mn) nsplit = launch_cl_reduce<T, false, true, false>(pl, xs, nullptr, part, mn, mx, C, s);
      else nsplit = launch_cl_reduce<T, false, false, false>(pl, xs, nullptr, part, nullptr, nullptr, C, s);
    }
  } else {
    const PlainInput<T> xs{static_cast<const T*>(x), pl.F};
    if (mn) launch_reduce<T, false, true>(pl, xs, nullptr, part, mn, mx, N, HW, s);
    else launch_reduce<T, false, false>(pl, xs, nullptr, part, nullptr, nullptr, N, HW, s);
  }
  bn_forward_finalize_kernel<<<dim3((unsigned)((C + kWaves - 1) / kWaves)), dim3(kThreads), 0, s>>>(
      part, weight, bias, running_mean, running_var, save_mean, save_invstd, coef, N, C, HW, pl.L, nsplit,
      pl.slots, momentum, eps);
  ACTNN_RETURN_LAUNCH_STATUS();
}

// y = a*x + b from the coefficients the statistics step left in the workspace; with a sink the
// same pass also writes the packed copy of x.
template <typename T>
int forward_apply_t(const Plan& pl, const void* x, void* y, const float* ws, const PackSink* sink, int64_t N,
                    int64_t C, int64_t HW, hipStream_t s) {
  const float* coef = ws + pl.part_floats;
  const PackSink none{};
  if (pl.any_shape) {
    const int64_t total = N * C * HW;
    int64_t blocks = (total + kThreads - 1) / kThreads;
    if (blocks > 65536) blocks = 65536;
    if (pl.channels_last)
      bn_any_apply_kernel<T, false, true><<<dim3((unsigned)blocks), dim3(kThreads), 0, s>>>(
          static_cast<const T*>(x), nullptr, coef, static_cast<T*>(y), total, C, HW);
    else
      bn_any_apply_kernel<T, false, false><<<dim3((unsigned)blocks), dim3(kThreads), 0, s>>>(
          static_cast<const T*>(x), nullptr, coef, static_cast<T*>(y), total, C, HW);
    ACTNN_RETURN_LAUNCH_STATUS();
  }
  if (pl.channels_last) {
    const PlainRows<T> xs{static_cast<const T*>(x), C};
    if constexpr (sizeof(T) == 2) {
      if (sink && sink->relu_mask) {
        if (sink->relu_add) launch_cl_apply<T, false, true, PlainRows<T>, 2>(pl, xs, nullptr, coef, y, C, *sink, s);
        else launch_cl_apply<T, false, true, PlainRows<T>, 1>(pl, xs, nullptr, coef, y, C, *sink, s);
        ACTNN_RETURN_LAUNCH_STATUS();
      }
    }
    if (sink) { launch_cl_apply<T, false, true>(pl, xs, nullptr, coef, y, C, *sink, s); ACTNN_RETURN_LAUNCH_STATUS(); }
    launch_cl_apply<T, false, false>(pl, xs, nullptr, coef, y, C, none, s);
  } else {
    const PlainInput<T> xs{static_cast<const T*>(x), pl.F};
    if (sink) { launch_apply<T, false, true>(pl, xs, nullptr, coef, y, N, HW, *sink, s); ACTNN_RETURN_LAUNCH_STATUS(); }
    launch_apply<T, false, false>(pl, xs, nullptr, coef, y, N, HW, none, s);
  }
  ACTNN_RETURN_LAUNCH_STATUS();
}

template <typename T, typename XS>
int backward_t(const Plan& pl, const XS& xs, const void* dy, const float* weight, const float* save_mean,
               const float* save_invstd, void* dx, float* dweight, float* dbias, float* ws, int64_t N,
               int64_t C, int64_t HW, float* sumsq, hipStream_t s, bool eval = false,
               const ReluRows* relu = nullptr) {
  float* part = ws;
  float* coef = ws + pl.part_floats;
  int nsplit = pl.nsplit;
  if constexpr (XS::kRows && XS::kInFlight == 2 && sizeof(T) == 2) {
    if (relu) {        // dy is the gradient of a ReLU's output: masked as it is read, in both passes
      if (pl.big) nsplit = launch_cl_reduce<T, true, false, true, XS, true>(pl, xs, dy, part, nullptr, nullptr, C, s, *relu);
      else nsplit = launch_cl_reduce<T, true, false, false, XS, true>(pl, xs, dy, part, nullptr, nullptr, C, s, *relu);
      bn_backward_finalize_kernel<<<dim3((unsigned)((C + kWaves - 1) / kWaves)), dim3(kThreads), 0, s>>>(
          part, weight, save_mean, save_invstd, dweight, dbias, coef, N, C, HW, pl.L, nsplit, pl.slots, eval);
      if (dx) {
        PackSink extra{};
        extra.sumsq = sumsq;
        launch_cl_apply<T, true, false, XS, 1>(pl, xs, dy, coef, dx, C, extra, s, *relu);
      }
      ACTNN_RETURN_LAUNCH_STATUS();
    }
  }
  if constexpr (XS::kRows) {
    if (pl.big) nsplit = launch_cl_reduce<T, true, false, true>(pl, xs, dy, part, nullptr, nullptr, C, s);
    else nsplit = launch_cl_reduce<T, true, false, false>(pl, xs, dy, part, nullptr, nullptr, C, s);
  }
  else launch_reduce<T, true, false>(pl, xs, dy, part, nullptr, nullptr, N, HW, s);
  bn_backward_finalize_kernel<<<dim3((unsigned)((C + kWaves - 1) / kWaves)), dim3(kThreads), 0, s>>>(
      part, weight, save_mean, save_invstd, dweight, dbias, coef, N, C, HW, pl.L, nsplit, pl.slots, eval);
  if (dx) {
    PackSink extra{};
    extra.sumsq = sumsq;
    if constexpr (XS::kRows) launch_cl_apply<T, true, false>(pl, xs, dy, coef, dx, C, extra, s);
    else launch_apply<T, true, false>(pl, xs, dy, coef, dx, N, HW, extra, s);
  }
  ACTNN_RETURN_LAUNCH_STATUS();
}

template <typename T, bool CL>
int backward_any(const Plan& pl, const void* x, const void* dy, const float* weight, const float* save_mean,
                 const float* save_invstd, void* dx, float* dweight, float* dbias, float* ws, int64_t N,
                 int64_t C, int64_t HW, hipStream_t s, bool eval) {
  float* part = ws;
  float* coef = ws + pl.part_floats;
  const T* px = static_cast<const T*>(x);
  const T* pd = static_cast<const T*>(dy);
  bn_any_reduce_kernel<T, true, CL><<<dim3((unsigned)C, (unsigned)pl.nsplit), dim3(kThreads), 0, s>>>(
      px, pd, part, N, C, HW, pl.any_per_block);
  bn_backward_finalize_kernel<<<dim3((unsigned)((C + kWaves - 1) / kWaves)), dim3(kThreads), 0, s>>>(
      part, weight, save_mean, save_invstd, dweight, dbias, coef, N, C, HW, pl.L, pl.nsplit, pl.slots, eval);
  if (dx) {
    const int64_t total = N * C * HW;
    int64_t blocks = (total + kThreads - 1) / kThreads;
    if (blocks > 65536) blocks = 65536;
    bn_any_apply_kernel<T, true, CL><<<dim3((unsigned)blocks), dim3(kThreads), 0, s>>>(
        px, pd, coef, static_cast<T*>(dx), total, C, HW);
  }
  ACTNN_RETURN_LAUNCH_STATUS();
}

template <typename T>
int backward_plain(const Plan& pl, const void* x, const void* dy, const float* weight, const float* save_mean,
                   const float* save_invstd, void* dx, float* dweight, float* dbias, float* ws, int64_t N,
                   int64_t C, int64_t HW, float* sumsq, hipStream_t s, bool eval = false) {
  if (pl.any_shape) {
    if (pl.channels_last) return backward_any<T, true>(pl, x, dy, weight, save_mean, save_invstd, dx, dweight, dbias, ws, N, C, HW, s, eval);
    return backward_any<T, false>(pl, x, dy, weight, save_mean, save_invstd, dx, dweight, dbias, ws, N, C, HW, s, eval);
  }
  if (pl.channels_last) {
    const PlainRows<T> xs{static_cast<const T*>(x), C};
    return backward_t<T>(pl, xs, dy, weight, save_mean, save_invstd, dx, dweight, dbias, ws, N, C, HW, sumsq, s, eval);
  }
  const PlainInput<T> xs{static_cast<const T*>(x), pl.F};
  return backward_t<T>(pl, xs, dy, weight, save_mean, save_invstd, dx, dweight, dbias, ws, N, C, HW, sumsq, s, eval);
}

template <typename T>
int backward_packed(const Plan& pl, const int32_t* packed, const int32_t* bits, const int32_t* prefix,
                    const void* scale, const void* mn, const void* dy, const float* weight,
                    const float* save_mean, const float* save_invstd, void* dx, float* dweight,
                    float* dbias, float* ws, int64_t N, int64_t C, int64_t HW, float* sumsq, hipStream_t s,
                    const int32_t* relu_mask = nullptr) {
  const PackedInput<T> in{packed, bits, prefix, static_cast<const T*>(scale), static_cast<const T*>(mn),
                          pl.F / 256, 0, 0u, false};
  if (pl.channels_last) {
    // (32-bit positions inside a sample and over the tensor's groups)
    if (C * HW >= ((int64_t)1 << 32) || N * (pl.F / 256) >= 0x7fffffffLL) return ACTNN_EINVAL;
    const PackedRows<T> xs{in, C, (uint32_t)HW, FastDiv((uint32_t)HW), 0u, 0u, 0u, 0u, 1, packed};
    const ReluRows relu{relu_mask, (N * pl.F) >> 9};
    return backward_t<T>(pl, xs, dy, weight, save_mean, save_invstd, dx, dweight, dbias, ws, N, C, HW, sumsq, s,
                         false, relu_mask ? &relu : nullptr);
  }
  if (relu_mask) return ACTNN_EINVAL;
  return backward_t<T>(pl, in, dy, weight, save_mean, save_invstd, dx, dweight, dbias, ws, N, C, HW, sumsq, s);
}

}  // namespace
}  // namespace actnn

extern "C" int64_t actnn_batch_norm_workspace_bytes(int64_t N, int64_t C, int64_t HW, int dtype,
                                                    int channels_last) {
  actnn::Plan pl;
  if (!actnn::make_plan(N, C, HW, dtype, channels_last, pl)) return -1;
  return actnn::workspace_floats(pl, C) * (int64_t)sizeof(float);
}

extern "C" int64_t actnn_batch_norm_backward_sumsq_entries(int64_t N, int64_t C, int64_t HW, int dtype,
                                                           int channels_last) {
  actnn::Plan pl;
  if (!actnn::make_plan(N, C, HW, dtype, channels_last, pl)) return -1;
  return actnn::apply_waves(pl);
}

extern "C" int actnn_batch_norm_groups_align(int64_t N, int64_t C, int64_t HW, int dtype, int channels_last) {
  actnn::Plan pl;
  if (!actnn::make_plan(N, C, HW, dtype, channels_last, pl)) return 0;
  return pl.groups_align && !pl.any_shape ? 1 : 0;
}

extern "C" int actnn_batch_norm_forward_stats(const void* x, const float* weight, const float* bias,
                                              float* running_mean, float* running_var, float* save_mean,
                                              float* save_invstd, void* mn, void* mx, void* workspace,
                                              int64_t workspace_bytes, int64_t N, int64_t C, int64_t HW,
                                              double momentum, double eps, int dtype, int channels_last,
                                              void* stream) {
  using namespace actnn;
  if (dtype < 0 || dtype > 2) return ACTNN_EDTYPE;
  Plan pl;
  if (!make_plan(N, C, HW, dtype, channels_last, pl)) return ACTNN_EINVAL;
  if (!x || !save_mean || !save_invstd || !workspace || (mn == nullptr) != (mx == nullptr)) return ACTNN_EINVAL;
  if (workspace_bytes < workspace_floats(pl, C) * (int64_t)sizeof(float)) return ACTNN_EINVAL;
  if (mn && !pl.groups_align) return ACTNN_EINVAL;
  if ((!pl.any_shape && !aligned16(x)) || !aligned16(workspace)) return ACTNN_EALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  float* ws = static_cast<float*>(workspace);
  switch (dtype) {
    case ACTNN_F32: return forward_stats_t<float>(pl, x, weight, bias, running_mean, running_var, save_mean, save_invstd, mn, mx, ws, N, C, HW, momentum, eps, s);
    case ACTNN_F16: return forward_stats_t<__half>(pl, x, weight, bias, running_mean, running_var, save_mean, save_invstd, mn, mx, ws, N, C, HW, momentum, eps, s);
    default: return forward_stats_t<bf16_t>(pl, x, weight, bias, running_mean, running_var, save_mean, save_invstd, mn, mx, ws, N, C, HW, momentum, eps, s);
  }
}

extern "C" int actnn_batch_norm_forward_apply(const void* x, void* y, const void* workspace,
                                              int64_t workspace_bytes, const int32_t* bits,
                                              const int32_t* prefix, const void* mn, const void* mx,
                                              void* scale, int32_t* packed, uint64_t seed, uint64_t offset,
                                              int64_t N, int64_t C, int64_t HW, int dtype, int channels_last,
                                              void* stream) {
  using namespace actnn;
  if (dtype < 0 || dtype > 2) return ACTNN_EDTYPE;
  Plan pl;
  if (!make_plan(N, C, HW, dtype, channels_last, pl)) return ACTNN_EINVAL;
  if (!x || !y || !workspace) return ACTNN_EINVAL;
  if (workspace_bytes < workspace_floats(pl, C) * (int64_t)sizeof(float)) return ACTNN_EINVAL;
  if ((!pl.any_shape && (!aligned16(x) || !aligned16(y))) || !aligned16(workspace)) return ACTNN_EALIGN;
  PackSink sink{bits, prefix, mn, mx, scale, packed, seed, offset, pl.F / 256};
  const bool pack = bits != nullptr;
  if (pack) {
    if (!pl.groups_align || !prefix || !mn || !mx || !scale || !packed) return ACTNN_EINVAL;
    // channels-last: 32-bit rows, groups and positions inside a sample
    if (channels_last && (pl.P > 0x7fffffffLL || C * HW >= ((int64_t)1 << 32) || N * (pl.F / 256) >= 0x7fffffffLL))
      return ACTNN_EINVAL;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const float* ws = static_cast<const float*>(workspace);
  switch (dtype) {
    case ACTNN_F32: return forward_apply_t<float>(pl, x, y, ws, pack ? &sink : nullptr, N, C, HW, s);
    case ACTNN_F16: return forward_apply_t<__half>(pl, x, y, ws, pack ? &sink : nullptr, N, C, HW, s);
    default: return forward_apply_t<bf16_t>(pl, x, y, ws, pack ? &sink : nullptr, N, C, HW, s);
  }
}

// _apply with the ReLU that follows the batch norm folded in: y = relu(bn(x)) as the ReLU operator
// would make it from the stored bn(x), with its 1-bit mask and the min / max of every group of 256
// outputs; packed copy of x as in _apply.
extern "C" int actnn_batch_norm_forward_apply_relu(const void* x, void* y, const void* workspace,
                                                   int64_t workspace_bytes, const int32_t* bits,
                                                   const int32_t* prefix, const void* mn, const void* mx,
                                                   void* scale, int32_t* packed, uint64_t seed, uint64_t offset,
                                                   int32_t* relu_mask, void* relu_mn, void* relu_mx,
                                                   const void* residual, int64_t N, int64_t C, int64_t HW,
                                                   int dtype, int channels_last, void* stream) {
  using namespace actnn;
  if (dtype != ACTNN_F16 && dtype != ACTNN_BF16) return ACTNN_EDTYPE;
  if (!aligned16(residual)) return ACTNN_EALIGN;
  Plan pl;
  if (!channels_last || !make_plan(N, C, HW, dtype, channels_last, pl) || pl.any_shape) return ACTNN_EINVAL;
  if (!x || !y || !workspace || !bits || !prefix || !mn || !mx || !scale || !packed || !relu_mask || !relu_mn || !relu_mx)
    return ACTNN_EINVAL;
  if (workspace_bytes < workspace_floats(pl, C) * (int64_t)sizeof(float)) return ACTNN_EINVAL;
  if (!aligned16(x) || !aligned16(y) || !aligned16(workspace)) return ACTNN_EALIGN;
  // a wave's step is one 512-element block of the mask or the same half of two, every step of every block is whole
  if (!pl.groups_align || !relu_mask_shape(pl, C)) return ACTNN_EINVAL;
  if (pl.P > 0x7fffffffLL || C * HW >= ((int64_t)1 << 32) || N * (pl.F / 256) >= 0x7fffffffLL) return ACTNN_EINVAL;
  PackSink sink{bits, prefix, mn, mx, scale, packed, seed, offset, pl.F / 256, nullptr, relu_mask, relu_mn, relu_mx,
                residual};
  hipStream_t s = static_cast<hipStream_t>(stream);
  const float* ws = static_cast<const float*>(workspace);
  if (dtype == ACTNN_F16) return forward_apply_t<__half>(pl, x, y, ws, &sink, N, C, HW, s);
  return forward_apply_t<bf16_t>(pl, x, y, ws, &sink, N, C, HW, s);
}

extern "C" int actnn_batch_norm_forward(const void* x, const float* weight, const float* bias,
                                        float* running_mean, float* running_var, void* y,
                                        float* save_mean, float* save_invstd, void* mn, void* mx,
                                        void* workspace, int64_t workspace_bytes, int64_t N, int64_t C,
                                        int64_t HW, double momentum, double eps, int dtype,
                                        int channels_last, void* stream) {
  if (!y) return ACTNN_EINVAL;
  const int rc = actnn_batch_norm_forward_stats(x, weight, bias, running_mean, running_var, save_mean,
                                                save_invstd, mn, mx, workspace, workspace_bytes, N, C, HW,
                                                momentum, eps, dtype, channels_last, stream);
  if (rc != ACTNN_OK) return rc;
  return actnn_batch_norm_forward_apply(x, y, workspace, workspace_bytes, nullptr, nullptr, nullptr, nullptr,
                                        nullptr, nullptr, 0, 0, N, C, HW, dtype, channels_last, stream);
}

// Evaluation mode: the running estimates take the place of the batch statistics.
extern "C" int actnn_batch_norm_forward_eval(const void* x, const float* weight, const float* bias,
                                             const float* running_mean, const float* running_var, void* y,
                                             float* save_mean, float* save_invstd, void* workspace,
                                             int64_t workspace_bytes, int64_t N, int64_t C, int64_t HW, double eps,
                                             int dtype, int channels_last, void* stream) {
  using namespace actnn;
  if (dtype < 0 || dtype > 2) return ACTNN_EDTYPE;
  Plan pl;
  if (!make_plan(N, C, HW, dtype, channels_last, pl)) return ACTNN_EINVAL;
  if (!x || !y || !running_mean || !running_var || !workspace) return ACTNN_EINVAL;
  if (workspace_bytes < workspace_floats(pl, C) * (int64_t)sizeof(float)) return ACTNN_EINVAL;
  if ((!pl.any_shape && (!aligned16(x) || !aligned16(y))) || !aligned16(workspace)) return ACTNN_EALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  float* ws = static_cast<float*>(workspace);
  bn_eval_coefficients_kernel<<<dim3((unsigned)((C + kThreads - 1) / kThreads)), dim3(kThreads), 0, s>>>(
      weight, bias, running_mean, running_var, save_mean, save_invstd, ws + pl.part_floats, C, eps);
  switch (dtype) {
    case ACTNN_F32: return forward_apply_t<float>(pl, x, y, ws, nullptr, N, C, HW, s);
    case ACTNN_F16: return forward_apply_t<__half>(pl, x, y, ws, nullptr, N, C, HW, s);
    default: return forward_apply_t<bf16_t>(pl, x, y, ws, nullptr, N, C, HW, s);
  }
}

extern "C" int actnn_batch_norm_backward_eval(const void* x, const void* dy, const float* weight,
                                              const float* mean, const float* invstd, void* dx,
                                              float* dweight, float* dbias, void* workspace,
                                              int64_t workspace_bytes, int64_t N, int64_t C, int64_t HW,
                                              int dtype, int channels_last, void* stream) {
  using namespace actnn;
  if (dtype < 0 || dtype > 2) return ACTNN_EDTYPE;
  Plan pl;
  if (!make_plan(N, C, HW, dtype, channels_last, pl)) return ACTNN_EINVAL;
  if (!x || !dy || !mean || !invstd || !workspace) return ACTNN_EINVAL;
  if (workspace_bytes < workspace_floats(pl, C) * (int64_t)sizeof(float)) return ACTNN_EINVAL;
  if ((!pl.any_shape && (!aligned16(x) || !aligned16(dy) || (dx && !aligned16(dx)))) || !aligned16(workspace)) return ACTNN_EALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  float* ws = static_cast<float*>(workspace);
  switch (dtype) {
    case ACTNN_F32: return backward_plain<float>(pl, x, dy, weight, mean, invstd, dx, dweight, dbias, ws, N, C, HW, nullptr, s, true);
    case ACTNN_F16: return backward_plain<__half>(pl, x, dy, weight, mean, invstd, dx, dweight, dbias, ws, N, C, HW, nullptr, s, true);
    default: return backward_plain<bf16_t>(pl, x, dy, weight, mean, invstd, dx, dweight, dbias, ws, N, C, HW, nullptr, s, true);
  }
}

// ------------------------------------------------------------------------------------------
// The forward pass for callers that cannot allocate and have no workspace to hand over: the partial
// sums and coefficients live in a fixed array in device memory instead of a workspace argument.
// Every GPU the library runs on holds its own copy of the array, at its own address, until the
// process ends.  In host code the array's name is only a stand-in for the symbol, not a device
// address: the address of this device's copy is asked for once per device, with that device
// current, and that pointer is what the kernels are given.
namespace actnn {
namespace {
constexpr int64_t kStaticScratchBytes = (int64_t)16 << 20;
static __device__ __align__(256) float scratch[kStaticScratchBytes / sizeof(float)];

constexpr int kMaxDevices = 64;
float* g_scratch_of_device[kMaxDevices];          // device address of `scratch`, per device
std::mutex g_scratch_mutex;

// -> ACTNN_OK and *out = the copy of the array on the current device, or an error code
int static_scratch(float** out, int* device) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return ACTNN_EINVAL;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_of_device[dev]) {
    float* ptr = nullptr;
    e = hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!ptr) return ACTNN_EINVAL;
    g_scratch_of_device[dev] = ptr;
  }
  *out = g_scratch_of_device[dev];
  *device = dev;
  return ACTNN_OK;
}
}  // namespace
}  // namespace actnn

// Also the set-up call: it looks up the array's address on the current device, so that a later
// actnn_batch_norm_forward_static on this device (under graph capture, say) finds it resolved.
extern "C" int64_t actnn_batch_norm_forward_static_limit(void) {
  float* ws = nullptr;
  int dev = -1;
  (void)actnn::static_scratch(&ws, &dev);          // an error here is reported by the forward call
  return actnn::kStaticScratchBytes;
}

extern "C" int actnn_batch_norm_forward_static(const void* x, const float* weight, const float* bias,
                                               float* running_mean, float* running_var, void* y,
                                               float* save_mean, float* save_invstd, void* mn, void* mx,
                                               int64_t N, int64_t C, int64_t HW, double momentum,
                                               double eps, int dtype, int channels_last, void* stream) {
  using namespace actnn;
  if (dtype < 0 || dtype > 2) return ACTNN_EDTYPE;
  Plan pl;
  if (!make_plan(N, C, HW, dtype, channels_last, pl)) return ACTNN_EINVAL;
  const int64_t need = workspace_floats(pl, C) * (int64_t)sizeof(float);
  if (need > kStaticScratchBytes) return ACTNN_ETOOBIG;
  float* ws = nullptr;
  int dev = -1;
  const int rc = static_scratch(&ws, &dev);
  if (rc != ACTNN_OK) return rc;
  // the array was looked up on the current device: a stream of another GPU would hand that GPU's
  // kernels an address of this one
  int stream_dev = -1;
  const hipError_t e = hipStreamGetDevice(static_cast<hipStream_t>(stream), &stream_dev);
  if (e != hipSuccess) return (int)e;
  if (stream_dev != dev) return ACTNN_EINVAL;
  // every partial sum and coefficient the second kernel reads is written by the first ones in this
  // call: nothing in the array has to start at zero
  return actnn_batch_norm_forward(x, weight, bias, running_mean, running_var, y, save_mean, save_invstd, mn,
                                  mx, ws, need, N, C, HW, momentum, eps, dtype, channels_last, stream);
}

extern "C" int actnn_batch_norm_backward(const void* x, const void* dy, const float* weight,
                                         const float* save_mean, const float* save_invstd, void* dx,
                                         float* dweight, float* dbias, void* workspace,
                                         int64_t workspace_bytes, float* sumsq, int64_t sumsq_entries,
                                         int64_t N, int64_t C, int64_t HW, int dtype, int channels_last,
                                         void* stream) {
  using namespace actnn;
  if (dtype < 0 || dtype > 2) return ACTNN_EDTYPE;
  Plan pl;
  if (!make_plan(N, C, HW, dtype, channels_last, pl)) return ACTNN_EINVAL;
  if (!x || !dy || !save_mean || !save_invstd || !workspace) return ACTNN_EINVAL;
  if (sumsq && (!dx || sumsq_entries < apply_waves(pl))) return ACTNN_EINVAL;
  if (workspace_bytes < workspace_floats(pl, C) * (int64_t)sizeof(float)) return ACTNN_EINVAL;
  if ((!pl.any_shape && (!aligned16(x) || !aligned16(dy) || (dx && !aligned16(dx)))) || !aligned16(workspace)) return ACTNN_EALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  float* ws = static_cast<float*>(workspace);
  switch (dtype) {
    case ACTNN_F32: return backward_plain<float>(pl, x, dy, weight, save_mean, save_invstd, dx, dweight, dbias, ws, N, C, HW, sumsq, s);
    case ACTNN_F16: return backward_plain<__half>(pl, x, dy, weight, save_mean, save_invstd, dx, dweight, dbias, ws, N, C, HW, sumsq, s);
    default: return backward_plain<bf16_t>(pl, x, dy, weight, save_mean, save_invstd, dx, dweight, dbias, ws, N, C, HW, sumsq, s);
  }
}

extern "C" int actnn_batch_norm_backward_packed(const int32_t* packed, const int32_t* bits,
                                                const int32_t* prefix, const void* scale, const void* mn,
                                                const void* dy, const float* weight,
                                                const float* save_mean, const float* save_invstd,
                                                void* dx, float* dweight, float* dbias, void* workspace,
                                                int64_t workspace_bytes, float* sumsq,
                                                int64_t sumsq_entries, int64_t N, int64_t C,
                                                int64_t HW, int dtype, int channels_last,
                                                void* stream) {
  using namespace actnn;
  if (dtype != ACTNN_F16 && dtype != ACTNN_BF16 && dtype != ACTNN_F32) return ACTNN_EDTYPE;
  Plan pl;
  if (!make_plan(N, C, HW, dtype, channels_last, pl) || !pl.groups_align) return ACTNN_EINVAL;
  if (channels_last && pl.P > 0x7fffffffLL) return ACTNN_EINVAL;
  if (sumsq && (!dx || sumsq_entries < apply_waves(pl))) return ACTNN_EINVAL;
  if (!packed || !bits || !prefix || !scale || !mn || !dy || !save_mean || !save_invstd || !workspace) return ACTNN_EINVAL;
  if (workspace_bytes < workspace_floats(pl, C) * (int64_t)sizeof(float)) return ACTNN_EINVAL;
  if (!aligned16(dy) || (dx && !aligned16(dx)) || !aligned16(workspace)) return ACTNN_EALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  float* ws = static_cast<float*>(workspace);
  if (dtype == ACTNN_F16)
    return backward_packed<__half>(pl, packed, bits, prefix, scale, mn, dy, weight, save_mean, save_invstd, dx, dweight, dbias, ws, N, C, HW, sumsq, s);
  if (dtype == ACTNN_F32)
    return backward_packed<float>(pl, packed, bits, prefix, scale, mn, dy, weight, save_mean, save_invstd, dx, dweight, dbias, ws, N, C, HW, sumsq, s);
  return backward_packed<bf16_t>(pl, packed, bits, prefix, scale, mn, dy, weight, save_mean, save_invstd, dx, dweight, dbias, ws, N, C, HW, sumsq, s);
}

// The same for a batch norm whose output went through a ReLU: `grad_out` is the gradient of the
// ReLU's output and `relu_mask` the ReLU's mask; both passes zero what actnn_relu_backward would
// have zeroed as they read, so the masked gradient is never written.  Shapes as
// actnn_batch_norm_forward_apply_relu takes them.
extern "C" int actnn_batch_norm_backward_packed_relu(const int32_t* packed, const int32_t* bits,
                                                     const int32_t* prefix, const void* scale, const void* mn,
                                                     const void* grad_out, const int32_t* relu_mask,
                                                     const float* weight, const float* save_mean,
                                                     const float* save_invstd, void* dx, float* dweight,
                                                     float* dbias, void* workspace, int64_t workspace_bytes,
                                                     float* sumsq, int64_t sumsq_entries, int64_t N, int64_t C,
                                                     int64_t HW, int dtype, int channels_last, void* stream) {
  using namespace actnn;
  if (dtype != ACTNN_F16 && dtype != ACTNN_BF16) return ACTNN_EDTYPE;
  Plan pl;
  if (!channels_last || !make_plan(N, C, HW, dtype, channels_last, pl) || pl.any_shape || !pl.groups_align) return ACTNN_EINVAL;
  if (!relu_mask_shape(pl, C) || pl.P > 0x7fffffffLL) return ACTNN_EINVAL;
  if (sumsq && (!dx || sumsq_entries < apply_waves(pl))) return ACTNN_EINVAL;
  if (!packed || !bits || !prefix || !scale || !mn || !grad_out || !relu_mask || !save_mean || !save_invstd || !workspace)
    return ACTNN_EINVAL;
  if (workspace_bytes < workspace_floats(pl, C) * (int64_t)sizeof(float)) return ACTNN_EINVAL;
  if (!aligned16(grad_out) || (dx && !aligned16(dx)) || !aligned16(workspace)) return ACTNN_EALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  float* ws = static_cast<float*>(workspace);
  if (dtype == ACTNN_F16)
    return backward_packed<__half>(pl, packed, bits, prefix, scale, mn, grad_out, weight, save_mean, save_invstd, dx, dweight, dbias, ws, N, C, HW, sumsq, s, relu_mask);
  return backward_packed<bf16_t>(pl, packed, bits, prefix, scale, mn, grad_out, weight, save_mean, save_invstd, dx, dweight, dbias, ws, N, C, HW, sumsq, s, relu_mask);
}
