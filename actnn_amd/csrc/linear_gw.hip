// Fused QLinear weight gradient (replaces dequantize_activation + grad_output.t().mm(input) in
// linear.backward, actnn/actnn/ops.py:407-421):
//
//     grad_w[O, I] = grad_out[M, O]^T @ dequant(x)[M, I]
//
// x stays in the stream the pack kernels wrote - the fixed-width stream (byte
// ((m / w) * I/256 + g) * 256 + d holds the w = 8/bits rows m of feature g*256 + d) or the
// mixed-width stream (per-sample widths, 32-lane ballot words) - with scale/min[M, I/256].  The
// full precision input is never written to memory: every k-step the tile is unpacked, dequantised
// and narrowed to the 16-bit format of grad_out straight into the LDS tile that feeds
// v_mfma_f32_32x32x16_bf16 / _f16, fp32 accumulation.
//
// Tiling: the reduction runs over the samples m (K of the GEMM).  A 256-thread block (one per CU)
// owns a 256 (O) x 256 (I) output tile - one whole quantisation group, so a block needs one
// scale/min per sample - as 4 waves of 128 (O) x 128 (I), one per SIMD, 256 accumulator registers
// each: a fragment read from LDS feeds four MFMAs (with 8 waves of 64 x 128 it feeds two or four:
// a third more LDS traffic).  Per k-step of 64 samples, LDS tiles double-buffered, one barrier a step:
//   * Both operand tiles lie in LDS the way they lie in memory: [sample][column], 512 bytes a row.
//     MFMA fragments want 8 consecutive samples of one column per lane; the transposing LDS read
//     (ds_read_b64_tr_b16: a 16-lane block that points at four rows of four 8-byte units gets back,
//     lane by lane, four consecutive samples of 16 consecutive columns) delivers exactly that, two
//     reads per fragment and no register transposes.  The 16-byte chunks of a row are stored at
//     chunk ^ ((sample & 7) << 2): the four rows that 32 lanes of such a read touch (64 bytes each)
//     then fall into the four quarters of the 64 banks, and the two reads of a fragment into
//     different halves of the row (measured: 1.4 times the rate of a swizzle that only separates
//     the rows within 16 lanes, 2.7 times no swizzle; 16-byte reads reach 1.3 times more still,
//     but need sample-contiguous tiles, i.e. register transposes of grad_out).
//   * grad_out tiles go from global memory straight into LDS (global_load_lds, 16 bytes per lane,
//     the swizzle applied to the source address): no registers, no VALU work.
//   * the 2-bit fixed-width stream: a thread takes one 32-bit load = 4 features x 4 samples.  The
//     four possible values of a sample, code / scale + min exactly as unpack_single rounds them,
//     are a table of eight bytes per sample (computed once per wave and step); v_perm_b32 with the
//     2-bit codes as byte selectors picks the low and the high bytes of four values at a time: 1.5
//     VALU instructions per value instead of extract + convert + multiply-add + narrow.
//   * any other stream (mixed widths; fixed 1, 4, 8 bits) takes a general loader: a lane unpacks
//     8 consecutive features of one sample (bit transpose as in unpack_mixed, or byte fields),
//     dequantises them with the unpack kernels' arithmetic and writes 16 bytes of the row.
//   The roles of the operands are chosen so that an accumulator register quad holds four
//   consecutive columns of grad_w: the epilogue stores 16 bytes (fp32) per lane and register quad.
// All work of a step other than the MFMAs is cut into pieces that sit between the MFMAs (see the
// schedule in the kernel).  Loads of packed data and scale/min run one step ahead of the staging
// code (widths and stream offsets of the mixed stream two steps ahead).
//
// Shapes with few output tiles and many samples (fewer than half the CUs busy) split the sum over the
// samples across blocks: every block writes its fp32 tile into a workspace and a second kernel adds
// the tiles in a fixed order (bit-reproducible, no atomics).
//
// What bounds it on MI355X: the matrix pipes themselves.  A kernel that issues the same 8.4 M
// v_mfma_f32_32x32x16 from registers and nothing else (actnn_matrix_pipe_probe) takes 0.167 ms with
// normally distributed operands against 0.127 ms with zeros: in both cases the pipes are busy 79 % of
// the cycles, but the part lowers its clock from 2.49 to 2.01 GHz when the operands switch many bits.
// 1650 TFLOP/s (66 % of the published 2.5 PFLOP/s) is therefore the ceiling of a 16-bit GEMM on
// N(0,1) data; this kernel reaches 0.25 ms = 1090 TFLOP/s on [8192, 4096]^T x [8192, 4096] with the
// 2-bit stream, level with rocBLAS on the dequantised copy (0.24 ms) and ahead of unpack + rocBLAS.
// The general loader decodes every element with shifts and a multiply-add (six times the vector
// instructions of the table loader) and loses to unpack + rocBLAS by 3-4x: the layers route only the
// 2-bit fixed-width stream here by default.
#include <type_traits>

#include "quant_math.h"

namespace actnn {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short i16x4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;
constexpr int NE = 4;               // 32-column fragments of the activation tile per wave (128 columns)
constexpr int NA = 4;               // 32-row fragments of the grad_out tile per wave (128 rows)
constexpr int kGroup = NE * NA;     // MFMAs per k-block and wave
constexpr int kSlots = 4 * kGroup;  // MFMAs per step and wave
constexpr int kSamplesPerWave = 64 / kWaves;
constexpr int BM = 256;             // output rows (O) per block
constexpr int BN = 256;             // output columns (I) per block: one quantisation group
constexpr int BK = 64;              // samples per k-step
constexpr int kRowBytes = 512;      // one sample of either tile: 256 16-bit values
constexpr int kTileBytes = BK * kRowBytes;
constexpr int kTabWave = kSamplesPerWave * 8;       // table bytes per wave and buffer: 8 per sample
constexpr int kTabBytes = kWaves * 2 * kTabWave;

template <int N> struct Slot { static constexpr int value = N; };
template <int N, typename F> ACTNN_DEV void for_each_slot(F&& f) {
  if constexpr (N > 0) {
    for_each_slot<N - 1>(f);
    f(Slot<N - 1>{});
  }
}

// byte offset of 16-byte chunk `ch` of row `k` inside a tile (the swizzle described above)
ACTNN_DEV int chunk_offset(int k, int ch) { return k * kRowBytes + ((ch ^ ((k & 7) << 2)) << 4); }

template <typename TG> struct Mma;
template <> struct Mma<bf16_t> {
  static ACTNN_DEV uint32_t pack2(float lo, float hi) { return pack_bf16x2(lo, hi); }
  static ACTNN_DEV uint32_t bits16(float v) { return float_to_bf16_bits(v); }
  static ACTNN_DEV f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};
template <> struct Mma<__half> {
  static ACTNN_DEV uint32_t pack2(float lo, float hi) {
    return float_to_half_bits(lo) | (float_to_half_bits(hi) << 16);
  }
  static ACTNN_DEV uint32_t bits16(float v) { return float_to_half_bits(v); }
  static ACTNN_DEV f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};

template <typename TO> ACTNN_DEV void store_out4(TO* p, float a, float b, float c, float d);
template <> ACTNN_DEV void store_out4<float>(float* p, float a, float b, float c, float d) {
  store16(p, (u32x4){as_uint(a), as_uint(b), as_uint(c), as_uint(d)});
}
template <> ACTNN_DEV void store_out4<__half>(__half* p, float a, float b, float c, float d) {
  *reinterpret_cast<u32x2*>(p) = (u32x2){float_to_half_bits(a) | (float_to_half_bits(b) << 16),
                                         float_to_half_bits(c) | (float_to_half_bits(d) << 16)};
}
template <> ACTNN_DEV void store_out4<bf16_t>(bf16_t* p, float a, float b, float c, float d) {
  *reinterpret_cast<u32x2*>(p) = (u32x2){pack_bf16x2(a, b), pack_bf16x2(c, d)};
}

// A scale / min value exactly as loaded: nothing may consume a load where it is issued (the wave would
// wait out the memory latency there), so prefetched values stay raw until the staging code runs.
template <typename T> struct RawScalar;
template <> struct RawScalar<float> {
  static ACTNN_DEV uint32_t load(const float* p, int64_t i) { return as_uint(p[i]); }
  static ACTNN_DEV float widen(uint32_t v) { return as_float(v); }
};
template <> struct RawScalar<__half> {
  static ACTNN_DEV uint32_t load(const __half* p, int64_t i) { return reinterpret_cast<const uint16_t*>(p)[i]; }
  static ACTNN_DEV float widen(uint32_t v) { return half_bits_to_float(v); }
};
template <> struct RawScalar<bf16_t> {
  static ACTNN_DEV uint32_t load(const bf16_t* p, int64_t i) { return p[i].bits; }
  static ACTNN_DEV float widen(uint32_t v) { return bf16_bits_to_float(v); }
};

// four consecutive samples of this lane's column (see the file comment for the lane pattern)
ACTNN_DEV u32x2 read_transposed(uint32_t lds_at) {
  const i16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (__attribute__((address_space(3))) i16x4*)(uintptr_t)lds_at);
  return __builtin_bit_cast(u32x2, v);
}

// What describes the packed input.  bits == nullptr: the fixed-width stream at `fixed_bits`.
struct Stream {
  const uint8_t* packed;
  const int32_t* bits;
  const int32_t* prefix;
  int fixed_bits;
};

// ------------------------------------------------------------------------------------------
// LDS is addressed by 32-bit numbers here: everything a lane contributes to an address is computed
// once, before the main loop, and what changes from step to step - the buffer, the k-block, the row
// of a staging store - is a compile-time constant that travels in the instruction's offset field
// (16 bits: the tiles are arranged so that every such constant stays below 64 KiB).  The main loop
// then spends no instructions on LDS addresses.
// ------------------------------------------------------------------------------------------
typedef __attribute__((address_space(3))) uint8_t* lds_ptr_t;
ACTNN_DEV uint32_t lds_address(const void* p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const uint8_t*)p;
}
template <typename V> ACTNN_DEV void lds_store(uint32_t address, V v) {
  *reinterpret_cast<__attribute__((address_space(3))) V*>((lds_ptr_t)(uintptr_t)address) = v;
}
template <typename V> ACTNN_DEV V lds_load(uint32_t address) {
  return *reinterpret_cast<const __attribute__((address_space(3))) V*>((lds_ptr_t)(uintptr_t)address);
}

// ------------------------------------------------------------------------------------------
// Loader of the 2-bit fixed-width stream (table + byte permutes)
// ------------------------------------------------------------------------------------------
template <typename TG, typename TS> struct TableLoader {
  static constexpr int Q = kSamplesPerWave / 4;      // sample quads per wave and step
  // Where the main loop places this loader's pieces (MFMA slot numbers of a step): in the slots that
  // read no fragments (the second half of each group of 16), so that no slot carries much more than
  // the half dozen instructions that fit beside one MFMA - table, read-back, then the 4 * Q staging
  // pieces, then the loads of the step after.
  static constexpr int kTableSlot = NE + NA, kReadbackSlot = NE + NA + 2, kPrefetchSlot = 2 * kGroup + NE + NA + 3;
  static_assert(NE + NA == 8 && kGroup == 16 && Q == 4, "the slot plan below is written for this tiling");
  // staging piece of a slot (-1: none): slots 11..15 -> 0..4, 24..31 -> 5..12, 40..42 -> 13..15
  static constexpr int stage_piece(int slot) {
    return slot >= 11 && slot <= 15 ? slot - 11 : slot >= 24 && slot <= 31 ? slot - 24 + 5
         : slot >= 40 && slot <= 42 ? slot - 40 + 13 : -1;
  }
  uint32_t rb[Q];          // this lane's 32-bit loads of the wave's sample quads
  uint32_t rsc, rmn;       // scale / min (raw) of sample lane / 4 of the wave's sixteen
  u32x2 tt[4 * Q];         // the wave's table entries, read back from LDS
  const uint8_t* pb0;      // this lane's bytes of quad 0
  const TS* psc0;          // scale / min of sample 0 in the block's group
  const TS* pmn0;
  int next;                // first sample of the step the next prefetch loads
  int M, G, quad_rows;     // quad_rows: bytes from one sample quad to the next in the stream
  // LDS addresses (buffer 0): this lane's table bytes, the wave's table, this lane's 8 bytes of
  // the wave's first sample row in the activation tile
  uint32_t tab_write, tab_read, stage;

  ACTNN_DEV void init(const Stream& st, const TS* scale, const TS* mn, int M_, int G_, int g, uint32_t tile_x0,
                      uint32_t tab0) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    M = M_;
    G = G_;
    next = 0;
    quad_rows = G * 256;
    pb0 = st.packed + (int64_t)g * 256 + lane * 4;
    psc0 = scale + g;
    pmn0 = mn + g;
    tab_read = tab0 + wave * 2 * kTabWave;
    tab_write = tab_read + (lane >> 2) * 8 + (lane & 3);
    stage = tile_x0 + wave * kSamplesPerWave * kRowBytes + ((lane >> 1) << 4) + (lane & 1) * 8;
  }
  // (no branches: out-of-range quads and samples read the last valid one and are ignored later -
  // the table gives samples past M the value 0 for every code - so that the loop body stays one
  // basic block and the compiler's wait counts for LDS stay exact)
  ACTNN_DEV void prefetch() {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int first = next + wave * kSamplesPerWave;
    const int last_quad = (M - 1) >> 2;
#pragma unroll
    for (int qq = 0; qq < Q; ++qq) {
      int quad = (first >> 2) + qq;
      quad = quad < last_quad ? quad : last_quad;
      rb[qq] = *reinterpret_cast<const uint32_t*>(pb0 + (int64_t)quad * quad_rows);
    }
    int smp = first + (lane >> 2);
    smp = smp < M - 1 ? smp : M - 1;
    rsc = RawScalar<TS>::load(psc0, (int64_t)smp * G);
    rmn = RawScalar<TS>::load(pmn0, (int64_t)smp * G);
    next += BK;
  }
  // The staging work of a step, cut into pieces that the main loop places between its MFMAs.
  // NB: the buffer that is being filled; kfirst: first sample of that tile.
  template <int SLOT, int NB> ACTNN_DEV void piece(int kfirst) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if constexpr (SLOT == kTableSlot) {
      // value of code (lane & 3) for sample lane / 4, rounded exactly as unpack_single rounds it
      const int smp = lane >> 2;
      const bool valid = kfirst + wave * kSamplesPerWave + smp < M;
      const Dequant<TS> dq(RawScalar<TS>::widen(rsc), RawScalar<TS>::widen(rmn));
      const uint32_t v = valid ? Mma<TG>::bits16(dq((uint32_t)(lane & 3))) : 0u;
      // low bytes of the sample's four values, then their high bytes
      lds_store<uint8_t>(tab_write + NB * kTabWave, (uint8_t)v);
      lds_store<uint8_t>(tab_write + NB * kTabWave + 4, (uint8_t)(v >> 8));
    } else if constexpr (SLOT == kReadbackSlot) {
      // same wave writes and reads: LDS operations of a wave complete in order
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
      for (int i = 0; i < 2 * Q; ++i) {
        const u32x4 two = lds_load<u32x4>(tab_read + NB * kTabWave + i * 16);
        tt[2 * i] = (u32x2){two.x, two.y};
        tt[2 * i + 1] = (u32x2){two.z, two.w};
      }
    } else if constexpr (stage_piece(SLOT) >= 0) {
      constexpr int qq = stage_piece(SLOT) / 4, j = stage_piece(SLOT) % 4;
      const uint32_t sel = (rb[qq] >> (2 * j)) & 0x03030303u;       // codes of 4 features as byte selectors
      const uint32_t lo = __builtin_amdgcn_perm(0u, tt[qq * 4 + j].x, sel);
      const uint32_t hi = __builtin_amdgcn_perm(0u, tt[qq * 4 + j].y, sel);
      const u32x2 out = {__builtin_amdgcn_perm(hi, lo, 0x05010400u), __builtin_amdgcn_perm(hi, lo, 0x07030602u)};
      // row k = 16 * wave + kk of the tile: chunk ch of it lies at ch ^ ((k & 7) << 2), i.e. the
      // lane's address with bits 6..8 flipped by kk & 7
      constexpr int kk = qq * 4 + j;
      lds_store<u32x2>((stage ^ ((kk & 7) << 6)) + NB * kTileBytes + kk * kRowBytes, out);
    } else if constexpr (SLOT == kPrefetchSlot) {
      prefetch();
    }
  }
};

// ------------------------------------------------------------------------------------------
// General loader: any fixed width, and the mixed-width stream.  A half-wave takes eight samples of
// a step; lane j unpacks features 8j .. 8j+7 of each.
// ------------------------------------------------------------------------------------------
template <typename TG, typename TS> struct GeneralLoader {
  static constexpr int U = BK / (kThreads / 32);      // samples per half-wave and step
  static constexpr int kStageSlot = kGroup, kPrefetchSlot = 2 * kGroup + 8;
  static_assert(U % 8 == 0, "the swizzle of a staging store must not depend on the half-wave");
  uint32_t w0[U], w1[U];               // packed data of the step being loaded
  uint32_t rsc[U], rmn[U];             // raw scale / min
  int wb[U];                           // widths that belong to w0/w1 (mixed stream)
  int nb[U];                           // widths and stream offsets of the step after (mixed stream)
  int64_t nbase[U];
  Stream st;
  const TS* scale;
  const TS* mn;
  int M, G, g, next_data, next_bits;
  uint32_t stage_at;                   // LDS address of this lane's 16 bytes of its half-wave's first row (buffer 0)

  ACTNN_DEV void init(const Stream& st_, const TS* scale_, const TS* mn_, int M_, int G_, int g_, uint32_t tile_x0,
                      uint32_t) {
    st = st_; scale = scale_; mn = mn_; M = M_; G = G_; g = g_;
    next_data = next_bits = 0;
    stage_at = tile_x0 + (threadIdx.x >> 5) * U * kRowBytes + ((threadIdx.x & 31) << 4);
#pragma unroll
    for (int u = 0; u < U; ++u) { nb[u] = 0; nbase[u] = 0; wb[u] = 0; w0[u] = w1[u] = 0u; rsc[u] = rmn[u] = 0u; }
    if (st.bits) prefetch_bits();
  }
  ACTNN_DEV void prefetch_bits() {
    const int hw = threadIdx.x >> 5;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int m = next_bits + hw * U + u;
      nb[u] = 0;
      nbase[u] = 0;
      if (m < M) {
        nb[u] = st.bits[m];
        nbase[u] = ((int64_t)st.prefix[m] * G + (int64_t)nb[u] * g) * 8;      // first word of (m, g)
      }
    }
    next_bits += BK;
  }
  ACTNN_DEV void prefetch() {
    const int hw = threadIdx.x >> 5, j = threadIdx.x & 31;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int m = next_data + hw * U + u;
      w0[u] = w1[u] = 0u;
      rsc[u] = rmn[u] = 0u;
      wb[u] = st.bits ? nb[u] : st.fixed_bits;
      if (m < M) {
        if (st.bits) {
          const int32_t* words = reinterpret_cast<const int32_t*>(st.packed) + nbase[u];
          const int n_words = 8 * wb[u];
          if (j < n_words) w0[u] = (uint32_t)words[j];
          if (32 + j < n_words) w1[u] = (uint32_t)words[32 + j];
        } else {
          const int wpt = 8 / st.fixed_bits;
          const u32x2 v = *reinterpret_cast<const u32x2*>(st.packed + ((int64_t)(m / wpt) * G + g) * 256 + j * 8);
          w0[u] = v.x;
          w1[u] = v.y;
        }
        rsc[u] = RawScalar<TS>::load(scale, (int64_t)m * G + g);
        rmn[u] = RawScalar<TS>::load(mn, (int64_t)m * G + g);
      }
    }
    next_data += BK;
    if (st.bits) prefetch_bits();
  }
  template <int SLOT, int NB> ACTNN_DEV void piece(int kfirst) {
    if constexpr (SLOT == kStageSlot) stage<NB>(kfirst);
    else if constexpr (SLOT == kPrefetchSlot) prefetch();
  }
  template <int NB> ACTNN_DEV void stage(int kfirst) {
    const int hw = threadIdx.x >> 5, j = threadIdx.x & 31;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int m = kfirst + hw * U + u;
      const int b = wb[u];
      u32x4 out = {0u, 0u, 0u, 0u};
      // the exchange below involves every lane: no lane may skip it (b is uniform per half-wave)
      uint64_t codes;
      int shift, step;
      if (st.bits) {
        codes = (uint64_t)transpose32(w0[u], (uint32_t)j) | ((uint64_t)transpose32(w1[u], (uint32_t)j) << 32);
        shift = 0;
        step = b;                       // code of feature 8j + e: bits [e*b, e*b + b)
      } else {
        codes = (uint64_t)w0[u] | ((uint64_t)w1[u] << 32);
        shift = (m % (8 / st.fixed_bits)) * b;      // byte e holds feature 8j + e, this sample at `shift`
        step = 8;
      }
      if (m < M && b >= 1 && b <= 8) {
        const uint32_t mask = (1u << b) - 1u;
        const Dequant<TS> dq(RawScalar<TS>::widen(rsc[u]), RawScalar<TS>::widen(rmn[u]));
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = dq((uint32_t)(codes >> (e * step + shift)) & mask);
        out = (u32x4){Mma<TG>::pack2(v[0], v[1]), Mma<TG>::pack2(v[2], v[3]),
                      Mma<TG>::pack2(v[4], v[5]), Mma<TG>::pack2(v[6], v[7])};
      }
      // row k = hw * U + u of the tile: its chunk j lies at j ^ ((k & 7) << 2) = j ^ ((u & 7) << 2)
      lds_store<u32x4>((stage_at ^ ((u & 7) << 6)) + NB * kTileBytes + u * kRowBytes, out);
    }
  }
};

template <typename TG, typename TS, bool TABLE>
__global__ __launch_bounds__(kThreads, 1) void linear_gw_kernel(
    const TG* __restrict__ gout, Stream st, const TS* __restrict__ scale, const TS* __restrict__ mn,
    void* __restrict__ gw_out, int out_dtype, int M, int O, int I, int splits, int rows_per_split) {
  // grad_out tiles first: the direct loads address LDS through M0, keep their targets low
  __shared__ __attribute__((aligned(1024))) uint8_t smem[4 * kTileBytes + kTabBytes];
  const uint32_t lds0 = lds_address(smem);
  const uint32_t tile_g0 = lds0, tile_x0 = lds0 + 2 * kTileBytes, tab0 = lds0 + 4 * kTileBytes;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wr = wave & 1, wn = wave >> 1;   // the wave's 128 rows (O) and 128 columns (I) of the tile
  const int G = I / 256;
  // Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.  Give every XCD whole
  // panels of grad_out rows (all column tiles of tile_m), so that a panel is pulled into one L2
  // only and reused there by the tiles_n blocks that need it.
  const int tiles_n = G;
  const int tiles_m = (O + BM - 1) / BM;
  int tile = blockIdx.x;
  int64_t out_slice = 0;                     // elements from gw_out to this block's output matrix
  if (splits > 1) {
    // Split reduction: the block takes rows [m0, m0 + M) of the sum and leaves its tile of partial
    // results (fp32) in slice `split` of the output buffer, [splits][O][I]; consecutive blocks are
    // the tiles of one split.  Every operand is moved to the block's first row (rows_per_split is a
    // multiple of BK, hence of the samples a byte of any fixed-width stream holds; the prefix sums of
    // the mixed-width stream are absolute).
    const int split = blockIdx.x / (tiles_m * tiles_n);
    tile = blockIdx.x % (tiles_m * tiles_n);
    const int m0 = split * rows_per_split;
    M = M - m0 < rows_per_split ? M - m0 : rows_per_split;
    gout += (int64_t)m0 * O;
    scale += (int64_t)m0 * G;
    mn += (int64_t)m0 * G;
    if (st.bits) {
      st.bits += m0;
      st.prefix += m0;
    } else {
      st.packed += (int64_t)(m0 / (8 / st.fixed_bits)) * G * 256;
    }
    out_slice = (int64_t)split * O * I;
  } else if (tiles_m % 8 == 0) {
    const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
    tile = (xcd * (tiles_m / 8) + idx / tiles_n) * tiles_n + idx % tiles_n;
  }
  const int o0 = (tile / tiles_n) * BM;
  const int g = tile % tiles_n;              // the block's columns are quantisation group g
  const int i0 = g * 256;

  // ---- grad_out tile: straight from global memory into LDS.  One instruction of a wave fills 1 KiB
  // of LDS (two rows); lane -> row 2*rp + lane/32, LDS chunk lane%32, which holds source chunk
  // lane%32 ^ swizzle(row).  Rows past M are read from the last row (their activations are staged as
  // zeros, so any finite value will do), columns past O from the block's first column (they only
  // reach output rows that are not stored): every lane loads, nothing else writes these tiles.
  // The source address is a scalar base (the first row of the pair) plus a lane offset that takes
  // one of two values: with or without the step to the pair's second row.
  const int g_row = lane >> 5;
  // rows of one instruction: 2 * rp + g_row with rp = kWaves * jj + wave, so (row & 7) only depends on the wave
  static_assert(kWaves % 4 == 0, "the swizzle of a direct load must not depend on jj");
  const int g_chunk = (lane & 31) ^ (((2 * (wave & 3) + g_row) & 7) << 2);
  const int g_col = o0 + g_chunk * 8 < O ? o0 + g_chunk * 8 : o0;
  const uint32_t g_off_first = (uint32_t)g_col * (uint32_t)sizeof(TG);                       // in the pair's first row
  const uint32_t g_off_pair = g_off_first + (uint32_t)g_row * (uint32_t)O * (uint32_t)sizeof(TG);  // in the lane's own row
  auto load_g_piece = [&](auto NB, int kfirst, int jj) {
    const int rp = jj * kWaves + wave;                    // row pair of the tile, uniform in the wave
    int m = kfirst + 2 * rp;
    const bool whole = m + 1 < M;                         // both rows of the pair exist
    m = m < M ? m : M - 1;
    const char* base = reinterpret_cast<const char*>(gout) + (int64_t)m * O * (int64_t)sizeof(TG);
    load_to_lds16_base(base, whole ? g_off_pair : g_off_first,
                       reinterpret_cast<const uint8_t*>(smem) + decltype(NB)::value * kTileBytes + rp * 2 * kRowBytes);
  };
  // The same for tiles that lie entirely below M (all but the last one or two): no clamping, and the
  // scalar base is a running pointer - the eight pieces of a tile are eight rows apart, and after the
  // eighth the pointer stands at the wave's first row pair of the next tile.
  const int64_t g_piece_bytes = (int64_t)2 * kWaves * O * (int64_t)sizeof(TG);
  const char* g_next = reinterpret_cast<const char*>(gout) + (int64_t)(BK + 2 * wave) * O * (int64_t)sizeof(TG);
  const uint8_t* g_lds_wave = reinterpret_cast<const uint8_t*>(smem) + wave * 2 * kRowBytes;
  auto load_g_piece_whole = [&](auto NB, auto JJ) {
    load_to_lds16_base(g_next, g_off_pair,
                       g_lds_wave + decltype(NB)::value * kTileBytes + decltype(JJ)::value * kWaves * 2 * kRowBytes);
    g_next += g_piece_bytes;
  };

  // ---- fragments: lane -> column n0 + lane%32, samples 16*kb + 8*(lane/32) + 0..7
  const int blk = lane >> 4, r = lane & 15;
  const int f_row = 8 * (blk >> 1) + (r >> 2);
  // chunk of column block n0 = 32*q: 4*q + 2*(blk&1) + ((r&3)>>1); bytes inside the chunk: (r&1)*8
  auto frag_offset = [&](int n0) {
    const int ch = n0 / 8 + 2 * (blk & 1) + ((r & 3) >> 1);
    return (uint32_t)(chunk_offset(f_row, ch) + (r & 1) * 8);
  };
  // LDS address of the first read of a fragment in buffer 0, k-block 0; the second read (4 rows on)
  // lies in the other half of the row: the address with bit 8 flipped, plus 4 rows
  uint32_t ax[NE], ag[NA];
#pragma unroll
  for (int e = 0; e < NE; ++e) ax[e] = tile_x0 + frag_offset(wn * 32 * NE + 32 * e);
#pragma unroll
  for (int a = 0; a < NA; ++a) ag[a] = tile_g0 + frag_offset(wr * 32 * NA + 32 * a);
  uint32_t ax2[NE], ag2[NA];
#pragma unroll
  for (int e = 0; e < NE; ++e) ax2[e] = ax[e] ^ 256u;
#pragma unroll
  for (int a = 0; a < NA; ++a) ag2[a] = ag[a] ^ 256u;

  f32x16 acc[NE][NA];
#pragma unroll
  for (int e = 0; e < NE; ++e)
#pragma unroll
    for (int a = 0; a < NA; ++a)
#pragma unroll
      for (int c = 0; c < 16; ++c) acc[e][a][c] = 0.0f;

  // fragment f of k-block kb: f = 0..NA-1 grad_out (MFMA columns), then NE activations (MFMA
  // rows); double-buffered in registers by the parity of kb.  They start as zeros: the first
  // step's leading MFMAs (the last k-block "of the step before") then add nothing.
  u32x4 fx[2][NE], fg[2][NA];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
#pragma unroll
    for (int e = 0; e < NE; ++e) fx[h][e] = (u32x4){0u, 0u, 0u, 0u};
#pragma unroll
    for (int a = 0; a < NA; ++a) fg[h][a] = (u32x4){0u, 0u, 0u, 0u};
  }
  auto read_fragment = [&](auto BUF, auto KB, auto F) {
    constexpr int buf = decltype(BUF)::value, kb = decltype(KB)::value, f = decltype(F)::value;
    constexpr bool is_g = f < NA;
    constexpr uint32_t at = buf * kTileBytes + kb * 16 * kRowBytes;
    const uint32_t a1 = is_g ? ag[is_g ? f : 0] : ax[is_g ? 0 : f - NA];
    const uint32_t a2 = is_g ? ag2[is_g ? f : 0] : ax2[is_g ? 0 : f - NA];
    const u32x2 lo = read_transposed(a1 + at);
    const u32x2 hi = read_transposed(a2 + at + 4 * kRowBytes);
    const u32x4 v = {lo.x, lo.y, hi.x, hi.y};
    if constexpr (is_g) fg[kb & 1][f] = v; else fx[kb & 1][f - NA] = v;
  };

  const int steps = (M + BK - 1) / BK;
  // The schedule.  Step t is multiplied out of LDS buffer t % 2; the tiles of step t+1 go into the
  // other buffer, whose last readers finished before the barrier that ended step t-1.  Between two
  // barriers a wave issues its 64 MFMAs of a step - the last k-block of the step before (its
  // fragments were read before the barrier) and the first three of this step - and everything else
  // is cut into pieces placed between them, so that the matrix pipe always has work queued while
  // the wave permutes bytes and waits for LDS:
  //   MFMA slot  0..15: k-block 3 of step t-1 | reads (t, 0), direct loads of G(t+1)
  //   MFMA slot 16..31: k-block 0 of step t   | reads (t, 1), table of X(t+1), first staging pieces
  //   MFMA slot 32..47: k-block 1             | reads (t, 2), staging pieces, loads for X(t+2)
  //   MFMA slot 48..63: k-block 2             | reads (t, 3)
  //   wait for the direct loads; barrier
  // The eight fragments of a k-block are read in the first eight slots of the group before the one
  // that multiplies them, into the register set the MFMAs of those slots do not read.
  // The body between two barriers has no branches and exists twice, once per buffer (the buffer is
  // what the offset fields of its LDS instructions encode).  Every step stages a next tile: after the
  // last step that tile lies past the rows and is filled from clamped addresses with values nobody
  // reads.
  constexpr int kDirectLoads = kTileBytes / (kThreads * 16);
  // WHOLE: the tile this step stages (step t + 1) lies entirely below M
  auto step = [&](auto& ld, auto BUF, auto WHOLE, int t) {
    constexpr int buf = decltype(BUF)::value, nb = 1 - buf;
    for_each_slot<kSlots>([&](auto S) {
      constexpr int slot = decltype(S)::value;
      constexpr int kb_mfma = (slot / kGroup + 3) % 4, e = (slot % kGroup) / NA, a = slot % NA;
      acc[e][a] = Mma<TG>::mfma(fx[kb_mfma & 1][e], fg[kb_mfma & 1][a], acc[e][a]);
      if constexpr (slot % kGroup < NE + NA) read_fragment(Slot<buf>{}, Slot<slot / kGroup>{}, Slot<slot % kGroup>{});
      if constexpr (slot < kDirectLoads) {
        if constexpr (decltype(WHOLE)::value != 0) load_g_piece_whole(Slot<nb>{}, Slot<slot>{});
        else load_g_piece(Slot<nb>{}, (t + 1) * BK, slot);
      }
      ld.template piece<slot, nb>((t + 1) * BK);
      __builtin_amdgcn_sched_barrier(0);
    });
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
  };
  auto run = [&](auto& ld) {
    using Loader = std::remove_reference_t<decltype(ld)>;
    if (steps > 0) {
      ld.prefetch();
      // the whole staging of tile 0 (every piece but the prefetch, which follows)
      for_each_slot<kSlots>([&](auto S) {
        constexpr int slot = decltype(S)::value;
        if constexpr (slot != Loader::kPrefetchSlot) ld.template piece<slot, 0>(0);
      });
#pragma unroll
      for (int jj = 0; jj < kDirectLoads; ++jj) load_g_piece(Slot<0>{}, 0, jj);
      ld.prefetch();
    }
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    // steps t = 0 .. whole - 1 stage a tile that lies entirely below M: (t + 2) * BK <= M
    const int whole = M / BK - 1;
    int t = 0;
    for (; t + 2 <= whole; t += 2) {
      step(ld, Slot<0>{}, Slot<1>{}, t);
      step(ld, Slot<1>{}, Slot<1>{}, t + 1);
    }
    for (; t + 2 <= steps; t += 2) {
      step(ld, Slot<0>{}, Slot<0>{}, t);
      step(ld, Slot<1>{}, Slot<0>{}, t + 1);
    }
    if (t < steps) step(ld, Slot<0>{}, Slot<0>{}, t);
    if (steps > 0) {
#pragma unroll
      for (int e = 0; e < NE; ++e)
#pragma unroll
        for (int a = 0; a < NA; ++a) acc[e][a] = Mma<TG>::mfma(fx[1][e], fg[1][a], acc[e][a]);
    }
  };
  if constexpr (TABLE) {
    TableLoader<TG, TS> ld;
    ld.init(st, scale, mn, M, G, g, tile_x0, tab0);
    run(ld);
  } else {
    GeneralLoader<TG, TS> ld;
    ld.init(st, scale, mn, M, G, g, tile_x0, tab0);
    run(ld);
  }

  // 32x32 accumulator layout: register c of a lane is fragment row 8*(c/4) + 4*(lane/32) + c%4 (a
  // column of grad_w: feature), fragment column lane%32 (a row of grad_w: output unit).
  auto store_all = [&](auto* gw) {
    using TO = std::remove_pointer_t<decltype(gw)>;
    gw += out_slice;
#pragma unroll
    for (int a = 0; a < NA; ++a) {
      const int row = o0 + wr * 32 * NA + 32 * a + (lane & 31);
      if (row < O) {
#pragma unroll
        for (int e = 0; e < NE; ++e) {
#pragma unroll
          for (int cq = 0; cq < 4; ++cq) {
            const int col = i0 + wn * 32 * NE + 32 * e + 8 * cq + 4 * (lane >> 5);
            store_out4<TO>(gw + (int64_t)row * I + col, acc[e][a][4 * cq], acc[e][a][4 * cq + 1],
                           acc[e][a][4 * cq + 2], acc[e][a][4 * cq + 3]);
          }
        }
      }
    }
  };
  if (out_dtype == ACTNN_F32) store_all(static_cast<float*>(gw_out));
  else if (out_dtype == ACTNN_F16) store_all(static_cast<__half*>(gw_out));
  else store_all(static_cast<bf16_t*>(gw_out));
}

// Sum of the `splits` partial tiles of a split reduction, narrowed to the output type.
template <typename TO>
__global__ __launch_bounds__(kThreads) void linear_gw_sum_splits_kernel(const float* __restrict__ part,
                                                                      TO* __restrict__ gw, int64_t quads,
                                                                      int splits) {
  const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i >= quads) return;
  float a = 0.0f, b = 0.0f, c = 0.0f, d = 0.0f;
  for (int sp = 0; sp < splits; ++sp) {                       // fixed order: the result is reproducible
    const u32x4 v = load16_nt(part + ((int64_t)sp * quads + i) * 4);
    a += as_float(v.x); b += as_float(v.y); c += as_float(v.z); d += as_float(v.w);
  }
  store_out4<TO>(gw + i * 4, a, b, c, d);
}

// How the reduction over the M samples is split over blocks.  The kernel's tile is fixed (one
// quantisation group of columns, 256 output rows), so a weight gradient with few tiles and many
// samples would leave most of the 256 CUs idle; its blocks then take slices of the samples each and a
// second kernel adds the slices.  The estimate: a k-step of one block takes about 2.1 us (config 4:
// 128 steps in 0.266 ms), the partial tiles are written and read back at about 4 TB/s, and the second
// launch costs about 6 us.  -> splits (1 = no split), rows per split (a multiple of BK).
struct SplitPlan { int splits, rows_per_split; };
SplitPlan plan_splits(int64_t M, int64_t O, int64_t I) {
  const int64_t tiles = ((O + BM - 1) / BM) * (I / BN);
  const int64_t steps = (M + BK - 1) / BK;
  constexpr int64_t kCUs = 256;
  auto cost_us = [&](int64_t sp) {
    const int64_t rounds = (tiles * sp + kCUs - 1) / kCUs;
    const int64_t per = (steps + sp - 1) / sp;
    double t = 2.1 * (double)(rounds * per) + 4.0;           // + prologue and epilogue of a block
    if (sp > 1) t += 6.0 + 2.0 * (double)sp * (double)O * (double)I * 4.0 / 4.0e6;
    return t;
  };
  int64_t best = 1;
  double best_t = cost_us(1);
  for (int64_t sp = 2; sp <= 64 && sp <= steps; sp *= 2) {
    const double t = cost_us(sp);
    if (t < 0.8 * best_t && t < cost_us(best)) { best = sp; best_t = t; }
  }
  if (best == 1) return SplitPlan{1, 0};
  const int64_t per = (steps + best - 1) / best;
  return SplitPlan{(int)((steps + per - 1) / per), (int)(per * BK)};
}

template <typename TO> void launch_sum_splits(const float* part, void* gw, int64_t quads, int splits, hipStream_t s) {
  linear_gw_sum_splits_kernel<TO><<<dim3((unsigned)((quads + kThreads - 1) / kThreads)), dim3(kThreads), 0, s>>>(
      part, static_cast<TO*>(gw), quads, splits);
}

template <typename TG, typename TS>
int launch_out(int out_dtype, const void* gout, const Stream& st, const void* scale, const void* mn,
               void* gw, int64_t M, int64_t O, int64_t I, void* workspace, int64_t workspace_bytes, hipStream_t s) {
  if (out_dtype != ACTNN_F32 && out_dtype != ACTNN_F16 && out_dtype != ACTNN_BF16) return ACTNN_EDTYPE;
  const int64_t tiles = ((O + BM - 1) / BM) * (I / BN);
  SplitPlan sp = plan_splits(M, O, I);
  if (sp.splits > 1 && (!workspace || workspace_bytes < (int64_t)sp.splits * O * I * 4)) sp = SplitPlan{1, 0};
  if (sp.splits > 1 && !aligned16(workspace)) return ACTNN_EALIGN;
  const int64_t blocks = tiles * sp.splits;
  if (blocks > 0x7fffffffLL) return ACTNN_EINVAL;
  const bool table = !st.bits && st.fixed_bits == 2;
  const dim3 grid((unsigned)blocks), blk(kThreads);
  // a split sum leaves fp32 partial tiles in the workspace; a second kernel adds them
  void* target = sp.splits > 1 ? workspace : gw;
  const int target_dtype = sp.splits > 1 ? (int)ACTNN_F32 : out_dtype;
  if (table)
    linear_gw_kernel<TG, TS, true><<<grid, blk, 0, s>>>(
        static_cast<const TG*>(gout), st, static_cast<const TS*>(scale), static_cast<const TS*>(mn), target,
        target_dtype, (int)M, (int)O, (int)I, sp.splits, sp.rows_per_split);
  else
    linear_gw_kernel<TG, TS, false><<<grid, blk, 0, s>>>(
        static_cast<const TG*>(gout), st, static_cast<const TS*>(scale), static_cast<const TS*>(mn), target,
        target_dtype, (int)M, (int)O, (int)I, sp.splits, sp.rows_per_split);
  if (sp.splits > 1) {
    const float* part = static_cast<const float*>(workspace);
    const int64_t quads = O * I / 4;
    if (out_dtype == ACTNN_F32) launch_sum_splits<float>(part, gw, quads, sp.splits, s);
    else if (out_dtype == ACTNN_F16) launch_sum_splits<__half>(part, gw, quads, sp.splits, s);
    else launch_sum_splits<bf16_t>(part, gw, quads, sp.splits, s);
  }
  ACTNN_RETURN_LAUNCH_STATUS();
}

template <typename TG>
int launch_sm(int sm_dtype, int out_dtype, const void* gout, const Stream& st, const void* scale,
              const void* mn, void* gw, int64_t M, int64_t O, int64_t I, void* ws, int64_t ws_bytes, hipStream_t s) {
  switch (sm_dtype) {
    case ACTNN_F32: return launch_out<TG, float>(out_dtype, gout, st, scale, mn, gw, M, O, I, ws, ws_bytes, s);
    case ACTNN_F16: return launch_out<TG, __half>(out_dtype, gout, st, scale, mn, gw, M, O, I, ws, ws_bytes, s);
    case ACTNN_BF16: return launch_out<TG, bf16_t>(out_dtype, gout, st, scale, mn, gw, M, O, I, ws, ws_bytes, s);
    default: return ACTNN_EDTYPE;
  }
}

}  // namespace
}  // namespace actnn

extern "C" int64_t actnn_linear_grad_weight_workspace_bytes(int64_t M, int64_t O, int64_t I) {
  using namespace actnn;
  if (M <= 0 || O <= 0 || I <= 0 || I % 256 != 0) return 0;
  const SplitPlan sp = plan_splits(M, O, I);
  return sp.splits > 1 ? (int64_t)sp.splits * O * I * 4 : 0;
}

extern "C" int actnn_linear_grad_weight_ws(const void* grad_out, const void* packed, const int32_t* bits,
                                           const int32_t* prefix, int fixed_bits, const void* scale,
                                           const void* mn, void* grad_w, int64_t M, int64_t O, int64_t I,
                                           int go_dtype, int sm_dtype, int out_dtype, void* workspace,
                                           int64_t workspace_bytes, void* stream) {
  using namespace actnn;
  if (M < 0 || O < 0 || I < 0 || I % 256 != 0 || O % 8 != 0) return ACTNN_EINVAL;
  if (M > 0x7fffffffLL - BK || O > 0x7fffffffLL - BM || I > 0x7fffffffLL) return ACTNN_EINVAL;
  if (bits) {
    if (!prefix) return ACTNN_EINVAL;
  } else if (fixed_bits != 1 && fixed_bits != 2 && fixed_bits != 4 && fixed_bits != 8) {
    return ACTNN_EBITS;
  }
  if (O == 0 || I == 0) return ACTNN_OK;
  if (!grad_w || (M > 0 && (!grad_out || !packed || !scale || !mn))) return ACTNN_EINVAL;
  if (M > 0 && (!aligned16(grad_out) || !aligned16(grad_w) || reinterpret_cast<uintptr_t>(packed) % 8 != 0 ||
                reinterpret_cast<uintptr_t>(scale) % 4 != 0 || reinterpret_cast<uintptr_t>(mn) % 4 != 0))
    return ACTNN_EALIGN;
  const Stream st{static_cast<const uint8_t*>(packed), bits, prefix, bits ? 0 : fixed_bits};
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (go_dtype) {
    case ACTNN_F16: return launch_sm<__half>(sm_dtype, out_dtype, grad_out, st, scale, mn, grad_w, M, O, I, workspace, workspace_bytes, s);
    case ACTNN_BF16: return launch_sm<bf16_t>(sm_dtype, out_dtype, grad_out, st, scale, mn, grad_w, M, O, I, workspace, workspace_bytes, s);
    default: return ACTNN_EDTYPE;
  }
}

extern "C" int actnn_linear_grad_weight(const void* grad_out, const void* packed, const int32_t* bits,
                                        const int32_t* prefix, int fixed_bits, const void* scale,
                                        const void* mn, void* grad_w, int64_t M, int64_t O, int64_t I,
                                        int go_dtype, int sm_dtype, int out_dtype, void* stream) {
  return actnn_linear_grad_weight_ws(grad_out, packed, bits, prefix, fixed_bits, scale, mn, grad_w, M, O, I,
                                     go_dtype, sm_dtype, out_dtype, nullptr, 0, stream);
}

extern "C" int actnn_linear_grad_weight_q2(const void* grad_out, const int8_t* packed, const void* scale,
                                           const void* mn, void* grad_w, int64_t M, int64_t O, int64_t I,
                                           int go_dtype, int sm_dtype, int out_dtype, void* stream) {
  if (M % 4 != 0) return ACTNN_EINVAL;
  return actnn_linear_grad_weight(grad_out, packed, nullptr, nullptr, 2, scale, mn, grad_w, M, O, I, go_dtype,
                                  sm_dtype, out_dtype, stream);
}
