// Fused QLinear weight gradient (replaces dequantize_activation + grad_output.t().mm(input) in
// linear.backward, actnn/actnn/ops.py:407-421):
//
//     grad_w[O, I] = grad_out[M, O]^T @ dequant(x)[M, I]
//
// x stays in the 2-bit fixed-width stream (byte ((m/4) * I/256 + g) * 256 + d holds rows
// 4*(m/4) .. +3 of feature g*256 + d, two bits each) with scale/min[M, I/256].  The full
// precision input is never written to memory: every k-step the 2-bit tile is unpacked,
// dequantised (code * (1/scale) + min) and narrowed to 16 bits straight into the LDS tile that feeds
// v_mfma_f32_32x32x16_bf16 (bf16 gradients) or v_mfma_f32_32x32x16_f16 (fp16 gradients), with
// fp32 accumulation.
//
// Tiling: the reduction runs over the samples m (K of the GEMM).  A 512-thread block (one per CU)
// owns a 256 (O) x 256 (I) output tile - one whole quantisation group, so a block needs one
// scale/min per sample - as 8 waves of 64 x 128, each 2 x 4 MFMA tiles of 32 x 32.  The large tile
// is what keeps the L2 -> CU traffic (grad_out is re-read once per column tile) below what the
// vector caches deliver.  Per k-step of 64 samples (LDS tiles double-buffered, one barrier a step):
//   * grad_out lies o-contiguous in memory but MFMA fragments want 8 consecutive k per row, so a
//     thread loads 4 consecutive k-rows x 8 o's (16-byte vectors, a wave covers whole rows of the
//     tile), transposes them in registers with 16 byte-permutes and writes 8 rows of 4 k's;
//   * the packed bytes already hold 4 consecutive k per feature: a thread unpacks 2 x (4 features
//     x 4 samples) from two 32-bit loads and writes them k-contiguous.  A wave works on 8
//     consecutive samples: 16 lanes fetch their 8 scales and 8 minima with one load and v_readlane
//     hands them out (scalar loads of one value per cache line were 40% of the kernel's time).
//   Both LDS tiles are [row][k] with a 144-byte pitch, every MFMA fragment is one 16-byte LDS read.
//   Rows are stored permuted - tile row o at LDS row (o % 8) * 32 + o / 8, tile column i at LDS row
//   (i % 4) * 64 + i / 4 - which makes lane pairs of a staging write fill 16 contiguous bytes of
//   consecutive LDS rows (no bank conflicts) and lets the epilogue store 4 consecutive columns
//   per lane.
// Global loads run two steps ahead of the MFMAs (two register sets), LDS writes one step ahead.
#include "device_utils.h"

namespace actnn {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kThreads = 512;
constexpr int BM = 256;            // output rows (O) per block
constexpr int BN = 256;            // output columns (I) per block: one quantisation group
constexpr int BK = 64;             // samples per k-step
constexpr int kPitch = BK + 8;     // 16-bit elements per row of either LDS tile (144 bytes)
constexpr int kTile = 256 * kPitch;                 // elements of one operand tile
constexpr int kLdsBytes = 2 * 2 * kTile * 2;        // two operands, two buffers

// The MFMA runs in the 16-bit format of grad_out, so its rows go to LDS exactly as loaded:
// bf16 gradients (bf16 autocast) use v_mfma_f32_32x32x16_bf16 and the dequantised activations are
// rounded to bf16 (nearest even); fp16 gradients use v_mfma_f32_32x32x16_f16 and the activations
// are narrowed to fp16 with v_cvt_pkrtz (truncation: 2^-11 relative, far below a 2-bit step).
template <typename TG> struct Mma;
template <> struct Mma<bf16_t> {
  static ACTNN_DEV uint32_t pack2(float lo, float hi) { return pack_bf16x2(lo, hi); }
  static ACTNN_DEV f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};
template <> struct Mma<__half> {
  static ACTNN_DEV uint32_t pack2(float lo, float hi) {
    return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(lo, hi));
  }
  static ACTNN_DEV f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};

template <typename T> struct RawScalar;          // a scale/min value exactly as loaded
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

template <typename TG, typename TS, typename TO>
__global__ __launch_bounds__(kThreads, 1) void linear_gw_q2_kernel(
    const TG* __restrict__ gout, const uint8_t* __restrict__ packed, const TS* __restrict__ scale,
    const TS* __restrict__ mn, TO* __restrict__ gw, int M, int O, int I) {
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  auto tileA = [&](int buf) { return smem + buf * 2 * kTile; };
  auto tileB = [&](int buf) { return smem + buf * 2 * kTile + kTile; };

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wr = wave & 3, wn = wave >> 2;   // the wave's 64-row group and 128-column half
  const int G = I / 256;
  // Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.  Give every XCD whole
  // panels of grad_out rows (all column tiles of tile_m), so that a panel is pulled into one L2
  // only and reused there by the tiles_n blocks that need it.
  const int tiles_n = G;
  const int tiles_m = (O + BM - 1) / BM;
  int tile = blockIdx.x;
  if (tiles_m % 8 == 0) {
    const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
    tile = (xcd * (tiles_m / 8) + idx / tiles_n) * tiles_n + idx % tiles_n;
  }
  const int o0 = (tile / tiles_n) * BM;
  const int g = tile % tiles_n;              // the block's columns are quantisation group g
  const int i0 = g * 256;

  // A wave stages the sample quads 2 * wave and 2 * wave + 1 (8 consecutive samples) of a step.
  // Neighbouring lanes take the two quads of the same row, so that the 32 lanes served by one LDS
  // cycle write 16 rows x 16 contiguous bytes: no bank conflicts with the 144-byte pitch.
  // A staging: thread -> k rows 4 * quad .. + 3, o offset ao * 8 (a wave: 2 quads x whole rows)
  // B staging: thread -> the same quad, features 4 * fl .. + 3 and 128 + 4 * fl .. + 3
  const int par = lane & 1;
  const int quad = 2 * wave + par;
  const int ao = lane >> 1, fl = lane >> 1;
  const bool ovalid = o0 + ao * 8 < O;       // O % 8 == 0: a vector is inside or outside as a whole
  // running pointers / indices, advanced by one k-step per prefetch
  const TG* pa = gout + (int64_t)(quad * 4) * O + o0 + ao * 8;
  const uint8_t* pb = packed + ((int64_t)quad * G + g) * 256 + fl * 4;
  int64_t si = (int64_t)(wave * 8) * G + g;  // index of the wave's first sample in scale / min
  const int64_t a_step = (int64_t)BK * O;
  const int64_t b_step = (int64_t)(BK / 4) * G * 256;
  const int64_t s_step = (int64_t)BK * G;

  f32x16 acc[2][4];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
      for (int c = 0; c < 16; ++c) acc[a][b][c] = 0.0f;

  // The prefetch registers hold the data of the step after the one being multiplied, exactly as
  // loaded (nothing may consume a load where it is issued, or the wave would wait out the memory
  // latency there).  They are refilled as soon as the staging code has read them, most of a
  // k-step before they are needed again.
  u32x4 ra[4];
  uint32_t rb[2];
  uint32_t rsm = 0u;                         // lanes 0..15: scale / min of the wave's 8 samples
  // lane l < 16 fetches for quad 2 * wave + l / 8: scale (l % 8 < 4) or min of its sample l % 4
  const int sm_h = (lane >> 3) & 1, sm_j = lane & 3;
  const TS* sm_base = (lane & 4) ? mn : scale;
  int ka_next = 0, kb_next = 0;              // first sample of the step the next prefetch loads

  auto prefetch_a = [&]() {
    const bool avalid = ovalid && ka_next + quad * 4 < M;   // M % 4 == 0: a quad is inside or outside as a whole
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      ra[r] = (u32x4){0u, 0u, 0u, 0u};
      if (avalid) ra[r] = load16(pa + (int64_t)r * O);
    }
    pa += a_step;
    ka_next += BK;
  };
  auto prefetch_b = [&]() {
    rb[0] = rb[1] = 0u;
    if (kb_next + quad * 4 < M) {
      rb[0] = *reinterpret_cast<const uint32_t*>(pb);
      rb[1] = *reinterpret_cast<const uint32_t*>(pb + 128);
    }
    rsm = 0u;
    if (lane < 16 && kb_next + (2 * wave + sm_h) * 4 < M)
      rsm = RawScalar<TS>::load(sm_base, si + (int64_t)(4 * sm_h + sm_j) * G);
    pb += b_step;
    si += s_step;
    kb_next += BK;
  };

  // 4 (k) x 8 (o) -> 8 (o) x 4 (k): word p of ra[r] holds o = 2p (low half) and 2p + 1 (high half)
  auto stage_a = [&](int buf) {
    uint16_t* sA = tileA(buf);
#pragma unroll
    for (int p2 = 0; p2 < 4; ++p2) {
      const uint32_t w0 = ra[0][p2], w1 = ra[1][p2], w2 = ra[2][p2], w3 = ra[3][p2];
      const u32x2 even = {__builtin_amdgcn_perm(w1, w0, 0x05040100u), __builtin_amdgcn_perm(w3, w2, 0x05040100u)};
      const u32x2 odd = {__builtin_amdgcn_perm(w1, w0, 0x07060302u), __builtin_amdgcn_perm(w3, w2, 0x07060302u)};
      *reinterpret_cast<u32x2*>(&sA[((2 * p2) * 32 + ao) * kPitch + quad * 4]) = even;
      *reinterpret_cast<u32x2*>(&sA[((2 * p2 + 1) * 32 + ao) * kPitch + quad * 4]) = odd;
    }
  };
  // the step whose first sample is kfirst (rows past M dequantise to 0; their grad_out rows were
  // loaded as 0)
  auto stage_b = [&](int buf, int kfirst) {
    uint16_t* sB = tileB(buf);
    const bool bvalid = kfirst + quad * 4 < M;
    float inv[4], m4[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t sc0 = (uint32_t)__builtin_amdgcn_readlane((int)rsm, j);
      const uint32_t mn0 = (uint32_t)__builtin_amdgcn_readlane((int)rsm, 4 + j);
      const uint32_t sc1 = (uint32_t)__builtin_amdgcn_readlane((int)rsm, 8 + j);
      const uint32_t mn1 = (uint32_t)__builtin_amdgcn_readlane((int)rsm, 12 + j);
      inv[j] = bvalid ? __builtin_amdgcn_rcpf(RawScalar<TS>::widen(par ? sc1 : sc0)) : 0.0f;
      m4[j] = bvalid ? RawScalar<TS>::widen(par ? mn1 : mn0) : 0.0f;
    }
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const uint32_t by = rb[h] >> (8 * e);
        const float x0 = fmaf((float)(by & 3u), inv[0], m4[0]);
        const float x1 = fmaf((float)((by >> 2) & 3u), inv[1], m4[1]);
        const float x2 = fmaf((float)((by >> 4) & 3u), inv[2], m4[2]);
        const float x3 = fmaf((float)((by >> 6) & 3u), inv[3], m4[3]);
        *reinterpret_cast<u32x2*>(&sB[(e * 64 + 32 * h + fl) * kPitch + quad * 4]) =
            (u32x2){Mma<TG>::pack2(x0, x1), Mma<TG>::pack2(x2, x3)};
      }
    }
  };

  // Fragments are double-buffered in registers: those of k-block kb+1 are requested before the
  // MFMAs of k-block kb are issued, so the matrix pipe does not wait for LDS inside a step.
  u32x4 fa[2][2], fb[2][4];
  auto fragments = [&](int buf, int kb) {
    const uint16_t* sA = tileA(buf) + ((2 * wr) * 32 + (lane & 31)) * kPitch + (lane >> 5) * 8;
    const uint16_t* sB = tileB(buf) + (wn * 32 + (lane & 31)) * kPitch + (lane >> 5) * 8;
#pragma unroll
    for (int a = 0; a < 2; ++a) fa[kb & 1][a] = *reinterpret_cast<const u32x4*>(sA + a * 32 * kPitch + kb * 16);
#pragma unroll
    for (int e = 0; e < 4; ++e) fb[kb & 1][e] = *reinterpret_cast<const u32x4*>(sB + e * 64 * kPitch + kb * 16);
  };
  auto mfmas = [&](int kb) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
      for (int a = 0; a < 2; ++a) acc[a][e] = Mma<TG>::mfma(fa[kb & 1][a], fb[kb & 1][e], acc[a][e]);
  };
  auto multiply_step = [&](int buf) {
    fragments(buf, 0);
#pragma unroll
    for (int kb = 0; kb < BK / 16; ++kb) {
      // keep the compiler from sinking the reads of kb+1 below the MFMAs of kb
      __builtin_amdgcn_sched_barrier(0);
      if (kb + 1 < BK / 16) fragments(buf, kb + 1);
      __builtin_amdgcn_sched_barrier(0);
      mfmas(kb);
    }
  };
  auto stage_step = [&](int j) {             // write tile j, then get the loads of tile j+1 in flight
    stage_a(j & 1);
    stage_b(j & 1, j * BK);
    prefetch_a();
    prefetch_b();
  };

  // Step t is multiplied out of LDS buffer t % 2 while the tile of step t+1 is written into the
  // other buffer (its last readers passed the barrier at the end of step t-1) and the loads of
  // step t+2 are issued: one barrier per step.
  const int steps = (M + BK - 1) / BK;
  prefetch_a();
  prefetch_b();
  if (steps > 0) stage_step(0);
  __syncthreads();
  for (int t = 0; t < steps; ++t) {
    if (t + 1 < steps) stage_step(t + 1);
    multiply_step(t & 1);
    __syncthreads();
  }

  // 32x32 accumulator layout: register c of a lane is fragment row 8*(c/4) + 4*(lane/32) + c%4,
  // fragment column lane%32.  Fragment row r of A-fragment a is tile row 8*r + 2*wr + a; fragment
  // column l of B-fragment e is tile column 128*wn + 4*l + e.
#pragma unroll
  for (int a = 0; a < 2; ++a) {
#pragma unroll
    for (int c = 0; c < 16; ++c) {
      const int r = 8 * (c >> 2) + 4 * (lane >> 5) + (c & 3);
      const int row = o0 + 8 * r + 2 * wr + a;
      const int col = i0 + 128 * wn + 4 * (lane & 31);
      if (row < O)
        store_out4<TO>(gw + (int64_t)row * I + col, acc[a][0][c], acc[a][1][c], acc[a][2][c], acc[a][3][c]);
    }
  }
}

template <typename TG, typename TS, typename TO>
int launch(const void* gout, const int8_t* packed, const void* scale, const void* mn, void* gw,
           int64_t M, int64_t O, int64_t I, hipStream_t s) {
  const int64_t blocks = ((O + BM - 1) / BM) * (I / BN);
  if (blocks > 0x7fffffffLL) return ACTNN_EINVAL;
  auto kernel = linear_gw_q2_kernel<TG, TS, TO>;
  // more than the 64 KB a kernel may use without asking
  const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
  if (e != hipSuccess) return (int)e;
  kernel<<<dim3((unsigned)blocks), dim3(kThreads), kLdsBytes, s>>>(
      static_cast<const TG*>(gout), reinterpret_cast<const uint8_t*>(packed),
      static_cast<const TS*>(scale), static_cast<const TS*>(mn), static_cast<TO*>(gw), (int)M, (int)O,
      (int)I);
  ACTNN_RETURN_LAUNCH_STATUS();
}

template <typename TG, typename TS>
int launch_out(int out_dtype, const void* gout, const int8_t* packed, const void* scale,
               const void* mn, void* gw, int64_t M, int64_t O, int64_t I, hipStream_t s) {
  switch (out_dtype) {
    case ACTNN_F32: return launch<TG, TS, float>(gout, packed, scale, mn, gw, M, O, I, s);
    case ACTNN_F16: return launch<TG, TS, __half>(gout, packed, scale, mn, gw, M, O, I, s);
    case ACTNN_BF16: return launch<TG, TS, bf16_t>(gout, packed, scale, mn, gw, M, O, I, s);
    default: return ACTNN_EDTYPE;
  }
}

template <typename TG>
int launch_sm(int sm_dtype, int out_dtype, const void* gout, const int8_t* packed, const void* scale,
              const void* mn, void* gw, int64_t M, int64_t O, int64_t I, hipStream_t s) {
  switch (sm_dtype) {
    case ACTNN_F32: return launch_out<TG, float>(out_dtype, gout, packed, scale, mn, gw, M, O, I, s);
    case ACTNN_F16: return launch_out<TG, __half>(out_dtype, gout, packed, scale, mn, gw, M, O, I, s);
    case ACTNN_BF16: return launch_out<TG, bf16_t>(out_dtype, gout, packed, scale, mn, gw, M, O, I, s);
    default: return ACTNN_EDTYPE;
  }
}

}  // namespace
}  // namespace actnn

extern "C" int actnn_linear_grad_weight_q2(const void* grad_out, const int8_t* packed,
                                           const void* scale, const void* mn, void* grad_w,
                                           int64_t M, int64_t O, int64_t I, int go_dtype,
                                           int sm_dtype, int out_dtype, void* stream) {
  using namespace actnn;
  if (M < 0 || O < 0 || I < 0 || M % 4 != 0 || I % 256 != 0 || O % 8 != 0) return ACTNN_EINVAL;
  if (M > 0x7fffffffLL || O > 0x7fffffffLL || I > 0x7fffffffLL) return ACTNN_EINVAL;
  if (O == 0 || I == 0) return ACTNN_OK;
  if (!grad_w || (M > 0 && (!grad_out || !packed || !scale || !mn))) return ACTNN_EINVAL;
  if (M > 0 && (!aligned16(grad_out) || !aligned16(grad_w) || reinterpret_cast<uintptr_t>(packed) % 4 != 0 ||
                reinterpret_cast<uintptr_t>(scale) % 4 != 0 || reinterpret_cast<uintptr_t>(mn) % 4 != 0))
    return ACTNN_EALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (go_dtype) {
    case ACTNN_F16: return launch_sm<__half>(sm_dtype, out_dtype, grad_out, packed, scale, mn, grad_w, M, O, I, s);
    case ACTNN_BF16: return launch_sm<bf16_t>(sm_dtype, out_dtype, grad_out, packed, scale, mn, grad_w, M, O, I, s);
    default: return ACTNN_EDTYPE;
  }
}
