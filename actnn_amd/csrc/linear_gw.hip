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
// Tiling: the reduction runs over the samples m (K of the GEMM).  A 256-thread block owns a
// 256 (O) x 128 (I) output tile - inside one quantisation group, so a block needs one scale/min
// per sample - as 4 waves of 64 x 128, each 2 x 4 MFMA tiles of 32 x 32.  Two blocks fit on a
// CU; they are not synchronised with each other, so one block's unpack/convert work overlaps the
// other's MFMAs.  Per k-step of 32 samples (LDS tiles are double-buffered, one barrier per step):
//   * grad_out rows are copied as they lie in memory (O contiguous, 16-byte vectors) into LDS as
//     [k][o]; the MFMA "A" fragments (8 consecutive k for one o) are gathered from there with
//     16-bit LDS reads;
//   * the packed bytes already hold 4 consecutive k per feature, so a thread unpacks 8 features x
//     4 samples and writes them k-contiguous: LDS [i][k], "B" fragments are single 16-byte reads.
// Global loads run two steps ahead of the MFMAs (register prefetch), LDS writes one step ahead.
#include "device_utils.h"

namespace actnn {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int BM = 256;            // output rows (O) per block
#ifndef GW_BN
#define GW_BN 128
#endif
constexpr int BN = GW_BN;          // output columns (I) per block: half a quantisation group (or a whole one)
constexpr int BK = 32;             // samples per k-step
constexpr int kPitchA = BM + 8;    // 16-bit elements per k-row of the A tile  (528 bytes)
constexpr int kPitchB = BK + 8;    // 16-bit elements per feature row of the B tile (80 bytes)
constexpr int WM = 64;             // wave tile: 64 (O) x 128 (I) = 2 x 4 MFMA tiles of 32 x 32
constexpr int NT = BN / 32;        // MFMA tiles per wave along I

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
  typedef float type;
  static ACTNN_DEV float widen(float v) { return v; }
};
template <> struct RawScalar<__half> {
  typedef uint16_t type;
  static ACTNN_DEV float widen(uint16_t v) { return half_bits_to_float(v); }
};
template <> struct RawScalar<bf16_t> {
  typedef uint16_t type;
  static ACTNN_DEV float widen(uint16_t v) { return bf16_bits_to_float(v); }
};

template <typename TG, typename TS, typename TO>
__global__ __launch_bounds__(kThreads, BN == 128 ? 2 : 1) void linear_gw_q2_kernel(
    const TG* __restrict__ gout, const uint8_t* __restrict__ packed, const TS* __restrict__ scale,
    const TS* __restrict__ mn, TO* __restrict__ gw, int M, int O, int I) {
  __shared__ __attribute__((aligned(16))) uint16_t sA[2][BK * kPitchA];
  __shared__ __attribute__((aligned(16))) uint16_t sB[2][BN * kPitchB];
  typedef typename RawScalar<TS>::type raw_t;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wm = (tid >> 6) * WM;            // wave's row offset inside the block tile
  const int G = I / 256;
  // Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.  Give every XCD whole
  // panels of grad_out rows (all column tiles of tile_m), so that a panel is pulled into one L2
  // only and reused there by the tiles_n blocks that need it.
  const int tiles_n = I / BN;
  const int tiles_m = (O + BM - 1) / BM;
  int tile = blockIdx.x;
  if (tiles_m % 8 == 0) {
    const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
    tile = (xcd * (tiles_m / 8) + idx / tiles_n) * tiles_n + idx % tiles_n;
  }
  const int o0 = (tile / tiles_n) * BM;
  const int i0 = (tile % tiles_n) * BN;
  const int g = i0 / 256;                    // the block's columns lie inside quantisation group g
  const int d0 = i0 % 256;                   // ... starting at feature d0 of the group

  // A staging: 4 vectors of 8 o's per thread: k rows ar + 8 * r, o offset (tid % 32) * 8
  // B staging: thread -> sample quad br = tid / 32 (4 consecutive k), features bi + 32 * e
  const int ar = tid >> 5;
  const int br = tid >> 5;
  const int bi = tid & 31;
  const bool ovalid = o0 + bi * 8 < O;       // O % 8 == 0: a vector is inside or outside as a whole
  // running pointers, advanced by one k-step per prefetch
  const TG* pa = gout + (int64_t)ar * O + o0 + bi * 8;
  const uint8_t* pb = packed + ((int64_t)br * G + g) * 256 + d0 + bi;
  const raw_t* psc = reinterpret_cast<const raw_t*>(scale) + (int64_t)(br * 4) * G + g;
  const raw_t* pmn = reinterpret_cast<const raw_t*>(mn) + (int64_t)(br * 4) * G + g;
  const int64_t a_step = (int64_t)BK * O, a_row8 = (int64_t)8 * O;
  const int64_t b_step = (int64_t)(BK / 4) * G * 256, s_step = (int64_t)BK * G;
  int k_next = 0;                            // first sample of the step the next prefetch loads

  f32x16 acc[2][NT];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < NT; ++b)
#pragma unroll
      for (int c = 0; c < 16; ++c) acc[a][b][c] = 0.0f;

  // Registers of the prefetch hold the data exactly as loaded: nothing may consume a load inside
  // `prefetch`, or the wave would wait out the memory latency there.
  u32x4 ra[4];
  uint32_t rb[NT];
  raw_t rsc[4], rmn[4];
  bool rvalid = false;

  auto prefetch = [&]() {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      ra[r] = (u32x4){0u, 0u, 0u, 0u};
      if (ovalid && k_next + ar + 8 * r < M) ra[r] = load16(pa + r * a_row8);
    }
    rvalid = k_next + br * 4 < M;            // M % 4 == 0: a quad is inside or outside as a whole
    if (rvalid) {
#pragma unroll
      for (int e = 0; e < NT; ++e) rb[e] = pb[32 * e];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        rsc[j] = psc[(int64_t)j * G];
        rmn[j] = pmn[(int64_t)j * G];
      }
    }
    pa += a_step;
    pb += b_step;
    psc += s_step;
    pmn += s_step;
    k_next += BK;
  };

  auto stage = [&](int buf) {
#pragma unroll
    for (int r = 0; r < 4; ++r)
      *reinterpret_cast<u32x4*>(&sA[buf][(ar + 8 * r) * kPitchA + bi * 8]) = ra[r];
    float inv[4], m4[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {            // rows past M dequantise to 0
      inv[j] = rvalid ? __builtin_amdgcn_rcpf(RawScalar<TS>::widen(rsc[j])) : 0.0f;
      m4[j] = rvalid ? RawScalar<TS>::widen(rmn[j]) : 0.0f;
    }
#pragma unroll
    for (int e = 0; e < NT; ++e) {
      const uint32_t by = rvalid ? rb[e] : 0u;
      const float x0 = fmaf((float)(by & 3u), inv[0], m4[0]);
      const float x1 = fmaf((float)((by >> 2) & 3u), inv[1], m4[1]);
      const float x2 = fmaf((float)((by >> 4) & 3u), inv[2], m4[2]);
      const float x3 = fmaf((float)((by >> 6) & 3u), inv[3], m4[3]);
      *reinterpret_cast<u32x2*>(&sB[buf][(bi + 32 * e) * kPitchB + br * 4]) =
          (u32x2){Mma<TG>::pack2(x0, x1), Mma<TG>::pack2(x2, x3)};
    }
  };

  const int steps = (M + BK - 1) / BK;
  prefetch();
  if (steps > 0) stage(0);
  __syncthreads();
  if (steps > 1) prefetch();

  for (int t = 0; t < steps; ++t) {
    const int cur = t & 1;
    // write the tile of step t+1 into the other buffer (its last readers passed the barrier at
    // the end of step t-1), then get the loads of step t+2 in flight, then multiply step t
    if (t + 1 < steps) stage(cur ^ 1);
    if (t + 2 < steps) prefetch();

    // all fragments of the step first (LDS reads return in order, so the MFMAs below can start
    // as soon as their operands are in), then the 2 x 2 x NT MFMAs
    u32x4 fa[BK / 16][2], fb[BK / 16][NT];
#pragma unroll
    for (int kb = 0; kb < BK / 16; ++kb) {
      const int kf = kb * 16 + (lane >> 5) * 8;      // this lane's first k in the step
#pragma unroll
      for (int b = 0; b < NT; ++b)
        fb[kb][b] = *reinterpret_cast<const u32x4*>(&sB[cur][(b * 32 + (lane & 31)) * kPitchB + kf]);
#pragma unroll
      for (int a = 0; a < 2; ++a) {
        const uint16_t* col = &sA[cur][kf * kPitchA + wm + a * 32 + (lane & 31)];
        uint32_t w[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
          w[j] = (uint32_t)col[(2 * j) * kPitchA] | ((uint32_t)col[(2 * j + 1) * kPitchA] << 16);
        fa[kb][a] = (u32x4){w[0], w[1], w[2], w[3]};
      }
    }
#pragma unroll
    for (int kb = 0; kb < BK / 16; ++kb)
#pragma unroll
      for (int b = 0; b < NT; ++b)
#pragma unroll
        for (int a = 0; a < 2; ++a) acc[a][b] = Mma<TG>::mfma(fa[kb][a], fb[kb][b], acc[a][b]);
    __syncthreads();
  }

  // 32x32 accumulator layout: register c of a lane is row 8*(c/4) + 4*(lane/32) + c%4, column lane%32
#pragma unroll
  for (int a = 0; a < 2; ++a) {
#pragma unroll
    for (int b = 0; b < NT; ++b) {
      const int col = i0 + b * 32 + (lane & 31);
#pragma unroll
      for (int c = 0; c < 16; ++c) {
        const int row = o0 + wm + a * 32 + 8 * (c >> 2) + 4 * (lane >> 5) + (c & 3);
        if (row < O) Conv<TO>::store(gw, (int64_t)row * I + col, acc[a][b][c]);
      }
    }
  }
}

template <typename TG, typename TS, typename TO>
int launch(const void* gout, const int8_t* packed, const void* scale, const void* mn, void* gw,
           int64_t M, int64_t O, int64_t I, hipStream_t s) {
  const int64_t blocks = ((O + BM - 1) / BM) * (I / BN);
  if (blocks > 0x7fffffffLL) return ACTNN_EINVAL;
  linear_gw_q2_kernel<TG, TS, TO><<<dim3((unsigned)blocks), dim3(kThreads), 0, s>>>(
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
  if (M > 0 && !aligned16(grad_out)) return ACTNN_EALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (go_dtype) {
    case ACTNN_F16: return launch_sm<__half>(sm_dtype, out_dtype, grad_out, packed, scale, mn, grad_w, M, O, I, s);
    case ACTNN_BF16: return launch_sm<bf16_t>(sm_dtype, out_dtype, grad_out, packed, scale, mn, grad_w, M, O, I, s);
    default: return ACTNN_EDTYPE;
  }
}
