// ReLU and Dropout with 1-bit masks (replaces quantization_cuda_kernel.cu:411-627).
//
// Mask layout (kept from the reference): elements are cut into blocks of 512; element
// t = 16*j + k of a block is bit j of the block's word k (16 int32 words per block).  Lane j
// of a 32-lane half-wave therefore owns 16 contiguous elements; two blocks fill a 32-bit
// register per lane and one 32x32 bit transpose leaves the 32 mask words of the two blocks in
// lanes 0..31, stored as one contiguous 128-byte run.  A 256-thread block covers 16 mask
// blocks (8192 elements).
#include "device_utils.h"

namespace actnn {
namespace {

constexpr int kThreads = 256;
constexpr int kMaskBlock = 512;
constexpr int kMaskBlocksPerBlock = (kThreads / 32) * 2;   // 16

enum class Op { kRelu, kDropout };

// Forward.  OP selects the keep rule: x > 0 (ReLU) or Philox r16 >= threshold (Dropout).
template <typename T, Op OP>
__global__ __launch_bounds__(kThreads) void mask_forward_kernel(const T* __restrict__ x,
                                                                T* __restrict__ y,
                                                                int32_t* __restrict__ mask, int64_t n,
                                                                int64_t n_mask_blocks, uint32_t thr,
                                                                float keep_div, uint64_t seed,
                                                                uint64_t offset, int64_t elem_offset,
                                                                const T* __restrict__ add = nullptr) {
  const uint32_t lane = threadIdx.x & 31;
  const int64_t mb0 = (int64_t)blockIdx.x * kMaskBlocksPerBlock + (threadIdx.x >> 5) * 2;
  uint32_t acc = 0;
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    const int64_t e0 = (mb0 + r) * kMaskBlock + lane * 16;
    if (e0 >= n) continue;
    float v[16];
    const bool full = e0 + 16 <= n;
    if (full) {
      load8(x + e0, reinterpret_cast<float(&)[8]>(v[0]));
      load8(x + e0 + 8, reinterpret_cast<float(&)[8]>(v[8]));
    } else {
#pragma unroll
      for (int k = 0; k < 16; ++k) v[k] = e0 + k < n ? Conv<T>::load(x, e0 + k) : 0.0f;
    }
    if (add) {                                       // the sum as a tensor addition rounds it, then the rule
      float a[16];
      if (full) {
        load8(add + e0, reinterpret_cast<float(&)[8]>(a[0]));
        load8(add + e0 + 8, reinterpret_cast<float(&)[8]>(a[8]));
      } else {
#pragma unroll
        for (int k = 0; k < 16; ++k) a[k] = e0 + k < n ? Conv<T>::load(add, e0 + k) : 0.0f;
      }
#pragma unroll
      for (int k = 0; k < 16; ++k) v[k] = Conv<T>::round(v[k] + a[k]);
    }
    uint32_t bitsr = 0;
    if (OP == Op::kRelu) {
#pragma unroll
      for (int k = 0; k < 16; ++k) {
        const bool keep = v[k] > 0.0f;
        v[k] = keep ? v[k] : 0.0f;
        bitsr |= (uint32_t)keep << k;
      }
    } else {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        uint32_t r16[8];
        philox_octet((uint64_t)((elem_offset + e0) >> 3) + h, seed, offset, r16);
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          const bool keep = r16[k] >= thr && e0 + h * 8 + k < n;
          v[h * 8 + k] = keep ? v[h * 8 + k] / keep_div : 0.0f;
          bitsr |= (uint32_t)keep << (h * 8 + k);
        }
      }
    }
    acc |= bitsr << (16 * r);
    if (full) {
      store8(y + e0, reinterpret_cast<const float(&)[8]>(v[0]));
      store8(y + e0 + 8, reinterpret_cast<const float(&)[8]>(v[8]));
    } else {
#pragma unroll
      for (int k = 0; k < 16; ++k)
        if (e0 + k < n) Conv<T>::store(y, e0 + k, v[k]);
    }
  }
  const uint32_t w = transpose32(acc, lane);       // lane p: word p % 16 of mask block mb0 + p / 16
  if (mb0 + (lane >> 4) < n_mask_blocks) mask[mb0 * 16 + lane] = (int32_t)w;
}

template <typename T>
__global__ __launch_bounds__(kThreads) void mask_backward_kernel(const T* __restrict__ gout,
                                                                 const int32_t* __restrict__ mask,
                                                                 T* __restrict__ gin, int64_t n,
                                                                 int64_t n_mask_blocks, float keep_div,
                                                                 bool divide, const T* __restrict__ acc = nullptr) {
  const uint32_t lane = threadIdx.x & 31;
  const int64_t mb0 = (int64_t)blockIdx.x * kMaskBlocksPerBlock + (threadIdx.x >> 5) * 2;
  uint32_t w = 0;
  if (mb0 + (lane >> 4) < n_mask_blocks) w = (uint32_t)mask[mb0 * 16 + lane];
  const uint32_t rows = transpose32(w, lane);       // bits 16*r + k: keep flag of element 16*lane + k of block r
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    const int64_t e0 = (mb0 + r) * kMaskBlock + lane * 16;
    if (e0 >= n) continue;
    float v[16];
    const bool full = e0 + 16 <= n;
    if (full) {
      load8(gout + e0, reinterpret_cast<float(&)[8]>(v[0]));
      load8(gout + e0 + 8, reinterpret_cast<float(&)[8]>(v[8]));
    } else {
#pragma unroll
      for (int k = 0; k < 16; ++k) v[k] = e0 + k < n ? Conv<T>::load(gout, e0 + k) : 0.0f;
    }
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const bool keep = (rows >> (16 * r + k)) & 1u;
      v[k] = keep ? (divide ? v[k] / keep_div : v[k]) : 0.0f;
    }
    if (acc) {                                       // the masked gradient added to another, as a tensor addition adds them
      float a[16];
      if (full) {
        load8(acc + e0, reinterpret_cast<float(&)[8]>(a[0]));
        load8(acc + e0 + 8, reinterpret_cast<float(&)[8]>(a[8]));
      } else {
#pragma unroll
        for (int k = 0; k < 16; ++k) a[k] = e0 + k < n ? Conv<T>::load(acc, e0 + k) : 0.0f;
      }
#pragma unroll
      for (int k = 0; k < 16; ++k) v[k] = a[k] + v[k];
    }
    if (full) {
      store8(gin + e0, reinterpret_cast<const float(&)[8]>(v[0]));
      store8(gin + e0 + 8, reinterpret_cast<const float(&)[8]>(v[8]));
    } else {
#pragma unroll
      for (int k = 0; k < 16; ++k)
        if (e0 + k < n) Conv<T>::store(gin, e0 + k, v[k]);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// 16-bit element types: whole-line streaming variant.  A wave handles 4 mask blocks (2048
// elements) with four wave-wide 16-byte non-temporal loads and stores, so that HBM sees only whole
// cache lines.  Lane l then holds elements 8l..8l+7 of each block, i.e. half of the 16 elements a
// mask row belongs to: lane pairs swap their 8-bit halves (one DPP move) so that the even lanes
// hold the rows of blocks A|B and the odd lanes those of C|D, two interleaved 32x32 bit
// transposes turn rows into mask words, and the 64 words leave as one 256-byte store.
constexpr int kTileElems = 4 * kMaskBlock;        // elements per wave and iteration
constexpr int kTilesPerBlock = kThreads / 64;

// MINMAX: also write the minimum and maximum of every group of 256 consecutive outputs (the lower
// and upper 32 lanes of each load own one group each) - what actnn_minimax returns for the output
// viewed as rows of 256, for a consumer that quantises it next.
// ADD: the rule is applied to x + add, rounded to T as the tensor addition it replaces rounds it
// (the closing `relu(out + identity)` of a residual block in one pass over the two operands).
template <typename T, Op OP, bool MINMAX = false, bool ADD = false>
__global__ __launch_bounds__(kThreads) void mask_forward16_kernel(const T* __restrict__ x, T* __restrict__ y,
                                                                  int32_t* __restrict__ mask, int64_t tiles,
                                                                  uint32_t thr, float keep_div,
                                                                  uint64_t seed, uint64_t offset,
                                                                  T* __restrict__ mn = nullptr,
                                                                  T* __restrict__ mx = nullptr,
                                                                  const T* __restrict__ add = nullptr) {
  const uint32_t lane = threadIdx.x & 63;
  const int64_t tile = (int64_t)blockIdx.x * kTilesPerBlock + (threadIdx.x >> 6);
  if (tile >= tiles) return;                       // whole waves leave together
  const int64_t e0 = tile * kTileElems + lane * 8;
  float v[4][8];
#pragma unroll
  for (int i = 0; i < 4; ++i) load8_nt(x + e0 + i * kMaskBlock, v[i]);
  if (ADD) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float a[8];
      load8_nt(add + e0 + i * kMaskBlock, a);
#pragma unroll
      for (int k = 0; k < 8; k += 2) {
        v[i][k] += a[k];
        v[i][k + 1] += a[k + 1];
        round_pair<T>(v[i][k], v[i][k + 1]);
      }
    }
  }
  uint32_t m[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    uint32_t r16[8];
    if (OP == Op::kDropout) philox_octet((uint64_t)((e0 + i * kMaskBlock) >> 3), seed, offset, r16);
    m[i] = 0;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const bool keep = OP == Op::kRelu ? v[i][k] > 0.0f : r16[k] >= thr;
      v[i][k] = keep ? (OP == Op::kRelu ? v[i][k] : v[i][k] / keep_div) : 0.0f;
      m[i] |= (uint32_t)keep << k;
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) store8_nt(y + e0 + i * kMaskBlock, v[i]);
  if (MINMAX) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float lo, hi;
      minmax_of<8>(v[i], lo, hi);
      lanes_minmax<2>(lo, hi);
      if ((lane & 31u) == 31u) {
        const int64_t g = tile * (kTileElems / 256) + i * (kMaskBlock / 256) + (lane >> 5);
        Conv<T>::store(mn, g, lo);
        Conv<T>::store(mx, g, hi);
      }
    }
  }
  const uint32_t w = rows_to_word(m, lane);
  // lane 2p+h holds word p % 16 of block 2h + p / 16
  mask[tile * 64 + (lane & 1u) * 32 + (lane >> 1)] = (int32_t)w;
}

// ACC: gin = acc + masked gradient (rounded to T as the tensor addition of the two rounds it): the
// gradient that arrives at a residual block's input over the skip connection, masked and added to the
// one from the block's first convolution in one pass.
template <typename T, bool ACC = false>
__global__ __launch_bounds__(kThreads) void mask_backward16_kernel(const T* __restrict__ gout,
                                                                   const int32_t* __restrict__ mask,
                                                                   T* __restrict__ gin, int64_t tiles,
                                                                   float keep_div, bool divide,
                                                                   const T* __restrict__ acc = nullptr) {
  const uint32_t lane = threadIdx.x & 63;
  const int64_t tile = (int64_t)blockIdx.x * kTilesPerBlock + (threadIdx.x >> 6);
  if (tile >= tiles) return;
  const int64_t e0 = tile * kTileElems + lane * 8;
  float v[4][8];
#pragma unroll
  for (int i = 0; i < 4; ++i) load8_nt(gout + e0 + i * kMaskBlock, v[i]);
  uint32_t m[4];
  word_to_rows((uint32_t)mask[tile * 64 + (lane & 1u) * 32 + (lane >> 1)], lane, m);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const bool keep = (m[i] >> k) & 1u;
      v[i][k] = keep ? (divide ? v[i][k] / keep_div : v[i][k]) : 0.0f;
    }
    if (ACC) {
      float a[8];
      load8_nt(acc + e0 + i * kMaskBlock, a);
#pragma unroll
      for (int k = 0; k < 8; ++k) v[i][k] = a[k] + v[i][k];
    }
    store8_nt(gin + e0 + i * kMaskBlock, v[i]);
  }
}

template <typename T, Op OP>
int launch_forward(const void* x, void* y, int32_t* mask, int64_t n, uint32_t thr, float keep_div,
                   uint64_t seed, uint64_t offset, hipStream_t s, const void* add = nullptr) {
  const T* xi = static_cast<const T*>(x);
  const T* ai = static_cast<const T*>(add);
  T* yo = static_cast<T*>(y);
  int64_t done = 0;                               // elements handled by the whole-line kernel
  if (sizeof(T) == 2) {
    const int64_t tiles = n / kTileElems;
    const int64_t tblocks = (tiles + kTilesPerBlock - 1) / kTilesPerBlock;
    if (tblocks > 0x7fffffffLL) return ACTNN_EINVAL;
    if (tiles > 0) {
      if (ai)
        mask_forward16_kernel<T, OP, false, true><<<dim3((unsigned)tblocks), dim3(kThreads), 0, s>>>(
            xi, yo, mask, tiles, thr, keep_div, seed, offset, nullptr, nullptr, ai);
      else
        mask_forward16_kernel<T, OP><<<dim3((unsigned)tblocks), dim3(kThreads), 0, s>>>(
            xi, yo, mask, tiles, thr, keep_div, seed, offset);
    }
    done = tiles * kTileElems;
  }
  const int64_t rest = n - done;
  if (rest > 0) {
    const int64_t nmb = (rest + kMaskBlock - 1) / kMaskBlock;
    const int64_t blocks = (nmb + kMaskBlocksPerBlock - 1) / kMaskBlocksPerBlock;
    if (blocks > 0x7fffffffLL) return ACTNN_EINVAL;
    mask_forward_kernel<T, OP><<<dim3((unsigned)blocks), dim3(kThreads), 0, s>>>(
        xi + done, yo + done, mask + done / 32, rest, nmb, thr, keep_div, seed, offset, done,
        ai ? ai + done : nullptr);
  }
  ACTNN_RETURN_LAUNCH_STATUS();
}

template <typename T>
int launch_backward(const void* gout, const int32_t* mask, void* gin, int64_t n, float keep_div,
                    bool divide, hipStream_t s, const void* acc = nullptr) {
  const T* go = static_cast<const T*>(gout);
  const T* ac = static_cast<const T*>(acc);
  T* gi = static_cast<T*>(gin);
  int64_t done = 0;
  if (sizeof(T) == 2) {
    const int64_t tiles = n / kTileElems;
    const int64_t tblocks = (tiles + kTilesPerBlock - 1) / kTilesPerBlock;
    if (tblocks > 0x7fffffffLL) return ACTNN_EINVAL;
    if (tiles > 0) {
      if (ac)
        mask_backward16_kernel<T, true><<<dim3((unsigned)tblocks), dim3(kThreads), 0, s>>>(go, mask, gi, tiles,
                                                                                           keep_div, divide, ac);
      else
        mask_backward16_kernel<T><<<dim3((unsigned)tblocks), dim3(kThreads), 0, s>>>(go, mask, gi, tiles,
                                                                                     keep_div, divide);
    }
    done = tiles * kTileElems;
  }
  const int64_t rest = n - done;
  if (rest > 0) {
    const int64_t nmb = (rest + kMaskBlock - 1) / kMaskBlock;
    const int64_t blocks = (nmb + kMaskBlocksPerBlock - 1) / kMaskBlocksPerBlock;
    if (blocks > 0x7fffffffLL) return ACTNN_EINVAL;
    mask_backward_kernel<T><<<dim3((unsigned)blocks), dim3(kThreads), 0, s>>>(
        go + done, mask + done / 32, gi + done, rest, nmb, keep_div, divide, ac ? ac + done : nullptr);
  }
  ACTNN_RETURN_LAUNCH_STATUS();
}

template <Op OP>
int dispatch_forward(const void* x, void* y, int32_t* mask, int64_t n, uint32_t thr, float keep_div,
                     uint64_t seed, uint64_t offset, int dtype, void* stream, const void* add = nullptr) {
  if (n < 0) return ACTNN_EINVAL;
  if (n == 0) return ACTNN_OK;
  if (!x || !y || !mask) return ACTNN_EINVAL;
  if (!aligned16(x) || !aligned16(y) || !aligned16(add)) return ACTNN_EALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case ACTNN_F32: return launch_forward<float, OP>(x, y, mask, n, thr, keep_div, seed, offset, s, add);
    case ACTNN_F16: return launch_forward<__half, OP>(x, y, mask, n, thr, keep_div, seed, offset, s, add);
    case ACTNN_BF16: return launch_forward<bf16_t, OP>(x, y, mask, n, thr, keep_div, seed, offset, s, add);
    default: return ACTNN_EDTYPE;
  }
}

int dispatch_backward(const void* gout, const int32_t* mask, void* gin, int64_t n, float keep_div,
                      bool divide, int dtype, void* stream, const void* acc = nullptr) {
  if (n < 0) return ACTNN_EINVAL;
  if (n == 0) return ACTNN_OK;
  if (!gout || !gin || !mask) return ACTNN_EINVAL;
  if (!aligned16(gout) || !aligned16(gin) || !aligned16(acc)) return ACTNN_EALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case ACTNN_F32: return launch_backward<float>(gout, mask, gin, n, keep_div, divide, s, acc);
    case ACTNN_F16: return launch_backward<__half>(gout, mask, gin, n, keep_div, divide, s, acc);
    case ACTNN_BF16: return launch_backward<bf16_t>(gout, mask, gin, n, keep_div, divide, s, acc);
    default: return ACTNN_EDTYPE;
  }
}

// keep iff r16 >= thr, r16 uniform on [0, 2^16): P(keep) = 1 - thr / 2^16 ~ 1 - p.
inline uint32_t dropout_threshold(float p) {
  double t = (double)p * 65536.0;
  t = t < 0.0 ? 0.0 : (t > 65536.0 ? 65536.0 : t);
  return (uint32_t)(t + 0.5);
}

}  // namespace
}  // namespace actnn

extern "C" int actnn_relu_forward(const void* x, void* y, int32_t* mask, int64_t n, int dtype,
                                  void* stream) {
  return actnn::dispatch_forward<actnn::Op::kRelu>(x, y, mask, n, 0u, 1.0f, 0, 0, dtype, stream);
}

extern "C" int actnn_relu_forward_minmax(const void* x, void* y, int32_t* mask, void* mn, void* mx,
                                         int64_t n, int dtype, void* stream) {
  using namespace actnn;
  if (n < 0 || n % kTileElems != 0) return ACTNN_EINVAL;       // whole tiles of 2048 elements only
  if (dtype != ACTNN_F16 && dtype != ACTNN_BF16) return ACTNN_EDTYPE;
  if (n == 0) return ACTNN_OK;
  if (!x || !y || !mask || !mn || !mx) return ACTNN_EINVAL;
  if (!aligned16(x) || !aligned16(y)) return ACTNN_EALIGN;
  const int64_t tiles = n / kTileElems;
  const int64_t blocks = (tiles + kTilesPerBlock - 1) / kTilesPerBlock;
  if (blocks > 0x7fffffffLL) return ACTNN_EINVAL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)blocks), blk(kThreads);
  if (dtype == ACTNN_F16)
    mask_forward16_kernel<__half, Op::kRelu, true><<<grid, blk, 0, s>>>(
        static_cast<const __half*>(x), static_cast<__half*>(y), mask, tiles, 0u, 1.0f, 0, 0,
        static_cast<__half*>(mn), static_cast<__half*>(mx));
  else
    mask_forward16_kernel<bf16_t, Op::kRelu, true><<<grid, blk, 0, s>>>(
        static_cast<const bf16_t*>(x), static_cast<bf16_t*>(y), mask, tiles, 0u, 1.0f, 0, 0,
        static_cast<bf16_t*>(mn), static_cast<bf16_t*>(mx));
  ACTNN_RETURN_LAUNCH_STATUS();
}

extern "C" int actnn_relu_add_forward(const void* x, const void* residual, void* y, int32_t* mask, void* mn,
                                      void* mx, int64_t n, int dtype, void* stream) {
  using namespace actnn;
  if ((mn == nullptr) != (mx == nullptr)) return ACTNN_EINVAL;
  if (n > 0 && !residual) return ACTNN_EINVAL;
  if (!mn) return dispatch_forward<Op::kRelu>(x, y, mask, n, 0u, 1.0f, 0, 0, dtype, stream, residual);
  if (n < 0 || n % kTileElems != 0) return ACTNN_EINVAL;       // whole tiles of 2048 elements only
  if (dtype != ACTNN_F16 && dtype != ACTNN_BF16) return ACTNN_EDTYPE;
  if (n == 0) return ACTNN_OK;
  if (!x || !y || !mask) return ACTNN_EINVAL;
  if (!aligned16(x) || !aligned16(residual) || !aligned16(y)) return ACTNN_EALIGN;
  const int64_t tiles = n / kTileElems;
  const int64_t blocks = (tiles + kTilesPerBlock - 1) / kTilesPerBlock;
  if (blocks > 0x7fffffffLL) return ACTNN_EINVAL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)blocks), blk(kThreads);
  if (dtype == ACTNN_F16)
    mask_forward16_kernel<__half, Op::kRelu, true, true><<<grid, blk, 0, s>>>(
        static_cast<const __half*>(x), static_cast<__half*>(y), mask, tiles, 0u, 1.0f, 0, 0,
        static_cast<__half*>(mn), static_cast<__half*>(mx), static_cast<const __half*>(residual));
  else
    mask_forward16_kernel<bf16_t, Op::kRelu, true, true><<<grid, blk, 0, s>>>(
        static_cast<const bf16_t*>(x), static_cast<bf16_t*>(y), mask, tiles, 0u, 1.0f, 0, 0,
        static_cast<bf16_t*>(mn), static_cast<bf16_t*>(mx), static_cast<const bf16_t*>(residual));
  ACTNN_RETURN_LAUNCH_STATUS();
}

extern "C" int actnn_relu_backward(const void* grad_out, const int32_t* mask, void* grad_in,
                                   int64_t n, int dtype, void* stream) {
  return actnn::dispatch_backward(grad_out, mask, grad_in, n, 1.0f, false, dtype, stream);
}

extern "C" int actnn_relu_backward_add(const void* grad_out, const int32_t* mask, const void* other,
                                       void* grad_in, int64_t n, int dtype, void* stream) {
  if (n > 0 && !other) return ACTNN_EINVAL;
  return actnn::dispatch_backward(grad_out, mask, grad_in, n, 1.0f, false, dtype, stream, other);
}

extern "C" int actnn_dropout_forward(const void* x, void* y, int32_t* mask, int64_t n, float p,
                                     uint64_t seed, uint64_t offset, int dtype, void* stream) {
  if (!(p >= 0.0f && p <= 1.0f)) return ACTNN_EINVAL;
  const float keep_div = (float)(1.0 - (double)p);     // x / (1.0 - p), .cu:540
  return actnn::dispatch_forward<actnn::Op::kDropout>(x, y, mask, n, actnn::dropout_threshold(p),
                                                      keep_div, seed, offset, dtype, stream);
}

extern "C" int actnn_dropout_backward(const void* grad_out, const int32_t* mask, void* grad_in,
                                      int64_t n, float p, int dtype, void* stream) {
  if (!(p >= 0.0f && p <= 1.0f)) return ACTNN_EINVAL;
  const float keep_div = (float)(1.0 - (double)p);     // .cu:601
  return actnn::dispatch_backward(grad_out, mask, grad_in, n, keep_div, true, dtype, stream);
}
