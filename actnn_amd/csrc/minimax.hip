// Per-row min/max (replaces minimax_cuda_kernel.cu:23-89 of the reference).
//
// HBM-bound streaming read.  A row of D elements is reduced by 16, 32 or 64 lanes so that each
// load instruction of a block covers 4 KiB of consecutive memory (one 16-byte non-temporal
// load per lane; a 256-element fp32 row is exactly one wave-wide load).  Lanes are combined
// with DPP steps (quad_perm, row mirrors, row broadcasts).  Small blocks that each sweep a
// short contiguous run measured faster on MI355X than blocks with many loads in flight per lane;
// eight rows per lane group (32 KiB per block for fp32 rows of 256) measured best.
#include "device_utils.h"

namespace actnn {
namespace {

constexpr int kThreads = 256;
constexpr int kRowGroups = kThreads / 16;     // rows per block in the generic kernel

constexpr int kRowsPerLaneGroup = 8;          // rows per lane group and block (8 measured best)

template <typename T> struct Vec16;           // running min/max over one 16-byte vector of T
template <> struct Vec16<float> {
  static constexpr int kElems = 4;
  static ACTNN_DEV void minmax(const float* p, float& lo, float& hi) {
    const u32x4 u = load16_nt(p);
    const float a = as_float(u.x), b = as_float(u.y), c = as_float(u.z), d = as_float(u.w);
    lo = min3_f32(min3_f32(lo, a, b), c, d);
    hi = max3_f32(max3_f32(hi, a, b), c, d);
  }
};
template <> struct Vec16<__half> {
  static constexpr int kElems = 8;
  static ACTNN_DEV void minmax(const __half* p, float& lo, float& hi) {
    const u32x4 u = load16_nt(p);
    const uint32_t w[4] = {u.x, u.y, u.z, u.w};
    float v[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = half_bits_to_float(w[i] & 0xffffu);
      v[2 * i + 1] = half_bits_to_float(w[i] >> 16);
    }
    float l8, h8;
    minmax_of<8>(v, l8, h8);
    lo = min_f32(lo, l8);
    hi = max_f32(hi, h8);
  }
};
template <> struct Vec16<bf16_t> {
  static constexpr int kElems = 8;
  static ACTNN_DEV void minmax(const bf16_t* p, float& lo, float& hi) {
    const u32x4 u = load16_nt(p);
    const uint32_t w[4] = {u.x, u.y, u.z, u.w};
    float v[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = as_float(w[i] << 16);
      v[2 * i + 1] = as_float(w[i] & 0xffff0000u);
    }
    float l8, h8;
    minmax_of<8>(v, l8, h8);
    lo = min_f32(lo, l8);
    hi = max_f32(hi, h8);
  }
};

// Vector path: a row is D = LPR * kElems * V elements, read by LPR lanes (16, 32 or 64) with V
// 16-byte loads each, so that every load instruction of a lane group covers LPR * 16
// contiguous bytes and a block sweeps kThreads * 16 contiguous bytes per instruction.  The
// base pointer is 16-byte aligned.  V == 0 means "runtime count" (vecs_per_lane).
template <typename T, int LPR, int V>
__global__ __launch_bounds__(kThreads) void minimax_vec_kernel(const T* __restrict__ data,
                                                               T* __restrict__ mn,
                                                               T* __restrict__ mx, int64_t M,
                                                               int64_t D, int vecs_per_lane) {
  constexpr int E = Vec16<T>::kElems;
  constexpr int kSlots = kThreads / LPR;
  constexpr int R = kRowsPerLaneGroup;
  const int sub = threadIdx.x % LPR;
  const int slot = threadIdx.x / LPR;
  const int64_t row0 = (int64_t)blockIdx.x * (kSlots * R) + slot;
  float lo[R], hi[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    lo[r] = INFINITY;
    hi[r] = -INFINITY;
    const int64_t row = row0 + r * kSlots;
    if (row < M) {
      const T* p = data + row * D + sub * E;
      if (V > 0) {
#pragma unroll
        for (int i = 0; i < V; ++i) Vec16<T>::minmax(p + i * LPR * E, lo[r], hi[r]);
      } else {
        for (int i = 0; i < vecs_per_lane; ++i) Vec16<T>::minmax(p + (int64_t)i * LPR * E, lo[r], hi[r]);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    float l = lo[r], h = hi[r];
    lanes_minmax<LPR / 16>(l, h);
    const int64_t row = row0 + r * kSlots;
    if (sub == LPR - 1 && row < M) {      // the last lane of the group holds the combined result
      Conv<T>::store(mn, row, l);
      Conv<T>::store(mx, row, h);
    }
  }
}

// Generic path: any D, element-wise loads, one 16-lane group per row.
template <typename T>
__global__ __launch_bounds__(kThreads) void minimax_generic_kernel(const T* __restrict__ data,
                                                                   T* __restrict__ mn,
                                                                   T* __restrict__ mx, int64_t M,
                                                                   int64_t D) {
  const int sub = threadIdx.x & 15;
  const int64_t row = (int64_t)blockIdx.x * kRowGroups + (threadIdx.x >> 4);
  float lo = INFINITY, hi = -INFINITY;
  if (row < M) {
    const T* p = data + row * D;
    for (int64_t i = sub; i < D; i += 16) {
      const float v = Conv<T>::load(p, i);
      lo = min_f32(lo, v);
      hi = max_f32(hi, v);
    }
  }
  lanes_minmax<1>(lo, hi);
  if (sub == 0 && row < M) {
    Conv<T>::store(mn, row, lo);
    Conv<T>::store(mx, row, hi);
  }
}

template <typename T, int LPR>
int launch_vec(const T* d, T* lo, T* hi, int64_t M, int64_t D, int64_t vecs, hipStream_t s) {
  constexpr int kRows = (kThreads / LPR) * kRowsPerLaneGroup;
  const int64_t blocks = (M + kRows - 1) / kRows;
  if (blocks > 0x7fffffffLL || vecs > 0x7fffffffLL) return ACTNN_EINVAL;
  const dim3 grid((unsigned)blocks), blk(kThreads);
  if (vecs == 1) minimax_vec_kernel<T, LPR, 1><<<grid, blk, 0, s>>>(d, lo, hi, M, D, 1);
  else if (vecs == 2) minimax_vec_kernel<T, LPR, 2><<<grid, blk, 0, s>>>(d, lo, hi, M, D, 2);
  else minimax_vec_kernel<T, LPR, 0><<<grid, blk, 0, s>>>(d, lo, hi, M, D, (int)vecs);
  ACTNN_RETURN_LAUNCH_STATUS();
}

template <typename T>
int launch_minimax(const void* data, void* mn, void* mx, int64_t M, int64_t D, hipStream_t s) {
  constexpr int E = Vec16<T>::kElems;
  const T* d = static_cast<const T*>(data);
  T* lo = static_cast<T*>(mn);
  T* hi = static_cast<T*>(mx);
  if (D % (16 * E) == 0 && aligned16(data)) {
    const int64_t nvec = D / E;                       // 16-byte vectors per row, a multiple of 16
    if (nvec % 64 == 0) return launch_vec<T, 64>(d, lo, hi, M, D, nvec / 64, s);
    if (nvec % 32 == 0) return launch_vec<T, 32>(d, lo, hi, M, D, nvec / 32, s);
    return launch_vec<T, 16>(d, lo, hi, M, D, nvec / 16, s);
  }
  const int64_t blocks = (M + kRowGroups - 1) / kRowGroups;
  if (blocks > 0x7fffffffLL) return ACTNN_EINVAL;
  minimax_generic_kernel<T><<<dim3((unsigned)blocks), dim3(kThreads), 0, s>>>(d, lo, hi, M, D);
  ACTNN_RETURN_LAUNCH_STATUS();
}

// Per-sample sensitivity of the bit allocation: out[n] = factor * mult * sum_g (mx[n,g] - mn[n,g])^2
// (the difference rounded to T, as the tensor subtraction of qscheme.py:80 rounds it; the sum is
// kept in fp32 in a fixed order).  mult: nothing, one device scalar or one value per sample.
template <typename T>
__global__ __launch_bounds__(kThreads) void range_sqr_kernel(const T* __restrict__ mn,
                                                             const T* __restrict__ mx,
                                                             float* __restrict__ out, int64_t G,
                                                             float factor, const float* __restrict__ mult,
                                                             int mult_stride) {
  __shared__ float s_part[kThreads];
  const int64_t n = blockIdx.x;
  float acc = 0.0f;
  for (int64_t g = threadIdx.x; g < G; g += kThreads) {
    const float d = Conv<T>::round(Conv<T>::load(mx, n * G + g) - Conv<T>::load(mn, n * G + g));
    acc = fmaf(d, d, acc);
  }
  s_part[threadIdx.x] = acc;
  __syncthreads();
  for (int w = kThreads / 2; w > 0; w >>= 1) {
    if ((int)threadIdx.x < w) s_part[threadIdx.x] += s_part[threadIdx.x + w];
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    float v = s_part[0] * factor;
    if (mult) v *= mult[n * mult_stride];
    out[n] = v;
  }
}

// Squared L2 norm of every sample (the gradient statistic of the bit allocation, qscheme.py:47-55):
// part[n * B + b] = sum of squares over slice b of row n, fp32, in a fixed order; the caller adds
// the B slices.  Rows are read with 16-byte non-temporal loads; 16-bit types use the dot-product
// instructions (exact products, fp32 accumulation).
template <typename T> ACTNN_DEV float square_sum16(const T* p);
template <> ACTNN_DEV float square_sum16<float>(const float* p) {
  const u32x4 u = load16_nt(p);
  const float a = as_float(u.x), b = as_float(u.y), c = as_float(u.z), d = as_float(u.w);
  return fmaf(a, a, fmaf(b, b, fmaf(c, c, d * d)));
}
typedef _Float16 f16x2_mm __attribute__((ext_vector_type(2)));
template <> ACTNN_DEV float square_sum16<__half>(const __half* p) {
  const u32x4 u = load16_nt(p);
  float q = 0.0f;
  const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
  for (int i = 0; i < 4; ++i)
    q = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_mm, w[i]), __builtin_bit_cast(f16x2_mm, w[i]), q, false);
  return q;
}
template <> ACTNN_DEV float square_sum16<bf16_t>(const bf16_t* p) {
  const u32x4 u = load16_nt(p);
  float q = 0.0f;
  const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
  for (int i = 0; i < 4; ++i)
    q = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, w[i]), __builtin_bit_cast(bf16x2_t, w[i]), q, false);
  return q;
}

template <typename T>
__global__ __launch_bounds__(kThreads) void sample_sqnorm_kernel(const T* __restrict__ x, float* __restrict__ part,
                                                                int64_t F, int64_t slice) {
  constexpr int E = Vec16<T>::kElems;
  __shared__ float s_part[kThreads];
  const int64_t n = blockIdx.y;
  const int64_t lo = (int64_t)blockIdx.x * slice;
  const int64_t hi = lo + slice < F ? lo + slice : F;
  const T* row = x + n * F;
  float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  int64_t i = lo + (int64_t)threadIdx.x * E;
  for (; i + 3 * (int64_t)kThreads * E < hi; i += 4 * (int64_t)kThreads * E) {
#pragma unroll
    for (int u = 0; u < 4; ++u) acc[u] += square_sum16<T>(row + i + (int64_t)u * kThreads * E);
  }
  for (; i < hi; i += (int64_t)kThreads * E) acc[0] += square_sum16<T>(row + i);
  s_part[threadIdx.x] = (acc[0] + acc[1]) + (acc[2] + acc[3]);
  __syncthreads();
  for (int w = kThreads / 2; w > 0; w >>= 1) {
    if ((int)threadIdx.x < w) s_part[threadIdx.x] += s_part[threadIdx.x + w];
    __syncthreads();
  }
  if (threadIdx.x == 0) part[n * gridDim.x + blockIdx.x] = s_part[0];
}

}  // namespace
}  // namespace actnn

extern "C" int actnn_range_sqr(const void* mn, const void* mx, float* out, int64_t N, int64_t G,
                               float factor, const float* mult, int mult_per_sample, int dtype,
                               void* stream) {
  using namespace actnn;
  if (N < 0 || G < 0 || N > 0x7fffffffLL) return ACTNN_EINVAL;
  if (N == 0) return ACTNN_OK;
  if (!out || (G > 0 && (!mn || !mx))) return ACTNN_EINVAL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)N), blk(kThreads);
  const int stride = mult_per_sample ? 1 : 0;
  switch (dtype) {
    case ACTNN_F32:
      range_sqr_kernel<float><<<grid, blk, 0, s>>>(static_cast<const float*>(mn), static_cast<const float*>(mx),
                                                   out, G, factor, mult, stride);
      break;
    case ACTNN_F16:
      range_sqr_kernel<__half><<<grid, blk, 0, s>>>(static_cast<const __half*>(mn), static_cast<const __half*>(mx),
                                                    out, G, factor, mult, stride);
      break;
    case ACTNN_BF16:
      range_sqr_kernel<bf16_t><<<grid, blk, 0, s>>>(static_cast<const bf16_t*>(mn), static_cast<const bf16_t*>(mx),
                                                    out, G, factor, mult, stride);
      break;
    default: return ACTNN_EDTYPE;
  }
  ACTNN_RETURN_LAUNCH_STATUS();
}

extern "C" int actnn_minimax(const void* data, void* mn, void* mx, int64_t M, int64_t D, int dtype,
                             void* stream) {
  using namespace actnn;
  if (M < 0 || D < 1) return ACTNN_EINVAL;
  if (M == 0) return ACTNN_OK;
  if (!data || !mn || !mx) return ACTNN_EINVAL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case ACTNN_F32: return launch_minimax<float>(data, mn, mx, M, D, s);
    case ACTNN_F16: return launch_minimax<__half>(data, mn, mx, M, D, s);
    case ACTNN_BF16: return launch_minimax<bf16_t>(data, mn, mx, M, D, s);
    default: return ACTNN_EDTYPE;
  }
}

extern "C" int actnn_sample_sqnorm(const void* x, float* part, int64_t N, int64_t F, int slices, int dtype,
                                   void* stream) {
  using namespace actnn;
  if (N < 0 || F < 0 || slices < 1 || slices > 65535 || N > 65535) return ACTNN_EINVAL;
  if (N == 0) return ACTNN_OK;
  if (!x || !part) return ACTNN_EINVAL;
  const int elems = dtype == ACTNN_F32 ? 4 : 8;
  if (F % elems != 0) return ACTNN_EINVAL;
  if (!aligned16(x)) return ACTNN_EALIGN;
  int64_t slice = (F + slices - 1) / slices;
  slice = (slice + elems - 1) / elems * elems;                 // whole 16-byte vectors
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)slices, (unsigned)N), blk(kThreads);
  switch (dtype) {
    case ACTNN_F32: sample_sqnorm_kernel<float><<<grid, blk, 0, s>>>(static_cast<const float*>(x), part, F, slice); break;
    case ACTNN_F16: sample_sqnorm_kernel<__half><<<grid, blk, 0, s>>>(static_cast<const __half*>(x), part, F, slice); break;
    case ACTNN_BF16: sample_sqnorm_kernel<bf16_t><<<grid, blk, 0, s>>>(static_cast<const bf16_t*>(x), part, F, slice); break;
    default: return ACTNN_EDTYPE;
  }
  ACTNN_RETURN_LAUNCH_STATUS();
}
