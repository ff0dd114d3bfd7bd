// Per-row min/max (replaces minimax_cuda_kernel.cu:23-89 of the reference).
//
// HBM-bound streaming read.  A row is reduced by one DPP row (16 lanes): every lane issues
// independent 16-byte loads (each load instruction of the wave covers four 256-byte
// contiguous segments), keeps running min/max in registers and the 16 lanes are combined
// with four DPP steps.  A 256-thread block owns kRowsPerGroup rows per 16-lane group so
// that many loads are in flight per lane.
#include "device_utils.h"

namespace actnn {
namespace {

constexpr int kThreads = 256;
constexpr int kRowGroups = kThreads / 16;     // 16-lane groups per block
constexpr int kRowsPerGroup = 4;              // rows reduced by one 16-lane group
constexpr int kRowsPerBlock = kRowGroups * kRowsPerGroup;

template <typename T> struct Vec16;           // 16-byte vector of T as floats
template <> struct Vec16<float> {
  static constexpr int kElems = 4;
  static ACTNN_DEV void minmax(const float* p, float& lo, float& hi) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    lo = fminf(fminf(lo, v.x), fminf(v.y, fminf(v.z, v.w)));
    hi = fmaxf(fmaxf(hi, v.x), fmaxf(v.y, fmaxf(v.z, v.w)));
  }
};
template <> struct Vec16<__half> {
  static constexpr int kElems = 8;
  static ACTNN_DEV void minmax(const __half* p, float& lo, float& hi) {
    float v[8];
    load8(p, v);
#pragma unroll
    for (int i = 0; i < 8; ++i) { lo = fminf(lo, v[i]); hi = fmaxf(hi, v[i]); }
  }
};
template <> struct Vec16<bf16_t> {
  static constexpr int kElems = 8;
  static ACTNN_DEV void minmax(const bf16_t* p, float& lo, float& hi) {
    float v[8];
    load8(p, v);
#pragma unroll
    for (int i = 0; i < 8; ++i) { lo = fminf(lo, v[i]); hi = fmaxf(hi, v[i]); }
  }
};

// Fast path: D * sizeof(T) is a multiple of 16 bytes and the base pointer is 16-byte aligned.
template <typename T, int kVecPerLane>   // kVecPerLane > 0: D == 16 * kVecPerLane * kElems exactly
__global__ __launch_bounds__(kThreads) void minimax_vec_kernel(const T* __restrict__ data,
                                                               T* __restrict__ mn,
                                                               T* __restrict__ mx, int64_t M,
                                                               int64_t D) {
  constexpr int E = Vec16<T>::kElems;
  const int sub = threadIdx.x & 15;
  const int grp = threadIdx.x >> 4;
  const int64_t row0 = (int64_t)blockIdx.x * kRowsPerBlock + (int64_t)grp * kRowsPerGroup;
  float lo[kRowsPerGroup], hi[kRowsPerGroup];
#pragma unroll
  for (int r = 0; r < kRowsPerGroup; ++r) { lo[r] = INFINITY; hi[r] = -INFINITY; }

  if (kVecPerLane > 0) {
#pragma unroll
    for (int r = 0; r < kRowsPerGroup; ++r) {
      const int64_t row = row0 + r;
      if (row < M) {
        const T* p = data + row * D + sub * E;
#pragma unroll
        for (int i = 0; i < kVecPerLane; ++i) Vec16<T>::minmax(p + i * 16 * E, lo[r], hi[r]);
      }
    }
  } else {
    const int64_t nvec = D / E;
#pragma unroll
    for (int r = 0; r < kRowsPerGroup; ++r) {
      const int64_t row = row0 + r;
      if (row < M) {
        const T* p = data + row * D;
        for (int64_t v = sub; v < nvec; v += 16) Vec16<T>::minmax(p + v * E, lo[r], hi[r]);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < kRowsPerGroup; ++r) {
    lo[r] = row16_min(lo[r]);
    hi[r] = row16_max(hi[r]);
  }
  // lane r of the group writes row r: four adjacent outputs per group.
  float wlo = lo[0], whi = hi[0];
#pragma unroll
  for (int r = 1; r < kRowsPerGroup; ++r) {
    if (sub == r) { wlo = lo[r]; whi = hi[r]; }
  }
  const int64_t row = row0 + sub;
  if (sub < kRowsPerGroup && row < M) {
    Conv<T>::store(mn, row, wlo);
    Conv<T>::store(mx, row, whi);
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
      lo = fminf(lo, v);
      hi = fmaxf(hi, v);
    }
  }
  lo = row16_min(lo);
  hi = row16_max(hi);
  if (sub == 0 && row < M) {
    Conv<T>::store(mn, row, lo);
    Conv<T>::store(mx, row, hi);
  }
}

template <typename T>
int launch_minimax(const void* data, void* mn, void* mx, int64_t M, int64_t D, hipStream_t s) {
  constexpr int E = Vec16<T>::kElems;
  const T* d = static_cast<const T*>(data);
  T* lo = static_cast<T*>(mn);
  T* hi = static_cast<T*>(mx);
  if (D % E == 0 && aligned16(data)) {
    const int64_t blocks = (M + kRowsPerBlock - 1) / kRowsPerBlock;
    if (blocks > 0x7fffffffLL) return ACTNN_EINVAL;
    const int64_t vec_per_lane = (D % (16 * E) == 0) ? D / (16 * E) : 0;
    if (vec_per_lane == 4)
      minimax_vec_kernel<T, 4><<<dim3((unsigned)blocks), dim3(kThreads), 0, s>>>(d, lo, hi, M, D);
    else if (vec_per_lane == 2)
      minimax_vec_kernel<T, 2><<<dim3((unsigned)blocks), dim3(kThreads), 0, s>>>(d, lo, hi, M, D);
    else
      minimax_vec_kernel<T, 0><<<dim3((unsigned)blocks), dim3(kThreads), 0, s>>>(d, lo, hi, M, D);
  } else {
    const int64_t blocks = (M + kRowGroups - 1) / kRowGroups;
    if (blocks > 0x7fffffffLL) return ACTNN_EINVAL;
    minimax_generic_kernel<T><<<dim3((unsigned)blocks), dim3(kThreads), 0, s>>>(d, lo, hi, M, D);
  }
  ACTNN_RETURN_LAUNCH_STATUS();
}

}  // namespace
}  // namespace actnn

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
