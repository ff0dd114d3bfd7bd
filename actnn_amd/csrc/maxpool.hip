// MaxPool2d with int8 arg-max-in-window indices (replaces quantization_cuda_kernel.cu:630-754).
//
// Forward: one thread per output element scans its clipped window in row-major order and
// keeps the first strict maximum (index relative to the unclipped window origin).
// Backward: a gather - one thread per input element sums, in a fixed order, the
// grad_output of the windows whose stored index points at it.  Unlike the reference's
// atomicAdd scatter this needs no zero-fill pass and is bit-reproducible.
#include "device_utils.h"

namespace actnn {
namespace {

constexpr int kThreads = 256;

struct PoolGeom {
  int H, W, Ho, Wo, KH, KW, SH, SW, PH, PW;
};

template <typename T>
__global__ __launch_bounds__(kThreads) void max_pool2d_forward_kernel(const T* __restrict__ x,
                                                                      T* __restrict__ y,
                                                                      int8_t* __restrict__ idx,
                                                                      int64_t total, PoolGeom g) {
  const int64_t id = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (id >= total) return;
  const int w = (int)(id % g.Wo);
  const int h = (int)((id / g.Wo) % g.Ho);
  const int64_t nc = id / ((int64_t)g.Wo * g.Ho);
  const int h_base = h * g.SH - g.PH, w_base = w * g.SW - g.PW;
  const int h_start = h_base > 0 ? h_base : 0, h_end = h_base + g.KH < g.H ? h_base + g.KH : g.H;
  const int w_start = w_base > 0 ? w_base : 0, w_end = w_base + g.KW < g.W ? w_base + g.KW : g.W;
  // the reference starts from -1e10 narrowed to the element type (-inf for f16), .cu:656
  float v = Conv<T>::round(-1e10f);
  int index = 0;
  const T* plane = x + nc * (int64_t)g.H * g.W;
  for (int i = h_start; i < h_end; ++i) {
    for (int j = w_start; j < w_end; ++j) {
      const float c = Conv<T>::load(plane, (int64_t)i * g.W + j);
      if (c > v) {
        v = c;
        index = (i - h_base) * g.KW + (j - w_base);
      }
    }
  }
  Conv<T>::store(y, id, v);
  idx[id] = (int8_t)index;
}

template <typename T>
__global__ __launch_bounds__(kThreads) void max_pool2d_backward_kernel(const T* __restrict__ gout,
                                                                       const int8_t* __restrict__ idx,
                                                                       T* __restrict__ gin,
                                                                       int64_t total, PoolGeom g) {
  const int64_t id = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (id >= total) return;
  const int w = (int)(id % g.W);
  const int h = (int)((id / g.W) % g.H);
  const int64_t nc = id / ((int64_t)g.W * g.H);
  // windows (ho, wo) that contain (h, w): ho*SH - PH <= h < ho*SH - PH + KH
  int ho_lo = h + g.PH - g.KH + 1;
  ho_lo = ho_lo > 0 ? (ho_lo + g.SH - 1) / g.SH : 0;
  int ho_hi = (h + g.PH) / g.SH;
  ho_hi = ho_hi < g.Ho - 1 ? ho_hi : g.Ho - 1;
  int wo_lo = w + g.PW - g.KW + 1;
  wo_lo = wo_lo > 0 ? (wo_lo + g.SW - 1) / g.SW : 0;
  int wo_hi = (w + g.PW) / g.SW;
  wo_hi = wo_hi < g.Wo - 1 ? wo_hi : g.Wo - 1;
  const int64_t obase = nc * (int64_t)g.Ho * g.Wo;
  float acc = 0.0f;
  for (int ho = ho_lo; ho <= ho_hi; ++ho) {
    const int kh = h - (ho * g.SH - g.PH);
    for (int wo = wo_lo; wo <= wo_hi; ++wo) {
      const int kw = w - (wo * g.SW - g.PW);
      const int64_t o = obase + (int64_t)ho * g.Wo + wo;
      if ((int)idx[o] == kh * g.KW + kw) acc += Conv<T>::load(gout, o);
    }
  }
  Conv<T>::store(gin, id, acc);
}

template <typename T>
int launch_fwd(const void* x, void* y, int8_t* idx, int64_t total, const PoolGeom& g, hipStream_t s) {
  const int64_t blocks = (total + kThreads - 1) / kThreads;
  if (blocks > 0x7fffffffLL) return ACTNN_EINVAL;
  max_pool2d_forward_kernel<T><<<dim3((unsigned)blocks), dim3(kThreads), 0, s>>>(
      static_cast<const T*>(x), static_cast<T*>(y), idx, total, g);
  ACTNN_RETURN_LAUNCH_STATUS();
}

template <typename T>
int launch_bwd(const void* gout, const int8_t* idx, void* gin, int64_t total, const PoolGeom& g,
               hipStream_t s) {
  const int64_t blocks = (total + kThreads - 1) / kThreads;
  if (blocks > 0x7fffffffLL) return ACTNN_EINVAL;
  max_pool2d_backward_kernel<T><<<dim3((unsigned)blocks), dim3(kThreads), 0, s>>>(
      static_cast<const T*>(gout), idx, static_cast<T*>(gin), total, g);
  ACTNN_RETURN_LAUNCH_STATUS();
}

int check_geom(int64_t N, int64_t C, int64_t H, int64_t W, int64_t Ho, int64_t Wo, int KH, int KW,
               int SH, int SW, int PH, int PW) {
  if (N < 0 || C < 0 || H < 1 || W < 1 || Ho < 0 || Wo < 0) return ACTNN_EINVAL;
  if (KH < 1 || KW < 1 || SH < 1 || SW < 1 || PH < 0 || PW < 0) return ACTNN_EINVAL;
  if (KH * KW >= 16) return ACTNN_EINVAL;                      // quantization.cc:162
  if (H > 0x3fffffff || W > 0x3fffffff || Ho > 0x3fffffff || Wo > 0x3fffffff) return ACTNN_EINVAL;
  // every window must overlap the input, otherwise the stored index would be undefined
  if (Ho > 0 && ((Ho - 1) * SH - PH >= H || PH >= KH)) return ACTNN_EINVAL;
  if (Wo > 0 && ((Wo - 1) * SW - PW >= W || PW >= KW)) return ACTNN_EINVAL;
  return ACTNN_OK;
}

}  // namespace
}  // namespace actnn

extern "C" int actnn_max_pool2d_forward(const void* x, void* y, int8_t* idx, int64_t N, int64_t C,
                                        int64_t H, int64_t W, int64_t Ho, int64_t Wo, int KH, int KW,
                                        int SH, int SW, int PH, int PW, int dtype, void* stream) {
  using namespace actnn;
  const int rc = check_geom(N, C, H, W, Ho, Wo, KH, KW, SH, SW, PH, PW);
  if (rc != ACTNN_OK) return rc;
  const int64_t total = N * C * Ho * Wo;
  if (total == 0) return ACTNN_OK;
  if (!x || !y || !idx) return ACTNN_EINVAL;
  const PoolGeom g{(int)H, (int)W, (int)Ho, (int)Wo, KH, KW, SH, SW, PH, PW};
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case ACTNN_F32: return launch_fwd<float>(x, y, idx, total, g, s);
    case ACTNN_F16: return launch_fwd<__half>(x, y, idx, total, g, s);
    case ACTNN_BF16: return launch_fwd<bf16_t>(x, y, idx, total, g, s);
    default: return ACTNN_EDTYPE;
  }
}

extern "C" int actnn_max_pool2d_backward(const void* grad_out, const int8_t* idx, void* grad_in,
                                         int64_t N, int64_t C, int64_t H, int64_t W, int64_t Ho,
                                         int64_t Wo, int KH, int KW, int SH, int SW, int PH, int PW,
                                         int dtype, void* stream) {
  using namespace actnn;
  const int rc = check_geom(N, C, H, W, Ho, Wo, KH, KW, SH, SW, PH, PW);
  if (rc != ACTNN_OK) return rc;
  const int64_t total = N * C * H * W;
  if (total == 0) return ACTNN_OK;
  if (!grad_out || !grad_in || !idx) return ACTNN_EINVAL;
  const PoolGeom g{(int)H, (int)W, (int)Ho, (int)Wo, KH, KW, SH, SW, PH, PW};
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case ACTNN_F32: return launch_bwd<float>(grad_out, idx, grad_in, total, g, s);
    case ACTNN_F16: return launch_bwd<__half>(grad_out, idx, grad_in, total, g, s);
    case ACTNN_BF16: return launch_bwd<bf16_t>(grad_out, idx, grad_in, total, g, s);
    default: return ACTNN_EDTYPE;
  }
}
