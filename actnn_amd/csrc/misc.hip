// Library-level helpers: error strings, version, the plain streaming copy used to calibrate
// bandwidth counters, and the matrix-pipe probe the benchmark prices the fused GEMM against.
#include "device_utils.h"

namespace actnn {
namespace {

__global__ __launch_bounds__(256) void stream_copy_kernel(const uint4* __restrict__ src,
                                                          uint4* __restrict__ dst, int64_t nvec) {
  // each block copies a contiguous run of 4 * 256 vectors (16 KiB); four loads in flight per lane
  const int64_t base = (int64_t)blockIdx.x * 1024 + threadIdx.x;
  uint4 v[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    if (base + i * 256 < nvec) v[i] = src[base + i * 256];      // plain loads and stores on purpose:
#pragma unroll
  for (int i = 0; i < 4; ++i)
    if (base + i * 256 < nvec) dst[base + i * 256] = v[i];      // this kernel is the calibration yardstick
}

// What the matrix pipes alone sustain: every wave (one per SIMD, as in the fused weight-gradient
// GEMM) loads eight 16-byte operand fragments once and then issues nothing but
// v_mfma_f32_32x32x16_bf16 on them - 16 per k-block into 16 independent accumulators, the operand
// registers rotated between k-blocks so that every instruction meets a fresh pair.  No loads, no
// LDS, no other arithmetic in the loop.
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
__global__ __launch_bounds__(256, 1) void matrix_pipe_kernel(const u32x4* __restrict__ operands,
                                                             float* __restrict__ out, int kblocks) {
  f32x16_t acc[4][4];
#pragma unroll
  for (int e = 0; e < 4; ++e)
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int c = 0; c < 16; ++c) acc[e][a][c] = 0.0f;
  u32x4 f[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) f[i] = operands[((size_t)blockIdx.x * 8 + i) * 256 + threadIdx.x];
  for (int kb = 0; kb < kblocks; ++kb) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
      for (int a = 0; a < 4; ++a)
        acc[e][a] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, f[e]),
                                                            __builtin_bit_cast(bf16x8_t, f[4 + a]), acc[e][a], 0, 0, 0);
    const u32x4 t = f[0];
#pragma unroll
    for (int i = 0; i < 7; ++i) f[i] = f[i + 1];
    f[7] = t;
  }
  float sum = 0.0f;
#pragma unroll
  for (int e = 0; e < 4; ++e)
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int c = 0; c < 16; ++c) sum += acc[e][a][c];
  out[(size_t)blockIdx.x * 256 + threadIdx.x] = sum;
}

}  // namespace
}  // namespace actnn

extern "C" int actnn_matrix_pipe_probe(const void* operands, float* out, int blocks, int kblocks, void* stream) {
  using namespace actnn;
  if (blocks <= 0 || kblocks < 0 || !operands || !out) return ACTNN_EINVAL;
  if (!aligned16(operands)) return ACTNN_EALIGN;
  matrix_pipe_kernel<<<dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<const u32x4*>(operands), out, kblocks);
  ACTNN_RETURN_LAUNCH_STATUS();
}

extern "C" int actnn_stream_copy(const void* src, void* dst, int64_t bytes, void* stream) {
  using namespace actnn;
  if (bytes < 0 || bytes % 16 != 0) return ACTNN_EINVAL;
  if (bytes == 0) return ACTNN_OK;
  if (!src || !dst) return ACTNN_EINVAL;
  if (!aligned16(src) || !aligned16(dst)) return ACTNN_EALIGN;
  const int64_t nvec = bytes / 16;
  const int64_t blocks = (nvec + 1023) / 1024;
  if (blocks > 0x7fffffffLL) return ACTNN_EINVAL;
  stream_copy_kernel<<<dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<const uint4*>(src), static_cast<uint4*>(dst), nvec);
  ACTNN_RETURN_LAUNCH_STATUS();
}

// The three allocation steps of a layer in one call (one crossing of the language boundary instead
// of three): sensitivities, greedy widths on the device, exclusive prefix of the widths.
extern "C" int actnn_range_sqr(const void* mn, const void* mx, float* out, int64_t N, int64_t G, float factor,
                               const float* mult, int mult_per_sample, int dtype, void* stream);
extern "C" int actnn_calc_precision_device(const float* C, int32_t* bits, int64_t N, int initial_bits,
                                           int64_t target, void* stream);
extern "C" int actnn_bits_prefix(const int32_t* bits, int32_t* prefix, int64_t N, void* stream);

extern "C" int actnn_allocate_bits_device(const void* mn, const void* mx, float factor, const float* mult,
                                          int mult_per_sample, float* sensitivity, int32_t* bits,
                                          int32_t* prefix, int64_t N, int64_t G, int initial_bits,
                                          int64_t target, int dtype, void* stream) {
  int rc = actnn_range_sqr(mn, mx, sensitivity, N, G, factor, mult, mult_per_sample, dtype, stream);
  if (rc != ACTNN_OK) return rc;
  rc = actnn_calc_precision_device(sensitivity, bits, N, initial_bits, target, stream);
  if (rc != ACTNN_OK) return rc;
  return actnn_bits_prefix(bits, prefix, N, stream);
}

// One crossing of the language boundary for a layer's whole forward-side sequence: the calls below
// on one stream, arguments as theirs.  Nothing is launched unless the arguments of the first step
// pass; a later step that refuses its arguments leaves the earlier ones launched (their outputs are
// then simply unused).
extern "C" int actnn_batch_norm_forward_stats(const void* x, const float* weight, const float* bias,
                                              float* running_mean, float* running_var, float* save_mean,
                                              float* save_invstd, void* mn, void* mx, void* workspace,
                                              int64_t workspace_bytes, int64_t N, int64_t C, int64_t HW,
                                              double momentum, double eps, int dtype, int channels_last,
                                              void* stream);
extern "C" int actnn_batch_norm_forward_apply(const void* x, void* y, const void* workspace,
                                              int64_t workspace_bytes, const int32_t* bits,
                                              const int32_t* prefix, const void* mn, const void* mx, void* scale,
                                              int32_t* packed, uint64_t seed, uint64_t offset, int64_t N,
                                              int64_t C, int64_t HW, int dtype, int channels_last, void* stream);
extern "C" int actnn_batch_norm_forward_apply_relu(const void* x, void* y, const void* workspace,
                                                   int64_t workspace_bytes, const int32_t* bits,
                                                   const int32_t* prefix, const void* mn, const void* mx,
                                                   void* scale, int32_t* packed, uint64_t seed, uint64_t offset,
                                                   int32_t* relu_mask, void* relu_mn, void* relu_mx,
                                                   const void* residual, int64_t N, int64_t C, int64_t HW,
                                                   int dtype, int channels_last, void* stream);
extern "C" int actnn_minimax(const void* data, void* mn, void* mx, int64_t M, int64_t D, int dtype, void* stream);
extern "C" int actnn_pack_mixed(const void* data, const void* mn, const void* mx, const int32_t* bits,
                                const int32_t* prefix, void* scale, int32_t* packed, const void* noise,
                                uint64_t seed, uint64_t offset, int64_t N, int64_t G, int64_t gs, int dtype,
                                void* stream);

extern "C" int actnn_batch_norm_forward_quantize(
    const void* x, const float* weight, const float* bias, float* running_mean, float* running_var, void* y,
    float* save_mean, float* save_invstd, void* mn, void* mx, void* workspace, int64_t workspace_bytes,
    float factor, const float* mult, int mult_per_sample, float* sensitivity, int32_t* bits, int32_t* prefix,
    int initial_bits, int64_t target, void* scale, int32_t* packed, uint64_t seed, uint64_t offset,
    int32_t* relu_mask, void* relu_mn, void* relu_mx, const void* residual, int64_t N, int64_t C, int64_t HW,
    double momentum, double eps, int dtype, int channels_last, void* stream) {
  if (!mn || !mx || !bits || !prefix || !scale || !packed || !sensitivity || !y) return ACTNN_EINVAL;
  if (N <= 0 || C <= 0 || HW <= 0 || (C * HW) % 256 != 0) return ACTNN_EINVAL;
  const bool relu = relu_mask || relu_mn || relu_mx;
  if (relu && (!relu_mask || !relu_mn || !relu_mx)) return ACTNN_EINVAL;
  if (residual && !relu) return ACTNN_EINVAL;
  if (!actnn::aligned16(residual)) return ACTNN_EALIGN;
  // (what the last step will ask, before anything is launched)
  if (relu && (!channels_last || (dtype != ACTNN_F16 && dtype != ACTNN_BF16) ||
               !((C <= 256 && 256 % C == 0) || C % 512 == 0) || (N * HW) % (2048 / (C < 256 ? C : 256)) != 0))
    return ACTNN_EINVAL;
  int rc = actnn_batch_norm_forward_stats(x, weight, bias, running_mean, running_var, save_mean, save_invstd, mn,
                                          mx, workspace, workspace_bytes, N, C, HW, momentum, eps, dtype,
                                          channels_last, stream);
  if (rc != ACTNN_OK) return rc;
  rc = actnn_allocate_bits_device(mn, mx, factor, mult, mult_per_sample, sensitivity, bits, prefix, N,
                                  C * HW / 256, initial_bits, target, dtype, stream);
  if (rc != ACTNN_OK) return rc;
  if (relu)
    return actnn_batch_norm_forward_apply_relu(x, y, workspace, workspace_bytes, bits, prefix, mn, mx, scale,
                                               packed, seed, offset, relu_mask, relu_mn, relu_mx, residual, N, C, HW,
                                               dtype, channels_last, stream);
  return actnn_batch_norm_forward_apply(x, y, workspace, workspace_bytes, bits, prefix, mn, mx, scale, packed,
                                        seed, offset, N, C, HW, dtype, channels_last, stream);
}

extern "C" int actnn_quantize_activation(const void* data, void* mn, void* mx, int minmax_known, float factor,
                                         const float* mult, int mult_per_sample, float* sensitivity,
                                         int32_t* bits, int32_t* prefix, int initial_bits, int64_t target,
                                         void* scale, int32_t* packed, uint64_t seed, uint64_t offset, int64_t N,
                                         int64_t G, int dtype, void* stream) {
  if (!data || !mn || !mx || !bits || !prefix || !scale || !packed || !sensitivity) return ACTNN_EINVAL;
  if (N <= 0 || G <= 0) return ACTNN_EINVAL;
  int rc = ACTNN_OK;
  if (!minmax_known) {
    rc = actnn_minimax(data, mn, mx, N * G, 256, dtype, stream);
    if (rc != ACTNN_OK) return rc;
  }
  rc = actnn_allocate_bits_device(mn, mx, factor, mult, mult_per_sample, sensitivity, bits, prefix, N, G,
                                  initial_bits, target, dtype, stream);
  if (rc != ACTNN_OK) return rc;
  return actnn_pack_mixed(data, mn, mx, bits, prefix, scale, packed, nullptr, seed, offset, N, G, 256, dtype,
                          stream);
}

extern "C" const char* actnn_strerror(int code) {
  switch (code) {
    case ACTNN_OK: return "success";
    case ACTNN_EINVAL: return "invalid size, null pointer or unsupported combination";
    case ACTNN_EDTYPE: return "unknown dtype";
    case ACTNN_EBITS: return "unsupported bit width";
    case ACTNN_EALIGN: return "pointer is not aligned as required (16 bytes)";
    case ACTNN_ETOOBIG: return "the problem needs more scratch memory than the library's fixed buffer holds";
    default: return code > 0 ? hipGetErrorString(static_cast<hipError_t>(code)) : "unknown error";
  }
}

extern "C" const char* actnn_version(void) { return "actnn_amd 0.1 (gfx950)"; }
