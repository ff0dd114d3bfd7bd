// Greedy per-sample bit allocation on the device, for the case the layers use at every step:
// all items start at the same width and have unit weight (replaces the host round trip around
// calc_precision.cc:9-50 in QScheme.compute_quantization_bits, actnn/actnn/qscheme.py:83-94).
//
// The reference pops, K = N * initial - target times, the largest (delta, index) pair of a
// priority queue and pushes the popped item's next step.  The steps of one item get strictly more
// expensive (delta more negative) as its width shrinks - or stay equal when C is 0 - so the popped
// set is exactly the K largest of all N * (initial - 1) candidate steps under the order
// (delta, index, earlier step first).  The kernel builds those candidates with the reference's
// arithmetic (delta evaluated in double, narrowed to float), sorts them in LDS with a bitonic
// network and counts, per item, how many of its steps are at or above the K-th one.
#include "device_utils.h"

namespace actnn {
namespace {

constexpr int kThreads = 1024;
constexpr int kMaxCand = 8192;           // 64 KiB of keys

// Key of step `l` (width initial - l -> initial - l - 1) of item i: larger key = popped earlier.
ACTNN_DEV uint64_t step_key(float C, const double* factor, int i, int l) {
  float d = (float)((double)C * factor[l]);            // calc_precision.cc:24-28, weight 1
  if (d == 0.0f) d = -0.0f;                            // one representation for "no cost"
  const uint32_t u = as_uint(d);
  const uint32_t ord = (u & 0x80000000u) ? ~u : (u | 0x80000000u);   // monotone in the float order
  return ((uint64_t)ord << 32) | (uint32_t)(i * 8 + (7 - l));
}

__global__ __launch_bounds__(kThreads) void calc_precision_device_kernel(
    const float* __restrict__ C, int32_t* __restrict__ bits, int N, int initial, int64_t K, int P) {
  __shared__ uint64_t keys[kMaxCand];                  // all of the 64 KiB a kernel gets without asking
  const int L = initial - 1;
  const int total = N * L;
  double factor[8];                                    // 1/(2^b - 1)^2 - 1/(2^(b-1) - 1)^2 per step
#pragma unroll
  for (int l = 0; l < 8; ++l) {
    const int b = initial - l > 1 ? initial - l : 2;
    const int64_t full = ((int64_t)1 << b) - 1, less = ((int64_t)1 << (b - 1)) - 1;
    factor[l] = 1.0 / (double)(full * full) - 1.0 / (double)(less * less);
  }
  if (K <= 0 || K >= total) {                          // nothing to take, or everything
    for (int i = threadIdx.x; i < N; i += kThreads) bits[i] = K <= 0 ? initial : 1;
    return;
  }
  for (int c = threadIdx.x; c < P; c += kThreads)
    keys[c] = c < total ? step_key(C[c / L], factor, c / L, c % L) : 0ull;   // padding sorts last
  __syncthreads();
  for (int k = 2; k <= P; k <<= 1) {                   // bitonic sort, descending
    for (int j = k >> 1; j > 0; j >>= 1) {
      for (int idx = threadIdx.x; idx < P; idx += kThreads) {
        const int other = idx ^ j;
        if (other > idx) {
          const uint64_t a = keys[idx], b = keys[other];
          const bool descending = (idx & k) == 0;
          if ((a < b) == descending) {
            keys[idx] = b;
            keys[other] = a;
          }
        }
      }
      __syncthreads();
    }
  }
  const uint64_t kth = keys[K - 1];
  for (int i = threadIdx.x; i < N; i += kThreads) {
    const float c = C[i];
    int taken = 0;
    for (int l = 0; l < L; ++l) taken += step_key(c, factor, i, l) >= kth ? 1 : 0;
    bits[i] = initial - taken;
  }
}

}  // namespace
}  // namespace actnn

extern "C" int actnn_calc_precision_device(const float* C, int32_t* bits, int64_t N, int initial_bits,
                                           int64_t target, void* stream) {
  using namespace actnn;
  if (N < 0) return ACTNN_EINVAL;
  if (N == 0) return ACTNN_OK;
  if (!C || !bits) return ACTNN_EINVAL;
  if (initial_bits < 1 || initial_bits > 8) return ACTNN_EBITS;
  const int64_t total = N * (initial_bits - 1);
  if (total > kMaxCand) return ACTNN_EINVAL;           // larger batches take the host routine
  int P = 2;
  while (P < total) P <<= 1;
  const int64_t K = N * initial_bits - target;         // widths to take away
  calc_precision_device_kernel<<<dim3(1), dim3(kThreads), 0, static_cast<hipStream_t>(stream)>>>(
      C, bits, (int)N, initial_bits, K, P);
  ACTNN_RETURN_LAUNCH_STATUS();
}
