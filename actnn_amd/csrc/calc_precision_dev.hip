// Greedy per-sample bit allocation on the device, for the case the layers use at every step:
// all items start at the same width and have unit weight (replaces the host round trip around
// calc_precision.cc:9-50 in QScheme.compute_quantization_bits, actnn/actnn/qscheme.py:83-94).
//
// The reference pops, K = N * initial - target times, the largest (delta, index) pair of a
// priority queue and pushes the popped item's next step.  The steps of one item get strictly more
// expensive (delta more negative) as its width shrinks - or stay equal when C is 0 - so the popped
// set is exactly the K largest of all N * (initial - 1) candidate steps under the order
// (delta, index, earlier step first).  Every block builds the keys of all candidates in LDS with
// the reference's arithmetic (delta evaluated in double, narrowed to float) and ranks the steps of
// a few items by counting the keys above each of them - 16 threads per step, each over a 16th of
// the keys - so the whole allocation is one launch of independent blocks: no sort, no atomics.
#include "device_utils.h"

namespace actnn {
namespace {

constexpr int kThreads = 256;
constexpr int kMaxCand = 8192;           // 64 KiB of keys: all a kernel gets without asking
constexpr int kSlots = 16;               // candidate steps ranked per block (16 threads each)

// Key of step `l` (width initial - l -> initial - l - 1) of item i: larger key = popped earlier.
ACTNN_DEV uint64_t step_key(float C, double factor, int i, int l) {
  float d = (float)((double)C * factor);               // calc_precision.cc:24-28, weight 1
  if (d == 0.0f) d = -0.0f;                            // one representation for "no cost"
  const uint32_t u = as_uint(d);
  const uint32_t ord = (u & 0x80000000u) ? ~u : (u | 0x80000000u);   // monotone in the float order
  return ((uint64_t)ord << 32) | (uint32_t)(i * 8 + (7 - l));
}

__global__ __launch_bounds__(kThreads) void fill_kernel(int32_t* __restrict__ out, int n, int value) {
  const int i = blockIdx.x * kThreads + threadIdx.x;
  if (i < n) out[i] = value;
}

__global__ __launch_bounds__(kThreads) void calc_precision_device_kernel(
    const float* __restrict__ C, int32_t* __restrict__ bits, int N, int initial, int64_t K) {
  __shared__ uint64_t keys[kMaxCand];
  const int L = initial - 1;
  const int total = N * L;
  const int items_per_block = kSlots / L;
  const int item0 = blockIdx.x * items_per_block;
  if (K <= 0 || K >= total) {                          // nothing to take, or everything
    if ((int)threadIdx.x < items_per_block && item0 + (int)threadIdx.x < N)
      bits[item0 + threadIdx.x] = K <= 0 ? initial : 1;
    return;
  }
  // 1/(2^b - 1)^2 - 1/(2^(b-1) - 1)^2 for the L steps: held in the tail of the key array until the
  // keys that would overwrite it are built (total < kMaxCand leaves room; otherwise per key)
  const bool shared_factors = total + 8 <= kMaxCand;
  double* factors = reinterpret_cast<double*>(keys + kMaxCand - 8);
  auto factor_of = [&](int l) {
    const int b = initial - l;
    const int64_t full = ((int64_t)1 << b) - 1, less = ((int64_t)1 << (b - 1)) - 1;
    return 1.0 / (double)(full * full) - 1.0 / (double)(less * less);
  };
  if (shared_factors) {
    if ((int)threadIdx.x < L) factors[threadIdx.x] = factor_of(threadIdx.x);
    __syncthreads();
  }
  for (int c = threadIdx.x; c < total; c += kThreads) {
    const int i = c / L, l = c - i * L;
    keys[c] = step_key(C[i], shared_factors ? factors[l] : factor_of(l), i, l);
  }
  __syncthreads();
  // thread -> (slot = candidate of this block, seg = which 16th of the keys it counts over)
  const int slot = threadIdx.x >> 4, seg = threadIdx.x & 15;
  const int cand = item0 * L + slot;
  const bool live = slot < items_per_block * L && cand < total;
  const uint64_t mine = live ? keys[cand] : ~0ull;
  int above = 0;
  for (int m = seg; m < total; m += 16) above += keys[m] > mine ? 1 : 0;
  above += __shfl_xor(above, 1);
  above += __shfl_xor(above, 2);
  above += __shfl_xor(above, 4);
  above += __shfl_xor(above, 8);                       // the 16 threads of a slot are 16 consecutive lanes
  __shared__ int taken[kSlots];
  if (seg == 0) taken[slot] = live && above < K ? 1 : 0;
  __syncthreads();
  if ((int)threadIdx.x < items_per_block && item0 + (int)threadIdx.x < N) {
    int t = 0;
    for (int l = 0; l < L; ++l) t += taken[threadIdx.x * L + l];
    bits[item0 + threadIdx.x] = initial - t;
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
  const int64_t K = N * initial_bits - target;         // widths to take away
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (initial_bits == 1) {                             // no steps to take: every item keeps its one bit
    fill_kernel<<<dim3((unsigned)((N + kThreads - 1) / kThreads)), dim3(kThreads), 0, s>>>(bits, (int)N, 1);
    ACTNN_RETURN_LAUNCH_STATUS();
  }
  const int items_per_block = kSlots / (initial_bits - 1);
  const int64_t blocks = (N + items_per_block - 1) / items_per_block;
  calc_precision_device_kernel<<<dim3((unsigned)blocks), dim3(kThreads), 0, s>>>(C, bits, (int)N, initial_bits, K);
  ACTNN_RETURN_LAUNCH_STATUS();
}
