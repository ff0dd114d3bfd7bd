// Greedy per-sample bit allocation on the device, for the case the layers use at every step:
// all items start at the same width and have unit weight (replaces the host round trip around
// calc_precision.cc:9-50 in QScheme.compute_quantization_bits, actnn/actnn/qscheme.py:83-94).
//
// The reference pops, K = N * initial - target times, the largest (delta, index) pair of a
// priority queue and pushes the popped item's next step.  The steps of one item get strictly more
// expensive (delta more negative) as its width shrinks - or stay equal when C is 0 - so the popped
// set is exactly the K largest of all N * (initial - 1) candidate steps under the order
// (delta, index, earlier step first).  Every block builds the keys of all candidates with the
// reference's arithmetic (delta evaluated in double, narrowed to float) - each thread a 256th of
// them, in registers - and ranks the steps of a few items by counting the keys above each of
// them, so the whole allocation is one launch of independent blocks: no sort, no atomics.
#include "device_utils.h"

namespace actnn {
namespace {

constexpr int kThreads = 256;
constexpr int kMaxCand = 8192;           // a thread counts at most 32 keys per candidate (8-bit counters)
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
  constexpr int kWaves = kThreads / 64;
  __shared__ double factors[8];
  __shared__ float C_s[kMaxCand];                      // N <= kMaxCand / L
  __shared__ uint64_t mine_s[kSlots];
  __shared__ int above_s[kWaves][kSlots];
  __shared__ int taken[kSlots];
  const int L = initial - 1;
  const int total = N * L;
  const int items_per_block = kSlots / L;
  const int nslot = items_per_block * L;
  const int item0 = blockIdx.x * items_per_block;
  if (K <= 0 || K >= total) {                          // nothing to take, or everything
    if ((int)threadIdx.x < items_per_block && item0 + (int)threadIdx.x < N)
      bits[item0 + threadIdx.x] = K <= 0 ? initial : 1;
    return;
  }
  for (int n = threadIdx.x; n < N; n += kThreads) C_s[n] = C[n];      // one trip to memory for all keys
  // 1/(2^b - 1)^2 - 1/(2^(b-1) - 1)^2 for the L steps
  if ((int)threadIdx.x < L) {
    const int b = initial - (int)threadIdx.x;
    const int64_t full = ((int64_t)1 << b) - 1, less = ((int64_t)1 << (b - 1)) - 1;
    factors[threadIdx.x] = 1.0 / (double)(full * full) - 1.0 / (double)(less * less);
  }
  __syncthreads();
  // the block's own candidates: steps item0 * L + slot
  if ((int)threadIdx.x < kSlots) {
    const int slot = threadIdx.x, cand = item0 * L + slot;
    uint64_t key = ~0ull;                              // nothing ranks above a dead slot
    if (slot < nslot && cand < total) {
      const int i = cand / L, l = cand - i * L;
      key = step_key(C_s[i], factors[l], i, l);
    }
    mine_s[slot] = key;
  }
  __syncthreads();
  uint64_t mine[kSlots];
#pragma unroll
  for (int sl = 0; sl < kSlots; ++sl) mine[sl] = mine_s[sl];
  // every thread builds a 256th of all keys in registers and counts, for each of the block's
  // candidates, the keys above it (the counts of a thread stay below 256: four to a register)
  uint32_t packed[kSlots / 4];
#pragma unroll
  for (int q = 0; q < kSlots / 4; ++q) packed[q] = 0u;
  int i = (int)threadIdx.x / L, l = (int)threadIdx.x - i * L;
  const int di = kThreads / L, dl = kThreads - di * L;
  for (int c = threadIdx.x; c < total; c += kThreads) {
    const uint64_t key = step_key(C_s[i], factors[l], i, l);
#pragma unroll
    for (int sl = 0; sl < kSlots; ++sl) packed[sl / 4] += (key > mine[sl] ? 1u : 0u) << (8 * (sl % 4));
    i += di;
    l += dl;
    if (l >= L) { l -= L; ++i; }
  }
  // counts of the block: butterfly inside each wave, then across the waves through LDS
#pragma unroll
  for (int sl = 0; sl < kSlots; ++sl) {
    int v = (int)((packed[sl / 4] >> (8 * (sl % 4))) & 0xffu);
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) v += __shfl_xor(v, d);
    if ((threadIdx.x & 63) == 0) above_s[threadIdx.x >> 6][sl] = v;
  }
  __syncthreads();
  if ((int)threadIdx.x < kSlots) {
    const int slot = threadIdx.x;
    int above = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) above += above_s[w][slot];
    const bool live = slot < nslot && item0 * L + slot < total;
    taken[slot] = live && above < K ? 1 : 0;
  }
  __syncthreads();
  if ((int)threadIdx.x < items_per_block && item0 + (int)threadIdx.x < N) {
    int t = 0;
    for (int k = 0; k < L; ++k) t += taken[threadIdx.x * L + k];
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
