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
// them, so the whole allocation is one launch of independent blocks: no sort.
//
// When the caller also wants the prefix sum of the widths (where each sample's words start in the
// stream), the block that finishes last computes it: every block publishes its widths (fence), then
// takes a ticket from a counter in device memory; the block that draws the last ticket knows all
// widths are written, scans them, and puts the counter back to zero for the next launch.  Nobody
// waits for anybody.  The counter is one word per GPU inside this library: launches that overlap in
// time on one GPU (different streams) would share it, launches on one stream are ordered.
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

__device__ unsigned int g_ticket = 0;

// prefix[0] = 0, prefix[i + 1] = bits[0] + ... + bits[i], by one block; the widths were written by
// other blocks, so they are read past this CU's cache.
ACTNN_DEV void block_prefix(const int32_t* bits, int32_t* __restrict__ prefix, int N) {
  __shared__ int32_t s_part[kThreads];
  const int per = (N + kThreads - 1) / kThreads;
  const int lo = (int)threadIdx.x * per;
  const int hi = lo + per < N ? lo + per : N;
  int32_t sum = 0;
  for (int i = lo; i < hi; ++i) sum += __hip_atomic_load(bits + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  s_part[threadIdx.x] = sum;
  __syncthreads();
  for (int off = 1; off < kThreads; off <<= 1) {         // inclusive Hillis-Steele scan
    const int32_t add = (int)threadIdx.x >= off ? s_part[threadIdx.x - off] : 0;
    __syncthreads();
    s_part[threadIdx.x] += add;
    __syncthreads();
  }
  int32_t run = threadIdx.x == 0 ? 0 : s_part[threadIdx.x - 1];
  if (threadIdx.x == 0) prefix[0] = 0;
  for (int i = lo; i < hi; ++i) {
    run += __hip_atomic_load(bits + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    prefix[i + 1] = run;
  }
}

// Called by every thread of every block after the block's widths are stored: the last block to
// arrive computes the prefix sum.
ACTNN_DEV void finish_with_prefix(const int32_t* bits, int32_t* __restrict__ prefix, int N) {
  __shared__ bool s_last;
  __threadfence();                                       // this block's widths are visible device-wide
  __syncthreads();
  if (threadIdx.x == 0) s_last = atomicAdd(&g_ticket, 1u) == gridDim.x - 1;
  __syncthreads();
  if (!s_last) return;
  __threadfence();
  block_prefix(bits, prefix, N);
  if (threadIdx.x == 0) atomicExch(&g_ticket, 0u);
}

template <bool PREFIX>
__global__ __launch_bounds__(kThreads) void calc_precision_device_kernel(
    const float* __restrict__ C, int32_t* bits, int32_t* __restrict__ prefix, int N, int initial, int64_t K) {
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
    if constexpr (PREFIX) finish_with_prefix(bits, prefix, N);
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
  if constexpr (PREFIX) finish_with_prefix(bits, prefix, N);
}

}  // namespace

// bits as actnn_calc_precision_device; with `prefix` (N + 1 entries) the same launch also leaves
// the exclusive prefix sum of the widths.  -> ACTNN_OK, an error code, or 1 when the widths are
// written but the prefix is left to the caller (the one-bit case, which launches no ranking kernel).
int calc_precision_device_launch(const float* C, int32_t* bits, int32_t* prefix, int64_t N, int initial_bits,
                                 int64_t target, hipStream_t s) {
  if (N < 0) return ACTNN_EINVAL;
  if (N == 0) return prefix ? 1 : ACTNN_OK;
  if (!C || !bits) return ACTNN_EINVAL;
  if (initial_bits < 1 || initial_bits > 8) return ACTNN_EBITS;
  const int64_t total = N * (initial_bits - 1);
  if (total > kMaxCand) return ACTNN_EINVAL;           // larger batches take the host routine
  const int64_t K = N * initial_bits - target;         // widths to take away
  if (initial_bits == 1) {                             // no steps to take: every item keeps its one bit
    fill_kernel<<<dim3((unsigned)((N + kThreads - 1) / kThreads)), dim3(kThreads), 0, s>>>(bits, (int)N, 1);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? (prefix ? 1 : ACTNN_OK) : (int)e;
  }
  const int items_per_block = kSlots / (initial_bits - 1);
  const int64_t blocks = (N + items_per_block - 1) / items_per_block;
  if (prefix)
    calc_precision_device_kernel<true><<<dim3((unsigned)blocks), dim3(kThreads), 0, s>>>(C, bits, prefix, (int)N, initial_bits, K);
  else
    calc_precision_device_kernel<false><<<dim3((unsigned)blocks), dim3(kThreads), 0, s>>>(C, bits, nullptr, (int)N, initial_bits, K);
  ACTNN_RETURN_LAUNCH_STATUS();
}

}  // namespace actnn

extern "C" int actnn_calc_precision_device(const float* C, int32_t* bits, int64_t N, int initial_bits,
                                           int64_t target, void* stream) {
  return actnn::calc_precision_device_launch(C, bits, nullptr, N, initial_bits, target,
                                             static_cast<hipStream_t>(stream));
}
