// Fixed-width pack / unpack (replaces quantization_cuda_kernel.cu:210-405).
//
// Stream layout (kept from the reference): byte ((no * G + g) * gs + d) holds the codes of
// the 8/bits consecutive samples n = no * (8/bits) + ni at bit offset ni * bits.
//
// A lane owns 8 consecutive d of one (no, g): it loads 8 elements of each of the 8/bits
// samples (one 16-byte load per sample for 16-bit types, two for f32), quantises them and
// writes its 8 output bytes with a single 8-byte store, so a wave writes 512 contiguous bytes.
// The per-group scale is produced by a small kernel first (N * G values).
//
// fp32 unpack takes its own kernel: with 8 elements per lane a lane's 32 bytes are two half-used
// 16-byte stores per cache line.  There a lane owns 4 consecutive d (one 16-byte non-temporal store
// per sample, a wave instruction covers 1 KiB contiguous) and reads 4 bytes: 3.9 -> 7.2 TB/s.  (The
// same split for fp32 pack was measured slower: twice the waves each with as many samples in
// flight.)
#include "quant_math.h"

namespace actnn {
namespace {

constexpr int kThreads = 256;

template <typename T, bool DET>
__global__ __launch_bounds__(kThreads) void scale_single_kernel(const T* __restrict__ mn,
                                                                const T* __restrict__ mx,
                                                                T* __restrict__ scale, int bits,
                                                                int64_t count) {
  const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i < count) {
    float mul, sub;
    Conv<T>::store(scale, i, GroupQuant<T, DET>::prepare(Conv<T>::load(mn, i), Conv<T>::load(mx, i), bits, mul, sub));
  }
}


// Where a thread works: the grid's x dimension runs over the G * chunks positions of one row of the
// stream (chunks = lanes per group), y over the rows (groups of 8/bits samples), so that the group
// and the offset inside it come out of one 32-bit shift or division and the sample from blockIdx -
// no 64-bit divisions per thread (they cost more instructions than the quantisation of the thread's
// elements: 4-bit pack of bf16 [512,256,56,56] 0.198 -> 0.180 ms, unpack 0.173 -> 0.155 ms).
struct SingleGeom {
  int64_t N, G;
  int gs, chunks, chunk_shift;     // chunk_shift < 0: chunks is not a power of two
  int64_t rows;                    // ceil(N / (8 / bits))
  uint32_t per_row;                // G * chunks
};
struct SingleAt { uint32_t g; int d0; bool live; };
template <int ELEMS> ACTNN_DEV SingleAt single_at(const SingleGeom& q) {
  const uint32_t i = blockIdx.x * kThreads + threadIdx.x;
  SingleAt a;
  a.live = i < q.per_row;
  a.g = q.chunk_shift >= 0 ? i >> q.chunk_shift : i / (uint32_t)q.chunks;
  a.d0 = (int)(q.chunk_shift >= 0 ? i & (uint32_t)(q.chunks - 1) : i % (uint32_t)q.chunks) * ELEMS;
  return a;
}

template <typename T, int BITS, bool DET>
__global__ __launch_bounds__(kThreads) void pack_single_kernel(
    const T* __restrict__ data, const T* __restrict__ mn, const T* __restrict__ scale,
    int8_t* __restrict__ packed, const T* __restrict__ noise, uint64_t seed, uint64_t offset,
    SingleGeom q) {
  constexpr int WPT = 8 / BITS;
  constexpr float Bf = (float)((1 << BITS) - 1);
  const SingleAt at = single_at<8>(q);
  if (!at.live) return;
  const int64_t N = q.N, G = q.G;
  const int gs = q.gs, chunks = q.chunks, d0 = at.d0;
  const int64_t g = at.g;
  for (int64_t no = blockIdx.y; no < q.rows; no += gridDim.y) {
  const int64_t og = no * G + g;

  float v[WPT][8];
  float nz[DET ? WPT : 1][8];
  float mul[WPT], sub[WPT];
#pragma unroll
  for (int ni = 0; ni < WPT; ++ni) {
    const int64_t n = no * WPT + ni;
    if (n < N) {
      const int64_t gi = n * G + g;
      const int64_t e = gi * gs + d0;
      load8_nt(data + e, v[ni]);        // 16-bit types: one whole-line access per wave instruction
      if (DET) load8(noise + e, nz[DET ? ni : 0]);
      const float sc = Conv<T>::load(scale, gi);
      const float m = Conv<T>::load(mn, gi);
      if (DET) {
        mul[ni] = sc;
        sub[ni] = Conv<T>::round(m - Conv<T>::round(1e-6f));    // shifted minimum, ops.py:31
      } else {
        RngFixed<T>::params(sc, m, BITS, mul[ni], sub[ni]);
      }
    } else {                            // samples past the end of the batch: code 0
#pragma unroll
      for (int k = 0; k < 8; ++k) v[ni][k] = 0.0f;
      mul[ni] = 0.0f;
      sub[ni] = 0.0f;
    }
  }
  uint32_t lo = 0, hi = 0;   // bytes 0..3 and 4..7
  if constexpr (DET) {
#pragma unroll
    for (int ni = 0; ni < WPT; ++ni) {
      const int64_t n = no * WPT + ni;
      if (n < N) {
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          const uint32_t c = det_code<T>(v[ni][k], nz[ni][k], mul[ni], sub[ni], Bf);
          if (k < 4) lo |= c << (8 * k + ni * BITS);
          else hi |= c << (8 * (k - 4) + ni * BITS);
        }
      }
    }
  } else {
    // Noise of the lane's octet in each sample.  Lane ^ 1 holds the neighbouring octet of the same
    // samples when a group has an even number of octets (units is then even too, so the two lanes
    // are here together), and the two share their Philox calls.
    uint32_t rw[WPT][Noise<T>::kWords];
    const uint64_t o0 = (uint64_t)(((no * WPT * G + g) * gs + d0) >> 3);    // sample no * WPT
    const uint64_t per_sample = (uint64_t)(G * gs) >> 3;
    if (WPT >= 2 && (chunks & 1) == 0) {
#pragma unroll
      for (int ni = 0; ni + 1 < WPT; ni += 2)
        Noise<T>::octets(o0 + ni * per_sample, o0 + (ni + 1) * per_sample, seed, offset, rw[ni], rw[ni + 1]);
    } else {
#pragma unroll
      for (int ni = 0; ni < WPT; ++ni) Noise<T>::octet(o0 + ni * per_sample, seed, offset, rw[ni]);
    }
    constexpr float kUnit = (float)(1u << (32 - BITS - Noise<T>::kBits));
    CodeShifter<BITS, false> slo, shi;     // last byte first, last sample first within a byte
#pragma unroll
    for (int k = 3; k >= 0; --k) {
#pragma unroll
      for (int ni = WPT - 1; ni >= 0; --ni) {
        slo.push(RngFixed<T>::word(v[ni][k], Noise<T>::at(rw[ni], k), mul[ni], sub[ni], kUnit));
        shi.push(RngFixed<T>::word(v[ni][k + 4], Noise<T>::at(rw[ni], k + 4), mul[ni], sub[ni], kUnit));
      }
    }
    lo = slo.lo;
    hi = shi.lo;
  }
  *reinterpret_cast<uint2*>(packed + og * gs + d0) = make_uint2(lo, hi);
  }
}

template <typename T, int BITS>
__global__ __launch_bounds__(kThreads) void unpack_single_kernel(
    const int8_t* __restrict__ packed, const T* __restrict__ scale, const T* __restrict__ mn,
    T* __restrict__ out, SingleGeom q) {
  constexpr int WPT = 8 / BITS;
  constexpr uint32_t kMask = (1u << BITS) - 1u;
  const SingleAt at = single_at<8>(q);
  if (!at.live) return;
  const int64_t N = q.N, G = q.G, g = at.g;
  const int gs = q.gs, d0 = at.d0;
  for (int64_t no = blockIdx.y; no < q.rows; no += gridDim.y) {
    const int64_t og = no * G + g;
    const uint2 w = *reinterpret_cast<const uint2*>(packed + og * gs + d0);
#pragma unroll
    for (int ni = 0; ni < WPT; ++ni) {
      const int64_t n = no * WPT + ni;
      if (n < N) {
        const int64_t gi = n * G + g;
        const Dequant<T> dq(Conv<T>::load(scale, gi), Conv<T>::load(mn, gi));
        float v[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          const uint32_t word = k < 4 ? w.x : w.y;
          v[k] = dq((word >> (8 * (k & 3) + ni * BITS)) & kMask);
        }
        store8_nt(out + gi * gs + d0, v);
      }
    }
  }
}

// ---------------------------------------------------------------------------- fp32 unpack: 4 elements per lane
template <int BITS>
__global__ __launch_bounds__(kThreads) void unpack_single_f32_kernel(
    const int8_t* __restrict__ packed, const float* __restrict__ scale, const float* __restrict__ mn,
    float* __restrict__ out, SingleGeom q) {
  constexpr int WPT = 8 / BITS;
  constexpr uint32_t kMask = (1u << BITS) - 1u;
  const SingleAt at = single_at<4>(q);
  if (!at.live) return;
  const int64_t N = q.N, G = q.G, g = at.g;
  const int gs = q.gs, d0 = at.d0;
  for (int64_t no = blockIdx.y; no < q.rows; no += gridDim.y) {
    const int64_t og = no * G + g;
    const uint32_t w = *reinterpret_cast<const uint32_t*>(packed + og * gs + d0);
#pragma unroll
    for (int ni = 0; ni < WPT; ++ni) {
      const int64_t n = no * WPT + ni;
      if (n < N) {
        const int64_t gi = n * G + g;
        const Dequant<float> dq(scale[gi], mn[gi]);
        u32x4 v;
#pragma unroll
        for (int k = 0; k < 4; ++k) v[k] = as_uint(dq((w >> (8 * k + ni * BITS)) & kMask));
        store16_nt(out + gi * gs + d0, v);
      }
    }
  }
}

// grid: x over the G * (gs / elems) lane positions of a stream row, y over the rows (capped; the
// kernels stride over the rest)
bool single_geometry(int64_t N, int64_t G, int64_t gs, int bits, int elems, SingleGeom& q, dim3& grid) {
  const int wpt = 8 / bits;
  q.N = N;
  q.G = G;
  q.gs = (int)gs;
  q.chunks = (int)(gs / elems);
  q.chunk_shift = -1;
  for (int sh = 0; sh < 31; ++sh)
    if ((1 << sh) == q.chunks) q.chunk_shift = sh;
  q.rows = (N + wpt - 1) / wpt;
  const int64_t per_row = G * q.chunks;
  if (per_row > 0x7fffffffLL || gs > 0x7fffffffLL) return false;
  q.per_row = (uint32_t)per_row;
  const int64_t bx = (per_row + kThreads - 1) / kThreads;
  grid = dim3((unsigned)bx, (unsigned)(q.rows < 65535 ? q.rows : 65535));
  return true;
}

template <typename T, bool DET>
int launch_pack_bits(int bits, const T* data, const T* mn, const T* scale, int8_t* packed,
                     const T* noise, uint64_t seed, uint64_t offset, int64_t N, int64_t G, int gs,
                     hipStream_t s) {
  SingleGeom q;
  dim3 grid;
  if (!single_geometry(N, G, gs, bits, 8, q, grid)) return ACTNN_EINVAL;
  const dim3 blk(kThreads);
  switch (bits) {
    case 1: pack_single_kernel<T, 1, DET><<<grid, blk, 0, s>>>(data, mn, scale, packed, noise, seed, offset, q); break;
    case 2: pack_single_kernel<T, 2, DET><<<grid, blk, 0, s>>>(data, mn, scale, packed, noise, seed, offset, q); break;
    case 4: pack_single_kernel<T, 4, DET><<<grid, blk, 0, s>>>(data, mn, scale, packed, noise, seed, offset, q); break;
    case 8: pack_single_kernel<T, 8, DET><<<grid, blk, 0, s>>>(data, mn, scale, packed, noise, seed, offset, q); break;
    default: return ACTNN_EBITS;
  }
  ACTNN_RETURN_LAUNCH_STATUS();
}

template <typename T>
int launch_pack(const void* data, const void* mn, const void* mx, int bits, void* scale,
                int8_t* packed, const void* noise, uint64_t seed, uint64_t offset, int64_t N,
                int64_t G, int64_t gs, hipStream_t s) {
  const int64_t count = N * G;
  const int64_t sblocks = (count + kThreads - 1) / kThreads;
  if (sblocks > 0x7fffffffLL) return ACTNN_EINVAL;
  const T* lo = static_cast<const T*>(mn);
  const T* hi = static_cast<const T*>(mx);
  T* sc = static_cast<T*>(scale);
  if (noise) scale_single_kernel<T, true><<<dim3((unsigned)sblocks), dim3(kThreads), 0, s>>>(lo, hi, sc, bits, count);
  else scale_single_kernel<T, false><<<dim3((unsigned)sblocks), dim3(kThreads), 0, s>>>(lo, hi, sc, bits, count);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return (int)e;
  if (noise)
    return launch_pack_bits<T, true>(bits, static_cast<const T*>(data), lo, sc, packed,
                                     static_cast<const T*>(noise), seed, offset, N, G, (int)gs, s);
  return launch_pack_bits<T, false>(bits, static_cast<const T*>(data), lo, sc, packed, nullptr, seed,
                                    offset, N, G, (int)gs, s);
}

template <typename T>
int launch_unpack(const int8_t* packed, int bits, const void* scale, const void* mn, void* out,
                  int64_t N, int64_t G, int64_t gs, hipStream_t s) {
  SingleGeom q;
  dim3 grid;
  const dim3 blk(kThreads);
  if constexpr (sizeof(T) == 4) {
    if (gs % 4 != 0 || !single_geometry(N, G, gs, bits, 4, q, grid)) return ACTNN_EINVAL;
    const float* sc4 = static_cast<const float*>(scale);
    const float* lo4 = static_cast<const float*>(mn);
    float* o4 = static_cast<float*>(out);
    switch (bits) {
      case 1: unpack_single_f32_kernel<1><<<grid, blk, 0, s>>>(packed, sc4, lo4, o4, q); break;
      case 2: unpack_single_f32_kernel<2><<<grid, blk, 0, s>>>(packed, sc4, lo4, o4, q); break;
      case 4: unpack_single_f32_kernel<4><<<grid, blk, 0, s>>>(packed, sc4, lo4, o4, q); break;
      case 8: unpack_single_f32_kernel<8><<<grid, blk, 0, s>>>(packed, sc4, lo4, o4, q); break;
      default: return ACTNN_EBITS;
    }
    ACTNN_RETURN_LAUNCH_STATUS();
  }
  if (!single_geometry(N, G, gs, bits, 8, q, grid)) return ACTNN_EINVAL;
  const T* sc = static_cast<const T*>(scale);
  const T* lo = static_cast<const T*>(mn);
  T* o = static_cast<T*>(out);
  switch (bits) {
    case 1: unpack_single_kernel<T, 1><<<grid, blk, 0, s>>>(packed, sc, lo, o, q); break;
    case 2: unpack_single_kernel<T, 2><<<grid, blk, 0, s>>>(packed, sc, lo, o, q); break;
    case 4: unpack_single_kernel<T, 4><<<grid, blk, 0, s>>>(packed, sc, lo, o, q); break;
    case 8: unpack_single_kernel<T, 8><<<grid, blk, 0, s>>>(packed, sc, lo, o, q); break;
    default: return ACTNN_EBITS;
  }
  ACTNN_RETURN_LAUNCH_STATUS();
}

inline bool single_bits_ok(int bits) { return bits == 1 || bits == 2 || bits == 4 || bits == 8; }

}  // namespace
}  // namespace actnn

extern "C" int actnn_pack_single(const void* data, const void* mn, const void* mx, int bits,
                                 void* scale, int8_t* packed, const void* noise, uint64_t seed,
                                 uint64_t offset, int64_t N, int64_t G, int64_t gs, int dtype,
                                 void* stream) {
  using namespace actnn;
  if (!single_bits_ok(bits)) return ACTNN_EBITS;       // TORCH_CHECK(8 % bits == 0), .cu:272
  if (N < 0 || G < 0 || gs < 8 || gs % 8 != 0) return ACTNN_EINVAL;
  if (N == 0 || G == 0) return ACTNN_OK;
  if (!data || !mn || !mx || !scale || !packed) return ACTNN_EINVAL;
  if (!aligned16(data) || (noise && !aligned16(noise)) ||
      (reinterpret_cast<uintptr_t>(packed) & 7u) != 0)
    return ACTNN_EALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case ACTNN_F32: return launch_pack<float>(data, mn, mx, bits, scale, packed, noise, seed, offset, N, G, gs, s);
    case ACTNN_F16: return launch_pack<__half>(data, mn, mx, bits, scale, packed, noise, seed, offset, N, G, gs, s);
    case ACTNN_BF16: return launch_pack<bf16_t>(data, mn, mx, bits, scale, packed, noise, seed, offset, N, G, gs, s);
    default: return ACTNN_EDTYPE;
  }
}

extern "C" int actnn_unpack_single(const int8_t* packed, int bits, const void* scale,
                                   const void* mn, void* out, int64_t N, int64_t G, int64_t gs,
                                   int dtype, void* stream) {
  using namespace actnn;
  if (!single_bits_ok(bits)) return ACTNN_EBITS;
  if (N < 0 || G < 0 || gs < 8 || gs % 8 != 0) return ACTNN_EINVAL;
  if (N == 0 || G == 0) return ACTNN_OK;
  if (!packed || !scale || !mn || !out) return ACTNN_EINVAL;
  if (!aligned16(out) || (reinterpret_cast<uintptr_t>(packed) & 7u) != 0) return ACTNN_EALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case ACTNN_F32: return launch_unpack<float>(packed, bits, scale, mn, out, N, G, gs, s);
    case ACTNN_F16: return launch_unpack<__half>(packed, bits, scale, mn, out, N, G, gs, s);
    case ACTNN_BF16: return launch_unpack<bf16_t>(packed, bits, scale, mn, out, N, G, gs, s);
    default: return ACTNN_EDTYPE;
  }
}
