// MaxPool2d with int8 arg-max-in-window indices (replaces quantization_cuda_kernel.cu:630-754).
//
// Index storage: one int8 per output element as in the reference, or (template parameter NIB of
// every kernel, the *_nibble entry points) two outputs per byte - an index is below 16 - with
// output o of the flat output order in bits 4 * (o & 1) .. of byte o >> 1.
//
// Forward: every output element scans its clipped window in row-major order and keeps the first
// strict maximum (index relative to the unclipped window origin).
// Backward: a gather - every input element sums, in a fixed order, the grad_output of the
// windows whose stored index points at it.  Unlike the reference's atomicAdd scatter this needs no
// zero-fill pass and is bit-reproducible.
//
// Both run tiled through LDS: a block owns a band of rows of one (n, c) plane, copies the rows it
// needs (a contiguous span of the plane) into LDS with 16-byte loads, and then works out of LDS,
// so HBM sees each input byte once and all global accesses are coalesced.  Planes too wide for
// the LDS budget fall back to direct global loads.
#include "device_utils.h"

namespace actnn {
namespace {

constexpr int kThreads = 256;             // general kernels
// Stride-2 kernels (measured on 256x64x112x112 f16): the forward likes tall bands and streamed
// (non-temporal) staging loads; the backward, whose bands share their edge rows and whose cache
// lines are split between neighbouring blocks, likes short bands and cached loads (256 threads:
// 0.114 ms, two passes per block: 0.138 ms, against 0.105 ms).  The backward issues as many vector
// instructions as fit its run time (counters: one per 4 cycles and SIMD), so what it saves in
// staging and index arithmetic shows directly: staging both spans in one round and dividing by
// multiply-high took it from 0.117 to 0.105 ms on the same machine.
constexpr int kFwdS2Threads = 256, kFwdS2Passes = 4;
constexpr int kBwdS2Threads = 128, kBwdS2Passes = 1;

struct PoolGeom {
  int H, W, Ho, Wo, KH, KW, SH, SW, PH, PW;
};

// index of output o
template <bool NIB> ACTNN_DEV int read_index(const int8_t* __restrict__ idx, int64_t o) {
  if (NIB) return ((int)(uint8_t)idx[o >> 1] >> (4 * (int)(o & 1))) & 15;
  return (int)idx[o];
}
// the same from a staged copy: i counts outputs from the first staged one, whose byte is s[0]
// and whose parity is folded into i by the caller
template <bool NIB> ACTNN_DEV int staged_index(const int8_t* s, int i) {
  if (NIB) return ((int)(uint8_t)s[i >> 1] >> (4 * (i & 1))) & 15;
  return (int)s[i];
}
// E (4 or 8) indices of outputs o .. o + E - 1 (o a multiple of E) as fields of kBits bits of one
// integer, field e = output o + e: what the kernels that own several adjacent outputs store and load
template <bool NIB> struct IndexFields {
  static constexpr int kBits = NIB ? 4 : 8;
  static constexpr uint32_t kMask = NIB ? 0xfu : 0xffu;
  static ACTNN_DEV int get(uint64_t fields, int e) { return (int)((uint32_t)(fields >> (kBits * e)) & kMask); }
  // bytes from the start of idx to the field of output o (o even)
  static ACTNN_DEV uint32_t byte_of(uint32_t o) { return NIB ? o >> 1 : o; }
  static ACTNN_DEV int64_t byte_of(int64_t o) { return NIB ? o >> 1 : o; }
  template <int E, typename P> static ACTNN_DEV void store(P* idx, int64_t o, uint64_t fields) {
    P* at = idx + (NIB ? o >> 1 : o);
    if constexpr (E * kBits == 16) *reinterpret_cast<uint16_t*>(at) = (uint16_t)fields;
    else if constexpr (E * kBits == 32) *reinterpret_cast<uint32_t*>(at) = (uint32_t)fields;
    else *reinterpret_cast<uint64_t*>(at) = fields;
  }
  template <int E, typename P> static ACTNN_DEV uint64_t load(const P* idx, int64_t o) {
    const P* at = idx + (NIB ? o >> 1 : o);
    if constexpr (E * kBits == 16) return *reinterpret_cast<const uint16_t*>(at);
    else if constexpr (E * kBits == 32) return *reinterpret_cast<const uint32_t*>(at);
    else return *reinterpret_cast<const uint64_t*>(at);
  }
};

template <typename T, bool NIB>
__global__ __launch_bounds__(kThreads) void max_pool2d_forward_kernel(const T* __restrict__ x,
                                                                      T* __restrict__ y,
                                                                      int8_t* __restrict__ idx,
                                                                      int64_t total, PoolGeom g) {
  const int64_t id = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  const bool live = id < total;
  int index = 0;
  if (live) {
    const int w = (int)(id % g.Wo);
    const int h = (int)((id / g.Wo) % g.Ho);
    const int64_t nc = id / ((int64_t)g.Wo * g.Ho);
    const int h_base = h * g.SH - g.PH, w_base = w * g.SW - g.PW;
    const int h_start = h_base > 0 ? h_base : 0, h_end = h_base + g.KH < g.H ? h_base + g.KH : g.H;
    const int w_start = w_base > 0 ? w_base : 0, w_end = w_base + g.KW < g.W ? w_base + g.KW : g.W;
    // the reference starts from -1e10 narrowed to the element type (-inf for f16), .cu:656
    float v = Conv<T>::round(-1e10f);
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
    if (!NIB) idx[id] = (int8_t)index;
  }
  if (NIB) {
    // the even thread writes the byte of outputs id and id + 1 (0 for an output past the end)
    const int next = lane_xor<1>(index);
    if (live && !(id & 1)) idx[id >> 1] = (int8_t)(index | (next << 4));
  }
}

template <typename T, bool NIB>
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
      if (read_index<NIB>(idx, o) == kh * g.KW + kw) acc += Conv<T>::load(gout, o);
    }
  }
  Conv<T>::store(gin, id, acc);
}


constexpr int kLdsBudget = 48 * 1024;     // bytes of dynamic LDS a block may use

// Copy the contiguous span [first, first + count) of `src` (element indices into a tensor of
// `total` elements whose base is 16-byte aligned) into LDS so that element first + i lands at
// dst[shift + i], shift = first % (16 / sizeof(T)); aligned 16-byte loads wherever they stay
// inside the tensor.  Returns shift.
// Copy nvec 16-byte vectors from global memory (streamed, non-temporal) into LDS.  Loads are issued
// in batches of 8 per thread before the first LDS write so that several are in flight at once.
template <int THREADS, bool NT>
ACTNN_DEV void copy_vectors(const void* __restrict__ src, void* dst, int nvec) {
  constexpr int U = 8;
  const u32x4* s = reinterpret_cast<const u32x4*>(src);
  u32x4* d = reinterpret_cast<u32x4*>(dst);
  for (int v0 = threadIdx.x; v0 < nvec; v0 += U * THREADS) {
    u32x4 t[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (v0 + u * THREADS < nvec) t[u] = NT ? load16_nt(s + v0 + u * THREADS) : load16(s + v0 + u * THREADS);
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (v0 + u * THREADS < nvec) d[v0 + u * THREADS] = t[u];
  }
}

template <typename T, int THREADS = kThreads, bool NT = false>
ACTNN_DEV int stage_span(const T* __restrict__ src, int64_t first, int count, int64_t total, T* dst) {
  constexpr int V = 16 / (int)sizeof(T);
  const int shift = (int)(first % V);
  const int64_t base = first - shift;                    // aligned element index
  const int nvec = (shift + count + V - 1) / V;
  // only the last vector can reach past the end of the tensor
  const bool ragged = base + (int64_t)nvec * V > total;
  copy_vectors<THREADS, NT>(src + base, dst, ragged ? nvec - 1 : nvec);
  if (ragged) {
    const int64_t e = base + (int64_t)(nvec - 1) * V;
    for (int i = threadIdx.x; i < V; i += THREADS)
      if (e + i < total) dst[(nvec - 1) * V + i] = src[e + i];
  }
  return shift;
}

// Two spans staged together: the loads of both are issued before the first LDS write, so a short
// band pays one round trip to memory, not two.
template <typename T> struct Span {
  const T* base;          // aligned start
  int whole;              // 16-byte vectors that lie inside the tensor
  int tail;               // elements of the ragged last vector (0: none)
  int shift;              // position of the span's first element in the staged copy
};
template <typename T> ACTNN_DEV Span<T> span_of(const T* __restrict__ src, int64_t first, int count, int64_t total) {
  constexpr int V = 16 / (int)sizeof(T);
  Span<T> sp;
  sp.shift = (int)(first & (V - 1));
  const int64_t base = first - sp.shift;
  const int nvec = (sp.shift + count + V - 1) / V;
  const bool ragged = base + (int64_t)nvec * V > total;          // only the last vector can reach past the end
  sp.base = src + base;
  sp.whole = ragged ? nvec - 1 : nvec;
  sp.tail = ragged ? (int)(total - base - (int64_t)(nvec - 1) * V) : 0;
  return sp;
}
template <int THREADS, typename A, typename B>
ACTNN_DEV void stage_two(const Span<A>& a, A* da, const Span<B>& b, B* db) {
  constexpr int VA = 16 / (int)sizeof(A), VB = 16 / (int)sizeof(B);
  const int most = a.whole > b.whole ? a.whole : b.whole;
#pragma unroll 1
  for (int v = threadIdx.x; v < most; v += THREADS) {
    u32x4 x, y;
    const bool in_a = v < a.whole, in_b = v < b.whole;
    if (in_a) x = load16(a.base + v * VA);
    if (in_b) y = load16(b.base + v * VB);
    if (in_a) reinterpret_cast<u32x4*>(da)[v] = x;
    if (in_b) reinterpret_cast<u32x4*>(db)[v] = y;
  }
#pragma unroll 1
  for (int i = threadIdx.x; i < a.tail; i += THREADS) da[a.whole * VA + i] = a.base[a.whole * VA + i];
#pragma unroll 1
  for (int i = threadIdx.x; i < b.tail; i += THREADS) db[b.whole * VB + i] = b.base[b.whole * VB + i];
}

template <typename T> ACTNN_DEV float lds_value(const T* p, int i);
template <> ACTNN_DEV float lds_value<float>(const float* p, int i) { return p[i]; }
template <> ACTNN_DEV float lds_value<__half>(const __half* p, int i) { return __half2float(p[i]); }
template <> ACTNN_DEV float lds_value<bf16_t>(const bf16_t* p, int i) { return bf16_bits_to_float(p[i].bits); }

// Geometry presets: with PRESET != 0 the window parameters are compile-time constants (loops
// unroll, divisions become shifts); PRESET 0 reads them from the argument.
//   1: 3x3 stride 2 pad 1 (ResNet stem)   2: 2x2 stride 2 pad 0   3: 3x3 stride 1 pad 1
template <int PRESET> struct Win {
  int KH, KW, SH, SW, PH, PW;
  __device__ __forceinline__ explicit Win(const PoolGeom& g)
      : KH(PRESET == 1 || PRESET == 3 ? 3 : PRESET == 2 ? 2 : g.KH),
        KW(PRESET == 1 || PRESET == 3 ? 3 : PRESET == 2 ? 2 : g.KW),
        SH(PRESET == 1 || PRESET == 2 ? 2 : PRESET == 3 ? 1 : g.SH),
        SW(PRESET == 1 || PRESET == 2 ? 2 : PRESET == 3 ? 1 : g.SW),
        PH(PRESET == 1 || PRESET == 3 ? 1 : PRESET == 2 ? 0 : g.PH),
        PW(PRESET == 1 || PRESET == 3 ? 1 : PRESET == 2 ? 0 : g.PW) {}
};

inline int preset_of(const PoolGeom& g) {
  if (g.KH == 3 && g.KW == 3 && g.SH == 2 && g.SW == 2 && g.PH == 1 && g.PW == 1) return 1;
  if (g.KH == 2 && g.KW == 2 && g.SH == 2 && g.SW == 2 && g.PH == 0 && g.PW == 0) return 2;
  if (g.KH == 3 && g.KW == 3 && g.SH == 1 && g.SW == 1 && g.PH == 1 && g.PW == 1) return 3;
  return 0;
}

template <typename T, int PRESET, bool NIB>      // NIB: Wo even, so the two outputs of a byte sit in one row
__global__ __launch_bounds__(kThreads) void max_pool2d_forward_lds_kernel(
    const T* __restrict__ x, T* __restrict__ y, int8_t* __restrict__ idx, int64_t total_in,
    PoolGeom g, int rows_per_band, int bands) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  T* s_in = reinterpret_cast<T*>(smem);
  const Win<PRESET> k(g);
  const int64_t nc = blockIdx.x / bands;
  const int ho0 = (int)(blockIdx.x % bands) * rows_per_band;
  const int rows_out = g.Ho - ho0 < rows_per_band ? g.Ho - ho0 : rows_per_band;
  int h_lo = ho0 * k.SH - k.PH;
  h_lo = h_lo > 0 ? h_lo : 0;
  int h_hi = (ho0 + rows_out - 1) * k.SH - k.PH + k.KH;
  h_hi = h_hi < g.H ? h_hi : g.H;
  const int shift = stage_span(x, nc * (int64_t)g.H * g.W + (int64_t)h_lo * g.W, (h_hi - h_lo) * g.W,
                               total_in, s_in);
  __syncthreads();
  const float init = Conv<T>::round(-1e10f);         // as the reference, .cu:656
  const int lane = threadIdx.x & 63;
  for (int r = threadIdx.x >> 6; r < rows_out; r += kThreads / 64) {     // one output row per wave
    const int ho = ho0 + r;
    const int h_base = ho * k.SH - k.PH;
    const int64_t orow = (nc * g.Ho + ho) * (int64_t)g.Wo;
    for (int wo = lane; wo < g.Wo; wo += 64) {
      const int w_base = wo * k.SW - k.PW;
      float v = init;
      int index = 0;
      for (int a = 0; a < k.KH; ++a) {
        const int i = h_base + a;
        if (i < 0 || i >= g.H) continue;
        const T* row = s_in + shift + (i - h_lo) * g.W;
        for (int b = 0; b < k.KW; ++b) {
          const int j = w_base + b;
          if (j < 0 || j >= g.W) continue;
          const float c = lds_value<T>(row, j);
          if (c > v) {
            v = c;
            index = a * k.KW + b;
          }
        }
      }
      Conv<T>::store(y, orow + wo, v);
      if (NIB) {
        const int next = lane_xor<1>(index);           // lane and wo have the same parity
        if (!(wo & 1)) idx[(orow + wo) >> 1] = (int8_t)(index | (next << 4));
      } else {
        idx[orow + wo] = (int8_t)index;
      }
    }
  }
}

template <typename T, int PRESET, bool NIB>
__global__ __launch_bounds__(kThreads) void max_pool2d_backward_lds_kernel(
    const T* __restrict__ gout, const int8_t* __restrict__ idx, T* __restrict__ gin,
    int64_t total_out, PoolGeom g, int rows_per_band, int bands, int max_out_rows) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  // [grad_output rows | index rows], each with room for the alignment shift
  T* s_g = reinterpret_cast<T*>(smem);
  int8_t* s_i = reinterpret_cast<int8_t*>(smem + (((size_t)max_out_rows * g.Wo + 16) * sizeof(T) + 15) / 16 * 16);
  const Win<PRESET> k(g);
  const int64_t nc = blockIdx.x / bands;
  const int h0 = (int)(blockIdx.x % bands) * rows_per_band;
  const int rows_in = g.H - h0 < rows_per_band ? g.H - h0 : rows_per_band;
  // output rows whose window touches input rows [h0, h0 + rows_in)
  int ho_lo = h0 + k.PH - k.KH + 1;
  ho_lo = ho_lo > 0 ? (ho_lo + k.SH - 1) / k.SH : 0;
  int ho_hi = (h0 + rows_in - 1 + k.PH) / k.SH;
  ho_hi = ho_hi < g.Ho - 1 ? ho_hi : g.Ho - 1;
  int shift_g = 0, shift_i = 0;
  if (ho_hi >= ho_lo) {
    const int64_t first = (nc * g.Ho + ho_lo) * (int64_t)g.Wo;
    const int count = (ho_hi - ho_lo + 1) * g.Wo;
    shift_g = stage_span(gout, first, count, total_out, s_g);
    if (NIB) {
      const int64_t b0 = first >> 1, b1 = (first + count + 1) >> 1;
      shift_i = 2 * stage_span(idx, b0, (int)(b1 - b0), (total_out + 1) >> 1, s_i) + (int)(first & 1);
    } else {
      shift_i = stage_span(idx, first, count, total_out, s_i);
    }
  }
  __syncthreads();
  const int lane = threadIdx.x & 63;
  for (int r = threadIdx.x >> 6; r < rows_in; r += kThreads / 64) {       // one input row per wave
    const int h = h0 + r;
    int a_lo = h + k.PH - k.KH + 1;
    a_lo = a_lo > 0 ? (a_lo + k.SH - 1) / k.SH : 0;
    int a_hi = (h + k.PH) / k.SH;
    a_hi = a_hi < g.Ho - 1 ? a_hi : g.Ho - 1;
    const int64_t irow = (nc * g.H + h) * (int64_t)g.W;
    for (int w = lane; w < g.W; w += 64) {
      int b_lo = w + k.PW - k.KW + 1;
      b_lo = b_lo > 0 ? (b_lo + k.SW - 1) / k.SW : 0;
      int b_hi = (w + k.PW) / k.SW;
      b_hi = b_hi < g.Wo - 1 ? b_hi : g.Wo - 1;
      float acc = 0.0f;
      for (int ho = a_lo; ho <= a_hi; ++ho) {
        const int kh = h - (ho * k.SH - k.PH);
        const int rr = (ho - ho_lo) * g.Wo;
        for (int wo = b_lo; wo <= b_hi; ++wo) {
          const int kw = w - (wo * k.SW - k.PW);
          if (staged_index<NIB>(s_i, shift_i + rr + wo) == kh * k.KW + kw) acc += lds_value<T>(s_g, shift_g + rr + wo);
        }
      }
      Conv<T>::store(gin, irow + w, acc);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Stride-2 fast path (3x3 pad 1 and 2x2 pad 0 with W % 8 == 0, Wo == W / 2, Ho == H / 2): the
// shapes of every stem / VGG-style pooling layer.  A thread produces 4 adjacent outputs from three
// 16-byte LDS reads (forward) or 8 adjacent inputs of two rows from a handful of LDS reads
// (backward), compares against compile-time window positions, and writes 8/16-byte pieces that are
// contiguous across the wave.  Padding is handled by data, not by branches: the row above the
// plane is staged as the initial value, out-of-range windows get an index that matches nothing.
template <typename T> ACTNN_DEV void store4(T* p, const float (&v)[4]);
template <> ACTNN_DEV void store4<float>(float* p, const float (&v)[4]) {
  store16(p, (u32x4){as_uint(v[0]), as_uint(v[1]), as_uint(v[2]), as_uint(v[3])});
}
template <> ACTNN_DEV void store4<__half>(__half* p, const float (&v)[4]) {
  *reinterpret_cast<u32x2*>(p) = (u32x2){float_to_half_bits(v[0]) | (float_to_half_bits(v[1]) << 16),
                                         float_to_half_bits(v[2]) | (float_to_half_bits(v[3]) << 16)};
}
template <> ACTNN_DEV void store4<bf16_t>(bf16_t* p, const float (&v)[4]) {
  *reinterpret_cast<u32x2*>(p) = (u32x2){pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
}

// 4 consecutive elements from LDS (8/16-byte aligned)
ACTNN_DEV void load4(const float* p, float (&v)[4]) {
  const u32x4 a = *reinterpret_cast<const u32x4*>(p);
  v[0] = as_float(a.x), v[1] = as_float(a.y), v[2] = as_float(a.z), v[3] = as_float(a.w);
}
ACTNN_DEV void load4(const __half* p, float (&v)[4]) {
  const u32x2 a = *reinterpret_cast<const u32x2*>(p);
  const uint32_t lo = a.x, hi = a.y;
  v[0] = half_bits_to_float(lo & 0xffffu), v[1] = half_bits_to_float(lo >> 16);
  v[2] = half_bits_to_float(hi & 0xffffu), v[3] = half_bits_to_float(hi >> 16);
}
ACTNN_DEV void load4(const bf16_t* p, float (&v)[4]) {
  const u32x2 a = *reinterpret_cast<const u32x2*>(p);
  const uint32_t lo = a.x, hi = a.y;
  v[0] = as_float(lo << 16), v[1] = as_float(lo & 0xffff0000u);
  v[2] = as_float(hi << 16), v[3] = as_float(hi & 0xffff0000u);
}

template <typename T, int K, int P, bool NIB>
__global__ __launch_bounds__(kFwdS2Threads) void max_pool2d_forward_s2_kernel(
    const T* __restrict__ x, T* __restrict__ y, int8_t* __restrict__ idx, PoolGeom g, int rows_per_band,
    int bands) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  constexpr int V = 16 / (int)sizeof(T);
  T* s_in = reinterpret_cast<T*>(smem) + 8;             // front pad: column -1 of the first row is addressable
  const int64_t nc = blockIdx.x / bands;
  const int ho0 = (int)(blockIdx.x % bands) * rows_per_band;
  const int rows_out = g.Ho - ho0 < rows_per_band ? g.Ho - ho0 : rows_per_band;
  const int W = g.W, cpr = g.Wo >> 2;
  const int i_first = 2 * ho0 - P;                      // -1 for the first band when P == 1
  const int rows_in = 2 * (rows_out - 1) + K;
  const int skip = i_first < 0 ? 1 : 0;
  const float init = Conv<T>::round(-1e10f);            // as the reference, .cu:656
  {
    const T* src = x + (nc * g.H + i_first + skip) * (int64_t)W;
    T* dst = s_in + skip * W;
    copy_vectors<kFwdS2Threads, true>(src, dst, (rows_in - skip) * (W / V));
    if (skip)
      for (int v = threadIdx.x; v < W; v += kFwdS2Threads) Conv<T>::store(s_in, v, init);
  }
  __syncthreads();
  const int items = rows_out * cpr;
  for (int item = threadIdx.x; item < items; item += kFwdS2Threads) {
    const int r = item / cpr, q = item - r * cpr;
    float cc[K][9];                                     // cc[a][1 + e]: column 8q + e of window row a
#pragma unroll
    for (int a = 0; a < K; ++a) {
      const T* row = s_in + (2 * r + a) * W + 8 * q;
      load8(row, reinterpret_cast<float(&)[8]>(cc[a][1]));
      const float left = lds_value<T>(row, -1);         // the front pad keeps this inside LDS
      cc[a][0] = P == 1 && q > 0 ? left : init;
    }
    float out[4];
    uint64_t packed_idx = 0;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      float v = init;
      uint32_t index = 0;
#pragma unroll
      for (int a = 0; a < K; ++a)
#pragma unroll
        for (int b = 0; b < K; ++b) {
          const float c = cc[a][2 * u - P + b + 1];
          if (c > v) {
            v = c;
            index = a * K + b;
          }
        }
      out[u] = v;
      packed_idx |= (uint64_t)index << (IndexFields<NIB>::kBits * u);
    }
    const int64_t o = (nc * g.Ho + ho0 + r) * (int64_t)g.Wo + 4 * q;
    store4<T>(y + o, out);
    IndexFields<NIB>::template store<4>(idx, o, packed_idx);
  }
}

template <typename T, int K, int P, bool NIB>
__global__ __launch_bounds__(kBwdS2Threads) void max_pool2d_backward_s2_kernel(
    const T* __restrict__ gout, const int8_t* __restrict__ idx, T* __restrict__ gin, int64_t total_out,
    PoolGeom g, int pairs_per_band, int bands, int max_out_rows, FastDiv by_cpr) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  constexpr int EXTRA = K == 3 ? 1 : 0;                 // windows of the next output row reach odd input rows
  constexpr int NW = 4 + EXTRA;                         // output columns that touch 8 input columns
  T* s_g = reinterpret_cast<T*>(smem);
  int8_t* s_i = reinterpret_cast<int8_t*>(smem + (((size_t)max_out_rows * g.Wo + 16) * sizeof(T) + 15) / 16 * 16);
  const int64_t nc = blockIdx.x / bands;
  const int s0 = (int)(blockIdx.x % bands) * pairs_per_band;
  const int pairs = g.Ho - s0 < pairs_per_band ? g.Ho - s0 : pairs_per_band;
  const int ho_hi = s0 + pairs - 1 + EXTRA < g.Ho - 1 ? s0 + pairs - 1 + EXTRA : g.Ho - 1;
  const int64_t first = (nc * g.Ho + s0) * (int64_t)g.Wo;
  const int count = (ho_hi - s0 + 1) * g.Wo;
  int shift_g, shift_i;
  if constexpr (NIB) {
    // (first and count are multiples of 4: whole bytes in the two-per-byte format)
    const Span<T> span_g = span_of(gout, first, count, total_out);
    const Span<int8_t> span_i = span_of(idx, first >> 1, count >> 1, total_out >> 1);
    stage_two<kBwdS2Threads>(span_g, s_g, span_i, s_i);
    shift_g = span_g.shift;
    shift_i = 2 * span_i.shift;
  } else {
    // (one index per byte: staged one span after the other; in one round it measured 10 % faster on
    // one machine and 19 % slower on another)
    shift_g = stage_span<T, kBwdS2Threads, false>(gout, first, count, total_out, s_g);
    shift_i = stage_span<int8_t, kBwdS2Threads, false>(idx, first, count, total_out, s_i);
  }
  __syncthreads();
  const int cpr = g.W >> 3;
  const int items = pairs * cpr;
  for (int item = threadIdx.x; item < items; item += kBwdS2Threads) {
    const int r = (int)by_cpr.div((uint32_t)item), q = item - r * cpr;
    float gv[1 + EXTRA][NW];
    int iv[1 + EXTRA][NW];
#pragma unroll
    for (int j = 0; j <= EXTRA; ++j) {
      const int at = (r + j) * g.Wo + 4 * q;
      const bool row_ok = s0 + r + j < g.Ho;
      // Wo % 4 == 0 makes both positions 4-element aligned
      load4(s_g + shift_g + at, reinterpret_cast<float(&)[4]>(gv[j][0]));
      const uint64_t i4 = IndexFields<NIB>::template load<4>(s_i, (int64_t)(shift_i + at));
#pragma unroll
      for (int t = 0; t < 4; ++t) iv[j][t] = row_ok ? IndexFields<NIB>::get(i4, t) : -1;
      if (EXTRA) {
        gv[j][NW - 1] = lds_value<T>(s_g, shift_g + at + 4);
        iv[j][NW - 1] = row_ok && q < cpr - 1 ? staged_index<NIB>(s_i, shift_i + at + 4) : -1;
      }
    }
#pragma unroll
    for (int rr = 0; rr < 2; ++rr) {
      float out[8];
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        float acc = 0.0f;
#pragma unroll
        for (int j = 0; j <= EXTRA; ++j) {
          const int kh = rr + P - 2 * j;
          if (kh < 0 || kh >= K) continue;
#pragma unroll
          for (int t = 0; t < NW; ++t) {
            const int kw = c + P - 2 * t;
            if (kw < 0 || kw >= K) continue;
            acc += iv[j][t] == kh * K + kw ? gv[j][t] : 0.0f;
          }
        }
        out[c] = acc;
      }
      store8_nt(gin + (nc * g.H + 2 * (s0 + r) + rr) * (int64_t)g.W + 8 * q, out);
    }
  }
}

// the stride-2 kernels' shape requirements; K = 3 (pad 1) or 2 (pad 0)
inline int s2_kernel_of(const PoolGeom& g) {
  const int p = preset_of(g);
  if (p != 1 && p != 2) return 0;
  if (g.W % 8 != 0 || g.Wo * 2 != g.W || g.Ho * 2 != g.H) return 0;
  return p == 1 ? 3 : 2;
}

// rows per band so that a block has about `want` elements of work and the LDS need (computed by
// `bytes(rows)`) fits the budget; 0 if even one row does not fit.
template <typename F> int pick_rows(int rows_total, int row_elems, int want, F bytes) {
  int rows = (want + row_elems - 1) / row_elems;
  rows = rows < 1 ? 1 : (rows > rows_total ? rows_total : rows);
  while (rows > 1 && bytes(rows) > (size_t)kLdsBudget) --rows;
  return bytes(rows) <= (size_t)kLdsBudget ? rows : 0;
}

// Band height for the stride-2 kernels: `units` rows (or row pairs) of `per_unit` work items each
// are cut into bands of equal height; a block of `threads` walks its band in passes of `threads` items.  Picks
// the height with the fewest idle thread slots among those that fit the LDS budget and need at
// most `max_passes` passes, preferring taller bands (fewer halo rows) on ties.  0 if nothing fits.
template <typename F> int pick_band(int units, int per_unit, int threads, int max_passes, F bytes) {
  int best = 0;
  double best_eff = 0.0;
  for (int rows = 1; rows <= units; ++rows) {
    if (bytes(rows) > (size_t)kLdsBudget) break;
    const int passes = (rows * per_unit + threads - 1) / threads;
    if (passes > max_passes && best > 0) break;
    const int full = units / rows, rest = units % rows;
    const int64_t slots = (int64_t)full * passes * threads +
                          (rest ? (int64_t)((rest * per_unit + threads - 1) / threads) * threads : 0);
    const double eff = (double)units * per_unit / (double)slots;
    if (eff >= best_eff) {
      best_eff = eff;
      best = rows;
    }
  }
  return best;
}

template <typename T, bool NIB>
int launch_fwd(const void* x, void* y, int8_t* idx, int64_t total, const PoolGeom& g, hipStream_t s) {
  const int64_t planes = total / ((int64_t)g.Ho * g.Wo);
  auto need = [&](int rows) { return ((size_t)((rows - 1) * g.SH + g.KH) * g.W + 16) * sizeof(T); };
  if (const int k = s2_kernel_of(g); k != 0 && aligned16(x) && aligned16(y) && aligned16(idx)) {
    const int rb = pick_band(g.Ho, g.Wo / 4, kFwdS2Threads, kFwdS2Passes, need);
    const int bands = rb > 0 ? (g.Ho + rb - 1) / rb : 0;
    if (rb > 0 && planes * bands <= 0x7fffffffLL) {
      const dim3 grid((unsigned)(planes * bands)), blk(kFwdS2Threads);
      const T* xi = static_cast<const T*>(x);
      T* yo = static_cast<T*>(y);
      if (k == 3) max_pool2d_forward_s2_kernel<T, 3, 1, NIB><<<grid, blk, need(rb), s>>>(xi, yo, idx, g, rb, bands);
      else max_pool2d_forward_s2_kernel<T, 2, 0, NIB><<<grid, blk, need(rb), s>>>(xi, yo, idx, g, rb, bands);
      ACTNN_RETURN_LAUNCH_STATUS();
    }
  }
  const int rb = pick_rows(g.Ho, g.Wo, 1024, need);
  if (rb > 0 && aligned16(x) && (!NIB || g.Wo % 2 == 0)) {
    const int bands = (g.Ho + rb - 1) / rb;
    if (planes * bands <= 0x7fffffffLL) {
      const dim3 grid((unsigned)(planes * bands)), blk(kThreads);
      const T* xi = static_cast<const T*>(x);
      T* yo = static_cast<T*>(y);
      const int64_t tin = planes * g.H * g.W;
      switch (preset_of(g)) {
        case 1: max_pool2d_forward_lds_kernel<T, 1, NIB><<<grid, blk, need(rb), s>>>(xi, yo, idx, tin, g, rb, bands); break;
        case 2: max_pool2d_forward_lds_kernel<T, 2, NIB><<<grid, blk, need(rb), s>>>(xi, yo, idx, tin, g, rb, bands); break;
        case 3: max_pool2d_forward_lds_kernel<T, 3, NIB><<<grid, blk, need(rb), s>>>(xi, yo, idx, tin, g, rb, bands); break;
        default: max_pool2d_forward_lds_kernel<T, 0, NIB><<<grid, blk, need(rb), s>>>(xi, yo, idx, tin, g, rb, bands); break;
      }
      ACTNN_RETURN_LAUNCH_STATUS();
    }
  }
  const int64_t blocks = (total + kThreads - 1) / kThreads;
  if (blocks > 0x7fffffffLL) return ACTNN_EINVAL;
  max_pool2d_forward_kernel<T, NIB><<<dim3((unsigned)blocks), dim3(kThreads), 0, s>>>(
      static_cast<const T*>(x), static_cast<T*>(y), idx, total, g);
  ACTNN_RETURN_LAUNCH_STATUS();
}

template <typename T, bool NIB>
int launch_bwd(const void* gout, const int8_t* idx, void* gin, int64_t total, const PoolGeom& g,
               hipStream_t s) {
  const int64_t planes = total / ((int64_t)g.H * g.W);
  // output rows a band of `rows` input rows can touch
  auto out_rows = [&](int rows) { return (rows + g.KH - 2) / g.SH + 2; };
  auto need = [&](int rows) {
    const size_t elems = (size_t)out_rows(rows) * g.Wo + 16;
    return (elems * sizeof(T) + 15) / 16 * 16 + elems + 16;
  };
  if (const int k = s2_kernel_of(g); k != 0 && aligned16(gout) && aligned16(idx) && aligned16(gin)) {
    // bands of input-row pairs; pair s reads output rows s (and s + 1 for 3x3)
    auto need2 = [&](int pairs) {
      const size_t elems = (size_t)(pairs + 2) * g.Wo + 16;
      return (elems * sizeof(T) + 15) / 16 * 16 + elems + 16;
    };
    const int pb = pick_band(g.Ho, g.W / 8, kBwdS2Threads, kBwdS2Passes, need2);
    const int bands = pb > 0 ? (g.Ho + pb - 1) / pb : 0;
    if (pb > 0 && planes * bands <= 0x7fffffffLL) {
      const dim3 grid((unsigned)(planes * bands)), blk(kBwdS2Threads);
      const T* go = static_cast<const T*>(gout);
      T* gi = static_cast<T*>(gin);
      const int64_t tout = planes * g.Ho * g.Wo;
      if (k == 3) max_pool2d_backward_s2_kernel<T, 3, 1, NIB><<<grid, blk, need2(pb), s>>>(go, idx, gi, tout, g, pb, bands, pb + 2, FastDiv((uint32_t)(g.W / 8)));
      else max_pool2d_backward_s2_kernel<T, 2, 0, NIB><<<grid, blk, need2(pb), s>>>(go, idx, gi, tout, g, pb, bands, pb + 2, FastDiv((uint32_t)(g.W / 8)));
      ACTNN_RETURN_LAUNCH_STATUS();
    }
  }
  const int rb = pick_rows(g.H, g.W, 2048, need);
  if (rb > 0 && aligned16(gout) && aligned16(idx)) {
    const int bands = (g.H + rb - 1) / rb;
    if (planes * bands <= 0x7fffffffLL) {
      const dim3 grid((unsigned)(planes * bands)), blk(kThreads);
      const T* go = static_cast<const T*>(gout);
      T* gi = static_cast<T*>(gin);
      const int64_t tout = planes * g.Ho * g.Wo;
      const int orows = out_rows(rb);
      switch (preset_of(g)) {
        case 1: max_pool2d_backward_lds_kernel<T, 1, NIB><<<grid, blk, need(rb), s>>>(go, idx, gi, tout, g, rb, bands, orows); break;
        case 2: max_pool2d_backward_lds_kernel<T, 2, NIB><<<grid, blk, need(rb), s>>>(go, idx, gi, tout, g, rb, bands, orows); break;
        case 3: max_pool2d_backward_lds_kernel<T, 3, NIB><<<grid, blk, need(rb), s>>>(go, idx, gi, tout, g, rb, bands, orows); break;
        default: max_pool2d_backward_lds_kernel<T, 0, NIB><<<grid, blk, need(rb), s>>>(go, idx, gi, tout, g, rb, bands, orows); break;
      }
      ACTNN_RETURN_LAUNCH_STATUS();
    }
  }
  const int64_t blocks = (total + kThreads - 1) / kThreads;
  if (blocks > 0x7fffffffLL) return ACTNN_EINVAL;
  max_pool2d_backward_kernel<T, NIB><<<dim3((unsigned)blocks), dim3(kThreads), 0, s>>>(
      static_cast<const T*>(gout), idx, static_cast<T*>(gin), total, g);
  ACTNN_RETURN_LAUNCH_STATUS();
}

// ------------------------------------------------------------------ channels-last ([N, H, W, C])
// A thread owns one 16-byte chunk of channels of one pixel; consecutive threads take consecutive
// chunks, then the next pixel, so every access of a wave is a run of whole cache lines and the
// overlap between neighbouring windows is served by the caches.  Same scan order and strict
// compare as the default-layout kernels, hence the same values and indices.
template <typename T> struct PoolChunk;
template <> struct PoolChunk<float> { static constexpr int kElems = 4; };
template <> struct PoolChunk<__half> { static constexpr int kElems = 8; };
template <> struct PoolChunk<bf16_t> { static constexpr int kElems = 8; };

template <typename T, int E> ACTNN_DEV void widen_chunk(const T* p, float (&v)[E]) {
  if constexpr (E == 4) {
    const u32x4 u = load16(p);
    v[0] = as_float(u.x); v[1] = as_float(u.y); v[2] = as_float(u.z); v[3] = as_float(u.w);
  } else {
    load8(p, v);
  }
}
// a dword filled with the value v of type T
template <typename T> ACTNN_DEV uint32_t dword_of(float v);
template <> ACTNN_DEV uint32_t dword_of<float>(float v) { return as_uint(v); }
template <> ACTNN_DEV uint32_t dword_of<__half>(float v) { return float_to_half_bits(v) * 0x10001u; }
template <> ACTNN_DEV uint32_t dword_of<bf16_t>(float v) { return float_to_bf16_bits(v) * 0x10001u; }
template <typename T, int E> ACTNN_DEV void raw_widen_chunk(const u32x4& u, float (&v)[E]) {
  if constexpr (E == 4) {
    v[0] = as_float(u.x); v[1] = as_float(u.y); v[2] = as_float(u.z); v[3] = as_float(u.w);
  } else {
    Raw8<T> r;
    r.a = u;
    raw8_widen(r, v);
  }
}
template <typename T, int E> ACTNN_DEV void narrow_chunk(T* p, const float (&v)[E]) {
  if constexpr (E == 4) store16(p, u32x4{as_uint(v[0]), as_uint(v[1]), as_uint(v[2]), as_uint(v[3])});
  else store8(p, v);
}
// the same as a streamed store: for tensors that are written once and not read by the kernel
template <typename T, int E> ACTNN_DEV void narrow_chunk_nt(T* p, const float (&v)[E]) {
  if constexpr (E == 4) store16_nt(p, u32x4{as_uint(v[0]), as_uint(v[1]), as_uint(v[2]), as_uint(v[3])});
  else store8_nt(p, v);
}

template <typename T, bool NIB>
__global__ __launch_bounds__(kThreads) void max_pool2d_forward_cl_kernel(
    const T* __restrict__ x, T* __restrict__ y, int8_t* __restrict__ idx, int64_t chunks, int cpp /* chunks per pixel */,
    int64_t C, PoolGeom g) {
  constexpr int E = PoolChunk<T>::kElems;
  // (neighbouring output rows share input rows: their blocks stay on one XCD)
  const int64_t id = xcd_block() * kThreads + threadIdx.x;
  if (id >= chunks) return;
  const int c = (int)(id % cpp) * E;
  const int64_t pix = id / cpp;
  const int w = (int)(pix % g.Wo);
  const int h = (int)((pix / g.Wo) % g.Ho);
  const int64_t n = pix / ((int64_t)g.Wo * g.Ho);
  const int h_base = h * g.SH - g.PH, w_base = w * g.SW - g.PW;
  const int h_start = h_base > 0 ? h_base : 0, h_end = h_base + g.KH < g.H ? h_base + g.KH : g.H;
  const int w_start = w_base > 0 ? w_base : 0, w_end = w_base + g.KW < g.W ? w_base + g.KW : g.W;
  float best[E];
  int where[E];
  const float init = Conv<T>::round(-1e10f);      // .cu:656, narrowed to the element type
#pragma unroll
  for (int e = 0; e < E; ++e) { best[e] = init; where[e] = 0; }
  const T* img = x + n * (int64_t)g.H * g.W * C + c;
  for (int i = h_start; i < h_end; ++i) {
    for (int j = w_start; j < w_end; ++j) {
      float v[E];
      widen_chunk<T, E>(img + ((int64_t)i * g.W + j) * C, v);
      const int k = (i - h_base) * g.KW + (j - w_base);
#pragma unroll
      for (int e = 0; e < E; ++e)
        if (v[e] > best[e]) { best[e] = v[e]; where[e] = k; }
    }
  }
  narrow_chunk<T, E>(y + pix * C + c, best);
  uint64_t fields = 0;
#pragma unroll
  for (int e = 0; e < E; ++e) fields |= (uint64_t)where[e] << (IndexFields<NIB>::kBits * e);
  IndexFields<NIB>::template store<E>(idx, pix * C + c, fields);
}

// Where a thread of the window kernels below works, without 64-bit arithmetic (which costs more
// instructions than the window itself: these kernels are bound by the vector ALUs, not by memory).
// Blocks are numbered image by image; a thread's number inside its image (below 2^31) splits into
// pixel row, column and chunk of channels by multiply-high divisions, and every address is a
// uniform base (image, window position) plus one 32-bit lane offset.
struct ClGeom {
  uint32_t cpp, cols;                     // chunks per pixel; pixels per row of the thread grid
  uint32_t per_image;                     // threads per image: rows * cols * cpp
  uint32_t blocks_per_image, blocks;
  FastDiv by_cpp, by_cols, by_blocks_per_image;
};
struct ClAt {
  uint32_t n, i, row, col, chunk;
  bool live;
};
ACTNN_DEV ClAt cl_at(const ClGeom& q) {
  ClAt a;
  // (neighbouring rows share input rows or windows: their blocks stay on one XCD)
  const uint32_t block = (blockIdx.x % kXcds) * (gridDim.x / kXcds) + blockIdx.x / kXcds;
  a.n = q.by_blocks_per_image.div(block);
  a.i = (block - a.n * q.blocks_per_image) * kThreads + threadIdx.x;
  a.live = block < q.blocks && a.i < q.per_image;
  const uint32_t pixel = q.by_cpp.div(a.i);
  a.chunk = a.i - pixel * q.cpp;
  a.row = q.by_cols.div(pixel);
  a.col = pixel - a.row * q.cols;
  return a;
}

// Forward for the windows known at compile time (the presets): all loads of the window are issued
// before the first comparison (taken one at a time their latencies add up); positions outside the
// image get the start value, which never wins the strict compare.  Same scan order as above.
template <typename T, int PRESET, bool NIB>
__global__ __launch_bounds__(kThreads) void max_pool2d_forward_cl_window_kernel(
    const T* __restrict__ x, T* __restrict__ y, int8_t* __restrict__ idx, ClGeom q, PoolGeom g) {
  constexpr int E = PoolChunk<T>::kElems;
  constexpr int KH = PRESET == 2 ? 2 : 3, KW = KH;
  const Win<PRESET> k(g);
  const ClAt at = cl_at(q);
  if (!at.live) return;
  const uint32_t C = q.cpp * E;
  const int i0 = (int)at.row * k.SH - k.PH, j0 = (int)at.col * k.SW - k.PW;
  // the lane's offset counts from the window origin moved by the padding, so it is never negative;
  // the uniform bases take the padding back
  const uint32_t lane = ((at.row * k.SH) * (uint32_t)g.W + at.col * k.SW) * C + at.chunk * E;
  const T* img = x + (int64_t)at.n * g.H * g.W * C;
  const float init = Conv<T>::round(-1e10f);      // .cu:656, narrowed to the element type
  const uint32_t fill = dword_of<T>(init);
  u32x4 raw[KH * KW];
#pragma unroll
  for (int a = 0; a < KH; ++a)
#pragma unroll
    for (int b = 0; b < KW; ++b) {
      const bool inside = (uint32_t)(i0 + a) < (uint32_t)g.H && (uint32_t)(j0 + b) < (uint32_t)g.W;
      const T* base = img + ((int64_t)(a - k.PH) * g.W + (b - k.PW)) * (int64_t)C;
      // pixels that no other window reads (every pixel of a 2x2 stride-2 window, the centre of a 3x3
      // stride-2 one) are streamed; the others are read again by the neighbours and stay cached
      const bool once = PRESET == 2 || (PRESET == 1 && a == 1 && b == 1);   // (constant after unrolling)
      raw[a * KW + b] = inside ? (once ? load16_nt(base + lane) : load16(base + lane)) : u32x4{fill, fill, fill, fill};
    }
  float best[E];
  int where[E];
#pragma unroll
  for (int e = 0; e < E; ++e) { best[e] = init; where[e] = 0; }
#pragma unroll
  for (int p = 0; p < KH * KW; ++p) {
    float v[E];
    raw_widen_chunk<T, E>(raw[p], v);
#pragma unroll
    for (int e = 0; e < E; ++e)
      if (v[e] > best[e]) { best[e] = v[e]; where[e] = p; }
  }
  const int64_t image_o = (int64_t)at.n * q.per_image * E;     // outputs before this image
  const uint32_t lane_o = at.i * E;
  narrow_chunk_nt<T, E>(y + image_o + lane_o, best);
  uint64_t fields = 0;
#pragma unroll
  for (int e = 0; e < E; ++e) fields |= (uint64_t)where[e] << (IndexFields<NIB>::kBits * e);
  IndexFields<NIB>::template store<E>(idx + IndexFields<NIB>::byte_of(image_o), (int64_t)lane_o, fields);
}

// Gather form of the backward pass: every input position sums the gradients of the windows that
// chose it, in a fixed order (no atomics, no zero fill).
template <typename T, bool NIB>
__global__ __launch_bounds__(kThreads) void max_pool2d_backward_cl_kernel(
    const T* __restrict__ gout, const int8_t* __restrict__ idx, T* __restrict__ gin, int64_t chunks, int cpp,
    int64_t C, PoolGeom g) {
  constexpr int E = PoolChunk<T>::kElems;
  const int64_t id = xcd_block() * kThreads + threadIdx.x;
  if (id >= chunks) return;
  const int c = (int)(id % cpp) * E;
  const int64_t pix = id / cpp;
  const int w = (int)(pix % g.W);
  const int h = (int)((pix / g.W) % g.H);
  const int64_t n = pix / ((int64_t)g.W * g.H);
  int ho_lo = h + g.PH - g.KH + 1;
  ho_lo = ho_lo > 0 ? (ho_lo + g.SH - 1) / g.SH : 0;
  int ho_hi = (h + g.PH) / g.SH;
  ho_hi = ho_hi < g.Ho - 1 ? ho_hi : g.Ho - 1;
  int wo_lo = w + g.PW - g.KW + 1;
  wo_lo = wo_lo > 0 ? (wo_lo + g.SW - 1) / g.SW : 0;
  int wo_hi = (w + g.PW) / g.SW;
  wo_hi = wo_hi < g.Wo - 1 ? wo_hi : g.Wo - 1;
  float acc[E];
#pragma unroll
  for (int e = 0; e < E; ++e) acc[e] = 0.0f;
  const int64_t obase = n * (int64_t)g.Ho * g.Wo;
  for (int ho = ho_lo; ho <= ho_hi; ++ho) {
    const int kh = h - (ho * g.SH - g.PH);
    for (int wo = wo_lo; wo <= wo_hi; ++wo) {
      const int k = kh * g.KW + (w - (wo * g.SW - g.PW));
      const int64_t o = (obase + (int64_t)ho * g.Wo + wo) * C + c;
      float v[E];
      widen_chunk<T, E>(gout + o, v);
      const uint64_t fields = IndexFields<NIB>::template load<E>(idx, o);
#pragma unroll
      for (int e = 0; e < E; ++e)
        if (IndexFields<NIB>::get(fields, e) == k) acc[e] += v[e];
    }
  }
  narrow_chunk<T, E>(gin + pix * C + c, acc);
}

// Backward for the stride-2 windows of the stem / VGG-style layers (3x3 pad 1 and 2x2 pad 0, H and W
// even): a thread owns the 2x2 block of input pixels (2a.., 2b..) of one chunk of channels.  The windows
// that reach the block are (a..a+1) x (b..b+1) (3x3) or (a, b) alone (2x2): one (gradient, index) load
// per input pixel where the general kernel needs 2.25 (3x3).  Every pixel adds its windows in the
// general kernel's order (rows, then columns), hence the same bits.  grad_in is written once and
// not read: streamed stores (measured 0.104 -> 0.079 ms on f16 [256,64,112,112]).
template <typename T, int K, int P, bool NIB>
__global__ __launch_bounds__(kThreads) void max_pool2d_backward_cl_s2_kernel(
    const T* __restrict__ gout, const int8_t* __restrict__ idx, T* __restrict__ gin, ClGeom q, PoolGeom g) {
  constexpr int E = PoolChunk<T>::kElems;
  constexpr int NWIN = K == 3 ? 2 : 1;
  constexpr uint64_t kNone = ~uint64_t(0);             // fields that match no window position (K * K < 15)
  const ClAt at = cl_at(q);                            // rows and columns of windows
  if (!at.live) return;
  const uint32_t C = q.cpp * E;
  const int64_t image_o = (int64_t)at.n * q.per_image * E;
  const uint32_t lane_o = at.i * E;                    // window (row, col) of this chunk inside the image
  const T* gimg = gout + image_o;
  const int8_t* iimg = idx + IndexFields<NIB>::byte_of(image_o);
  u32x4 raw[NWIN][NWIN];
  uint64_t fields[NWIN][NWIN];
#pragma unroll
  for (int j = 0; j < NWIN; ++j)
#pragma unroll
    for (int t = 0; t < NWIN; ++t) {
      const bool inside = at.row + j < (uint32_t)g.Ho && at.col + t < (uint32_t)g.Wo;
      const int64_t step = ((int64_t)j * g.Wo + t) * C;              // uniform
      raw[j][t] = inside ? load16(gimg + step + lane_o) : u32x4{0, 0, 0, 0};
      fields[j][t] = inside ? IndexFields<NIB>::template load<E>(iimg + IndexFields<NIB>::byte_of(step), (int64_t)lane_o) : kNone;
    }
  float acc[2][2][E];
#pragma unroll
  for (int rr = 0; rr < 2; ++rr)
#pragma unroll
    for (int cc = 0; cc < 2; ++cc)
#pragma unroll
      for (int e = 0; e < E; ++e) acc[rr][cc][e] = 0.0f;
#pragma unroll
  for (int j = 0; j < NWIN; ++j) {
#pragma unroll
    for (int t = 0; t < NWIN; ++t) {
      float v[E];
      raw_widen_chunk<T, E>(raw[j][t], v);
      // input row 2a + rr sits at window row kh = rr + P - 2j of window row a + j; columns alike
#pragma unroll
      for (int rr = 0; rr < 2; ++rr) {
        const int kh = rr + P - 2 * j;
        if (kh < 0 || kh >= K) continue;
#pragma unroll
        for (int cc = 0; cc < 2; ++cc) {
          const int kw = cc + P - 2 * t;
          if (kw < 0 || kw >= K) continue;
#pragma unroll
          for (int e = 0; e < E; ++e)
            if (IndexFields<NIB>::get(fields[j][t], e) == kh * K + kw) acc[rr][cc][e] += v[e];
        }
      }
    }
  }
  T* out = gin + (int64_t)at.n * g.H * g.W * C;
  const uint32_t lane_in = (2 * at.row * (uint32_t)g.W + 2 * at.col) * C + at.chunk * E;
#pragma unroll
  for (int rr = 0; rr < 2; ++rr)
#pragma unroll
    for (int cc = 0; cc < 2; ++cc)
      narrow_chunk_nt<T, E>(out + ((int64_t)rr * g.W + cc) * C + lane_in, acc[rr][cc]);
}

// thread positions for rows x cols pixels per image; false when an image is too large for 32-bit offsets
inline bool cl_geometry(int64_t N, int64_t rows, int64_t cols, int64_t cpp, int64_t image_elems, ClGeom& q) {
  const int64_t per_image = rows * cols * cpp;
  if (image_elems >= 0x7fffffffLL || per_image >= 0x7fffffffLL || per_image == 0) return false;
  const int64_t bpi = (per_image + kThreads - 1) / kThreads;
  if (N * bpi > 0x7ffffff0LL) return false;
  q.cpp = (uint32_t)cpp;
  q.cols = (uint32_t)cols;
  q.per_image = (uint32_t)per_image;
  q.blocks_per_image = (uint32_t)bpi;
  q.blocks = (uint32_t)(N * bpi);
  q.by_cpp = FastDiv((uint32_t)cpp);
  q.by_cols = FastDiv((uint32_t)cols);
  q.by_blocks_per_image = FastDiv((uint32_t)bpi);
  return true;
}

template <typename T, bool NIB>
int launch_cl(bool forward, const void* a, const int8_t* idx_in, int8_t* idx_out, void* out, int64_t N, int64_t C,
              const PoolGeom& g, hipStream_t s) {
  constexpr int E = PoolChunk<T>::kElems;
  if (C % E != 0 || C / E > 0x7fffffffLL) return ACTNN_EINVAL;
  // a thread stores or loads the E indices of its chunk as one integer of E * (4 or 8) bits
  constexpr uintptr_t kIdxAlign = E * (NIB ? 4 : 8) / 8;
  if (!aligned16(a) || !aligned16(out)) return ACTNN_EALIGN;
  if (reinterpret_cast<uintptr_t>(forward ? idx_out : idx_in) % kIdxAlign != 0) return ACTNN_EALIGN;
  const int cpp = (int)(C / E);
  const int64_t pixels = forward ? N * g.Ho * g.Wo : N * (int64_t)g.H * g.W;
  const int64_t chunks = pixels * cpp;
  const int64_t blocks = (chunks + kThreads - 1) / kThreads;
  if (blocks > 0x7ffffff0LL) return ACTNN_EINVAL;
  if (blocks == 0) return ACTNN_OK;
  ClGeom q;
  // the padded input image must fit 32-bit element offsets for the window kernels
  const int64_t image_elems = ((int64_t)g.H + 2) * ((int64_t)g.W + 2) * C;
  const int p = preset_of(g);
  if (forward) {
    const T* xi = static_cast<const T*>(a);
    T* yo = static_cast<T*>(out);
    if (p != 0 && cl_geometry(N, g.Ho, g.Wo, cpp, image_elems, q)) {
      const dim3 grid(xcd_grid(q.blocks)), blk(kThreads);
      switch (p) {
        case 1: max_pool2d_forward_cl_window_kernel<T, 1, NIB><<<grid, blk, 0, s>>>(xi, yo, idx_out, q, g); break;
        case 2: max_pool2d_forward_cl_window_kernel<T, 2, NIB><<<grid, blk, 0, s>>>(xi, yo, idx_out, q, g); break;
        default: max_pool2d_forward_cl_window_kernel<T, 3, NIB><<<grid, blk, 0, s>>>(xi, yo, idx_out, q, g); break;
      }
    } else {
      max_pool2d_forward_cl_kernel<T, NIB><<<dim3(xcd_grid(blocks)), dim3(kThreads), 0, s>>>(xi, yo, idx_out, chunks, cpp, C, g);
    }
  } else if ((p == 1 || p == 2) && g.H == 2 * g.Ho && g.W == 2 * g.Wo && cl_geometry(N, g.Ho, g.Wo, cpp, image_elems, q)) {
    const dim3 grid(xcd_grid(q.blocks)), blk(kThreads);
    if (p == 1)
      max_pool2d_backward_cl_s2_kernel<T, 3, 1, NIB><<<grid, blk, 0, s>>>(
          static_cast<const T*>(a), idx_in, static_cast<T*>(out), q, g);
    else
      max_pool2d_backward_cl_s2_kernel<T, 2, 0, NIB><<<grid, blk, 0, s>>>(
          static_cast<const T*>(a), idx_in, static_cast<T*>(out), q, g);
  } else {
    max_pool2d_backward_cl_kernel<T, NIB><<<dim3(xcd_grid(blocks)), dim3(kThreads), 0, s>>>(
        static_cast<const T*>(a), idx_in, static_cast<T*>(out), chunks, cpp, C, g);
  }
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

// The four operators (forward / backward, default / channels-last layout) with either index format.
namespace actnn {
namespace {
template <bool NIB>
int pool_forward(bool cl, const void* x, void* y, int8_t* idx, int64_t N, int64_t C, int64_t H, int64_t W,
                 int64_t Ho, int64_t Wo, int KH, int KW, int SH, int SW, int PH, int PW, int dtype, void* stream) {
  const int rc = check_geom(N, C, H, W, Ho, Wo, KH, KW, SH, SW, PH, PW);
  if (rc != ACTNN_OK) return rc;
  const int64_t total = N * C * Ho * Wo;
  if (total == 0) return ACTNN_OK;
  if (!x || !y || !idx) return ACTNN_EINVAL;
  const PoolGeom g{(int)H, (int)W, (int)Ho, (int)Wo, KH, KW, SH, SW, PH, PW};
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case ACTNN_F32: return cl ? launch_cl<float, NIB>(true, x, nullptr, idx, y, N, C, g, s) : launch_fwd<float, NIB>(x, y, idx, total, g, s);
    case ACTNN_F16: return cl ? launch_cl<__half, NIB>(true, x, nullptr, idx, y, N, C, g, s) : launch_fwd<__half, NIB>(x, y, idx, total, g, s);
    case ACTNN_BF16: return cl ? launch_cl<bf16_t, NIB>(true, x, nullptr, idx, y, N, C, g, s) : launch_fwd<bf16_t, NIB>(x, y, idx, total, g, s);
    default: return ACTNN_EDTYPE;
  }
}
template <bool NIB>
int pool_backward(bool cl, const void* grad_out, const int8_t* idx, void* grad_in, int64_t N, int64_t C, int64_t H,
                  int64_t W, int64_t Ho, int64_t Wo, int KH, int KW, int SH, int SW, int PH, int PW, int dtype,
                  void* stream) {
  const int rc = check_geom(N, C, H, W, Ho, Wo, KH, KW, SH, SW, PH, PW);
  if (rc != ACTNN_OK) return rc;
  const int64_t total = N * C * H * W;
  if (total == 0) return ACTNN_OK;
  if (!grad_out || !grad_in || !idx) return ACTNN_EINVAL;
  const PoolGeom g{(int)H, (int)W, (int)Ho, (int)Wo, KH, KW, SH, SW, PH, PW};
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case ACTNN_F32: return cl ? launch_cl<float, NIB>(false, grad_out, idx, nullptr, grad_in, N, C, g, s) : launch_bwd<float, NIB>(grad_out, idx, grad_in, total, g, s);
    case ACTNN_F16: return cl ? launch_cl<__half, NIB>(false, grad_out, idx, nullptr, grad_in, N, C, g, s) : launch_bwd<__half, NIB>(grad_out, idx, grad_in, total, g, s);
    case ACTNN_BF16: return cl ? launch_cl<bf16_t, NIB>(false, grad_out, idx, nullptr, grad_in, N, C, g, s) : launch_bwd<bf16_t, NIB>(grad_out, idx, grad_in, total, g, s);
    default: return ACTNN_EDTYPE;
  }
}
}  // namespace
}  // namespace actnn

#define ACTNN_POOL_GEOM_PARAMS int64_t N, int64_t C, int64_t H, int64_t W, int64_t Ho, int64_t Wo, int KH, int KW, \
                               int SH, int SW, int PH, int PW, int dtype, void* stream
#define ACTNN_POOL_GEOM_ARGS N, C, H, W, Ho, Wo, KH, KW, SH, SW, PH, PW, dtype, stream

extern "C" int actnn_max_pool2d_forward(const void* x, void* y, int8_t* idx, ACTNN_POOL_GEOM_PARAMS) {
  return actnn::pool_forward<false>(false, x, y, idx, ACTNN_POOL_GEOM_ARGS);
}
extern "C" int actnn_max_pool2d_backward(const void* grad_out, const int8_t* idx, void* grad_in, ACTNN_POOL_GEOM_PARAMS) {
  return actnn::pool_backward<false>(false, grad_out, idx, grad_in, ACTNN_POOL_GEOM_ARGS);
}
extern "C" int actnn_max_pool2d_forward_cl(const void* x, void* y, int8_t* idx, ACTNN_POOL_GEOM_PARAMS) {
  return actnn::pool_forward<false>(true, x, y, idx, ACTNN_POOL_GEOM_ARGS);
}
extern "C" int actnn_max_pool2d_backward_cl(const void* grad_out, const int8_t* idx, void* grad_in, ACTNN_POOL_GEOM_PARAMS) {
  return actnn::pool_backward<false>(true, grad_out, idx, grad_in, ACTNN_POOL_GEOM_ARGS);
}
extern "C" int actnn_max_pool2d_forward_nibble(const void* x, void* y, uint8_t* idx, ACTNN_POOL_GEOM_PARAMS) {
  return actnn::pool_forward<true>(false, x, y, reinterpret_cast<int8_t*>(idx), ACTNN_POOL_GEOM_ARGS);
}
extern "C" int actnn_max_pool2d_backward_nibble(const void* grad_out, const uint8_t* idx, void* grad_in, ACTNN_POOL_GEOM_PARAMS) {
  return actnn::pool_backward<true>(false, grad_out, reinterpret_cast<const int8_t*>(idx), grad_in, ACTNN_POOL_GEOM_ARGS);
}
extern "C" int actnn_max_pool2d_forward_cl_nibble(const void* x, void* y, uint8_t* idx, ACTNN_POOL_GEOM_PARAMS) {
  return actnn::pool_forward<true>(true, x, y, reinterpret_cast<int8_t*>(idx), ACTNN_POOL_GEOM_ARGS);
}
extern "C" int actnn_max_pool2d_backward_cl_nibble(const void* grad_out, const uint8_t* idx, void* grad_in, ACTNN_POOL_GEOM_PARAMS) {
  return actnn::pool_backward<true>(true, grad_out, reinterpret_cast<const int8_t*>(idx), grad_in, ACTNN_POOL_GEOM_ARGS);
}
