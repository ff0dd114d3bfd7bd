// Greedy per-sample bit allocation on the host (replaces calc_precision.cc:9-50).
//
//   minimise sum_i C_i / (2^b_i - 1)^2   s.t.   sum_i b_i w_i <= target,  b_i >= 1
//
// Start from the given widths and repeatedly take one bit from the item whose objective
// grows least per unit weight.  The candidate order must reproduce the reference's
// std::priority_queue<std::pair<float, int64_t>>: larger (float-narrowed) delta first, ties
// to the larger index.  A binary max-heap over (delta, index) with that total order pops
// the same sequence whatever its internal arrangement.
#include <algorithm>
#include <cstdint>
#include <vector>

#include "../../include/actnn_hip.h"

namespace {

struct Cand {
  float delta;
  int64_t index;
};

inline bool cand_less(const Cand& a, const Cand& b) {   // strict weak order of std::pair
  if (a.delta < b.delta) return true;
  if (b.delta < a.delta) return false;
  return a.index < b.index;
}

// Objective change when item goes from b to b - 1 bits, sign as in the reference
// (negative), evaluated in double and divided by the weight (calc_precision.cc:24-28,:33).
inline float step_delta(float C, int b, int w) {
  const int64_t full = ((int64_t)1 << b) - 1;
  const int64_t less = ((int64_t)1 << (b - 1)) - 1;
  const double c1 = (double)(full * full);
  const double c2 = (double)(less * less);              // 0 for b == 1: the step costs +inf
  const double d = (double)C * (1.0 / c1 - 1.0 / c2);
  return (float)(d / w);
}

}  // namespace

extern "C" int actnn_calc_precision(int32_t* b, const float* C, const int32_t* w, int64_t N,
                                    double target) {
  if (N < 0) return ACTNN_EINVAL;
  if (N == 0) return ACTNN_OK;
  if (!b || !C || !w) return ACTNN_EINVAL;
  for (int64_t i = 0; i < N; ++i)
    if (b[i] < 1 || b[i] > 30 || w[i] == 0) return ACTNN_EBITS;

  std::vector<Cand> heap;
  heap.reserve((size_t)N);
  double b_sum = 0.0;
  for (int64_t i = 0; i < N; ++i) {
    heap.push_back(Cand{step_delta(C[i], b[i], w[i]), i});
    b_sum += (double)b[i] * w[i];
  }
  std::make_heap(heap.begin(), heap.end(), cand_less);

  while (b_sum > target) {
    if (heap.empty()) break;            // every item already at 1 bit: cannot go lower
    std::pop_heap(heap.begin(), heap.end(), cand_less);
    const int64_t i = heap.back().index;
    heap.pop_back();
    b[i] -= 1;
    b_sum -= w[i];
    if (b[i] > 1) {
      heap.push_back(Cand{step_delta(C[i], b[i], w[i]), i});
      std::push_heap(heap.begin(), heap.end(), cand_less);
    }
  }
  return ACTNN_OK;
}

// Dynamic-programming allocation with keep probabilities (replaces calc_precision.cc:58-125):
//
//   minimise sum_i (1 - p_i) / p_i * A_i + C_i / (p_i * (2^b_i - 1)^2)
//   s.t.     sum_i b_i * (states * p_i) == target * N * states,
//   b_i in 1..max_b,  p_i in {1/states, ..., 1}.
//
// f[i][t] = best objective of the first i items that spend exactly t units.  Items are relaxed
// one after the other from the spent amounts upwards, choices in the order (b, p), and a new
// value replaces the old one only when strictly smaller - the reference's order, so ties
// resolve the same way.  Only two rows of objectives are alive at a time; the choice taken to
// reach each (i, t) is kept as one byte for the walk back from (N, total).
extern "C" int actnn_calc_precision_dp(const float* A, const float* C, int64_t N, int max_b, int target,
                                       int states, float* b_out, float* p_out) {
  if (N < 0 || max_b < 1 || max_b > 30 || states < 1 || target < 0) return ACTNN_EINVAL;
  if ((int64_t)max_b * states > 255) return ACTNN_EINVAL;      // choices are stored as bytes
  if (N == 0) return ACTNN_OK;
  if (!A || !C || !b_out || !p_out) return ACTNN_EINVAL;
  if ((int64_t)target > (((int64_t)1 << 40) / N) / states) return ACTNN_EINVAL;
  const int64_t total = (int64_t)target * N * states;
  const float kUnreached = 1e20f;
  const int choices = max_b * states;
  constexpr uint8_t kNone = 255;

  std::vector<float> prev((size_t)total + 1, kUnreached), next((size_t)total + 1);
  std::vector<uint8_t> taken((size_t)N * ((size_t)total + 1), kNone);
  std::vector<float> delta((size_t)choices);
  std::vector<int64_t> cost((size_t)choices);
  prev[0] = 0.0f;
  for (int64_t i = 0; i < N; ++i) {
    for (int b = 1; b <= max_b; ++b)
      for (int p = 1; p <= states; ++p) {
        const float p0 = (float)p / states;
        const float B = (float)(((int64_t)1 << b) - 1);
        delta[(size_t)(b - 1) * states + (p - 1)] = (1 - p0) / p0 * A[i] + C[i] / (p0 * B * B);
        cost[(size_t)(b - 1) * states + (p - 1)] = (int64_t)b * p;
      }
    std::fill(next.begin(), next.end(), kUnreached);
    uint8_t* how = taken.data() + (size_t)i * ((size_t)total + 1);
    for (int64_t t = 0; t < total; ++t) {
      const float base = prev[(size_t)t];
      for (int c = 0; c < choices; ++c) {
        const int64_t to = t + cost[(size_t)c];
        if (to > total) continue;
        const float value = base + delta[(size_t)c];
        if (value < next[(size_t)to]) {
          next[(size_t)to] = value;
          how[to] = (uint8_t)c;
        }
      }
    }
    prev.swap(next);
  }
  int64_t t = total;
  for (int64_t i = N - 1; i >= 0; --i) {
    const uint8_t c = taken[(size_t)i * ((size_t)total + 1) + (size_t)t];
    if (c == kNone) return ACTNN_EINVAL;                       // "DP Failed: no path to initial state!"
    const int b = c / states + 1, p = c % states + 1;
    b_out[i] = (float)b;
    p_out[i] = (float)p / states;
    t -= (int64_t)b * p;
  }
  return t == 0 ? ACTNN_OK : ACTNN_EINVAL;
}
