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
