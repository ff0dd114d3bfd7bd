"""Greedy bit allocation (test infrastructure).  Follows calc_precision.cc:9-50.

minimise  sum_i C_i / (2^b_i - 1)^2   subject to  sum_i b_i w_i <= target, b_i >= 1,
by repeatedly taking one bit from the item whose objective grows least per unit weight.
The reference keeps ``std::pair<float, int64_t>`` in a ``std::priority_queue`` (max-heap,
lexicographic), so ties on the (float-narrowed) delta go to the larger index.
"""
import heapq
import itertools

import numpy as np


def _delta(C, b, w):
    """calc_precision.cc:24-28, :33: evaluated in double, divided by the int weight, then
    narrowed to float when stored in the heap's pair<float, int64_t>."""
    coeff_1 = ((1 << b) - 1) ** 2
    coeff_2 = ((1 << (b - 1)) - 1) ** 2
    with np.errstate(divide="ignore", invalid="ignore"):
        inv2 = np.float64(1.0) / np.float64(coeff_2) if coeff_2 != 0 else np.float64(np.inf)
        d = np.float64(np.float32(C)) * (np.float64(1.0) / np.float64(coeff_1) - inv2)
        return np.float32(d / np.float64(w))


def calc_precision(b, C, w, target):
    """b int32 [N] (copied, not mutated), C float32 [N], w int32 [N]; returns int32 [N]."""
    b = np.array(b, dtype=np.int32).copy()
    C = np.asarray(C, dtype=np.float32)
    w = np.asarray(w, dtype=np.int32)
    N = b.shape[0]
    heap = []          # max-heap on (delta, i)  ==  min-heap on (-delta, -i)
    b_sum = 0.0
    for i in range(N):
        heap.append((-float(_delta(C[i], int(b[i]), int(w[i]))), -i))
        b_sum += float(b[i]) * float(w[i])
    heapq.heapify(heap)
    while b_sum > target:
        _, neg_i = heapq.heappop(heap)
        i = -neg_i
        b[i] -= 1
        b_sum -= float(w[i])
        if b[i] > 1:
            heapq.heappush(heap, (-float(_delta(C[i], int(b[i]), int(w[i]))), -i))
    return b


def objective(b, C):
    b = np.asarray(b, dtype=np.int64)
    return float(np.sum(np.asarray(C, np.float64) / ((2.0 ** b - 1.0) ** 2)))


def brute_force_optimum(b0, C, w, target):
    """Exhaustive minimum of the objective over 1 <= b_i <= b0_i with sum b_i w_i <= target."""
    best = None
    for cand in itertools.product(*[range(1, int(x) + 1) for x in b0]):
        if sum(c * int(wi) for c, wi in zip(cand, w)) <= target:
            o = objective(cand, C)
            if best is None or o < best:
                best = o
    return best
