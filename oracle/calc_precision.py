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


def calc_precision_dp(A, C, max_b, target, states):
    """Follows calc_precision.cc:58-125 step by step in float32: f[i][t] over the first i items and
    t spent units, relaxed from every t < total with the choices in (b, p) order, strict
    improvement only; walk back from (N, total).  Returns (b float32 [N], p float32 [N]);
    raises ValueError where the reference's TORCH_CHECK fails."""
    A = np.asarray(A, dtype=np.float32)
    C = np.asarray(C, dtype=np.float32)
    N = A.shape[0]
    total = int(target) * N * int(states)
    big = np.float32(1e20)
    obj = np.full((N + 1, total + 1), big, dtype=np.float32)
    how_b = np.zeros((N + 1, total + 1), dtype=np.int64)
    how_p = np.zeros((N + 1, total + 1), dtype=np.int64)
    obj[0, 0] = np.float32(0)
    one = np.float32(1)
    for i in range(1, N + 1):
        for t in range(total):
            old = obj[i - 1, t]
            for b0 in range(1, max_b + 1):
                for p in range(1, states + 1):
                    if t + b0 * p <= total:
                        p0 = np.float32(np.float32(p) / np.float32(states))
                        B = np.float32((1 << b0) - 1)
                        delta = np.float32(np.float32(np.float32(one - p0) / p0) * A[i - 1]) \
                            + np.float32(C[i - 1] / np.float32(np.float32(p0 * B) * B))
                        value = np.float32(old + np.float32(delta))
                        if value < obj[i, t + b0 * p]:
                            obj[i, t + b0 * p] = value
                            how_b[i, t + b0 * p] = b0
                            how_p[i, t + b0 * p] = p
    b_vec = np.zeros(N, dtype=np.float32)
    p_vec = np.zeros(N, dtype=np.float32)
    t = total
    for i in range(N, 0, -1):
        if how_b[i, t] == 0:
            raise ValueError("DP Failed: no path to initial state!")
        b_vec[i - 1] = how_b[i, t]
        p_vec[i - 1] = np.float32(np.float32(how_p[i, t]) / np.float32(states))
        t -= int(how_b[i, t] * how_p[i, t])
    if t != 0:
        raise ValueError("DP Failed: no path to initial state!")
    return b_vec, p_vec


def dp_objective(b, p, A, C):
    b = np.asarray(b, np.float64)
    p = np.asarray(p, np.float64)
    return float(np.sum((1 - p) / p * np.asarray(A, np.float64)
                        + np.asarray(C, np.float64) / (p * (2.0 ** b - 1.0) ** 2)))


def dp_brute_force(A, C, max_b, target, states):
    """Exhaustive minimum of the objective over every (b_i, p_i) that spends exactly the budget."""
    N = len(A)
    total = target * N * states
    options = [(b, p) for b in range(1, max_b + 1) for p in range(1, states + 1)]
    best = None
    for cand in itertools.product(options, repeat=N):
        if sum(b * p for b, p in cand) == total:
            o = dp_objective([b for b, _ in cand], [p / states for _, p in cand], A, C)
            if best is None or o < best:
                best = o
    return best
