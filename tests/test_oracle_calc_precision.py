"""Greedy bit allocation: oracle pins, and the library's host entry point against the oracle."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import build_ref, calc_precision as cp


def test_degenerate_known_answer():
    # C == 0, N = 256, b0 = 8, target = 512: ties go to the largest index, so samples 255..37
    # drop to 1 bit, sample 36 loses 3 bits, samples 0..35 keep 8 (first-iteration state of
    # a layer whose gradient scale is still 0, qscheme.py:24).
    b = cp.calc_precision(np.full(256, 8, np.int32), np.zeros(256, np.float32), np.ones(256, np.int32), 512)
    assert (b[:36] == 8).all() and b[36] == 5 and (b[37:] == 1).all()
    assert b.sum() == 512


@pytest.mark.parametrize("seed", range(6))
def test_greedy_is_optimal_on_tiny_inputs(seed):
    # the objective is separable and convex in each b_i, so the greedy result is a global optimum
    rng = np.random.default_rng(seed)
    N = 4
    C = rng.lognormal(0, 2, N).astype(np.float32)
    b0 = np.full(N, 4, np.int32)
    w = np.ones(N, np.int32)
    target = int(rng.integers(N, 4 * N))
    b = cp.calc_precision(b0, C, w, target)
    assert b.sum() <= target and (b >= 1).all()
    assert cp.objective(b, C) <= cp.brute_force_optimum(b0, C, w, target) * (1 + 1e-9)


def _lib_calc(lib, b, C, w, target):
    b = np.ascontiguousarray(b, np.int32).copy()
    C = np.ascontiguousarray(C, np.float32)
    w = np.ascontiguousarray(w, np.int32)
    rc = lib.actnn_calc_precision(b.ctypes.data_as(ctypes.c_void_p), C.ctypes.data_as(ctypes.c_void_p),
                                  w.ctypes.data_as(ctypes.c_void_p), b.size, float(target))
    assert rc == 0
    return b


@pytest.mark.parametrize("seed", range(5))
def test_library_matches_oracle(lib, seed):
    rng = np.random.default_rng(100 + seed)
    N = int(rng.integers(1, 400))
    C = rng.lognormal(0, 3, N).astype(np.float32)
    C[rng.random(N) < 0.2] = 0.0
    w = rng.integers(1, 5, N).astype(np.int32) if seed % 2 else np.ones(N, np.int32)
    b0 = np.full(N, 8, np.int32)
    target = float(rng.uniform(1.0, 8.0) * w.sum())
    assert np.array_equal(_lib_calc(lib, b0, C, w, target), cp.calc_precision(b0, C, w, target))


def test_library_known_answer_and_errors(lib):
    b = _lib_calc(lib, np.full(256, 8), np.zeros(256), np.ones(256), 512)
    assert (b[:36] == 8).all() and b[36] == 5 and (b[37:] == 1).all()
    bad = np.zeros(4, np.int32)
    rc = lib.actnn_calc_precision(bad.ctypes.data_as(ctypes.c_void_p), bad.ctypes.data_as(ctypes.c_void_p),
                                  bad.ctypes.data_as(ctypes.c_void_p), 4, 1.0)
    assert rc != 0
    # target below N: everything ends at 1 bit and the call still terminates
    b = _lib_calc(lib, np.full(8, 3), np.ones(8), np.ones(8), 2)
    assert (b == 1).all()


def test_against_compiled_reference():
    ref = build_ref.load()
    if ref is None:
        pytest.skip("oracle/_ref not built (reference tree not mounted when build() ran)")
    rng = np.random.default_rng(7)
    for trial in range(20):
        N = int(rng.integers(1, 300))
        C = rng.lognormal(0, 3, N).astype(np.float32)
        if trial % 3 == 0:
            C[rng.random(N) < 0.3] = 0.0
        w = rng.integers(1, 6, N).astype(np.int32) if trial % 2 else np.ones(N, np.int32)
        b0 = np.full(N, 8, np.int32)
        target = float(rng.uniform(1.0, 8.0) * w.sum())
        got = ref.calc_precision(torch.from_numpy(b0.copy()), torch.from_numpy(C), torch.from_numpy(w), target)
        assert np.array_equal(got.numpy(), cp.calc_precision(b0, C, w, target))


# ------------------------------------------------------------------------------------------
# calc_precision_dp (calc_precision.cc:58-125)
# ------------------------------------------------------------------------------------------
def _dp_inputs(rng, N):
    A = rng.lognormal(0, 1, N).astype(np.float32)
    C = rng.lognormal(1, 2, N).astype(np.float32)
    return A, C


def test_dp_restatement_is_optimal_on_tiny_inputs():
    """The objective is separable and the budget an equality: brute force over every (b, p)
    assignment gives the same minimum (float64 objective of the float32 DP's choice)."""
    rng = np.random.default_rng(3)
    for N, max_b, target, states in ((3, 3, 2, 2), (4, 2, 1, 2), (2, 4, 3, 1), (3, 2, 2, 3)):
        A, C = _dp_inputs(rng, N)
        b, p = cp.calc_precision_dp(A, C, max_b, target, states)
        assert np.isclose(sum(b * p * states), target * N * states)
        assert ((b >= 1) & (b <= max_b) & (p > 0) & (p <= 1)).all()
        best = cp.dp_brute_force(A, C, max_b, target, states)
        assert cp.dp_objective(b, p, A, C) <= best * (1 + 1e-5)


def test_dp_known_cases():
    # one state, budget = max_b: every item keeps all its bits, p = 1
    b, p = cp.calc_precision_dp(np.ones(5, np.float32), np.ones(5, np.float32), 4, 4, 1)
    assert (b == 4).all() and (p == 1).all()
    # budget of one unit per item and state: the only way is b = 1, p = 1/states ... or b*p = states
    b, p = cp.calc_precision_dp(np.zeros(3, np.float32), np.array([1, 100, 1], np.float32), 2, 1, 1)
    assert (b == 1).all() and (p == 1).all()
    # an unreachable budget fails like the reference's TORCH_CHECK
    with pytest.raises(ValueError):
        cp.calc_precision_dp(np.ones(2, np.float32), np.ones(2, np.float32), 1, 3, 1)


def test_dp_library_routine_matches_the_restatement_and_the_compiled_reference():
    import actnn_amd.cpp_extension.calc_precision as ext
    ref = build_ref.load()
    rng = np.random.default_rng(11)
    for trial in range(12):
        N = int(rng.integers(1, 24))
        max_b, target, states = int(rng.integers(1, 5)), int(rng.integers(1, 4)), int(rng.integers(1, 4))
        A, C = _dp_inputs(rng, N)
        if trial % 4 == 0:
            C[rng.random(N) < 0.4] = 0.0                  # equal costs: the tie rule decides
        if target > max_b:                                # no assignment can spend that much
            with pytest.raises(RuntimeError):
                ext.calc_precision_dp(torch.from_numpy(A), torch.from_numpy(C), max_b, target, states)
            continue
        want_b, want_p = cp.calc_precision_dp(A, C, max_b, target, states)
        got_b, got_p = ext.calc_precision_dp(torch.from_numpy(A), torch.from_numpy(C), max_b, target, states)
        assert np.array_equal(got_b.numpy(), want_b) and np.array_equal(got_p.numpy(), want_p)
        if ref is not None:
            ref_b, ref_p = ref.calc_precision_dp(torch.from_numpy(A), torch.from_numpy(C), max_b, target, states)
            assert np.array_equal(ref_b.numpy(), want_b) and np.array_equal(ref_p.numpy(), want_p)
    with pytest.raises(RuntimeError):
        ext.calc_precision_dp(torch.ones(3, dtype=torch.float64), torch.ones(3), 2, 1, 1)
    # the reference's own sizing (N = 128, b = 2, s = 2: calc_precision.cc:73) in well under a second
    A, C = _dp_inputs(rng, 128)
    got_b, got_p = ext.calc_precision_dp(torch.from_numpy(A), torch.from_numpy(C), 8, 2, 2)
    assert float((got_b * got_p * 2).sum()) == 2 * 128 * 2
    if ref is not None:
        ref_b, ref_p = ref.calc_precision_dp(torch.from_numpy(A), torch.from_numpy(C), 8, 2, 2)
        assert torch.equal(ref_b, got_b) and torch.equal(ref_p, got_p)
