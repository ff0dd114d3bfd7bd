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
