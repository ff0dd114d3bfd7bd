"""Vectorised layout restatements against the literal per-thread re-enactments."""
import numpy as np
import pytest

from oracle import layouts


@pytest.mark.parametrize("gs", [64, 256])
def test_mixed_literal_vs_vectorised(gs):
    rng = np.random.default_rng(0)
    bits = np.array([1, 2, 3, 4, 5, 6, 7, 8, 2, 2], dtype=np.int32)
    N, G = bits.size, 3
    codes = np.stack([rng.integers(0, 2 ** int(b), (G, gs)) for b in bits]).astype(np.int32)
    lit = layouts.pack_mixed_literal(codes, bits)
    vec = layouts.pack_mixed(codes, bits)
    assert lit.shape == vec.shape == (layouts.mixed_total_words(bits, G, gs),)
    assert np.array_equal(lit, vec)
    assert np.array_equal(layouts.unpack_mixed_literal(lit, bits, N, G, gs), codes)
    assert np.array_equal(layouts.unpack_mixed(vec, bits, N, G, gs), codes)


def test_mixed_word_is_a_ballot():
    # closed form: for gs = 256, word k*b+i bit j == bit i of code[8*j+k]
    b, gs = 3, 256
    codes = np.random.default_rng(1).integers(0, 8, (1, 1, gs)).astype(np.int32)
    w = layouts.pack_mixed(codes, [b]).view(np.uint32)
    for k in range(8):
        for i in range(b):
            for j in range(32):
                assert (int(w[k * b + i]) >> j) & 1 == (int(codes[0, 0, 8 * j + k]) >> i) & 1


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
@pytest.mark.parametrize("N", [1, 5, 8])
def test_single_literal_vs_vectorised(bits, N):
    rng = np.random.default_rng(2)
    G, gs = 2, 64
    codes = rng.integers(0, 2 ** bits, (N, G, gs)).astype(np.int32)
    lit = layouts.pack_single_literal(codes, bits)
    vec = layouts.pack_single(codes, bits)
    assert lit.shape == vec.shape == (layouts.single_total_bytes(N, G, gs, bits),)
    assert np.array_equal(lit, vec)
    assert np.array_equal(layouts.unpack_single(vec, bits, N, G, gs), codes)


def test_single_sizes_follow_reference_formula():
    # (bits * N_round * G * gs + 8) / 8 with N rounded up to a multiple of 8/bits
    assert layouts.single_total_bytes(5, 2, 64, 2) == (2 * 8 * 2 * 64 + 8) // 8
    assert layouts.single_total_bytes(4, 1, 256, 8) == 4 * 256 + 1


@pytest.mark.parametrize("n", [1, 31, 512, 513, 1500, 2048])
def test_mask_literal_vs_vectorised(n):
    bit = np.random.default_rng(n).integers(0, 2, n)
    lit = layouts.mask_words_literal(bit)
    vec = layouts.mask_words(bit)
    assert np.array_equal(lit, vec)
    assert vec.size == (n + 511) // 512 * 16
    assert np.array_equal(layouts.mask_bits(vec, n), bit)
