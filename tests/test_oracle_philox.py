"""Philox4x32-10 restatement against the Random123 known-answer vectors."""
import numpy as np

from oracle import philox


def _run(ctr, key):
    return [int(x) for x in philox.philox4x32_10(np.array([ctr], dtype=np.uint32), key)[0]]


def test_kat_zero():
    assert _run([0, 0, 0, 0], (0, 0)) == [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]


def test_kat_ones():
    f = 0xFFFFFFFF
    assert _run([f, f, f, f], (f, f)) == [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]


def test_kat_pi():
    assert _run([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], (0xa4093822, 0x299f31d0)) == \
        [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1]


def test_noise16_mapping():
    # element e uses half (e & 1) of word (e & 7) >> 1 of the call with counter e >> 3
    seed, off = 0x1234567890ABCDEF, 0x55AA000012345678
    e = np.arange(64, dtype=np.uint64)
    got = philox.noise16(e, seed, off)
    for o in range(8):
        r = philox.philox4x32_10(np.array([[o, 0, off & 0xFFFFFFFF, off >> 32]], dtype=np.uint32),
                                 (seed & 0xFFFFFFFF, seed >> 32))[0]
        for k in range(8):
            assert int(got[8 * o + k]) == (int(r[k >> 1]) >> (16 * (k & 1))) & 0xFFFF


def test_noise16_uniform():
    r = philox.noise16(np.arange(1 << 18, dtype=np.uint64), 7, 0).astype(np.float64)
    assert abs(r.mean() - 32767.5) < 120
    assert abs(r.var() - (65536.0 ** 2 - 1) / 12) / (65536.0 ** 2 / 12) < 0.01


def test_noise8_mapping():
    # element e uses byte (e & 3) of word (e & 15) >> 2 of the call with counter e >> 4
    seed, off = 0x1234567890ABCDEF, 0x55AA000012345678
    e = np.arange(96, dtype=np.uint64)
    got = philox.noise8(e, seed, off)
    for o in range(6):
        r = philox.philox4x32_10(np.array([[o, 0, off & 0xFFFFFFFF, off >> 32]], dtype=np.uint32),
                                 (seed & 0xFFFFFFFF, seed >> 32))[0]
        for k in range(16):
            assert int(got[16 * o + k]) == (int(r[k >> 2]) >> (8 * (k & 3))) & 0xFF


def test_noise8_uniform():
    r = philox.noise8(np.arange(1 << 18, dtype=np.uint64), 7, 0).astype(np.float64)
    assert abs(r.mean() - 127.5) < 0.5
    assert abs(r.var() - (256.0 ** 2 - 1) / 12) / (256.0 ** 2 / 12) < 0.01
    assert np.bincount(r.astype(np.int64), minlength=256).min() > 0.8 * (1 << 18) / 256
