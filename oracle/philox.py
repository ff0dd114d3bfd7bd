"""Philox4x32-10 counter-based generator (test infrastructure).

The reference draws its rounding noise from cuRAND's Philox4_32_10
(quantization_cuda_kernel.cu:61-63, :242-252, :533-535); cuRAND is a CUDA-toolkit
dependency that is not part of the reference tree, so the algorithm restated here is the
published one (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3", SC'11),
pinned by the Random123 known-answer vectors in ``tests/test_oracle_philox.py``.
Bit-compatibility with cuRAND's *stream order* is not claimed (parity unpinned): the
reference's own tests only check the distribution.
"""
import numpy as np

M0 = np.uint64(0xD2511F53)
M1 = np.uint64(0xCD9E8D57)
W0 = 0x9E3779B9
W1 = 0xBB67AE85
MASK32 = np.uint64(0xFFFFFFFF)


def philox4x32_10(ctr, key):
    """ctr: uint32 array [..., 4]; key: (k0, k1) python ints.  Returns uint32 [..., 4]."""
    c = [np.asarray(ctr[..., i], dtype=np.uint64) for i in range(4)]
    k0, k1 = int(key[0]) & 0xFFFFFFFF, int(key[1]) & 0xFFFFFFFF
    for _ in range(10):
        p0 = M0 * c[0]
        p1 = M1 * c[2]
        hi0, lo0 = p0 >> np.uint64(32), p0 & MASK32
        hi1, lo1 = p1 >> np.uint64(32), p1 & MASK32
        c = [hi1 ^ c[1] ^ np.uint64(k0), lo1, hi0 ^ c[3] ^ np.uint64(k1), lo0]
        k0 = (k0 + W0) & 0xFFFFFFFF
        k1 = (k1 + W1) & 0xFFFFFFFF
    return np.stack([x.astype(np.uint32) for x in c], axis=-1)


def noise16(elem_index, seed, offset):
    """16-bit noise of flat element index ``e`` as the HIP kernels define it:
    one Philox call per 8 consecutive elements, counter = (lo(e>>3), hi(e>>3), lo(offset),
    hi(offset)), key = (lo(seed), hi(seed)); element ``e & 7`` takes the (e&1)-th 16-bit
    half (low first) of output word ``(e & 7) >> 1``."""
    e = np.asarray(elem_index, dtype=np.uint64)
    o = e >> np.uint64(3)
    ctr = np.stack([(o & MASK32).astype(np.uint32), (o >> np.uint64(32)).astype(np.uint32),
                    np.full(o.shape, offset & 0xFFFFFFFF, np.uint32),
                    np.full(o.shape, (offset >> 32) & 0xFFFFFFFF, np.uint32)], axis=-1)
    r = philox4x32_10(ctr, (seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF))
    k = (e & np.uint64(7)).astype(np.int64)
    w = np.take_along_axis(r, (k >> 1)[..., None], axis=-1)[..., 0]
    return ((w >> ((k & 1) * 16).astype(np.uint32)) & np.uint32(0xFFFF)).astype(np.uint32)


def noise8(elem_index, seed, offset):
    """8-bit noise of flat element index ``e`` as the HIP kernels define it for fp16 / bf16 tensors:
    one Philox call per 16 consecutive elements, counter = (lo(e>>4), hi(e>>4), lo(offset),
    hi(offset)), key = (lo(seed), hi(seed)); element ``e & 15`` takes byte ``e & 3`` (low first) of
    output word ``(e & 15) >> 2``."""
    e = np.asarray(elem_index, dtype=np.uint64)
    o = e >> np.uint64(4)
    ctr = np.stack([(o & MASK32).astype(np.uint32), (o >> np.uint64(32)).astype(np.uint32),
                    np.full(o.shape, offset & 0xFFFFFFFF, np.uint32),
                    np.full(o.shape, (offset >> 32) & 0xFFFFFFFF, np.uint32)], axis=-1)
    r = philox4x32_10(ctr, (seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF))
    k = (e & np.uint64(15)).astype(np.int64)
    w = np.take_along_axis(r, (k >> 2)[..., None], axis=-1)[..., 0]
    return ((w >> ((k & 3) * 8).astype(np.uint32)) & np.uint32(0xFF)).astype(np.uint32)
