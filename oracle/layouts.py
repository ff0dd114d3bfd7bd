"""Bit-stream layouts of the reference's packed tensors (test infrastructure).

Each layout has two restatements:
* ``*_literal``: pure-Python loops that re-enact the reference kernel thread by thread,
  using the kernel's own index expressions (small inputs only);
* a vectorised numpy version used by the parity tests, checked against the literal one
  in ``tests/test_oracle_layouts.py``.
"""
import numpy as np


# ----------------------------------------------------------------------------------
# mixed precision: quantization_cuda_kernel.cu:37-80 (pack), :145-172 (unpack)
# ----------------------------------------------------------------------------------
def mixed_total_words(bits, G, gs):
    """.cu:97-100: ceil(sum(bits) * G * gs / 32) int32 words."""
    total_bits = int(np.sum(np.asarray(bits, dtype=np.int64))) * G * gs
    return (total_bits + 31) // 32


def pack_mixed_literal(codes, bits):
    """codes int [N,G,gs]; bits int [N].  Literal re-enactment of .cu:51-79."""
    codes = np.asarray(codes)
    N, G, gs = codes.shape
    bits = [int(b) for b in bits]
    out = np.zeros(mixed_total_words(bits, G, gs), dtype=np.uint32)
    prefix = np.cumsum(bits)
    for n in range(N):
        b = bits[n]
        shared_len = gs * b // 32                                   # :55
        for g in range(G):
            shared = [0] * shared_len
            for d in range(gs):                                     # one thread per d
                val = int(codes[n, g, d])
                offset = d * b                                      # :66
                for i in range(b):                                  # :69-71
                    shared[(offset + i) % shared_len] |= (1 & (val >> i)) << ((offset + i) // shared_len)
            global_offset = ((0 if n == 0 else int(prefix[n - 1])) * G * gs + b * g * gs) // 32   # :75-76
            for t in range(shared_len):
                out[global_offset + t] = shared[t] & 0xFFFFFFFF
    return out.view(np.int32)


def unpack_mixed_literal(words, bits, N, G, gs):
    """Literal re-enactment of .cu:156-169 (integer part only)."""
    words = np.asarray(words).view(np.uint32)
    bits = [int(b) for b in bits]
    prefix = np.cumsum(bits)
    out = np.zeros((N, G, gs), dtype=np.int32)
    for n in range(N):
        b = bits[n]
        shared_len = gs * b // 32
        for g in range(G):
            global_offset = ((0 if n == 0 else int(prefix[n - 1])) * G * gs + b * g * gs) // 32
            for d in range(gs):
                block_offset = d * b
                val = 0
                for i in range(b):
                    val |= (1 & (int(words[global_offset + (block_offset + i) % shared_len])
                                 >> ((block_offset + i) // shared_len))) << i
                out[n, g, d] = val
    return out


def pack_mixed(codes, bits):
    """Vectorised: for gs = 32*E, element d = E*j + k, bit i -> word k*b + i, bit j."""
    codes = np.asarray(codes).astype(np.uint32)
    N, G, gs = codes.shape
    assert gs % 32 == 0
    E = gs // 32
    bits = np.asarray(bits, dtype=np.int64)
    out = np.zeros(mixed_total_words(bits, G, gs), dtype=np.uint32)
    prefix = np.concatenate([[0], np.cumsum(bits)])
    jw = (np.uint32(1) << np.arange(32, dtype=np.uint32))
    for n in range(N):
        b = int(bits[n])
        c = codes[n].reshape(G, 32, E)                              # [g, j, k]
        i = np.arange(b, dtype=np.uint32)
        bitsel = (c[:, :, :, None] >> i) & np.uint32(1)             # [g, j, k, i]
        w = (bitsel * jw[None, :, None, None]).sum(axis=1, dtype=np.uint64).astype(np.uint32)   # [g, k, i]
        base = int(prefix[n]) * G * gs // 32
        out[base: base + G * E * b] = w.reshape(-1)
    return out.view(np.int32)


def unpack_mixed(words, bits, N, G, gs):
    words = np.asarray(words).view(np.uint32)
    E = gs // 32
    bits = np.asarray(bits, dtype=np.int64)
    prefix = np.concatenate([[0], np.cumsum(bits)])
    out = np.zeros((N, G, gs), dtype=np.int32)
    j = np.arange(32, dtype=np.uint32)
    for n in range(N):
        b = int(bits[n])
        base = int(prefix[n]) * G * gs // 32
        w = words[base: base + G * E * b].reshape(G, E, b)          # [g, k, i]
        bit = (w[:, None, :, :] >> j[None, :, None, None]) & np.uint32(1)   # [g, j, k, i]
        val = (bit << np.arange(b, dtype=np.uint32)).sum(axis=3, dtype=np.uint32)   # [g, j, k]
        out[n] = val.reshape(G, gs)
    return out


# ----------------------------------------------------------------------------------
# single precision: .cu:225-258 (pack), :333-361 (unpack); sizes :271-277
# ----------------------------------------------------------------------------------
def single_total_bytes(N, G, gs, bits):
    """.cu:271-277: N rounded up to a multiple of 8/bits; (total_bits + 8) / 8 bytes."""
    wpt = 8 // bits
    n_round = N + (wpt - N % wpt) % wpt
    return (bits * n_round * G * gs + 8) // 8


def pack_single_literal(codes, bits):
    codes = np.asarray(codes)
    N, G, gs = codes.shape
    wpt = 8 // bits
    out = np.zeros(single_total_bytes(N, G, gs, bits), dtype=np.uint8)
    for no in range((N + wpt - 1) // wpt):
        for g in range(G):
            for d in range(gs):
                tid = (no * G + g) * gs + d                         # :240
                local = 0
                for ni in range(wpt):
                    n = no * wpt + ni
                    if n >= N:
                        break
                    local |= (int(codes[n, g, d]) << (ni * bits))  # :254
                out[tid] = local & 0xFF
    return out.view(np.int8)


def pack_single(codes, bits):
    codes = np.asarray(codes).astype(np.uint32)
    N, G, gs = codes.shape
    wpt = 8 // bits
    n_round = N + (wpt - N % wpt) % wpt
    c = np.zeros((n_round, G, gs), dtype=np.uint32)
    c[:N] = codes
    c = c.reshape(n_round // wpt, wpt, G, gs)
    sh = (np.arange(wpt, dtype=np.uint32) * bits)[None, :, None, None]
    by = ((c << sh).sum(axis=1, dtype=np.uint32) & np.uint32(0xFF)).astype(np.uint8)
    out = np.zeros(single_total_bytes(N, G, gs, bits), dtype=np.uint8)
    out[: by.size] = by.reshape(-1)
    return out.view(np.int8)


def unpack_single(packed, bits, N, G, gs):
    """.cu:343-360, integer part."""
    p = np.asarray(packed).view(np.uint8)
    wpt = 8 // bits
    n_out = (N + wpt - 1) // wpt
    by = p[: n_out * G * gs].reshape(n_out, 1, G, gs).astype(np.uint32)
    sh = (np.arange(wpt, dtype=np.uint32) * bits)[None, :, None, None]
    v = (by >> sh) & np.uint32((1 << bits) - 1)
    return v.reshape(n_out * wpt, G, gs)[:N].astype(np.int32)


# ----------------------------------------------------------------------------------
# 1-bit masks of ReLU / Dropout: .cu:419-443 (write), :475-486 (read)
# ----------------------------------------------------------------------------------
MASK_BLOCK = 512      # ACT_QUANTIZED_RELU_NUM_THREADS, .cu:411


def mask_words_literal(bit):
    """bit: 0/1 array [n].  Literal re-enactment of .cu:419-443 for every block, with the
    tail block's 16 words all materialised (the reference allocates only ceil(n/32) words
    and its tail block stores past the end; the build allocates 16 words per block)."""
    bit = np.asarray(bit).astype(np.int64).reshape(-1)
    n = bit.size
    nblk = (n + MASK_BLOCK - 1) // MASK_BLOCK
    out = np.zeros(nblk * 16, dtype=np.uint32)
    for blk in range(nblk):
        shared = [0] * 16
        for t in range(MASK_BLOCK):
            idx = blk * MASK_BLOCK + t
            if idx < n:
                shared[t % 16] |= int(bit[idx]) << (t // 16)        # :437
        global_offset = blk * MASK_BLOCK // 32                      # :420
        for k in range(16):
            out[global_offset + k] = shared[k] & 0xFFFFFFFF
    return out.view(np.int32)


def mask_words(bit):
    bit = np.asarray(bit).astype(np.uint32).reshape(-1)
    n = bit.size
    nblk = (n + MASK_BLOCK - 1) // MASK_BLOCK
    padded = np.zeros(nblk * MASK_BLOCK, dtype=np.uint32)
    padded[:n] = bit
    c = padded.reshape(nblk, 32, 16)                                # [blk, j, k]
    jw = (np.uint32(1) << np.arange(32, dtype=np.uint32))[None, :, None]
    return (c * jw).sum(axis=1, dtype=np.uint64).astype(np.uint32).reshape(-1).view(np.int32)


def mask_bits(words, n):
    """Inverse of ``mask_words`` (.cu:480): bit of element blk*512 + 16*j + k."""
    w = np.asarray(words).view(np.uint32).reshape(-1, 1, 16)
    j = np.arange(32, dtype=np.uint32)[None, :, None]
    return ((w >> j) & np.uint32(1)).reshape(-1)[:n].astype(np.uint8)
