"""Max-pool with arg-max-in-window indices, dropout mask rule (test infrastructure).

Follows quantization_cuda_kernel.cu:634-670 (forward), :702-725 (backward) and the
checks of quantization.cc:156-162.  Values are pinned by torch's own
``F.max_pool2d`` forward/backward (as the reference's test does,
tests/test_act_quantized_ops.py:206-232); the index rule (first strict maximum in
row-major window order, offset relative to the *unclipped* window origin) comes from the
kernel source and is pinned by ``gather(input, index) == output`` and by a brute-force
loop version.
"""
import numpy as np


def out_size(H, k, s, p, d=1):
    """.cu:679-680."""
    return (H + 2 * p - d * (k - 1) - 1) // s + 1


def max_pool2d_forward(x, kernel, stride, padding, dilation=(1, 1)):
    """x float array [N,C,H,W] -> (out [N,C,Ho,Wo], idx int8 [N,C,Ho,Wo]).
    The window ignores dilation (only the output size uses it), .cu:649-654."""
    x = np.asarray(x)
    N, C, H, W = x.shape
    KH, KW = kernel
    SH, SW = stride
    PH, PW = padding
    Ho, Wo = out_size(H, KH, SH, PH, dilation[0]), out_size(W, KW, SW, PW, dilation[1])
    # the kernel starts from v = -1e10 narrowed to the input type (.cu:656): -inf in fp16
    init = x.dtype.type(-1e10) if x.dtype != np.float16 else np.float16(-np.inf)
    out = np.full((N, C, Ho, Wo), init, dtype=x.dtype)
    idx = np.zeros((N, C, Ho, Wo), dtype=np.int8)
    hb = np.arange(Ho) * SH - PH
    wb = np.arange(Wo) * SW - PW
    for kh in range(KH):
        for kw in range(KW):
            hi = hb + kh
            wi = wb + kw
            vh = (hi >= 0) & (hi < H)
            vw = (wi >= 0) & (wi < W)
            cand = x[:, :, np.clip(hi, 0, H - 1)][:, :, :, np.clip(wi, 0, W - 1)]
            valid = (vh[:, None] & vw[None, :])[None, None]
            better = valid & (cand > out)                       # strict '>' keeps the first
            out = np.where(better, cand, out)
            idx = np.where(better, np.int8(kh * KW + kw), idx)
    return out, idx


def max_pool2d_forward_literal(x, kernel, stride, padding, dilation=(1, 1)):
    """Thread-by-thread loop version of .cu:644-669 (tiny inputs)."""
    x = np.asarray(x)
    N, C, H, W = x.shape
    KH, KW = kernel
    SH, SW = stride
    PH, PW = padding
    Ho, Wo = out_size(H, KH, SH, PH, dilation[0]), out_size(W, KW, SW, PW, dilation[1])
    out = np.zeros((N, C, Ho, Wo), dtype=x.dtype)
    idx = np.zeros((N, C, Ho, Wo), dtype=np.int8)
    for n in range(N):
        for c in range(C):
            for h in range(Ho):
                for w in range(Wo):
                    h_base, w_base = h * SH - PH, w * SW - PW
                    v = x.dtype.type(-1e10) if x.dtype != np.float16 else np.float16(-np.inf)
                    index = 0
                    for i in range(max(h_base, 0), min(h_base + KH, H)):
                        for j in range(max(w_base, 0), min(w_base + KW, W)):
                            if x[n, c, i, j] > v:
                                v = x[n, c, i, j]
                                index = (i - h_base) * KW + j - w_base
                    out[n, c, h, w] = v
                    idx[n, c, h, w] = index
    return out, idx


def max_pool2d_backward(gout, idx, in_shape, kernel, stride, padding):
    """.cu:712-723: scatter-add grad_output to the arg-max position (accumulated in
    float64 here; the kernel's atomic order is unspecified)."""
    gout = np.asarray(gout)
    N, C, H, W = in_shape
    KH, KW = kernel
    SH, SW = stride
    PH, PW = padding
    _, _, Ho, Wo = gout.shape
    gin = np.zeros((N * C, H * W), dtype=np.float64)
    hb = (np.arange(Ho) * SH - PH)[:, None]
    wb = (np.arange(Wo) * SW - PW)[None, :]
    ii = idx.astype(np.int64)
    hh = hb[None, None] + ii // KW
    ww = wb[None, None] + ii % KW
    lin = (hh * W + ww).reshape(N * C, -1)
    g = gout.astype(np.float64).reshape(N * C, -1)
    for r in range(N * C):
        np.add.at(gin[r], lin[r], g[r])
    return gin.reshape(N, C, H, W)


def pack_index_nibbles(idx):
    """Two indices per byte, the format of the *_nibble operators of the library (the reference has
    none: it keeps one int8 per output, quantization_cuda_kernel.cu:683): element o of `idx` in memory order
    -> bits 4 * (o & 1) .. of byte o // 2; the spare half of the last byte of an odd count is 0."""
    flat = np.asarray(idx).reshape(-1).astype(np.uint8)
    assert flat.size == 0 or flat.max() < 16
    if flat.size & 1:
        flat = np.concatenate([flat, np.zeros(1, np.uint8)])
    return (flat[0::2] | (flat[1::2] << 4)).astype(np.uint8)


def unpack_index_nibbles(packed, count):
    packed = np.asarray(packed, dtype=np.uint8)
    out = np.empty(packed.size * 2, np.int8)
    out[0::2] = packed & 15
    out[1::2] = packed >> 4
    return out[:count]
