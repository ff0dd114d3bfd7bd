"""Max-pool oracle against torch's own max_pool2d (the check the reference's test uses)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import pool

CASES = [((3, 3), (2, 2), (1, 1)), ((2, 2), (2, 2), (0, 0)), ((3, 2), (1, 2), (1, 0)), ((3, 3), (1, 1), (1, 1))]


@pytest.mark.parametrize("k,s,p", CASES)
def test_forward_backward_vs_torch(k, s, p):
    torch.manual_seed(0)
    x = torch.randn(2, 3, 13, 14, requires_grad=True)
    y_t = F.max_pool2d(x, k, s, p)
    out, idx = pool.max_pool2d_forward(x.detach().numpy(), k, s, p)
    assert np.array_equal(out, y_t.detach().numpy())
    g = torch.randn_like(y_t)
    y_t.backward(g)
    gin = pool.max_pool2d_backward(g.numpy(), idx, x.shape, k, s, p)
    assert np.allclose(gin, x.grad.numpy(), atol=1e-6)
    assert idx.max() < k[0] * k[1] and idx.min() >= 0


@pytest.mark.parametrize("k,s,p", CASES[:3])
def test_literal_agrees_and_ties_take_first(k, s, p):
    rng = np.random.default_rng(0)
    x = rng.integers(0, 3, (1, 2, 9, 8)).astype(np.float32)      # many ties
    a = pool.max_pool2d_forward(x, k, s, p)
    b = pool.max_pool2d_forward_literal(x, k, s, p)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
    # gather(input, index) == output
    out, idx = a
    for h in range(out.shape[2]):
        for w in range(out.shape[3]):
            i = h * s[0] - p[0] + idx[0, 0, h, w] // k[1]
            j = w * s[1] - p[1] + idx[0, 0, h, w] % k[1]
            assert x[0, 0, i, j] == out[0, 0, h, w]


def test_index_nibbles_known_bytes_and_round_trip():
    idx = np.array([1, 8, 0, 14, 3], np.int8)
    packed = pool.pack_index_nibbles(idx)
    assert packed.dtype == np.uint8 and packed.tolist() == [0x81, 0xE0, 0x03]
    assert np.array_equal(pool.unpack_index_nibbles(packed, 5), idx)
    rng = np.random.default_rng(0)
    for n in (0, 1, 2, 17, 256):
        idx = rng.integers(0, 15, n).astype(np.int8)
        p = pool.pack_index_nibbles(idx)
        assert p.size == (n + 1) // 2
        assert np.array_equal(pool.unpack_index_nibbles(p, n), idx)
