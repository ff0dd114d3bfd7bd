"""Pins for the simulate-quantiser restatement (oracle/simulate.py)."""
import itertools

import numpy as np
import pytest
import torch

from oracle import simulate


def _case(N, G, gs, seed, scale=1.0, relu=True):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(N, G, gs, generator=g) * scale
    if relu:
        x = torch.relu(x)
    mn = x.min(dim=2, keepdim=True)[0]
    mx = x.max(dim=2, keepdim=True)[0]
    noise = torch.rand(N, G, gs, generator=g) - 0.5
    return x, mn, mx, noise


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 8])
@pytest.mark.parametrize("scale", [1.0, 1e-3, 300.0])
def test_torch_and_numpy_restatements_agree(bits, scale):
    x, mn, mx, noise = _case(6, 5, 256, 11, scale)
    q_t, s_t = simulate.quantize_simulate(x.clone(), bits, mn, mx, noise)
    q_n, s_n = simulate.quantize_simulate_np(x.numpy(), bits, mn.numpy(), mx.numpy(), noise.numpy())
    assert np.array_equal(q_t.numpy(), q_n)
    assert np.array_equal(s_t.numpy().view(np.uint32), s_n.view(np.uint32))
    d_t = simulate.dequantize_simulate(q_t, s_t, mn)
    d_n = simulate.dequantize_simulate_np(q_n, s_n, mn.numpy())
    assert np.array_equal(d_t.numpy().view(np.uint32), d_n.view(np.uint32))


def test_mixed_bits_tensor():
    x, mn, mx, noise = _case(8, 3, 256, 5)
    bits = torch.tensor([1, 2, 3, 4, 5, 6, 7, 8], dtype=torch.int32)
    q, s = simulate.quantize_simulate(x.clone(), bits, mn, mx, noise)
    q_n, s_n = simulate.quantize_simulate_np(x.numpy(), bits.numpy(), mn.numpy(), mx.numpy(), noise.numpy())
    assert np.array_equal(q.numpy(), q_n)
    for n in range(8):
        assert int(q[n].max()) <= 2 ** int(bits[n]) - 1 and int(q[n].min()) >= 0


def test_invariants_without_noise():
    x, mn, mx, _ = _case(4, 4, 256, 3)
    for bits in (1, 2, 4, 8):
        B = 2 ** bits - 1
        q, s = simulate.quantize_simulate(x.clone(), bits, mn, mx, None)
        # the group minimum maps to code 0 and the maximum to B
        assert (q.min(dim=2)[0] == 0).all() and (q.max(dim=2)[0] == B).all()
        # dequantisation error is at most half a step (+ the 1e-6 shifts)
        d = simulate.dequantize_simulate(q, s, mn)
        assert ((d - x).abs() <= 0.5 / s + 3e-6).all()


def test_half_to_even_rounding():
    # group = {0, 1, ..., B}: t is an exact integer grid up to the 1e-6 guards; with an explicit
    # noise of exactly +-0.5 on integer t the tie must go to the even code.  Build t directly:
    # mn = 0, mx = B so scale ~ 1 - 2e-6/B, then check against closed-form float arithmetic.
    B = 3
    x = torch.tensor([[[0.0, 1.0, 2.0, 3.0] * 64]])
    mn = torch.zeros(1, 1, 1)
    mx = torch.full((1, 1, 1), float(B))
    mn32, mx32 = np.float32(0) - np.float32(1e-6), np.float32(B) + np.float32(1e-6)
    scale = np.float32(B) / np.float32(mx32 - mn32)
    for nz in (0.5, -0.5, 0.25, 0.0):
        noise = torch.full_like(x, nz)
        q, s = simulate.quantize_simulate(x.clone(), 2, mn, mx, noise)
        t = (x.numpy().astype(np.float32) - mn32).astype(np.float32) * scale
        t = (t.astype(np.float32) + np.float32(nz)).astype(np.float32)
        exp = np.rint(np.clip(t, 0, B)).astype(np.int32)
        assert np.array_equal(q.numpy(), exp)
    # genuine ties: t + noise exactly k + 0.5
    t = torch.tensor([0.5, 1.5, 2.5, 3.5])
    assert torch.equal(t.round(), torch.tensor([0.0, 2.0, 2.0, 4.0]))


def test_brute_force_tiny_group():
    # every ordering of a 4-value group, 1 and 2 bits, against scalar python float32 arithmetic
    vals = [0.0, 0.3, 0.7, 1.9]
    f = np.float32
    for perm in itertools.permutations(vals):
        x = torch.tensor(perm, dtype=torch.float32).view(1, 1, 4).repeat(1, 1, 8)    # gs = 32
        mn = x.min(dim=2, keepdim=True)[0]
        mx = x.max(dim=2, keepdim=True)[0]
        noise = torch.linspace(-0.49, 0.49, 32).view(1, 1, 32)
        for bits in (1, 2):
            q, _ = simulate.quantize_simulate(x.clone(), bits, mn, mx, noise)
            B = f(2 ** bits - 1)
            mns, mxs = f(f(0.0) - f(1e-6)), f(f(1.9) + f(1e-6))
            sc = f(B / f(mxs - mns))
            for i in range(32):
                t = f(f(f(f(x[0, 0, i].item()) - mns) * sc) + f(noise[0, 0, i].item()))
                t = min(max(t, f(0)), B)
                assert int(q[0, 0, i]) == int(np.rint(t))


def test_group_view_padding():
    x = torch.arange(2 * 3 * 100, dtype=torch.float32).view(2, 3, 10, 10)   # 300 features -> 512
    gview = simulate.group_view(x, 256)
    assert gview.shape == (2, 2, 256)
    assert torch.equal(gview.view(2, -1)[:, :300], x.view(2, -1))
    assert (gview.view(2, -1)[:, 300:] == 0).all()
    y = torch.zeros(2, 512)
    assert simulate.group_view(y, 256).shape == (2, 2, 256)


def test_minimax_is_rowwise():
    x = torch.randn(100, 256)
    mn, mx = simulate.minimax(x)
    assert torch.equal(mn, torch.from_numpy(x.numpy().min(axis=1)))
    assert torch.equal(mx, torch.from_numpy(x.numpy().max(axis=1)))


def test_range_sqr_closed_form_and_torch_expression():
    """oracle.kernel_mode.range_sqr: a constant range r over G groups gives G * r^2 * factor, and on
    random fp32 data it agrees with the reference's tensor expression (qscheme.py:80) evaluated
    by torch on the CPU; 16-bit inputs round the subtraction to the tensor dtype first."""
    from oracle import kernel_mode
    N, G = 5, 37
    mn = np.full((N, G), -0.25, np.float32)
    mx = np.full((N, G), 1.25, np.float32)
    assert np.allclose(kernel_mode.range_sqr(mn, mx, 0.5), G * 1.5 ** 2 * 0.5, rtol=0, atol=1e-12)
    rng = np.random.default_rng(0)
    mn = rng.standard_normal((N, G)).astype(np.float32)
    mx = mn + rng.random((N, G)).astype(np.float32) * 3
    ref = torch.norm((torch.from_numpy(mx) - torch.from_numpy(mn)).view(N, -1), dim=1).float().square() * (256 / 49)
    mult = rng.random(N).astype(np.float32) + 0.5
    got = kernel_mode.range_sqr(mn, mx, 256 / 49, mult)
    assert np.allclose(got, ref.numpy().astype(np.float64) * mult, rtol=1e-5)
    # 16-bit inputs: the subtraction rounds to the tensor dtype (numpy float16 stands for it here)
    mnh, mxh = mn.astype(np.float16), mx.astype(np.float16)
    d = (torch.from_numpy(mxh) - torch.from_numpy(mnh)).float().numpy().astype(np.float64)
    assert np.allclose(kernel_mode.range_sqr(mnh, mxh), (d ** 2).sum(1), rtol=1e-12)
