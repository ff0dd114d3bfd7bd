"""Committed fixtures (tests/golden/, written by tests/golden/make_fixtures.py): the CPU
restatements must keep reproducing them, and so must the HIP kernels - bit for bit."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import calc_precision as o_calc
from oracle import kernel_mode, layouts, philox, pool, simulate

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
V = np.load(os.path.join(HERE, "vectors.npz"), allow_pickle=False)
KA = json.load(open(os.path.join(HERE, "known_answers.json")))
DTYPES = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}
N, G, GS = 8, 3, 256


def _tensor(name, tag):
    raw = torch.from_numpy(V[f"pack_{tag}_{name}"].copy())
    return raw.view(DTYPES[tag])


def test_known_answers_philox_and_degenerate_allocation():
    for k in KA["philox4x32_10"]:
        got = philox.philox4x32_10(np.array([k["counter"]], dtype=np.uint32), tuple(k["key"]))[0]
        assert [int(v) for v in got] == k["output"]
    z = KA["calc_precision_zero_sensitivity"]
    bits = o_calc.calc_precision(np.full(z["N"], z["initial_bits"], np.int32), np.zeros(z["N"], np.float32),
                                 np.ones(z["N"], np.int32), z["target"])
    assert [int(v) for v in bits] == z["bits"]
    # the first-step state of every layer: samples 0-35 keep 8 bits, sample 36 gets 5, the rest 1
    assert z["bits"][:36] == [8] * 36 and z["bits"][36] == 5 and z["bits"][37:] == [1] * 219


@pytest.mark.parametrize("tag", ["f32", "f16", "bf16"])
def test_oracle_reproduces_the_deterministic_vectors(tag):
    x, noise = _tensor("x", tag), _tensor("noise", tag)
    bits = torch.from_numpy(V["pack_bits"].copy())
    mn, mx = x.min(2, keepdim=True)[0], x.max(2, keepdim=True)[0]
    codes, scale = simulate.quantize_simulate(x.clone(), bits, mn, mx, noise)
    assert np.array_equal(layouts.pack_mixed(codes.numpy(), bits.numpy()).astype(np.int32), V[f"pack_{tag}_words"])
    assert torch.equal(scale, _tensor("scale", tag))
    assert torch.equal(simulate.dequantize_simulate(codes, scale, mn), _tensor("dequant", tag))


def test_oracle_reproduces_rng_mask_and_pool_vectors():
    x = _tensor("x", "f32")
    bits = torch.from_numpy(V["pack_bits"].copy())
    mn, mx = x.min(2, keepdim=True)[0], x.max(2, keepdim=True)[0]
    seed, offset = (int(v) for v in V["rng_seed_offset"])
    codes = kernel_mode.rng_codes(x, mn, kernel_mode.kernel_scale(mn, mx, bits), bits, seed, offset)
    assert np.array_equal(layouts.pack_mixed(np.asarray(codes), bits.numpy()).astype(np.int32), V["rng_words"])
    assert np.array_equal(layouts.mask_words(V["mask_input_positive"]).astype(np.int32), V["mask_words"])
    y, idx = pool.max_pool2d_forward(V["pool_x"], (3, 3), (2, 2), (1, 1))
    assert np.array_equal(y, V["pool_y"]) and np.array_equal(idx, V["pool_idx"])


# ------------------------------------------------------------------------------------------ GPU
@pytest.mark.gpu
@pytest.mark.parametrize("tag", ["f32", "f16", "bf16"])
def test_kernels_reproduce_the_deterministic_vectors(tag):
    import actnn_amd.cpp_extension.minimax as ext_minimax
    import actnn_amd.cpp_extension.quantization as ext_q
    dev = "cuda:0"
    x, noise = _tensor("x", tag).to(dev), _tensor("noise", tag).to(dev)
    host_bits = torch.from_numpy(V["pack_bits"].copy())
    bits = ext_q.attach_bits_host(host_bits.to(dev), host_bits)
    mn, mx = ext_minimax.minimax(x.view(-1, GS))
    mn, mx = mn.view(N, G, 1), mx.view(N, G, 1)
    packed, scale = ext_q.pack_mixed_precision(x, mn, mx, bits, True, noise=noise)
    assert np.array_equal(packed.cpu().numpy(), V[f"pack_{tag}_words"])
    assert torch.equal(scale.cpu(), _tensor("scale", tag))
    out = ext_q.unpack_mixed_precision(packed, bits, scale, mn, N, G, GS)
    assert torch.equal(out.cpu(), _tensor("dequant", tag))


@pytest.mark.gpu
def test_kernels_reproduce_rng_mask_and_pool_vectors():
    import actnn_amd.cpp_extension.minimax as ext_minimax
    import actnn_amd.cpp_extension.quantization as ext_q
    dev = "cuda:0"
    x = _tensor("x", "f32").to(dev)
    host_bits = torch.from_numpy(V["pack_bits"].copy())
    bits = ext_q.attach_bits_host(host_bits.to(dev), host_bits)
    mn, mx = ext_minimax.minimax(x.view(-1, GS))
    seed, offset = (int(v) for v in V["rng_seed_offset"])
    gen = torch.cuda.default_generators[0]
    gen.manual_seed(seed)
    gen.set_offset(offset)
    packed, _ = ext_q.pack_mixed_precision(x, mn.view(N, G, 1), mx.view(N, G, 1), bits, True)
    assert np.array_equal(packed.cpu().numpy(), V["rng_words"])
    pos = torch.from_numpy(V["mask_input_positive"].copy())
    xin = torch.where(pos, torch.ones(pos.numel()), -torch.ones(pos.numel())).to(dev)
    _, mask = ext_q.relu_forward(xin)
    assert np.array_equal(mask.cpu().numpy(), V["mask_words"])
    y, idx = ext_q.max_pool2d_forward(torch.from_numpy(V["pool_x"].copy()).to(dev), (3, 3), (2, 2), (1, 1), (1, 1))
    assert np.array_equal(y.cpu().numpy(), V["pool_y"]) and np.array_equal(idx.cpu().numpy(), V["pool_idx"])
