"""Writes the regression fixtures of this directory (run from the repository root:
`python tests/golden/make_fixtures.py`).

The reference ships no golden vectors for this path (its tests draw unseeded random data and
compare against torch operators), and nothing here comes from running the reference: the inputs are
seeded draws, the expected outputs come from the CPU restatements under `oracle/`, which are pinned
by the checks listed in `oracle/__init__.py`, plus published known answers (Random123 Philox4x32-10
vectors, the hand-derived degenerate bit allocation).  The fixtures freeze those results, so that a
later change of the restatement or of a kernel shows up as a difference against committed data.
"""
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import calc_precision as o_calc  # noqa: E402
from oracle import kernel_mode, layouts, philox, pool, simulate  # noqa: E402


def main():
    out = {}
    # 1. Philox4x32-10 known answers (Random123 kat_vectors)
    kat = [([0, 0, 0, 0], [0, 0], [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]),
           ([0xffffffff] * 4, [0xffffffff] * 2, [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]),
           ([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], [0xa4093822, 0x299f31d0],
            [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1])]
    json.dump({"philox4x32_10": [{"counter": c, "key": k, "output": o} for c, k, o in kat],
               # greedy allocation with all sensitivities zero: N = 256 items at 8 bits, budget 512
               "calc_precision_zero_sensitivity": {
                   "N": 256, "initial_bits": 8, "target": 512,
                   "bits": [int(v) for v in o_calc.calc_precision(
                       np.full(256, 8, np.int32), np.zeros(256, np.float32), np.ones(256, np.int32), 512)]}},
              open(os.path.join(HERE, "known_answers.json"), "w"), indent=1)

    # 2. deterministic-mode quantiser: seeded input and noise, every width once
    g = torch.Generator().manual_seed(2024)
    N, G, gs = 8, 3, 256
    x = torch.relu(torch.randn(N, G, gs, generator=g)) * torch.exp(torch.randn(1, G, 1, generator=g))
    noise = torch.rand(N, G, gs, generator=g) - 0.5
    bits = torch.tensor([1, 2, 3, 4, 5, 6, 7, 8], dtype=torch.int32)
    for name, dtype in (("f32", torch.float32), ("f16", torch.float16), ("bf16", torch.bfloat16)):
        xd, nd = x.to(dtype), noise.to(dtype)
        mn, mx = xd.min(2, keepdim=True)[0], xd.max(2, keepdim=True)[0]
        codes, scale = simulate.quantize_simulate(xd.clone(), bits, mn, mx, nd)
        words = layouts.pack_mixed(codes.numpy(), bits.numpy())
        deq = simulate.dequantize_simulate(codes, scale, mn)
        as_bits = (lambda t: t.contiguous().view(torch.int16).numpy()) if dtype != torch.float32 else \
            (lambda t: t.contiguous().view(torch.int32).numpy())
        out[f"pack_{name}_x"] = as_bits(xd)
        out[f"pack_{name}_noise"] = as_bits(nd)
        out[f"pack_{name}_words"] = words.astype(np.int32)
        out[f"pack_{name}_scale"] = as_bits(scale)
        out[f"pack_{name}_dequant"] = as_bits(deq)
    out["pack_bits"] = bits.numpy()

    # 3. in-kernel RNG mode: codes of the kernel-mode arithmetic with the Philox stream
    xr = x.to(torch.float32)
    mn, mx = xr.min(2, keepdim=True)[0], xr.max(2, keepdim=True)[0]
    seed, offset = 0x0123456789ABCDEF, 8
    sc = kernel_mode.kernel_scale(mn, mx, bits)
    rng = kernel_mode.rng_codes(xr, mn, sc, bits, seed, offset)
    out["rng_words"] = layouts.pack_mixed(np.asarray(rng), bits.numpy()).astype(np.int32)
    out["rng_seed_offset"] = np.array([seed, offset], dtype=np.uint64)

    # 4. ReLU mask words and max-pool indices
    m = torch.randn(3 * 512, generator=g) > 0
    out["mask_input_positive"] = m.numpy()
    out["mask_words"] = layouts.mask_words(m.numpy()).astype(np.int32)
    xp = torch.randn(2, 3, 9, 11, generator=g).numpy()
    yp, ip = pool.max_pool2d_forward(xp, (3, 3), (2, 2), (1, 1))
    out["pool_x"], out["pool_y"], out["pool_idx"] = xp, yp, ip
    np.savez_compressed(os.path.join(HERE, "vectors.npz"), **out)
    print("wrote", sorted(out))


if __name__ == "__main__":
    main()
