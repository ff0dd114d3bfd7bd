"""CPU oracle for the ActNN activation-compression path.  TEST INFRASTRUCTURE ONLY.

Nothing in the product package (``actnn_amd``) may import this package: it is the
checker used by ``tests/``, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py``.  Every function restates one piece of the
reference and cites the reference file:line it follows.

Pinning status (what fixes each function besides its own formula):

* ``simulate.quantize_simulate`` / ``dequantize_simulate`` - the reference's
  ``config.simulate`` branch is a dozen stock torch tensor ops; the restatement calls
  the same torch ops on CPU.  Pinned by an independent numpy-float32 step-by-step
  version, noise==0 half-to-even cases, range invariants and brute force on tiny groups.
* ``layouts.*`` - pure integer index arithmetic.  Pinned by a literal per-thread
  re-enactment of the reference kernels' index expressions (loops) on small cases and
  by pack/unpack round trips.
* ``philox.philox4x32_10`` - Random123 known-answer vectors.
* ``pool.*`` - ``torch.nn.functional.max_pool2d`` forward/backward (as the reference's
  own test does, tests/test_act_quantized_ops.py:206-232) + first-strict-max index rule.
* ``calc_precision.calc_precision`` - brute-force optimality on tiny inputs, the
  hand-derived degenerate allocation (C == 0) and, where it builds, the reference's own
  calc_precision.cc compiled into ``oracle/_ref`` (see ``oracle/build_ref.py``).
* ``kernel_mode.kernel_scale`` / ``kernel_dequant`` (arithmetic of the reference's CUDA
  kernels, which differs from ``config.simulate``) - pinned on the CPU by
  tests/test_oracle_kernel_mode.py: known answers where evaluating the scale in float instead
  of double, or narrowing double -> half directly, would store another value; an exact
  rational-arithmetic model of the rounding chain; constant groups (+inf in fp16) and B = 255.
* ``kernel_mode.fma32`` (correctly rounded float32 fma, used by the RNG model) - exact
  rational arithmetic on random and cancelling operands (tests/test_oracle_kernel_mode.py).
* ``kernel_mode.rng_codes`` and the rest of the in-kernel-RNG model - the arithmetic is pinned
  against the exact (x - min) * scale by brute force over every draw (8-bit noise) or a
  sweep (16-bit noise), and ``philox.noise8`` / ``noise16`` against the generator's words;
  the *stream values* of the reference's generator (cuRAND) are not reproducible here:
  parity unpinned for the values, the distribution (unbiasedness, closed-form variance) is
  pinned.
"""
