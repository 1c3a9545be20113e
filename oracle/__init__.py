"""CPU oracle for the MXFP8 MoE FFN forward path.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package imports this directory.  Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may use it,
and there only as the checker.

Pin status of each function (what independent evidence fixes its result):

* ``mxfp8.e4m3_decode``      -- exhaustive 256-entry comparison with torch's
  ``float8_e4m3fn`` view (library routine) and the C restatement.
* ``mxfp8.e4m3_encode``      -- every bf16 bit pattern and a dense fp32 sweep against
  torch's cast after an explicit clamp to +-448, and against the C restatement.
* ``mxfp8.e8m0_*``           -- closed form 2**(b-127), cross-checked with torch's
  ``float8_e8m0fnu``.
* ``mxfp8.mx_quantize``      -- the OCP MX v1.0 rule (documented in the docstring);
  property tests (power-of-two scale, max code magnitude in [256,448], idempotence,
  sign symmetry) plus the C restatement.  The rule used by the reference's absent
  third-party quantiser (mixture-of-kittens @ f3a8bd2, ``csrc/mxfp8.cuh``) cannot be
  read here: **parity unpinned** against that dependency; irrelevant to the metric
  because oracle and kernel consume the same pre-quantised bytes.
* ``moe_ffn.gptoss_swiglu``  -- closed form following
  campaigns/mok/host/act_gptoss_reference.py:16-21; special-value tests.
* ``moe_ffn.grouped_matmul`` -- brute-force triple loop on tiny shapes + the C
  restatement; reduces to ``torch.matmul`` per expert.
* accumulation order / bf16 epilogue rounding of the reference's
  ``expert_grouped_gemm_kernel`` (absent third-party source): **parity unpinned**;
  the stated tolerance (relative Frobenius <= 3e-2) is the bar instead.
"""
