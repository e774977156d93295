"""CPU oracle of the packed-state decode step.  TEST INFRASTRUCTURE ONLY.

This package restates, in plain torch on the CPU, the arithmetic of the reference's own torch implementation of the
packed decode path (the classes its tests use as the yardstick for its Triton kernels):

    formats.py   storage format and rounding          <- /root/reference/src/statequant/kernels/fold.py:123-191,
                                                          /root/reference/src/statequant/quantizer.py:159-193
    states.py    GDN / KDA / Mamba2 packed decode     <- fold.py:197-274 (ReferenceGDNState), kda.py:95-186
                 and the textbook fp32 recurrences       (ReferenceKDAState), mamba2.py:116-217
                                                          (ReferenceMamba2State), kda.py:44-52, mamba2.py:45-70
    slots.py     per-slot byte layout, read, write    <- slots.py:76-95, 210-252; kda.py:311-323, 351-386;
                                                          mamba2.py:359-370
    gga.py       mixed-width GGA / STEP slot, FP8     <- /root/reference/src/statequant/step_quant.py:35-96,
                 window, its byte layout                 methods_ext/gga.py:225-233, integrations/vllm_gga.py:86-217,
                                                          kernels/_gga_triton.py:3-13, 40-95

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import it, and only as
the checker; nothing under ``statequant_amd/`` does.  It runs wherever torch runs (no GPU, no HIP library).

How it is pinned (see tests/test_oracle_*.py; gga.py states its own pins in its header):
  * bit-for-bit against golden vectors produced by the reference's own classes on seeded inputs
    (tests/golden/*.pt, written by tests/golden/make_golden.py) -- every function below is covered by them;
  * independently of those: pack/unpack against a per-group brute force in NumPy with np.float16 and against the
    format's closed form on the reference tests' edge cases (all-zero groups, scales in the fp16 subnormal range,
    ragged last group); the step algebra with an fp32 state and fp32 buffer against the textbook recurrences; the
    m = 1 special case against per-token rounding of the textbook update; ``read`` + one textbook step against the
    next packed step; the byte layout against the reference's documented per-slot totals;
  * the stand-alone helpers that no golden record exercises -- ``gdn_gate``, ``GGAState.gate`` and the one-step
    textbook recurrences ``gdn_recurrence`` / ``kda_recurrence`` / ``mamba2_recurrence`` -- against torch's library
    softplus / sigmoid and float64 NumPy recurrences on inputs either side of the softplus threshold, with non-zero
    A_log / dt_bias, dt limits and the D term (tests/test_oracle_math_cpu.py).
"""
