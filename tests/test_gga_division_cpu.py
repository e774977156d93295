"""The two shortcuts the kernels take for their divisions (statequant_amd/csrc/sq_device.cuh: ``rcp_f16``, ``div_rc``
-- the GGA fit's divisions, every quantizer scale ``absmax / qmax``, the buffer entries ``x / scale`` and the pack
kernels' ``x / scale``), checked in exact rational arithmetic on the CPU: with fp32 fused multiply-adds modelled exactly,

  * one Newton step from ANY estimate within 1 ulp of 1 / d gives the correctly rounded fp32 reciprocal, for every
    fp16-valued divisor d (the row and column factors of the fit are fp16 values);
  * q = RN(x rc), r = fma(-q, d, x), RN(q + r rc) with that reciprocal is the correctly rounded x / d -- the quotient
    an IEEE division (torch's, the reference's ``div_rn``) returns -- also for x chosen to sit next to the rounding
    ties of the code grid, and for the divisors 3, 7, 31, 127 (qmax).

So the kernel's codes are those of true divisions, which the GPU tests can only show statistically.
"""
from fractions import Fraction

import numpy as np


def rn32(fr):
    """The fp32 value (as an exact Fraction) nearest to the Fraction fr, ties to even; normal range only."""
    if fr == 0:
        return Fraction(0)
    s = -1 if fr < 0 else 1
    a = abs(fr)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    assert -126 <= e <= 127, e
    ulp = Fraction(2) ** (e - 23)
    n, rem = divmod(a, ulp)
    n = int(n)
    if rem * 2 > ulp or (rem * 2 == ulp and n % 2 == 1):
        n += 1
    return s * n * ulp


def fma32(a, b, c):
    return rn32(a * b + c)


def fr(x):
    return Fraction(float(x))


def fp16_divisors():
    """Every positive fp16 value from 2^-24 (the fit clamps there) to 65504."""
    bits = np.arange(1, 0x7C00, dtype=np.uint16)
    return bits.view(np.float16).astype(np.float64)


def ulp_of(fr_val):
    a = abs(fr_val)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    return Fraction(2) ** (e - 23)


def test_newton_step_gives_the_correctly_rounded_reciprocal():
    ds = fp16_divisors()
    step = 7                                         # every 7th value, plus both ends and the powers of two's neighbours
    sample = list(ds[::step]) + list(ds[:40]) + list(ds[-40:])
    bad = 0
    for d in sample:
        d = fr(d)
        want = rn32(1 / d)
        u = ulp_of(want)
        for r0 in (want - u, want, want + u):        # any estimate within 1 ulp (the hardware's guarantee)
            e = fma32(-d, r0, Fraction(1))
            got = fma32(e, r0, r0)
            bad += got != want
    assert bad == 0, bad


def test_reciprocal_division_is_the_ieee_quotient():
    rng = np.random.default_rng(0)
    ds = fp16_divisors()
    divisors = [fr(d) for d in rng.choice(ds, 400, replace=False)] + [Fraction(q) for q in (3, 7, 31, 127)]
    bad = total = 0
    for d in divisors:
        rc = rn32(1 / d)
        xs = [fr(np.float32(v)) for v in rng.standard_normal(12) * float(d) * rng.choice([0.3, 3.0, 40.0, 120.0], 12)]
        # values whose quotient sits within a few ulp of k + 1/2, where a code flips
        for k in (0, 1, 6, 30, 126):
            t = (Fraction(2 * k + 1, 2)) * d
            base = rn32(t)
            u = ulp_of(base)
            xs += [base - u, base, base + u]
        for x in xs:
            if x == 0:
                continue
            q = rn32(x * rc)
            r = fma32(-q, d, x)
            got = fma32(r, rc, q)
            bad += got != rn32(x / d)
            total += 1
    assert total > 10000 and bad == 0, (bad, total)


def rn16_of_f32(fr32):
    """fp16 (as an exact Fraction) nearest to an fp32 value, ties to even, subnormals kept; below the overflow range."""
    if fr32 == 0:
        return Fraction(0)
    a = abs(fr32)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    e = max(e, -14)
    ulp = Fraction(2) ** (e - 10)
    n, rem = divmod(a, ulp)
    n = int(n)
    if rem * 2 > ulp or (rem * 2 == ulp and n % 2 == 1):
        n += 1
    return n * ulp


def test_scale_is_rounded_twice_as_the_reference_does():
    """``fp16_scale``: absmax / qmax as an fp32 quotient, THEN to fp16 -- two roundings, as torch's
    ``(amax / qmax).to(float16)``.  A single rounding of the exact value of the division's last fused multiply-add
    (what a fused fma-and-convert instruction would do) differs where the fp32 quotient is an fp16 tie; the absmax
    below, 7 x an fp16 midpoint, is one that the pack test's data contains."""
    rng = np.random.default_rng(1)
    xs = [fr(np.float32(1.45391845703125))]
    for qmax in (7, 127):
        # fp32 values that are exactly qmax x (an fp16 midpoint): the quotient is the midpoint itself
        mids = rng.integers(1024, 2048, 60) * 2 + 1                     # odd 12-bit significands
        xs += [Fraction(int(m), 4096) * Fraction(2) ** int(e) * qmax for m, e in zip(mids, rng.integers(-6, 6, 60))]
    xs += [fr(np.float32(v)) for v in np.abs(rng.standard_normal(400)) * 3]
    single = 0
    for qmax in (7, 127):
        d, rc = Fraction(qmax), rn32(Fraction(1, qmax))
        for x in xs:
            if rn32(x) != x:
                continue
            q = rn32(x * rc)
            r = fma32(-q, d, x)
            s32 = fma32(r, rc, q)
            assert s32 == rn32(x / d)
            assert rn16_of_f32(s32) == rn16_of_f32(rn32(x / d))         # what the kernel computes == the reference
            single += rn16_of_f32(r * rc + q) != rn16_of_f32(s32)       # one rounding of the unrounded sum instead
    assert single > 0                                                   # the fused form would differ on some of these
