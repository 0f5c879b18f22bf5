"""Pins the hi/lo (fp16) and b0/b1/b2 (bf16) splits of the oracle through the
invariants the published algorithm guarantees, using float64 as exact
arithmetic (every quantity involved has at most 24+11 significant bits)."""
import numpy as np


def _samples(rng, n):
    mant = rng.uniform(1.0, 2.0, n)
    exp = rng.integers(-13, 16, n)  # |a| in [2^-13, 2^16): hi normal and finite
    sign = rng.choice([-1.0, 1.0], n)
    return (sign * np.ldexp(mant, exp)).astype(np.float32)


def test_fp16_split_invariants(O):
    rng = np.random.default_rng(11)
    a = _samples(rng, 500_000)
    a = a[np.abs(a) <= 65504.0]
    hi, lo = O.split_fp16(a)
    a64, hi64, lo64 = a.astype(np.float64), hi.astype(np.float64), lo.astype(np.float64)
    # hi is the nearest fp16 (independent check: numpy cast)
    assert np.array_equal(hi, a.astype(np.float16).astype(np.float32))
    # (i) the residual is exact in FP32 and at most half an fp16 ulp
    r64 = a64 - hi64
    assert np.array_equal((a - hi).astype(np.float64), r64)
    e = np.floor(np.log2(np.abs(a64)))
    assert np.all(np.abs(r64) <= np.ldexp(1.0, (e - 11).astype(int)) * (1 + 1e-12))
    # (ii) scaling by 2^11 is exact; lo is its nearest fp16
    assert np.array_equal(lo, ((a - hi) * np.float32(2048.0)).astype(np.float16).astype(np.float32))
    # (iii) reconstruction error <= 2^-22 |a| whenever lo is a normal fp16
    normal_lo = (np.abs(r64) * 2048.0 >= 2.0 ** -14) | (r64 == 0)
    err = np.abs(a64 - (hi64 + lo64 / 2048.0))
    assert np.all(err[normal_lo] <= np.abs(a64[normal_lo]) * 2.0 ** -22)
    # the bound is nearly attained somewhere (so it is not vacuous)
    assert err.max() > 2.0 ** -26 * np.abs(a64).min()


def test_fp16_split_exact_for_22_bit_inputs(O):
    rng = np.random.default_rng(12)
    # 21-bit integers times a power of two: hi takes 11 bits, lo the rest exactly
    k = rng.integers(1, 2 ** 21, 200_000)
    s = rng.integers(-24, -8, 200_000)
    a = np.ldexp(k.astype(np.float64), s).astype(np.float32)
    a = a[(np.abs(a) >= 2.0 ** -3) & (np.abs(a) <= 60000.0)]
    hi, lo = O.split_fp16(a)
    assert np.array_equal(hi.astype(np.float64) + lo.astype(np.float64) / 2048.0, a.astype(np.float64))


def test_fp16_split_degrades_outside_range(O):
    big = np.array([70000.0, -1e6, 65520.0], dtype=np.float32)
    hi, lo = O.split_fp16(big)
    assert np.all(np.isinf(hi))
    tiny = np.array([2.0 ** -20, 3.0e-7, -2.0 ** -26], dtype=np.float32)
    hi, lo = O.split_fp16(tiny)
    # hi is subnormal (or zero) fp16, lo may flush: error no longer 2^-22 relative
    assert np.all(np.abs(hi) < 2.0 ** -14)
    zero = np.zeros(4, dtype=np.float32)
    hi, lo = O.split_fp16(zero)
    assert not hi.any() and not lo.any()


def test_bf16x3_split_invariants(O):
    rng = np.random.default_rng(13)
    mant = rng.uniform(1.0, 2.0, 300_000)
    exp = rng.integers(-60, 60, 300_000)
    a = (rng.choice([-1.0, 1.0], 300_000) * np.ldexp(mant, exp)).astype(np.float32)
    b0, b1, b2 = O.split_bf16x3(a)
    import torch
    as_bf16 = lambda x: torch.from_numpy(x.copy()).to(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(b0, as_bf16(a))
    assert np.array_equal(b1, as_bf16(a - b0))
    assert np.array_equal(b2, as_bf16((a - b0) - b1))
    # three 8-bit pieces carry all 24 bits: the sum is exact
    s = b0.astype(np.float64) + b1.astype(np.float64) + b2.astype(np.float64)
    assert np.array_equal(s, a.astype(np.float64))
    # two pieces: 16 bits
    s2 = b0.astype(np.float64) + b1.astype(np.float64)
    assert np.all(np.abs(s2 - a) <= np.abs(a) * 2.0 ** -16)
