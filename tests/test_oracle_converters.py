"""Pins the oracle's FP32->FP16 / FP32->BF16 converters against independent
implementations: numpy's float16 cast (exhaustively around every fp16 value and
every rounding boundary) and torch's bfloat16 cast."""
import numpy as np


def _all_f16_boundaries():
    h = np.arange(0, 0x7c00, dtype=np.uint16)  # all non-negative finite halves
    v = h.view(np.float16).astype(np.float64)
    nxt = np.arange(1, 0x7c01, dtype=np.uint16).view(np.float16).astype(np.float64)
    nxt[-1] = 65536.0  # the value after 65504 on the fp16 grid if it had more exponent
    mid = (v + nxt) / 2  # exact ties (representable in fp32: 12 significant bits)
    cands = [v, mid]
    for base in (v, mid):
        f = base.astype(np.float32)
        cands.append(np.nextafter(f, np.float32(np.inf)).astype(np.float64))
        cands.append(np.nextafter(f, np.float32(-np.inf)).astype(np.float64))
    x = np.concatenate(cands).astype(np.float32)
    return np.concatenate([x, -x])


def test_f16_exhaustive_against_numpy(O):
    x = _all_f16_boundaries()
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = O.f32_to_f16_bits(x)
    assert np.array_equal(got, want)


def test_f16_random_bit_patterns_against_numpy(O):
    rng = np.random.default_rng(123)
    bits = rng.integers(0, 2 ** 32, size=2_000_000, dtype=np.uint64).astype(np.uint32)
    x = bits.view(np.float32)
    x = x[~np.isnan(x)]
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(O.f32_to_f16_bits(x), want)


def test_f16_special_values(O):
    L = O.lib()
    assert L.oracle_f32_to_f16_bits(0.0) == 0
    assert L.oracle_f32_to_f16_bits(-0.0) == 0x8000
    assert L.oracle_f32_to_f16_bits(float("inf")) == 0x7c00
    assert L.oracle_f32_to_f16_bits(65504.0) == 0x7bff
    assert L.oracle_f32_to_f16_bits(65519.99) == 0x7bff
    assert L.oracle_f32_to_f16_bits(65520.0) == 0x7c00  # tie rounds to even = inf
    assert L.oracle_f32_to_f16_bits(2.0 ** -24) == 1  # smallest subnormal
    assert L.oracle_f32_to_f16_bits(2.0 ** -25) == 0  # tie to even
    assert L.oracle_f32_to_f16_bits(np.nextafter(np.float32(2.0 ** -25), np.float32(1))) == 1
    nan = L.oracle_f32_to_f16_bits(float("nan"))
    assert (nan & 0x7c00) == 0x7c00 and (nan & 0x3ff) != 0


def test_f16_widening_roundtrip(O):
    h = np.arange(0, 0x10000, dtype=np.uint32).astype(np.uint16)
    f = h.view(np.float16).astype(np.float32)
    L = O.lib()
    for bits in list(range(0, 0x10000, 97)) + [0x0001, 0x03ff, 0x0400, 0x7bff, 0x7c00, 0x8001, 0xfbff]:
        got = L.oracle_f16_bits_to_f32(bits)
        want = f[bits]
        assert (np.isnan(got) and np.isnan(want)) or got == want


def test_bf16_against_torch(O):
    import torch
    rng = np.random.default_rng(5)
    bits = rng.integers(0, 2 ** 32, size=1_000_000, dtype=np.uint64).astype(np.uint32)
    x = bits.view(np.float32)
    x = x[~np.isnan(x)]
    want = torch.from_numpy(x.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(O.f32_to_bf16_bits(x), want)
    # ties: values exactly half-way between two bf16 neighbours
    base = (rng.integers(0x0080, 0x7f00, size=10000, dtype=np.uint32) << 16) | np.uint32(0x8000)
    t = base.view(np.float32)
    want = torch.from_numpy(t.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(O.f32_to_bf16_bits(t), want)
