"""Pins the oracle's exponent statistics, scaling coefficients, launch-flag
packing and ring ids against brute-force recounts in numpy and closed forms."""
import zlib

import numpy as np
import pytest

FP16TCEC, TF32TCEC, UNDEFINED, SCALING = 1, 2, 10, 11


def _brute(x, ignore, under, tol):
    """Independent restatement with numpy reductions over the logical elements."""
    f = np.abs(x.view(np.float32) if x.dtype == np.complex64 else x).astype(np.float32)
    finite_max = np.float32(np.fmax.reduce(f, initial=np.float32(0)))
    bits = np.uint32(finite_max.view(np.uint32) & np.uint32(0x7f800000))
    max_exp = bits.view(np.float32)
    total = int(np.count_nonzero(f >= np.float32(ignore)))
    und = int(np.count_nonzero((f >= np.float32(ignore)) & (f < np.float32(under))))
    stage2 = False
    if np.float32(und) > np.float32(total) * np.float32(tol) or (max_exp > 0 and total == 0):
        stage2 = True
        np.seterr(invalid="ignore")  # inf * 0 thresholds compare false, as on the device
        it = np.float32(np.float32(ignore) / np.float32(2)) * max_exp
        ut = np.float32(np.float32(under) / np.float32(2)) * max_exp
        total = int(np.count_nonzero(f >= it))
        und = int(np.count_nonzero((f >= it) & (f < ut)))
        mode = SCALING if np.float32(und) <= np.float32(total) * np.float32(tol) else TF32TCEC
    else:
        mode = FP16TCEC
    return int(bits), total, und, mode, stage2


CASES = {
    "unit_normal": lambda rng: rng.standard_normal(20000).astype(np.float32),
    "tiny_normal": lambda rng: (rng.standard_normal(20000) * 2.0 ** -16).astype(np.float32),
    "wide_exponents": lambda rng: (rng.standard_normal(20000) * np.ldexp(1.0, rng.integers(-30, 31, 20000))).astype(np.float32),
    "all_zero": lambda rng: np.zeros(5000, dtype=np.float32),
    "one_huge": lambda rng: np.concatenate([np.full(4999, 1e-3), [3e30]]).astype(np.float32),
    "denormals": lambda rng: (rng.integers(1, 1000, 3000).astype(np.uint32)).view(np.float32),
    "with_nan_inf": lambda rng: np.array([1.0, np.nan, -np.inf, 2.0 ** -20, 0.0] * 100, dtype=np.float32),
    "scaled_small": lambda rng: (rng.uniform(0.5, 1.0, 8000) * 2.0 ** -17).astype(np.float32),
}


@pytest.mark.parametrize("name", sorted(CASES))
@pytest.mark.parametrize("params", [(0.0, 2.0 ** -15, 0.0), (2.0 ** -24, 2.0 ** -15, 0.1), (0.0, 2.0 ** -15, 0.5)])
def test_stats_match_bruteforce(O, name, params):
    rng = np.random.default_rng(zlib.crc32(name.encode()))
    x = CASES[name](rng)
    m, n = len(x) // 10, 10
    x = x[: m * n].copy()
    got = O.exp_stats(x, m, n, m, ignore=params[0], underflow=params[1], tol=params[2])
    want = _brute(x, *params)
    assert (got.max_exp_bits, got.total, got.underflow, got.mode, bool(got.stage2_ran)) == want
    assert O.exp_max_bits(x, m, n, m) == want[0]


def test_known_decisions(O):
    rng = np.random.default_rng(0)
    unit = rng.standard_normal(4096).astype(np.float32)
    unit[np.abs(unit) < 2.0 ** -14] = 0.5
    assert O.exp_stats(unit, 64, 64, 64).mode == FP16TCEC
    # all tiny but within a narrow band: scaling rescues it
    band = (rng.uniform(0.5, 1.0, 4096) * 2.0 ** -20).astype(np.float32)
    s = O.exp_stats(band, 64, 64, 64)
    assert s.mode == SCALING and s.stage2_ran == 1 and s.underflow == 0 and s.total == 4096
    # 60 binades of spread: even relative to the maximum, values underflow
    wide = (rng.standard_normal(4096) * np.ldexp(1.0, rng.integers(-30, 31, 4096))).astype(np.float32)
    assert O.exp_stats(wide, 64, 64, 64).mode == TF32TCEC
    z = O.exp_stats(np.zeros(16, dtype=np.float32), 4, 4, 4)
    # zeros: stage 1 sees 16 of 16 below the threshold, stage 2 (thresholds 0) none
    assert (z.max_exp_bits, z.total, z.underflow, z.mode, z.stage2_ran) == (0, 16, 0, SCALING, 1)


def test_view_semantics(O):
    rng = np.random.default_rng(1)
    m, n, ld, batch = 7, 5, 11, 3
    stride = ld * n + 4
    buf = (rng.standard_normal(stride * batch) * 2.0 ** -16).astype(np.float32)
    logical = np.stack([buf[b * stride: b * stride + ld * n].reshape(n, ld)[:, :m] for b in range(batch)])
    got = O.exp_stats(buf, m, n, ld, batch=batch, stride=stride)
    assert (got.max_exp_bits, got.total, got.underflow, got.mode) == _brute(logical.reshape(-1), 0.0, 2.0 ** -15, 0.0)[:4]
    # stride == 0: only the first matrix
    got0 = O.exp_stats(buf, m, n, ld, batch=batch, stride=0)
    assert (got0.max_exp_bits, got0.total, got0.underflow, got0.mode) == _brute(logical[0].reshape(-1), 0.0, 2.0 ** -15, 0.0)[:4]
    # complex: re and im counted separately
    z = (rng.standard_normal(40) * 2.0 ** -16 + 1j * rng.standard_normal(40)).astype(np.complex64)
    gz = O.exp_stats(z, 8, 5, 8)
    assert (gz.max_exp_bits, gz.total, gz.underflow, gz.mode) == _brute(z, 0.0, 2.0 ** -15, 0.0)[:4]
    assert gz.total == 80


def test_scaling_coefficients_and_roundtrip(O):
    L = O.lib()
    for e in (-20, -3, 0, 5, 14, 30):
        mx = float(2.0 ** e)
        assert L.oracle_scale_ab_coef(mx) == 2.0 ** (14 - e)
        assert L.oracle_reset_ab_coef(mx) == 2.0 ** (e - 14)
    assert L.oracle_scale_c_coef(2.0 ** 3, 2.0 ** -5, 0, 0) == 2.0 ** (3 - 5 - 28)
    assert L.oracle_scale_c_coef(2.0 ** 3, 2.0 ** -5, 1, 0x40 | 1) == 2.0 ** (3 - 14)
    assert L.oracle_scale_c_coef(2.0 ** 3, 2.0 ** -5, 1, 0x20 | 1) == 2.0 ** (-5 - 14)
    assert L.oracle_scale_c_coef(2.0 ** 3, 2.0 ** -5, 1, 0x60 | 1) == 2.0 ** (3 - 5 - 28)
    assert L.oracle_scale_c_coef(2.0 ** 3, 2.0 ** -5, 1, 1) == 1.0
    rng = np.random.default_rng(2)
    x = (rng.standard_normal(600) * 2.0 ** -18).astype(np.float32)
    bits = O.exp_max_bits(x, 20, 30, 20)
    mx = np.uint32(bits).view(np.float32)
    y = x.copy()
    O.scale_matrix(y, 20, 30, 20, L.oracle_scale_ab_coef(mx))
    assert 2.0 ** 14 <= np.abs(y).max() < 2.0 ** 15
    O.scale_matrix(y, 20, 30, 20, L.oracle_reset_ab_coef(mx))
    assert np.array_equal(x, y)  # a power-of-two scale is undone exactly


def test_flag_truth_table_and_ring(O):
    L = O.lib()
    for a in (FP16TCEC, SCALING, TF32TCEC):
        for b in (FP16TCEC, SCALING, TF32TCEC):
            f = L.oracle_combine_flag(a, b)
            if TF32TCEC in (a, b):
                assert f == TF32TCEC
            else:
                assert f & 0x1f == FP16TCEC
                assert bool(f & 0x40) == (a == SCALING) and bool(f & 0x20) == (b == SCALING)
    assert ((3 << 5) | FP16TCEC) == L.oracle_combine_flag(SCALING, SCALING)
    cur, seen = 1, []
    for _ in range(25):
        cur = L.oracle_next_ring_id(cur, 10)
        seen.append(cur)
    assert seen[:8] == [2, 3, 4, 5, 6, 7, 8, 9] and seen[8] == 2 and 0 not in seen and 1 not in seen
