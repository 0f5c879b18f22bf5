"""Exponent statistics, scaling and launch flags of the HIP path against the
oracle: counts, max-exponent bits and decisions must be bit-exact; scaled data
must be bit-identical (multiplication by a power of two)."""
import numpy as np
import pytest

from cumpsgemm_amd import inputs

pytestmark = pytest.mark.gpu

FP16TCEC, TF32TCEC, UNDEFINED, SCALING = 1, 2, 10, 11


def _bits(f):
    return int(np.float32(f).view(np.uint32))


def _cmp_stats(O, handle, dev, x, m, n, ld, batch=1, stride=0, params=(0.0, 2.0 ** -15, 0.0), offset=0):
    cplx = x.dtype == np.complex64
    handle.set_exp_stats_params(*params)
    d = dev.up(x)
    es = 8 if cplx else 4
    ptr = d.data_ptr() + offset * es
    sid = handle.exp_stats_ext(m, n, ptr, ld, batch, stride, cplx=cplx)
    under, total = handle.get_exp_stats(sid)
    got = (_bits(handle.get_max_exp(sid)), total, under, handle.get_exp_stats_compute_mode_level(sid))
    o = O.exp_stats(x[offset:], m, n, ld, batch=batch, stride=stride, ignore=params[0], underflow=params[1], tol=params[2])
    assert got == (o.max_exp_bits, o.total, o.underflow, o.mode)
    mid = handle.exp_max_ext(m, n, ptr, ld, batch, stride, cplx=cplx)
    assert _bits(handle.get_max_exp(mid)) == O.exp_max_bits(x[offset:], m, n, ld, batch=batch, stride=stride)
    handle.set_exp_stats_params(0.0, 2.0 ** -15, 0.0)
    return got


@pytest.mark.parametrize("shape", [(1000, 777), (1, 1), (3, 5), (4096, 4096), (1023, 513), (64, 1)])
@pytest.mark.parametrize("sigma", [1.0, 2.0 ** -16])
def test_stats_dense(O, handle, dev, shape, sigma):
    m, n = shape
    x = inputs.normal(7, m * n, sigma)
    _cmp_stats(O, handle, dev, x, m, n, m)
    _cmp_stats(O, handle, dev, x, m, n, m, params=(2.0 ** -24, 2.0 ** -15, 0.1))


def test_stats_unaligned_pointer_and_tails(O, handle, dev):
    x = inputs.normal(8, 5000, 2.0 ** -15)
    for off in (1, 2, 3):
        for count in (1, 2, 3, 5, 1021, 4097):
            _cmp_stats(O, handle, dev, x, count, 1, count, offset=off)


def test_stats_strided_views(O, handle, dev):
    m, n, ld, batch = 70, 33, 96, 4
    stride = ld * n + 17
    x = inputs.normal(9, stride * batch, 2.0 ** -16)
    _cmp_stats(O, handle, dev, x, m, n, ld)
    _cmp_stats(O, handle, dev, x, m, n, ld, batch=batch, stride=stride)
    _cmp_stats(O, handle, dev, x, m, n, ld, batch=batch, stride=0)  # first matrix only
    d = inputs.normal(10, m * n * batch, 2.0 ** -14)
    _cmp_stats(O, handle, dev, d, m, n, m, batch=batch, stride=m * n)  # dense batch


def test_stats_complex(O, handle, dev):
    z = inputs.complex_normal(11, 300 * 200, 2.0 ** -16)
    got = _cmp_stats(O, handle, dev, z, 300, 200, 300)
    assert got[1] == 2 * 300 * 200
    _cmp_stats(O, handle, dev, z, 150, 100, 300, batch=2, stride=300 * 100)


def test_stats_special_values(O, handle, dev):
    zeros = np.zeros(4096, dtype=np.float32)
    assert _cmp_stats(O, handle, dev, zeros, 64, 64, 64)[0] == 0
    x = inputs.normal(12, 4096)
    x[100] = np.nan
    x[200] = -np.inf
    assert _cmp_stats(O, handle, dev, x, 64, 64, 64)[0] == 0x7f800000
    x[200] = 3.0e38
    x[5] = -np.nan
    _cmp_stats(O, handle, dev, x, 64, 64, 64)
    den = np.arange(1, 4097, dtype=np.uint32).view(np.float32).copy()
    assert _cmp_stats(O, handle, dev, den, 64, 64, 64)[0] == 0


def test_three_way_decision(O, handle, dev):
    rng = np.random.default_rng(3)
    unit = inputs.normal(13, 256 * 256)
    unit[np.abs(unit) < 2.0 ** -14] = 0.25
    assert _cmp_stats(O, handle, dev, unit, 256, 256, 256)[3] == FP16TCEC
    band = (rng.uniform(0.5, 1.0, 65536) * 2.0 ** -20).astype(np.float32)
    assert _cmp_stats(O, handle, dev, band, 256, 256, 256)[3] == SCALING
    wide = inputs.exponent_spread(14, 256, 256, per_row=True)
    assert _cmp_stats(O, handle, dev, wide, 256, 256, 256)[3] == TF32TCEC


def test_c4_config_stats_bit_exact(O, handle, dev):
    """Benchmark configuration C4 inputs (4096^2, per-row / per-column exponents in [-30, 30])."""
    a = inputs.exponent_spread(3, 4096, 4096, per_row=True)
    b = inputs.exponent_spread(4, 4096, 4096, per_row=False)
    _cmp_stats(O, handle, dev, a, 4096, 4096, 4096)
    _cmp_stats(O, handle, dev, b, 4096, 4096, 4096)


def test_result_ring_ids(handle, dev, cg):
    handle.reset_exp_stats_buffer_id()
    assert handle.get_current_exp_stats_buffer_id() == 1
    x = dev.up(np.ones(16, np.float32))
    ids = [handle.exp_max_ext(4, 4, x, 4) for _ in range(3)]
    assert ids == [2, 3, 4] and handle.get_current_exp_stats_buffer_id() == 4
    # presets: slot 0 decides TF32TCEC, slot 1 FP16TCEC
    assert handle.get_exp_stats_compute_mode_level(0) == TF32TCEC
    assert handle.get_exp_stats_compute_mode_level(1) == FP16TCEC
    handle.reset_exp_stats_buffer_id()
    last = None
    for _ in range(10000):
        last = handle.exp_max_ext(4, 4, x, 4)
    assert last == 2 + (10000 - 1) % 9998  # 2..9999 cycle, the length is preserved


@pytest.mark.parametrize("cplx", [False, True])
def test_scaling_roundtrip_and_coefficients(O, handle, dev, cplx):
    m, n, ld = 300, 200, 320
    gen = inputs.complex_normal if cplx else inputs.normal
    a = gen(21, ld * n, 2.0 ** -19)
    b = gen(22, ld * n, 2.0 ** 9)
    dt = np.complex64 if cplx else np.float32
    da, db = dev.up(a), dev.up(b)
    ia = handle.exp_max_ext(m, n, da, ld, cplx=cplx)
    ib = handle.exp_max_ext(m, n, db, ld, cplx=cplx)
    ma, mb = handle.get_max_exp(ia), handle.get_max_exp(ib)
    L = O.lib()
    FLAG_BOTH = 1  # preset slot 1: FP16TCEC | scale A | scale B
    handle.scale_A(ia, FLAG_BOTH, m, n, da, ld, cplx=cplx)
    handle.scale_B(ib, FLAG_BOTH, m, n, db, ld, cplx=cplx)
    sa = O.scale_matrix(a.copy(), m, n, ld, L.oracle_scale_ab_coef(ma))
    sb = O.scale_matrix(b.copy(), m, n, ld, L.oracle_scale_ab_coef(mb))
    ga, gb = dev.down(da, dt), dev.down(db, dt)
    assert np.array_equal(ga.view(np.uint32), sa.view(np.uint32))  # padding rows untouched too
    assert np.array_equal(gb.view(np.uint32), sb.view(np.uint32))
    amax = np.abs(ga.view(np.float32).reshape(n, -1)[:, : m * (2 if cplx else 1)]).max()
    assert 2.0 ** 14 <= amax < 2.0 ** 15
    c = gen(23, ld * n, 1.0)
    dc = dev.up(c)
    handle.scale_C(ia, ib, FLAG_BOTH, m, n, dc, ld, cplx=cplx)
    sc = O.scale_matrix(c.copy(), m, n, ld, L.oracle_scale_c_coef(ma, mb, 1, 0x61))
    assert np.array_equal(dev.down(dc, dt).view(np.uint32), sc.view(np.uint32))
    handle.reset_scale_A(ia, FLAG_BOTH, m, n, da, ld, cplx=cplx)
    handle.reset_scale_B(ib, FLAG_BOTH, m, n, db, ld, cplx=cplx)
    assert np.array_equal(dev.down(da, dt).view(np.uint32), a.view(np.uint32))
    assert np.array_equal(dev.down(db, dt).view(np.uint32), b.view(np.uint32))
    # flag slot 0 (TF32TCEC, no scale bits): every scaling call is a no-op
    handle.scale_A(ia, 0, m, n, da, ld, cplx=cplx)
    handle.scale_C(ia, ib, 0, m, n, dc, ld, cplx=cplx)
    assert np.array_equal(dev.down(da, dt).view(np.uint32), a.view(np.uint32))
    assert np.array_equal(dev.down(dc, dt).view(np.uint32), sc.view(np.uint32))


def test_scaling_skips_all_zero_matrix(handle, dev):
    z = dev.up(np.zeros(64, np.float32))
    one = dev.up(np.ones(64, np.float32))
    iz = handle.exp_max_ext(8, 8, z, 8)
    io = handle.exp_max_ext(8, 8, one, 8)
    handle.scale_A(iz, 1, 8, 8, z, 8)
    handle.scale_C(iz, io, 1, 8, 8, one, 8)  # max_exp(A) == 0 -> C untouched
    assert not dev.down(z).any() and np.array_equal(dev.down(one), np.ones(64, np.float32))


def test_scaling_batched_strided(O, handle, dev):
    m, n, ld, batch = 40, 30, 48, 3
    stride = ld * n + 5
    x = inputs.normal(31, stride * batch, 2.0 ** -10)
    d = dev.up(x)
    sid = handle.exp_max_ext(m, n, d, ld, batch, stride)
    mx = handle.get_max_exp(sid)
    assert _bits(mx) == O.exp_max_bits(x, m, n, ld, batch=batch, stride=stride)
    handle.scale_A(sid, 1, m, n, d, ld, batch, stride)
    want = O.scale_matrix(x.copy(), m, n, ld, O.lib().oracle_scale_ab_coef(mx), batch=batch, stride=stride)
    assert np.array_equal(dev.down(d).view(np.uint32), want.view(np.uint32))


def test_launch_flag_combination(O, handle, dev):
    rng = np.random.default_rng(5)
    mats = {
        FP16TCEC: np.full(4096, 0.5, np.float32),
        SCALING: (rng.uniform(0.5, 1.0, 4096) * 2.0 ** -20).astype(np.float32),
        TF32TCEC: inputs.exponent_spread(15, 64, 64, per_row=True),
    }
    ids = {}
    for mode, x in mats.items():
        ids[mode] = handle.exp_stats_ext(64, 64, dev.up(x), 64)
        assert handle.get_exp_stats_compute_mode_level(ids[mode]) == mode
    for ma in mats:
        for mb in mats:
            fid = handle.get_next_dynamic_launch_buffer_id()
            handle.set_dynamic_launch_buffer_by_exp_stats(fid, ids[ma], ids[mb])
            assert handle.get_dynamic_launch_flag(fid) == O.lib().oracle_combine_flag(ma, mb)
    assert handle.get_dynamic_launch_flag(0) == TF32TCEC
    assert handle.get_dynamic_launch_flag(1) == (3 << 5) | FP16TCEC


@pytest.mark.parametrize("shapes", [((700, 300), (300, 900)), ((4096, 4096), (64, 64)), ((1, 1), (2048, 1024))])
def test_pair_launch_matches_two_single_launches(O, handle, dev, shapes):
    """A and B of a GEMM scanned by one launch per pass: the same slots, counts, maxima and
    decisions as one call per matrix (and as the oracle), and the launch flag of the pair."""
    (ma, na), (mb, nb) = shapes
    a = inputs.normal(81, ma * na, 2.0 ** -14)       # some elements below the underflow threshold
    b = inputs.normal(82, mb * nb, 1.0)
    da, db = dev.up(a), dev.up(b)
    handle.set_exp_stats_params(0.0, 2.0 ** -15, 0.0)
    flag = handle.get_next_dynamic_launch_buffer_id()
    ia, ib = handle.exp_stats_pair(ma, na, da, ma, mb, nb, db, mb, flag_id=flag)
    assert ib == ia + 1 or ib == 2
    for sid, x, mm, nn in ((ia, a, ma, na), (ib, b, mb, nb)):
        o = O.exp_stats(x, mm, nn, mm)
        assert handle.get_exp_stats(sid) == (o.underflow, o.total)
        assert int(np.float32(handle.get_max_exp(sid)).view(np.uint32)) == o.max_exp_bits
        assert handle.get_exp_stats_compute_mode_level(sid) == o.mode
    oa, ob = O.exp_stats(a, ma, na, ma), O.exp_stats(b, mb, nb, mb)
    assert handle.get_dynamic_launch_flag(flag) == O.lib().oracle_combine_flag(oa.mode, ob.mode)
    ja, jb = handle.exp_max_pair(ma, na, da, ma, mb, nb, db, mb)
    assert int(np.float32(handle.get_max_exp(ja)).view(np.uint32)) == oa.max_exp_bits
    assert int(np.float32(handle.get_max_exp(jb)).view(np.uint32)) == ob.max_exp_bits
