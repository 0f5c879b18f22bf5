"""Pins the oracle's GEMM restatement: exact cases, closed forms, layout and
conjugation identities, the reference's own accuracy bar (relative Frobenius
residual vs FP64 < 2^-23 * sqrt(K), test/main.cu:68-74) and the "within 2x of a
plain FP32 SGEMM" bar."""
import numpy as np
import pytest

N, T, C = 111, 112, 113
EC_MODES = [1, 2]        # FP16TCEC, TF32TCEC(bf16x3)
ALL_MODES = [1, 2, 3, 4, 12]


def _np_op(x, op):
    return x if op == N else (x.T if op == T else x.conj().T)


def _mk(rng, rows, cols, ld, cplx=False, ints=None):
    buf = np.zeros(ld * cols, dtype=np.complex64 if cplx else np.float32)
    if ints is not None:
        vals = rng.integers(-ints, ints + 1, (rows, cols)).astype(np.float32)
        if cplx:
            vals = vals + 1j * rng.integers(-ints, ints + 1, (rows, cols)).astype(np.float32)
    else:
        vals = rng.uniform(-1, 1, (rows, cols)).astype(np.float32)
        if cplx:
            vals = vals + 1j * rng.uniform(-1, 1, (rows, cols)).astype(np.float32)
    view = buf.reshape(cols, ld).T  # column-major view [row, col]
    view[:rows, :] = vals
    return buf, view[:rows, :]


def test_fp64_reference_matches_numpy(O):
    rng = np.random.default_rng(1)
    for cplx in (False, True):
        for opa in (N, T, C):
            for opb in (N, T, C):
                m, n, k = 13, 7, 9
                ar, ac = (m, k) if opa == N else (k, m)
                br, bc = (k, n) if opb == N else (n, k)
                a, av = _mk(rng, ar, ac, ar + 3, cplx)
                b, bv = _mk(rng, br, bc, br + 1, cplx)
                c, cv = _mk(rng, m, n, m + 2, cplx)
                alpha, beta = (0.75 - 0.5j, 0.3 + 2j) if cplx else (0.75, -1.25)
                ref = O.gemm_fp64(opa, opb, m, n, k, alpha, a, ar + 3, b, br + 1, beta, c, m + 2)
                want = alpha * (_np_op(av.astype(np.complex128 if cplx else np.float64), opa) @
                                _np_op(bv.astype(np.complex128 if cplx else np.float64), opb)) + \
                    beta * cv.astype(np.complex128 if cplx else np.float64)
                assert np.allclose(ref.reshape(n, m).T, want, rtol=1e-13, atol=1e-13)


@pytest.mark.parametrize("mode", ALL_MODES)
@pytest.mark.parametrize("cplx", [False, True])
def test_small_integers_are_exact(O, mode, cplx):
    """Integers up to 2^7 are exact in fp16 and bf16 and every partial sum is an
    exact FP32 integer: any correct split-and-correct GEMM returns the integer
    product exactly, whatever its summation order."""
    rng = np.random.default_rng(2)
    m, n, k = 37, 29, 53
    for opa in (N, T, C):
        for opb in (N, T, C):
            ar, ac = (m, k) if opa == N else (k, m)
            br, bc = (k, n) if opb == N else (n, k)
            a, av = _mk(rng, ar, ac, ar + 2, cplx, ints=100)
            b, bv = _mk(rng, br, bc, br + 5, cplx, ints=100)
            c, cv = _mk(rng, m, n, m + 1, cplx, ints=50)
            alpha, beta = (2.0, -3.0)
            want = alpha * (_np_op(av.astype(np.complex128), opa) @ _np_op(bv.astype(np.complex128), opb)) + beta * cv.astype(np.complex128)
            O.gemm(mode, opa, opb, m, n, k, alpha, a, ar + 2, b, br + 5, beta, c, m + 1)
            got = c.reshape(n, m + 1).T[:m, :]
            assert np.array_equal(got.astype(np.complex128), want)
            # padding rows of C are never written
            assert not c.reshape(n, m + 1).T[m:, :].any()


@pytest.mark.parametrize("mode", EC_MODES)
def test_identity_returns_split_reconstruction(O, mode):
    rng = np.random.default_rng(3)
    m = k = 64
    a = rng.uniform(-4, 4, m * k).astype(np.float32)
    eye = np.eye(k, dtype=np.float32).reshape(-1)
    c = np.zeros(m * k, dtype=np.float32)
    O.gemm(mode, N, N, m, k, k, 1.0, a, m, eye, k, 0.0, c, m)
    assert np.all(np.abs(c.astype(np.float64) - a) <= np.abs(a) * 2.0 ** -22)


def test_k1_is_outer_product_of_splits(O):
    rng = np.random.default_rng(4)
    m, n = 33, 17
    a = rng.uniform(-1, 1, m).astype(np.float32)
    b = rng.uniform(-1, 1, n).astype(np.float32)
    c = np.zeros(m * n, dtype=np.float32)
    O.gemm(1, N, N, m, n, 1, 1.0, a, m, b, 1, 0.0, c, m)
    ah, al = O.split_fp16(a)
    bh, bl = O.split_fp16(b)
    main = np.outer(bh, ah)  # [n, m] == column-major flat
    corr = (np.outer(bh, al) + np.outer(bl, ah)).astype(np.float32)
    want = (main + corr * np.float32(1.0 / 2048)).astype(np.float32)
    assert np.array_equal(c.reshape(n, m), want)


def test_beta_zero_never_reads_c(O):
    m = n = k = 8
    rng = np.random.default_rng(5)
    a = rng.uniform(-1, 1, m * k).astype(np.float32)
    b = rng.uniform(-1, 1, k * n).astype(np.float32)
    c = np.full(m * n, np.nan, dtype=np.float32)
    O.gemm(1, N, N, m, n, k, 1.0, a, m, b, k, 0.0, c, m)
    assert np.isfinite(c).all()


@pytest.mark.parametrize("mode", EC_MODES)
def test_layout_and_conjugate_identities(O, mode):
    rng = np.random.default_rng(6)
    m, n, k = 24, 20, 28
    a = (rng.uniform(-1, 1, (m, k)) + 1j * rng.uniform(-1, 1, (m, k))).astype(np.complex64)
    b = (rng.uniform(-1, 1, (k, n)) + 1j * rng.uniform(-1, 1, (k, n))).astype(np.complex64)
    col = lambda x: np.asfortranarray(x).reshape(-1, order="F")
    out = {}
    for name, opa, am in (("N", N, a), ("T", T, a.T), ("C", C, a.conj().T)):
        c = np.zeros(m * n, dtype=np.complex64)
        O.gemm(mode, opa, N, m, n, k, 1.0, col(am), am.shape[0], col(b), k, 0.0, c, m)
        out[name] = c
    assert np.array_equal(out["N"], out["T"]) and np.array_equal(out["N"], out["C"])
    c2 = np.zeros(m * n, dtype=np.complex64)
    O.gemm(mode, N, C, m, n, k, 1.0, col(a), m, col(b.conj().T), n, 0.0, c2, m)
    assert np.array_equal(out["N"], c2)
    # real data: op C behaves as op T
    ar = rng.uniform(-1, 1, (k, m)).astype(np.float32)
    br = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    c3 = np.zeros(m * n, dtype=np.float32)
    c4 = np.zeros(m * n, dtype=np.float32)
    O.gemm(mode, T, N, m, n, k, 1.0, col(ar), k, col(br), k, 0.0, c3, m)
    O.gemm(mode, C, N, m, n, k, 1.0, col(ar), k, col(br), k, 0.0, c4, m)
    assert np.array_equal(c3, c4)


@pytest.mark.parametrize("mode", EC_MODES)
@pytest.mark.parametrize("cplx", [False, True])
@pytest.mark.parametrize("k", [64, 1024])
def test_accuracy_bars(O, mode, cplx, k):
    from cumpsgemm_amd import inputs
    m = n = 96
    gen = (lambda s, c: inputs.complex_normal(s, c, 0.7)) if cplx else inputs.uniform
    a, b = gen(1, m * k), gen(2, k * n)
    ref = O.gemm_fp64(N, N, m, n, k, 1.0, a, m, b, k)
    c = np.zeros(m * n, dtype=a.dtype)
    O.gemm(mode, N, N, m, n, k, 1.0, a, m, b, k, 0.0, c, m)
    f = np.zeros(m * n, dtype=a.dtype)
    O.gemm(12, N, N, m, n, k, 1.0, a, m, b, k, 0.0, f, m)
    r_ec, r_f32 = O.residual(ref, c, m, n, m), O.residual(ref, f, m, n, m)
    assert r_ec < 2.0 ** -23 * np.sqrt(k)  # the reference's own threshold
    assert r_ec <= 2.0 * r_f32             # within 2x of plain FP32


def test_uncorrected_modes_are_visibly_worse(O):
    """A dropped correction term must fail the EC bar (guards against a
    restatement that silently computes only hi*hi)."""
    from cumpsgemm_amd import inputs
    m = n = k = 128
    a, b = inputs.uniform(1, m * k), inputs.uniform(2, k * n)
    ref = O.gemm_fp64(N, N, m, n, k, 1.0, a, m, b, k)
    res = {}
    for mode in ALL_MODES:
        c = np.zeros(m * n, dtype=np.float32)
        O.gemm(mode, N, N, m, n, k, 1.0, a, m, b, k, 0.0, c, m)
        res[mode] = O.residual(ref, c, m, n, m)
    assert res[3] > 100 * res[1] and res[3] < 2.0 ** -10 * np.sqrt(k)
    assert res[4] > 5 * res[2] and res[4] < 2.0 ** -10 * np.sqrt(k)


def test_residual_metric_closed_form(O):
    ref = np.array([3.0, 4.0, 0.0, 0.0])
    c = np.array([3.0, 4.0, 0.0, 5.0], dtype=np.float32)
    assert O.residual(ref, c, 2, 2, 2) == pytest.approx(1.0)
    assert O.residual(ref, ref.astype(np.float32), 2, 2, 2) == 0.0
