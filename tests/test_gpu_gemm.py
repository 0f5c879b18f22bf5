"""Parity of the HIP GEMM path (through the C ABI) with the oracle.

Tolerances (floating point, stated by the task): relative Frobenius error of
the error-corrected modes against an FP64 GEMM of the same inputs must be
within 2x of a plain FP32 SGEMM's error and below the reference's own bar
2^-23*sqrt(K) (test/main.cu:68-74); the uncorrected modes below 2^-10*sqrt(K).
Cases whose result is exactly representable must match the oracle bit for bit.
"""
import numpy as np
import pytest

from cumpsgemm_amd import inputs
from gpu_util import (N, T, C, assert_same_up_to_summation_order, make_operand, oracle_gemm, rel_diff, run_gemm,
                      stored_shape)

pytestmark = pytest.mark.gpu

FP16TCEC, TF32TCEC, FP16TC, TF32TC, FP32 = 1, 2, 3, 4, 12


def _gen(cplx):
    return (lambda s, c: inputs.complex_normal(s, c, 0.6)) if cplx else inputs.uniform


def _check(O, handle, dev, mode, opa, opb, m, n, k, cplx, alpha, beta, pads=(0, 0, 0), seed=1):
    gen = _gen(cplx)
    a, lda = make_operand(gen, seed, opa, m, k, pads[0])
    b, ldb = make_operand(gen, seed + 1, opb, k, n, pads[1])
    ldc = m + pads[2]
    c0 = gen(seed + 2, ldc * n)
    c, st = run_gemm(handle, dev, mode, opa, opb, m, n, k, alpha, a, lda, b, ldb, beta, c0, ldc, cplx)
    assert st == 0
    ref = O.gemm_fp64(opa, opb, m, n, k, alpha, a, lda, b, ldb, beta, c0, ldc)
    r_gpu = O.residual(ref, c, m, n, ldc)
    co = oracle_gemm(O, mode, opa, opb, m, n, k, alpha, a, lda, b, ldb, beta, c0, ldc)
    r_oracle = O.residual(ref, co, m, n, ldc)
    cf = oracle_gemm(O, FP32, opa, opb, m, n, k, alpha, a, lda, b, ldb, beta, c0, ldc)
    r_fp32 = O.residual(ref, cf, m, n, ldc)
    kk = max(k, 1)
    if mode in (FP16TCEC, TF32TCEC):
        # 2x the FP32 error, plus one FP32 rounding of slack for outputs so small
        # that plain FP32 happens to be exact
        assert r_gpu <= 2.0 * r_fp32 + 2.0 ** -23, (r_gpu, r_fp32)
        if alpha == 1.0 and beta == 0.0:  # the conditions of the reference's own bar
            assert r_gpu < 2.0 ** -23 * np.sqrt(kk)
        # GPU and oracle run the same algorithm in different summation orders
        assert rel_diff(c, co, m, n, ldc) < 2.0 ** -21 * np.sqrt(kk)
    else:
        assert r_gpu < 2.0 ** -10 * np.sqrt(kk)
        assert r_gpu <= 1.5 * r_oracle + 1e-7
    # rows between m and ldc are never written
    if pads[2]:
        assert np.array_equal(c.reshape(n, ldc)[:, m:], c0.reshape(n, ldc)[:, m:])
    return r_gpu


@pytest.mark.parametrize("mode", [FP16TCEC, TF32TCEC, FP16TC, TF32TC])
@pytest.mark.parametrize("opa", [N, T])
@pytest.mark.parametrize("opb", [N, T])
def test_sgemm_aligned_all_layouts(O, handle, dev, mode, opa, opb):
    _check(O, handle, dev, mode, opa, opb, 512, 384, 256, False, 1.0, 0.0)


@pytest.mark.parametrize("mode", [FP16TCEC, TF32TCEC])
@pytest.mark.parametrize("opa", [N, T])
@pytest.mark.parametrize("opb", [N, T])
@pytest.mark.parametrize("shape", [(131, 77, 45), (1, 1, 1), (33, 1, 7), (1, 65, 129), (257, 130, 33),
                                   (64, 64, 1), (5, 300, 1000)])
def test_sgemm_ragged_padded_alpha_beta(O, handle, dev, mode, opa, opb, shape):
    m, n, k = shape
    _check(O, handle, dev, mode, opa, opb, m, n, k, False, 1.5, -0.75, pads=(3, 5, 2))


@pytest.mark.parametrize("mode", [FP16TCEC, TF32TCEC, FP16TC, TF32TC])
@pytest.mark.parametrize("opa", [N, T, C])
@pytest.mark.parametrize("opb", [N, T, C])
def test_cgemm_all_ops(O, handle, dev, mode, opa, opb):
    _check(O, handle, dev, mode, opa, opb, 160, 96, 200, True, 1.0 + 0.5j, 0.25 - 1.0j, pads=(1, 0, 3))


@pytest.mark.parametrize("shape", [(96, 80, 72), (3, 2, 5), (129, 65, 31), (512, 512, 64)])
def test_cgemm_shapes_beta_zero(O, handle, dev, shape):
    m, n, k = shape
    _check(O, handle, dev, FP16TCEC, N, N, m, n, k, True, 1.0, 0.0)
    _check(O, handle, dev, TF32TCEC, C, T, m, n, k, True, -2.0j, 0.0, pads=(2, 2, 2))


def test_op_c_on_real_data_is_transpose(O, handle, dev):
    _check(O, handle, dev, FP16TCEC, C, C, 100, 90, 80, False, 1.0, 0.0)


@pytest.mark.parametrize("mode", [FP16TCEC, TF32TCEC, FP16TC, TF32TC])
@pytest.mark.parametrize("cplx", [False, True])
def test_exact_integer_products_match_oracle_bitwise(O, handle, dev, mode, cplx):
    rng = np.random.default_rng(7)
    m, n, k = 150, 70, 333
    def ints(count):
        v = rng.integers(-60, 61, count).astype(np.float32)
        if cplx:
            v = (v + 1j * rng.integers(-60, 61, count).astype(np.float32)).astype(np.complex64)
        return v
    for opa, opb in ((N, N), (T, N), (N, T), (C, C)):
        a, b, c0 = ints(m * k), ints(k * n), ints(m * n)
        lda = m if opa == N else k
        ldb = k if opb == N else n
        c, st = run_gemm(handle, dev, mode, opa, opb, m, n, k, 2.0, a, lda, b, ldb, -1.0, c0, m, cplx)
        co = oracle_gemm(O, mode, opa, opb, m, n, k, 2.0, a, lda, b, ldb, -1.0, c0, m)
        assert st == 0 and np.array_equal(c, co)


def test_subnormal_fp16_terms_are_kept(O, handle, dev):
    """hi values below 2^-14 are fp16 subnormals; they must not be flushed by the
    conversion or by the matrix unit: powers of two give an exact result."""
    m = n = k = 64
    a = np.full(m * k, 2.0 ** -20, dtype=np.float32)
    b = np.full(k * n, 2.0 ** -3, dtype=np.float32)
    c, st = run_gemm(handle, dev, FP16TCEC, N, N, m, n, k, 1.0, a, m, b, k, 0.0, np.zeros(m * n, np.float32), m, False)
    assert np.array_equal(c, np.full(m * n, k * 2.0 ** -23, dtype=np.float32))


def test_beta_zero_ignores_nan_in_c(O, handle, dev):
    m = n = k = 96
    a, b = inputs.uniform(1, m * k), inputs.uniform(2, k * n)
    c0 = np.full(m * n, np.nan, dtype=np.float32)
    c, st = run_gemm(handle, dev, FP16TCEC, N, N, m, n, k, 1.0, a, m, b, k, 0.0, c0, m, False)
    assert np.isfinite(c).all()


def test_split_k_path_small_output_long_k(O, handle, dev):
    m, n, k = 64, 48, 8192
    a, b = inputs.uniform(3, m * k), inputs.uniform(4, k * n)
    c0 = inputs.uniform(5, m * n)
    c, st, mid = run_gemm(handle, dev, FP16TCEC, N, N, m, n, k, 1.25, a, m, b, k, 0.5, c0, m, False, want_module_id=True)
    assert st == 0 and mid >= 100  # split-K took over
    ref = O.gemm_fp64(N, N, m, n, k, 1.25, a, m, b, k, 0.5, c0, m)
    cf = oracle_gemm(O, FP32, N, N, m, n, k, 1.25, a, m, b, k, 0.5, c0, m)
    assert O.residual(ref, c, m, n, m) <= 2.0 * O.residual(ref, cf, m, n, m)


@pytest.mark.parametrize("cplx", [False, True])
def test_strided_batch(O, handle, dev, cplx):
    m, n, k, batch = 70, 50, 90, 5
    gen = _gen(cplx)
    lda, ldb, ldc = m + 2, k, m + 1
    sa, sb, sc = lda * k + 7, ldb * n, ldc * n + 3
    a, b, c0 = gen(1, sa * batch), gen(2, sb * batch), gen(3, sc * batch)
    da, db, dc = dev.up(a), dev.up(b), dev.up(c0)
    st = handle.gemm_strided_batch(N, N, m, n, k, 1.0, da, lda, sa, db, ldb, sb, 0.5, dc, ldc, sc, batch,
                                   FP16TCEC, cplx=cplx)
    assert st == 0
    c = dev.down(dc, np.complex64 if cplx else np.float32)
    for i in range(batch):
        ai, bi, ci0 = a[i * sa:], b[i * sb:], c0[i * sc: i * sc + ldc * n]
        ref = O.gemm_fp64(N, N, m, n, k, 1.0, ai, lda, bi, ldb, 0.5, ci0, ldc)
        cf = oracle_gemm(O, FP32, N, N, m, n, k, 1.0, ai, lda, bi, ldb, 0.5, ci0, ldc)
        got = c[i * sc: i * sc + ldc * n]
        assert O.residual(ref, got, m, n, ldc) <= 2.0 * O.residual(ref, cf, m, n, ldc)
    # gaps between batch entries are untouched
    assert np.array_equal(c[ldc * n: sc], c0[ldc * n: sc])


def test_c1_config_1024_cubed(O, handle, dev):
    """Benchmark configuration C1: SGEMM NN 1024^3, uniform[-1,1], seeds (1,2)."""
    m = n = k = 1024
    a, b = inputs.uniform(1, m * k), inputs.uniform(2, k * n)
    for mode in (FP16TCEC, TF32TCEC):
        c, st = run_gemm(handle, dev, mode, N, N, m, n, k, 1.0, a, m, b, k, 0.0, np.zeros(m * n, np.float32), m, False)
        ref = O.gemm_fp64(N, N, m, n, k, 1.0, a, m, b, k)
        cf = oracle_gemm(O, FP32, N, N, m, n, k, 1.0, a, m, b, k, 0.0, np.zeros(m * n, np.float32), m)
        co = oracle_gemm(O, mode, N, N, m, n, k, 1.0, a, m, b, k, 0.0, np.zeros(m * n, np.float32), m)
        r, rf = O.residual(ref, c, m, n, m), O.residual(ref, cf, m, n, m)
        assert r <= 2.0 * rf and r < 2.0 ** -23 * 32
        assert rel_diff(c, co, m, n, m) < 2.0 ** -21 * 32


def test_invalid_arguments(handle, dev, cg):
    x = dev.up(np.zeros(64, np.float32))
    assert handle.gemm(N, N, 8, 8, 8, 1.0, x, 8, x, 8, 0.0, x, 8, cg.CUBLAS) == cg.STATUS_INVALID_VALUE
    assert handle.gemm(N, N, 8, 8, 8, 1.0, x, 4, x, 8, 0.0, x, 8, cg.FP16TCEC) == cg.STATUS_INVALID_VALUE
    assert handle.gemm(N, N, 8, 8, 8, 1.0, x, 8, x, 8, 0.0, x, 7, cg.FP16TCEC) == cg.STATUS_INVALID_VALUE
    assert handle.gemm(N, N, 0, 8, 8, 1.0, x, 8, x, 8, 0.0, x, 8, cg.FP16TCEC) == cg.STATUS_SUCCESS
    # null operands are refused on the host (on the device they would fault)
    assert handle.gemm(N, N, 8, 8, 8, 1.0, 0, 8, x, 8, 0.0, x, 8, cg.FP16TCEC) == cg.STATUS_INVALID_VALUE
    assert handle.gemm(N, N, 8, 8, 8, 1.0, x, 8, 0, 8, 0.0, x, 8, cg.FP16TCEC) == cg.STATUS_INVALID_VALUE
    assert handle.gemm(N, N, 8, 8, 8, 1.0, x, 8, x, 8, 0.0, 0, 8, cg.FP16TCEC) == cg.STATUS_INVALID_VALUE
    assert handle.gemm(N, N, 8, 8, 0, 1.0, 0, 8, 0, 8, 0.0, x, 8, cg.FP16TCEC) == cg.STATUS_SUCCESS   # k = 0 reads neither
    assert handle.gemm_Mx2x2(N, N, 16, 1.0, 0, 16, x, 2, 0.0, x, 16) == cg.STATUS_INVALID_VALUE
    before = handle.get_current_exp_stats_buffer_id()
    sid = handle.exp_max_ext(8, 8, 0, 8)              # logged, nothing launched; the ring still advances
    assert sid != before
    handle.scale_A(1, 1, 8, 8, 0, 8)
    assert not dev.down(x).any()


# ---- persistent (tile-walking) kernels -----------------------------------------
# Shapes made of interior, aligned tiles run on kernels in which one workgroup
# per CU slot walks a list of (tile, batch) pairs with the load pipeline running
# across tile boundaries.  They perform the same arithmetic in the same order as
# the one-tile-per-workgroup kernels, so the two must agree bit for bit; the
# environment switches select the tile class and turn the persistent path off.
def _with_env(monkeypatch, cls, persistent):
    monkeypatch.setenv("CUMPSGEMM_FORCE_TILE_CLASS", str(cls))
    if persistent:
        monkeypatch.delenv("CUMPSGEMM_NO_PERSISTENT", raising=False)
    else:
        monkeypatch.setenv("CUMPSGEMM_NO_PERSISTENT", "1")


@pytest.mark.parametrize("cls", [0, 1])
@pytest.mark.parametrize("mode", [FP16TCEC, TF32TCEC])
@pytest.mark.parametrize("cplx,opa,opb,m,n,k,batch,alpha,beta", [
    (False, N, N, 4096, 4096, 128, 1, 1.0, 0.0),     # 512 / 1024 tiles of 4 K-steps: every workgroup walks several
    (False, T, N, 2048, 1024, 160, 3, 0.75, -0.5),   # batches in the walk, beta != 0
    (False, N, T, 1024, 2048, 352, 2, 1.0, 0.0),
    (False, T, T, 512, 512, 128, 9, 1.0, 1.0),
    (True, N, N, 1024, 1024, 128, 3, 1.0, 0.0),
    (True, C, N, 512, 1024, 192, 5, 0.5, 0.25),
    (True, N, C, 512, 512, 224, 6, 1.0, 0.0),
])
def test_persistent_kernels_match_plain_kernels(O, handle, dev, monkeypatch, cls, mode, cplx, opa, opb,
                                                m, n, k, batch, alpha, beta):
    gen = _gen(cplx)
    ar, ac = (m, k) if opa == N else (k, m)
    br, bc = (k, n) if opb == N else (n, k)
    sa, sb, sc = ar * ac, br * bc, m * n
    a, b, c0 = gen(11, sa * batch), gen(12, sb * batch), gen(13, sc * batch)
    da, db = dev.up(a), dev.up(b)
    outs = []
    for persistent in (True, False):
        _with_env(monkeypatch, cls, persistent)
        dc = dev.up(c0)
        st = handle.gemm_strided_batch(opa, opb, m, n, k, alpha, da, ar, sa, db, br, sb, beta, dc, m, sc,
                                       batch, mode, cplx=cplx)
        assert st == 0
        outs.append(dev.down(dc, np.complex64 if cplx else np.float32))
    assert np.array_equal(outs[0], outs[1])
    # and the result is right: last batch entry against FP64 and the FP32 error
    i = batch - 1
    ai, bi, ci0 = a[i * sa:(i + 1) * sa], b[i * sb:(i + 1) * sb], c0[i * sc:(i + 1) * sc]
    ref = O.gemm_fp64(opa, opb, m, n, k, alpha, ai, ar, bi, br, beta, ci0, m)
    cf = oracle_gemm(O, FP32, opa, opb, m, n, k, alpha, ai, ar, bi, br, beta, ci0, m)
    got = outs[0][i * sc:(i + 1) * sc]
    assert O.residual(ref, got, m, n, m) <= 2.0 * O.residual(ref, cf, m, n, m) + 2.0 ** -23


def test_persistent_split_k(O, handle, dev, monkeypatch):
    # few tiles, long K: K is cut into chunks and each chunk's tiles are walked
    m, n, k = 256, 256, 16384
    a, b = inputs.uniform(21, m * k), inputs.uniform(22, k * n)
    c0 = inputs.uniform(23, m * n)
    outs = []
    for persistent in (True, False):
        _with_env(monkeypatch, 1, persistent)
        c, st, mid = run_gemm(handle, dev, FP16TCEC, N, N, m, n, k, 1.0, a, m, b, k, 0.5, c0, m, False,
                              want_module_id=True)
        assert st == 0 and mid == 101
        outs.append(c)
    ref = O.gemm_fp64(N, N, m, n, k, 1.0, a, m, b, k, 0.5, c0, m)
    cf = oracle_gemm(O, FP32, N, N, m, n, k, 1.0, a, m, b, k, 0.5, c0, m)
    for c in outs:  # atomic accumulation order differs from run to run
        assert O.residual(ref, c, m, n, m) <= 2.0 * O.residual(ref, cf, m, n, m)


# ---- edge tiles computed from an origin moved inwards ------------------------------
# A tile that sticks out over the edge of C is loaded from an origin moved back by
# the overhang; the rows / columns it shares with its neighbour must not be updated
# twice (beta != 0, split-K accumulation).  Forced tile classes make sure that large
# tiles meet small overhangs.
@pytest.mark.parametrize("cls", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("cplx,opa,opb,m,n,k,alpha,beta", [
    (False, N, N, 300, 200, 160, 1.5, -0.5),     # K a multiple of 32: persistent kernels
    (False, T, N, 257, 129, 96, 1.0, 1.0),
    (False, N, T, 511, 383, 75, 1.0, 0.25),      # ragged K: one-tile kernels with a guarded tail
    (False, T, T, 256, 131, 130, 2.0, 0.0),
    (True, N, N, 200, 150, 128, 1.0 - 0.5j, 0.5 + 0.25j),
    (True, C, T, 129, 65, 70, 1.0, 1.0),
    (True, N, C, 70, 260, 64, 0.5j, -1.0),
])
def test_edge_tiles_with_beta(O, handle, dev, monkeypatch, cls, cplx, opa, opb, m, n, k, alpha, beta):
    monkeypatch.setenv("CUMPSGEMM_FORCE_TILE_CLASS", str(cls))
    _check(O, handle, dev, FP16TCEC, opa, opb, m, n, k, cplx, alpha, beta, pads=(1, 3, 2), seed=41)
    _check(O, handle, dev, TF32TCEC, opa, opb, m, n, k, cplx, alpha, beta, pads=(0, 0, 0), seed=43)


@pytest.mark.parametrize("cls", [0, 1])
def test_edge_tiles_split_k(O, handle, dev, monkeypatch, cls):
    monkeypatch.setenv("CUMPSGEMM_FORCE_TILE_CLASS", str(cls))
    m, n, k = 300, 260, 8192
    a, b = inputs.uniform(51, m * k), inputs.uniform(52, k * n)
    c0 = inputs.uniform(53, m * n)
    c, st, mid = run_gemm(handle, dev, FP16TCEC, N, N, m, n, k, 1.0, a, m, b, k, 0.5, c0, m, False,
                          want_module_id=True)
    assert st == 0 and mid == 100 + cls
    ref = O.gemm_fp64(N, N, m, n, k, 1.0, a, m, b, k, 0.5, c0, m)
    cf = oracle_gemm(O, FP32, N, N, m, n, k, 1.0, a, m, b, k, 0.5, c0, m)
    assert O.residual(ref, c, m, n, m) <= 2.0 * O.residual(ref, cf, m, n, m)


# ---- C with a few columns, or a few rows -------------------------------------------
# Tile classes 3 (256 x 32) and 4 (32 x 256) serve products whose result is at most 32 wide or high:
# the long operand is streamed once, K is split so that every CU has a share, the narrow operand goes
# through the guarded loader (wide loads where a unit lies inside the matrix).
@pytest.mark.parametrize("mode", [FP16TCEC, TF32TCEC])
@pytest.mark.parametrize("opa,opb", [(N, N), (T, N), (N, T), (T, T)])
@pytest.mark.parametrize("m,n,k,want_cls", [
    (4096, 8, 4096, 3), (4100, 1, 1000, 3), (2048, 17, 515, 3), (8192, 32, 1024, 3),
    (8, 4096, 4096, 4), (5, 3000, 777, 4), (32, 8192, 1024, 4),
])
def test_narrow_results_on_the_streaming_tile_classes(O, handle, dev, monkeypatch, mode, opa, opb, m, n, k, want_cls):
    # (the planner takes these classes on its own for the large ones; forced, so that the small ones run them too)
    monkeypatch.setenv("CUMPSGEMM_FORCE_TILE_CLASS", str(want_cls))
    a, lda = make_operand(inputs.uniform, 61, opa, m, k, 1)
    b, ldb = make_operand(inputs.uniform, 62, opb, k, n, 2)
    ldc = m + 3
    c0 = inputs.uniform(63, ldc * n)
    c, st, mid = run_gemm(handle, dev, mode, opa, opb, m, n, k, 0.75, a, lda, b, ldb, -0.5, c0, ldc, False,
                          want_module_id=True)
    assert st == 0 and mid % 100 == want_cls, mid
    ref = O.gemm_fp64(opa, opb, m, n, k, 0.75, a, lda, b, ldb, -0.5, c0, ldc)
    cf = oracle_gemm(O, FP32, opa, opb, m, n, k, 0.75, a, lda, b, ldb, -0.5, c0, ldc)
    co = oracle_gemm(O, mode, opa, opb, m, n, k, 0.75, a, lda, b, ldb, -0.5, c0, ldc)
    assert O.residual(ref, c, m, n, ldc) <= 2.0 * O.residual(ref, cf, m, n, ldc) + 2.0 ** -24
    assert rel_diff(c, co, m, n, ldc) <= 4 * 2.0 ** -24 * np.sqrt(k)
    assert np.array_equal(c.reshape(n, ldc)[:, m:], c0.reshape(n, ldc)[:, m:])


# ---- pre-split (packed) path ------------------------------------------------------
# Large real FP16TCEC / bf16x3 problems split A and B once into fp16 / bf16 planes (workspace of the
# handle) and run a kernel that only copies them into LDS.  Same split, same products; the
# pre-split kernels add them 32 K-values per MFMA where the in-loop kernels add 16, so the
# two results agree up to the order of summation.
@pytest.mark.parametrize("opa,opb,m,n,k,pads,alpha,beta", [
    (N, N, 4096, 4096, 256, (0, 0, 0), 1.0, 0.0),
    (T, N, 4000, 3000, 300, (1, 3, 2), 1.5, -0.5),     # ragged M, N, K and odd leading dimensions
    (N, T, 2304, 4100, 1000, (0, 5, 0), 1.0, 1.0),
    (T, T, 3333, 2777, 129, (2, 0, 1), -1.0, 0.25),
])
@pytest.mark.parametrize("mode", [FP16TCEC, TF32TCEC, FP16TC, TF32TC])
def test_packed_path_matches_in_loop_split(O, handle, dev, monkeypatch, mode, opa, opb, m, n, k, pads, alpha, beta):
    a, lda = make_operand(inputs.uniform, 61, opa, m, k, pads[0])
    b, ldb = make_operand(inputs.uniform, 62, opb, k, n, pads[1])
    ldc = m + pads[2]
    c0 = inputs.uniform(63, ldc * n)
    outs = []
    for packed in ("1", "0"):
        monkeypatch.setenv("CUMPSGEMM_PACKED", packed)
        c, st, mid = run_gemm(handle, dev, mode, opa, opb, m, n, k, alpha, a, lda, b, ldb, beta, c0, ldc, False,
                              want_module_id=True)
        assert st == 0 and (mid == 200) == (packed == "1")
        outs.append(c)
    assert_same_up_to_summation_order(outs[0], outs[1], k)
    ref = O.gemm_fp64(opa, opb, m, n, k, alpha, a, lda, b, ldb, beta, c0, ldc)
    if mode in (FP16TCEC, TF32TCEC):
        cf = oracle_gemm(O, FP32, opa, opb, m, n, k, alpha, a, lda, b, ldb, beta, c0, ldc)
        assert O.residual(ref, outs[0], m, n, ldc) <= 2.0 * O.residual(ref, cf, m, n, ldc)
    else:  # the uncorrected modes: as accurate as one rounding of the operands to fp16 / two bf16 terms allows
        assert O.residual(ref, outs[0], m, n, ldc) <= (2.0 ** -10 if mode == FP16TC else 2.0 ** -14)
    if pads[2]:
        assert np.array_equal(outs[0].reshape(n, ldc)[:, m:], c0.reshape(n, ldc)[:, m:])


@pytest.mark.parametrize("opa,opb,m,n,k,pads,alpha,beta", [
    (N, N, 2048, 2048, 256, (0, 0, 0), 1.0, 0.0),
    (C, N, 2000, 1700, 300, (1, 3, 2), 1.5 - 0.5j, -0.5 + 0.25j),   # ragged M, N, K, conjugated A
    (N, T, 1280, 2100, 520, (0, 5, 0), 1.0, 1.0),
    (T, C, 1700, 1500, 129, (2, 0, 1), -1.0j, 0.25),
])
@pytest.mark.parametrize("mode", [FP16TCEC, TF32TCEC, FP16TC, TF32TC])
def test_complex_packed_path_matches_in_loop_split(O, handle, dev, monkeypatch, mode, opa, opb, m, n, k, pads, alpha,
                                                   beta):
    gen = _gen(True)
    a, lda = make_operand(gen, 65, opa, m, k, pads[0])
    b, ldb = make_operand(gen, 66, opb, k, n, pads[1])
    ldc = m + pads[2]
    c0 = gen(67, ldc * n)
    outs = []
    for packed in ("1", "0"):
        monkeypatch.setenv("CUMPSGEMM_PACKED", packed)
        c, st, mid = run_gemm(handle, dev, mode, opa, opb, m, n, k, alpha, a, lda, b, ldb, beta, c0, ldc, True,
                              want_module_id=True)
        assert st == 0 and (mid == 200) == (packed == "1")
        outs.append(c)
    assert_same_up_to_summation_order(outs[0], outs[1], k)
    ref = O.gemm_fp64(opa, opb, m, n, k, alpha, a, lda, b, ldb, beta, c0, ldc)
    if mode in (FP16TCEC, TF32TCEC):
        cf = oracle_gemm(O, FP32, opa, opb, m, n, k, alpha, a, lda, b, ldb, beta, c0, ldc)
        assert O.residual(ref, outs[0], m, n, ldc) <= 2.0 * O.residual(ref, cf, m, n, ldc)
    else:
        assert O.residual(ref, outs[0], m, n, ldc) <= (2.0 ** -10 if mode == FP16TC else 2.0 ** -14)
    if pads[2]:
        assert np.array_equal(outs[0].reshape(n, ldc)[:, m:], c0.reshape(n, ldc)[:, m:])


@pytest.mark.parametrize("mode", [FP16TCEC, TF32TCEC, FP16TC, TF32TC])
@pytest.mark.parametrize("cplx,opa,opb", [(False, N, N), (False, T, T), (True, N, N), (True, C, T), (True, T, C)])
def test_packed_path_is_exact_on_small_integers(handle, dev, monkeypatch, mode, cplx, opa, opb):
    """Operands with small integer values (Gaussian integers for complex data) are held exactly by
    every plane format and every partial sum fits FP32, so whatever the order of summation the
    pre-split kernels must return the exact product, bit for bit -- a misplaced plane, a wrong
    sign in the complex combination or a dropped K-step would show."""
    m, n, k = 3100, 2900, 292   # (the path needs at least one 256x128 tile per CU)
    rng = np.random.default_rng(77)

    def ints(count):
        if cplx:
            return (rng.integers(-8, 9, count) + 1j * rng.integers(-8, 9, count)).astype(np.complex64)
        return rng.integers(-8, 9, count).astype(np.float32)
    ra, ca = stored_shape(opa, m, k)
    rb, cb = stored_shape(opb, k, n)
    a, b = ints(ra * ca), ints(rb * cb)
    monkeypatch.setenv("CUMPSGEMM_PACKED", "1")
    c, st, mid = run_gemm(handle, dev, mode, opa, opb, m, n, k, 1.0, a, ra, b, rb, 0.0, np.zeros(m * n, a.dtype), m,
                          cplx, want_module_id=True)
    assert st == 0 and mid == 200

    def logical(x, op, rows, cols):       # column-major flat buffer -> op(X) as rows x cols, in wide integers
        r, cc = stored_shape(op, rows, cols)
        mat = x.reshape(cc, r).T.astype(np.complex128 if cplx else np.float64)
        if op != N:
            mat = mat.T
        return np.conj(mat) if op == C else mat
    want = logical(a, opa, m, k) @ logical(b, opb, k, n)          # exact: |sums| < 2^24
    got = c.reshape(n, m).T
    assert np.array_equal(got.astype(want.dtype), want)


@pytest.mark.parametrize("cplx,opa,opb,m,n,k,batch", [
    (False, N, T, 3700, 3700, 512, 3),      # both operands M/N-contiguous: pre-split from K = 512 on
    (True, N, N, 3072, 3072, 1024, 2),
])
def test_batch_of_large_matrices_takes_the_pre_split_path_one_by_one(cg, torch_gpu, monkeypatch, cplx, opa, opb,
                                                                     m, n, k, batch):
    """A strided batch whose matrices are each worth the pre-split path is issued matrix by
    matrix through it; the same result as the batched in-loop kernels up to the order of summation."""
    torch = torch_gpu
    dev_t = torch.device("cuda:0")
    es = 2 if cplx else 1
    h = cg.Handle()
    h.set_stream(torch.cuda.current_stream())
    try:
        g = torch.Generator(device=dev_t).manual_seed(123)
        sa, sb, sc = m * k + 64, k * n + 32, m * n + 16      # gaps between the matrices
        a = torch.rand(sa * batch * es, generator=g, device=dev_t) - 0.5
        b = torch.rand(sb * batch * es, generator=g, device=dev_t) - 0.5
        c0 = torch.rand(sc * batch * es, generator=g, device=dev_t) - 0.5
        lda = m                                   # op N: m x k
        ldb = n if opb == T else k
        outs = {}
        for packed in ("0", None):
            if packed is None:
                monkeypatch.delenv("CUMPSGEMM_PACKED", raising=False)
            else:
                monkeypatch.setenv("CUMPSGEMM_PACKED", packed)
            c = c0.clone()
            st = h.gemm_strided_batch(opa, opb, m, n, k, 1.5, a, lda, sa, b, ldb, sb, -0.5, c, m, sc, batch,
                                      FP16TCEC, cplx=cplx)
            torch.cuda.synchronize()
            assert st == 0
            assert (h.workspace_size() > 0) == (packed is None)
            outs[packed] = c
        assert_same_up_to_summation_order(outs["0"], outs[None], k)
        # ... and right: the last matrix against FP64
        i = batch - 1
        dt = torch.complex128 if cplx else torch.float64
        def mat(buf, off, rows, cols):
            x = buf[off * es:(off + rows * cols) * es].double()
            x = torch.view_as_complex(x.view(-1, 2)) if cplx else x
            return x.view(cols, rows).t()                                # column-major rows x cols
        A = mat(a, i * sa, m, k)
        B = mat(b, i * sb, n, k).t() if opb == T else mat(b, i * sb, k, n)
        ref = 1.5 * (A @ B) - 0.5 * mat(c0, i * sc, m, n)
        got = mat(outs[None], i * sc, m, n)
        assert (torch.linalg.norm(got - ref) / torch.linalg.norm(ref)).item() < 4 * 2.0 ** -23 * k ** 0.5
    finally:
        torch.cuda.synchronize()
        h.close()


@pytest.mark.parametrize("mode,cplx", [(FP16TCEC, False), (TF32TCEC, False), (FP16TCEC, True), (FP16TC, False),
                                       (TF32TC, False), (FP16TC, True), (TF32TC, True)])
# (the path needs at least one 256x128 tile per CU; the second shape ends one row and one column
# past a tile boundary, so the last tile row / column leaves whole waves without anything to
# store, and its tiles are five K-steps short: the walking form changes tile every few steps and
# must not count on the stores of a write-out when it waits for the next tile's planes)
@pytest.mark.parametrize("m,n,k", [(3100, 2900, 600), (3073, 2945, 160)])
def test_packed_kernels_walk_and_one_tile_forms_agree(handle, dev, monkeypatch, mode, cplx, m, n, k):
    """The pre-split kernels exist as persistent (tile-walking) and one-tile-per-workgroup
    forms, chosen by K; both do the same arithmetic in the same order."""
    gen = _gen(cplx)
    a, lda = make_operand(gen, 91, T, m, k, 3)
    b, ldb = make_operand(gen, 92, N, k, n, 0)
    c0 = gen(93, m * n)
    monkeypatch.setenv("CUMPSGEMM_PACKED", "1")
    outs = []
    for walk in ("1", "0"):
        monkeypatch.setenv("CUMPSGEMM_PACKED_WALK", walk)
        c, st, mid = run_gemm(handle, dev, mode, T, N, m, n, k, 1.25, a, lda, b, ldb, 0.5, c0, m, cplx,
                              want_module_id=True)
        assert st == 0 and mid == 200
        outs.append(c)
    assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))


# ---- column split for a partial last round --------------------------------------
# When the tile count is just above a multiple of the CU slots, C is cut into two
# column blocks that are planned separately.  Same numbers as the single launch up
# to the accumulation order of a split-K second part.
@pytest.mark.parametrize("cplx,opa,opb,m,n,k,alpha,beta", [
    (False, N, N, 3072, 3072, 512, 1.0, 0.0),
    (False, T, T, 2560, 2700, 384, 1.5, -0.5),
    (False, N, T, 3000, 3000, 300, 1.0, 1.0),
    (True, N, N, 2048, 1300, 256, 1.0 + 0.5j, 0.5),
    (True, C, T, 1536, 1700, 320, 1.0, 0.0),
])
def test_column_split_matches_single_launch(O, handle, dev, monkeypatch, cplx, opa, opb, m, n, k, alpha, beta):
    gen = _gen(cplx)
    a, lda = make_operand(gen, 71, opa, m, k, 1)
    b, ldb = make_operand(gen, 72, opb, k, n, 2)
    ldc = m + 3
    c0 = gen(73, ldc * n)
    outs = []
    for single in (False, True):
        if single:
            monkeypatch.setenv("CUMPSGEMM_NO_COLUMN_SPLIT", "1")
        else:
            monkeypatch.delenv("CUMPSGEMM_NO_COLUMN_SPLIT", raising=False)
        c, st = run_gemm(handle, dev, FP16TCEC, opa, opb, m, n, k, alpha, a, lda, b, ldb, beta, c0, ldc, cplx)
        assert st == 0
        outs.append(c)
    assert rel_diff(outs[0], outs[1], m, n, ldc) < 2.0 ** -22 * np.sqrt(k)
    ref = O.gemm_fp64(opa, opb, m, n, k, alpha, a, lda, b, ldb, beta, c0, ldc)
    cf = oracle_gemm(O, FP32, opa, opb, m, n, k, alpha, a, lda, b, ldb, beta, c0, ldc)
    for c in outs:
        assert O.residual(ref, c, m, n, ldc) <= 2.0 * O.residual(ref, cf, m, n, ldc) + 2.0 ** -23
        assert np.array_equal(c.reshape(n, ldc)[:, m:], c0.reshape(n, ldc)[:, m:])


# A problem that is worth the pre-split path but whose tiles leave the last round of CU slots
# mostly empty is cut where the whole rounds end: the first part takes the path (module id 200,
# workspace allocated), the rest is planned on its own.
@pytest.mark.parametrize("cplx,mode,opa,opb,m,n,k,alpha,beta", [
    (False, FP16TCEC, N, N, 4352, 4352, 1024, 1.0, 0.0),       # 17 x 34 tiles of 256 x 128 = 2.26 rounds
    (False, FP16TCEC, T, N, 4400, 4300, 1030, 1.5, -0.5),      # ragged; cut along the rows or the columns
    (False, FP16TC, N, T, 4352, 4352, 1024, 1.0, 1.0),         # the uncorrected mode, same tiles
    (True, FP16TCEC, C, N, 3072, 1536, 1024, 1.0 - 0.5j, 0.25), # 24 x 24 tiles of 128 x 64 = 2.25 rounds ...
    (True, FP16TCEC, N, N, 2200, 2200, 1024, 1.0, 0.0),        # ... and 18 x 35 = 2.46
])
def test_pre_split_path_on_the_whole_rounds_of_a_cut_problem(handle, dev, monkeypatch, cplx, mode, opa, opb,
                                                              m, n, k, alpha, beta):
    gen = _gen(cplx)
    a, lda = make_operand(gen, 75, opa, m, k, 1)
    b, ldb = make_operand(gen, 76, opb, k, n, 2)
    ldc = m + 3
    c0 = gen(77, ldc * n)
    outs = {}
    for form in ("cut", "in_loop"):
        monkeypatch.delenv("CUMPSGEMM_PACKED", raising=False)
        if form == "in_loop":
            monkeypatch.setenv("CUMPSGEMM_PACKED", "0")
        c, st, mid = run_gemm(handle, dev, mode, opa, opb, m, n, k, alpha, a, lda, b, ldb, beta, c0, ldc, cplx,
                              want_module_id=True)
        assert st == 0 and (mid == 200) == (form == "cut"), (form, mid)
        outs[form] = c
    # every element of C, both sides of the cut: the in-loop result up to the order of summation
    # (the second part of either form may split K)
    assert rel_diff(outs["cut"], outs["in_loop"], m, n, ldc) < 2.0 ** -22 * np.sqrt(k)
    x, y = outs["cut"].view(np.float32).astype(np.float64), outs["in_loop"].view(np.float32).astype(np.float64)
    assert np.abs(x - y).max() <= 2.0 ** -18 * np.sqrt(k) * np.abs(y).max()
    assert np.array_equal(outs["cut"].reshape(n, ldc)[:, m:], c0.reshape(n, ldc)[:, m:])


# ---- small problems: two wave groups per workgroup --------------------------------------
# A problem of no more small tiles than CUs (an operand K-contiguous) runs the 64 x 64 kernel with twice the waves:
# each group takes one K-slice of every step and the sums meet in LDS at the end.  Same products
# as the four-wave kernel, another order of summation.
@pytest.mark.parametrize("mode", [FP16TCEC, TF32TCEC, TF32TC])
@pytest.mark.parametrize("cplx,opa,opb,m,n,k,batch,alpha,beta", [
    (False, N, N, 1024, 1024, 1024, 1, 1.0, 0.0),        # 256 interior tiles
    (False, T, N, 1000, 900, 777, 1, 1.5, -0.5),         # edge tiles, ragged K, beta != 0
    (False, N, N, 300, 200, 4100, 1, 1.0, 1.0),          # K split between workgroups as well (atomic write-out)
    (False, T, N, 256, 192, 520, 16, -1.0, 0.25),        # a batch: 12 tiles x 16 matrices
    (False, N, N, 70, 33, 50, 1, 1.0, 0.0),              # one partial tile, two K-steps
    (False, T, T, 640, 500, 300, 1, 1.0, 0.0),           # op(B) = T: the groups trade operands
    (True, N, N, 512, 512, 512, 1, 1.0, 0.0),            # complex: every thread stages half a unit of A and of B
    (True, C, N, 500, 450, 333, 2, 1.0 - 0.5j, 0.5j),    # conjugated A, edge tiles, ragged K, complex scalars
])
def test_two_wave_groups_match_the_four_wave_kernel(O, handle, dev, monkeypatch, mode, cplx, opa, opb, m, n, k,
                                                    batch, alpha, beta):
    gen = _gen(cplx)   # (complex bf16x3 has no two-group form: both runs launch the same kernel)
    ar, ac = (m, k) if opa == N else (k, m)
    br, bc = (k, n) if opb == N else (n, k)
    lda, ldb, ldc = ar + 1, br + 2, m + 3
    sa, sb, sc = lda * ac + 5, ldb * bc + 3, ldc * n + 7
    a, b, c0 = gen(85, sa * batch), gen(86, sb * batch), gen(87, sc * batch)
    da, db = dev.up(a), dev.up(b)
    outs = []
    for plain in (False, True):
        if plain:
            monkeypatch.setenv("CUMPSGEMM_NO_KSLICE_GROUPS", "1")
        else:
            monkeypatch.delenv("CUMPSGEMM_NO_KSLICE_GROUPS", raising=False)
        dc = dev.up(c0)
        st = handle.gemm_strided_batch(opa, opb, m, n, k, alpha, da, lda, sa, db, ldb, sb, beta, dc, ldc, sc,
                                       batch, mode, cplx=cplx)
        assert st == 0
        outs.append(dev.down(dc, np.complex64 if cplx else np.float32))
    for i in (0, batch - 1):
        x, y = outs[0][i * sc:i * sc + ldc * n], outs[1][i * sc:i * sc + ldc * n]
        assert rel_diff(x, y, m, n, ldc) < 2.0 ** -22 * np.sqrt(k)
        assert np.array_equal(x.reshape(n, ldc)[:, m:], c0[i * sc:i * sc + ldc * n].reshape(n, ldc)[:, m:])
        ai, bi, ci0 = a[i * sa:(i + 1) * sa], b[i * sb:(i + 1) * sb], c0[i * sc:i * sc + ldc * n]
        ref = O.gemm_fp64(opa, opb, m, n, k, alpha, ai, lda, bi, ldb, beta, ci0, ldc)
        if mode == TF32TC:
            assert O.residual(ref, x, m, n, ldc) <= 2.0 ** -14
        else:
            cf = oracle_gemm(O, FP32, opa, opb, m, n, k, alpha, ai, lda, bi, ldb, beta, ci0, ldc)
            assert O.residual(ref, x, m, n, ldc) <= 2.0 * O.residual(ref, cf, m, n, ldc) + 2.0 ** -24
    # (the gaps between the matrices of the batch stay as they were)
    assert np.array_equal(outs[0][ldc * n:sc], c0[ldc * n:sc])


# ---- degenerate and skinny shapes ----------------------------------------------------
@pytest.mark.parametrize("cplx", [False, True])
def test_k_zero_scales_c(O, handle, dev, cplx):
    m, n = 37, 21
    gen = _gen(cplx)
    c0 = gen(81, (m + 2) * n)
    x = gen(82, 64)
    beta = (0.5 - 0.25j) if cplx else -1.5
    c, st = run_gemm(handle, dev, FP16TCEC, N, N, m, n, 0, 1.0, x, m, x, 1, beta, c0, m + 2, cplx)
    assert st == 0
    want = c0.copy().reshape(n, m + 2)
    want[:, :m] = (want[:, :m].astype(np.complex128 if cplx else np.float64) * beta).astype(c0.dtype)
    assert np.allclose(c.reshape(n, m + 2), want, rtol=1e-6, atol=0)
    assert np.array_equal(c.reshape(n, m + 2)[:, m:], c0.reshape(n, m + 2)[:, m:])


@pytest.mark.parametrize("cplx", [False, True])
@pytest.mark.parametrize("m,n,ldc,batch,stride_pad,offset", [
    (1030, 77, 1032, 1, 0, 0),   # 16-byte aligned columns, a tail of 2 floats per column
    (1027, 5, 1027, 1, 0, 0),    # odd ldc: element-wise path
    (513, 9, 516, 3, 8, 0),      # batches, aligned
    (513, 9, 516, 3, 3, 0),      # batch stride breaks the alignment
    (300, 300, 304, 1, 0, 1),    # base pointer off by one element
    (3, 70000, 4, 1, 0, 0),      # more column groups than a grid dimension holds
])
@pytest.mark.parametrize("beta", [0.0, -0.75])
def test_k_zero_prepares_c_exactly(handle, dev, torch_gpu, cplx, m, n, ldc, batch, stride_pad, offset, beta):
    """k = 0 is C = beta * C (the same kernel prepares C for split-K): exact products, padding and
    gaps between batches untouched, beta = 0 overwrites NaN."""
    torch = torch_gpu
    es = 2 if cplx else 1
    stride = ldc * n + stride_pad
    total = (offset + stride * batch) * es
    g = torch.Generator(device=dev.dev).manual_seed(77)
    c0 = torch.rand(total, generator=g, device=dev.dev) - 0.5
    if beta == 0.0:
        c0[offset * es] = float("nan")
    c = c0.clone()
    x = torch.zeros(64, device=dev.dev)
    ptr = c.data_ptr() + offset * es * 4
    if batch == 1:
        st = handle.gemm(N, N, m, n, 0, 1.0, x, m, x, 1, beta, ptr, ldc, FP16TCEC, cplx=cplx)
    else:
        st = handle.gemm_strided_batch(N, N, m, n, 0, 1.0, x, m, 0, x, 1, 0, beta, ptr, ldc, stride, batch,
                                       FP16TCEC, cplx=cplx)
    assert st == 0
    torch.cuda.synchronize()
    want = c0.clone()
    for bi in range(batch):
        first = (offset + bi * stride) * es
        body = want[first:first + ldc * n * es].view(n, ldc * es)
        body[:, :m * es] = 0.0 if beta == 0.0 else body[:, :m * es] * beta   # a real beta: exact products
    assert torch.equal(c.view(torch.int32), want.view(torch.int32))


@pytest.mark.parametrize("mode", [FP16TCEC, TF32TCEC])
@pytest.mark.parametrize("opa,opb,m,n,k", [
    (N, N, 1, 4096, 4096),      # row vector times matrix
    (T, N, 4096, 1, 300),       # matrix times column vector
    (N, T, 5, 7, 10000),        # tiny output, long K: split-K with guarded loads
    (T, T, 3, 1, 1),
    (N, N, 2000, 3, 64),
    (N, N, 31, 33, 17),
])
def test_skinny_shapes(O, handle, dev, mode, opa, opb, m, n, k):
    _check(O, handle, dev, mode, opa, opb, m, n, k, False, 1.25, 0.5, pads=(1, 2, 3), seed=91)


def test_skinny_complex(O, handle, dev):
    _check(O, handle, dev, FP16TCEC, C, N, 1, 513, 700, True, 1.0 - 1.0j, 0.5j, pads=(0, 1, 2), seed=93)
    _check(O, handle, dev, TF32TCEC, N, C, 257, 2, 90, True, 1.0, 0.0, pads=(3, 0, 0), seed=95)


def test_huge_leading_dimension_uses_64_bit_addressing(O, handle, dev, torch_gpu):
    """lda = 2^29: the per-thread byte offsets of a tile no longer fit 31 bits and
    the kernels must fall back to 64-bit element addressing."""
    torch = torch_gpu
    m, n, k, lda = 64, 48, 2, 1 << 29
    a_small = inputs.uniform(97, m * k).reshape(k, m)           # column-major: column j at a[j]
    b = inputs.uniform(98, k * n)
    da = torch.zeros((k - 1) * lda + m, device=dev.dev)         # 2 GiB of floats
    for j in range(k):
        da[j * lda: j * lda + m] = torch.from_numpy(a_small[j]).to(dev.dev)
    db, dc = dev.up(b), dev.up(np.zeros(m * n, np.float32))
    for opa, ld_used in ((N, lda),):
        st = handle.gemm(opa, N, m, n, k, 1.0, da, ld_used, db, k, 0.0, dc, m, FP16TCEC)
        assert st == 0
        c = dev.down(dc)
        ref = O.gemm_fp64(N, N, m, n, k, 1.0, a_small.reshape(-1), m, b, k)
        cf = oracle_gemm(O, FP32, N, N, m, n, k, 1.0, a_small.reshape(-1), m, b, k, 0.0, np.zeros(m * n, np.float32), m)
        assert O.residual(ref, c, m, n, m) <= 2.0 * O.residual(ref, cf, m, n, m) + 2.0 ** -23
    del da
    torch.cuda.empty_cache()


def test_seeded_random_shapes_all_paths(O, handle, dev):
    """Forty seeded random problems (shape, layout, mode, type, scalars, padding):
    whatever kernel form the planner picks -- one-tile or persistent, split-K,
    column split, moved edge tiles -- the result must meet the accuracy bars."""
    rng = np.random.default_rng(20240611)
    dims = [1, 2, 31, 32, 33, 64, 100, 127, 128, 129, 200, 255, 256, 257, 300, 384, 512, 640, 700, 1000]
    for case in range(40):
        m, n, k = (int(rng.choice(dims)) for _ in range(3))
        if case % 8 == 0:
            k = int(rng.choice([2048, 4096, 6000]))      # long K: split-K candidates
        if case % 10 == 5:
            m, n = 2560, int(rng.choice([1300, 2700]))     # column split candidates
            k = int(rng.choice([256, 288]))
        cplx = bool(rng.integers(0, 2))
        ops = [N, T, C] if cplx else [N, T]
        opa, opb = int(rng.choice(ops)), int(rng.choice(ops))
        mode = int(rng.choice([FP16TCEC, TF32TCEC, FP16TCEC, FP16TC, TF32TC]))
        alpha = complex(rng.normal(), rng.normal()) if cplx else float(rng.normal())
        beta = 0.0 if rng.integers(0, 3) == 0 else (complex(rng.normal(), rng.normal()) if cplx else float(rng.normal()))
        pads = tuple(int(x) for x in rng.integers(0, 4, 3))
        _check(O, handle, dev, mode, opa, opb, m, n, k, cplx, alpha, beta, pads=pads, seed=1000 + case)


# ---- the planner's choices ------------------------------------------------------
# The tile class behind a call is reported as the module id (class, + 100 with K split,
# 200 for the pre-split path).  These shapes sit where the cost model was fitted on
# timings of every class: four K-steps take the 128x128 class although the 256x128 one
# fills the chip, sixteen take the large one (for two M/N-contiguous operands and for
# bf16x2 that is the kernel on 16x16x32 MFMAs), and a long-K complex product keeps the
# 128x64 tile with K split.
@pytest.mark.parametrize("mode,cplx,opa,opb,m,n,k,expected", [
    (FP16TCEC, False, N, N, 4096, 4096, 128, (1,)),
    (FP16TCEC, False, N, T, 2560, 2560, 512, (0,)),
    (FP16TCEC, False, N, N, 2560, 2560, 512, (0,)),
    (TF32TCEC, False, N, N, 4096, 4096, 128, (1,)),
    (TF32TC, False, N, T, 2560, 2560, 512, (0,)),
    (FP16TCEC, True, N, T, 1024, 1024, 4096, (0, 100)),
])
def test_planner_takes_the_class_the_sweeps_found_best(handle, dev, mode, cplx, opa, opb, m, n, k, expected):
    gen = _gen(cplx)
    a, lda = make_operand(gen, 41, opa, m, k, 0)
    b, ldb = make_operand(gen, 42, opb, k, n, 0)
    c0 = gen(43, m * n)
    c, st, mid = run_gemm(handle, dev, mode, opa, opb, m, n, k, 1.0, a, lda, b, ldb, 0.0, c0, m, cplx,
                          want_module_id=True)
    assert st == 0 and mid in expected, mid


# ---- the large real FP16TCEC tile on 16x16x32 MFMAs ------------------------------
# A tile-walking launch that keeps every CU busy takes a second instance of the 256x128
# kernel, built on 16x16x32 instead of 32x32x16 MFMAs: the same products, 32 K-values per
# MFMA instead of 16.  Against the 32x32x16 instance (CUMPSGEMM_NO_EDGE16_TWIN): equal up
# to the order of summation on random data, bit for bit on small integers, where every
# partial sum is exact.
@pytest.mark.parametrize("opa,opb", [(N, N), (T, N), (T, T)])
# (512^2: eight 256x128 tiles per matrix, two per CU; 384^2: nine 128x128 tiles per matrix, nine per CU;
# the tables with such a pair of instances: real FP16TCEC both tiles, plain and with fused scaling, real
# bf16x3 128x128, real FP16TC 256x128)
@pytest.mark.parametrize("mode,scaled,m,n,k,batch", [
    (FP16TCEC, False, 512, 512, 288, 64), (FP16TCEC, True, 512, 512, 288, 64),
    (FP16TCEC, False, 384, 384, 288, 256), (FP16TCEC, True, 384, 384, 288, 256),
    (TF32TCEC, False, 384, 384, 288, 256), (FP16TC, False, 512, 512, 288, 64)])
def test_large_in_loop_tile_on_16x16x32_mfmas(cg, handle, dev, monkeypatch, opa, opb, mode, scaled, m, n, k, batch):
    ra, _ = stored_shape(opa, m, k)
    rb, _ = stored_shape(opb, k, n)
    sa, sb, sc = m * k, k * n, m * n
    rng = np.random.default_rng(5)
    for exact in (False, True):
        if exact:
            a = rng.integers(-8, 9, sa * batch).astype(np.float32)
            b = rng.integers(-8, 9, sb * batch).astype(np.float32)
        else:
            a, b = inputs.uniform(61, sa * batch), inputs.uniform(62, sb * batch)
        c0 = inputs.uniform(63, sc * batch)
        da, db = dev.up(a), dev.up(b)
        outs = []
        for twin in (True, False):
            if twin:
                monkeypatch.delenv("CUMPSGEMM_NO_EDGE16_TWIN", raising=False)
            else:
                monkeypatch.setenv("CUMPSGEMM_NO_EDGE16_TWIN", "1")
            dc = dev.up(c0)
            if scaled:
                st, _ = handle.gemm_pipeline(opa, opb, m, n, k, 1.0, da, ra, db, rb, 0.0, dc, m,
                                             cg.FP16TCEC_SCALING, stridea=sa, strideb=sb, stridec=sc, batch=batch)
            else:
                st = handle.gemm_strided_batch(opa, opb, m, n, k, 1.0, da, ra, sa, db, rb, sb, 0.0, dc, m, sc,
                                               batch, mode)
            assert st == 0
            outs.append(dev.down(dc))
        if exact:
            assert np.array_equal(outs[0], outs[1])
            A = a[:sa].reshape(-1, ra).T.astype(np.float64)
            B = b[:sb].reshape(-1, rb).T.astype(np.float64)
            A = A if opa == N else A.T
            B = B if opb == N else B.T
            assert np.array_equal(outs[0][:sc].reshape(n, m).T.astype(np.float64), A @ B)
        elif mode == FP16TC:
            # one product per block, one accumulator: a 16x16x32 MFMA adds its 32 K-values like two
            # 32x32x16 MFMAs add their 16 each, and the two instances agree bit for bit
            assert np.array_equal(outs[0], outs[1])
        else:
            assert not np.array_equal(outs[0], outs[1])      # (the two instances did run)
            assert_same_up_to_summation_order(outs[0], outs[1], k)
