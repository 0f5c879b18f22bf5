"""The HBM-streaming (M,2,2) / (2,N,2) kernels against the oracle's plain FP32
GEMM (semantics of the shapes the reference hands to cuGEMM-Mx2x2)."""
import numpy as np
import pytest

from cumpsgemm_amd import inputs
from gpu_util import N, T, C, oracle_gemm

pytestmark = pytest.mark.gpu
FP32 = 12


@pytest.mark.parametrize("cplx", [False, True])
@pytest.mark.parametrize("opa", [N, T, C])
@pytest.mark.parametrize("opb", [N, T, C])
@pytest.mark.parametrize("m", [1, 2, 64, 4096, 1 << 16, 1000])
def test_Mx2x2(O, handle, dev, cplx, opa, opb, m):
    gen = (lambda s, c: inputs.complex_normal(s, c, 0.7)) if cplx else inputs.uniform
    lda = m + 4 if opa == N else 2
    a = gen(1, lda * (2 if opa == N else m))
    b = gen(2, 4) if not cplx else inputs.random_unitary_2x2(2)
    ldc = m + 4
    c0 = gen(3, ldc * 2)
    alpha, beta = ((0.5 + 1j), (1 - 0.25j)) if cplx else (1.5, -0.5)
    da, db, dc = dev.up(a), dev.up(b), dev.up(c0)
    assert handle.gemm_Mx2x2(opa, opb, m, alpha, da, lda, db, 2, beta, dc, ldc, cplx=cplx) == 0
    got = dev.down(dc, c0.dtype)
    ref = O.gemm_fp64(opa, opb, m, 2, 2, alpha, a, lda, b, 2, beta, c0, ldc)
    assert O.residual(ref, got, m, 2, ldc) < 4e-7
    assert np.array_equal(got.reshape(2, ldc)[:, m:], c0.reshape(2, ldc)[:, m:])


@pytest.mark.parametrize("cplx", [False, True])
@pytest.mark.parametrize("opa", [N, T, C])
@pytest.mark.parametrize("opb", [N, T, C])
@pytest.mark.parametrize("n", [1, 8, 4096, 1000])
def test_2xNx2(O, handle, dev, cplx, opa, opb, n):
    gen = (lambda s, c: inputs.complex_normal(s, c, 0.7)) if cplx else inputs.uniform
    a = gen(1, 4)
    ldb = 2 if opb == N else n + 3
    b = gen(2, ldb * (n if opb == N else 2))
    ldc = 3
    c0 = gen(3, ldc * n)
    da, db, dc = dev.up(a), dev.up(b), dev.up(c0)
    assert handle.gemm_2xNx2(opa, opb, n, 1.0, da, 2, db, ldb, 0.0, dc, ldc, cplx=cplx) == 0
    got = dev.down(dc, c0.dtype)
    ref = O.gemm_fp64(opa, opb, 2, n, 2, 1.0, a, 2, b, ldb)
    assert O.residual(ref, got, 2, n, ldc) < 4e-7
    assert np.array_equal(got.reshape(n, ldc)[:, 2:], c0.reshape(n, ldc)[:, 2:])


def test_Mx2x2_batched_and_beta_zero_nan(O, handle, dev):
    m, batch = 512, 4
    a = inputs.complex_normal(4, m * 2 * batch, 0.7)
    b = np.concatenate([inputs.random_unitary_2x2(10 + i) for i in range(batch)])
    c0 = np.full(m * 2 * batch, np.nan + 0j, dtype=np.complex64)
    da, db, dc = dev.up(a), dev.up(b), dev.up(c0)
    assert handle.gemm_Mx2x2(N, N, m, 1.0, da, m, db, 2, 0.0, dc, m, cplx=True, stridea=2 * m, strideb=4,
                             stridec=2 * m, batch=batch) == 0
    got = dev.down(dc, np.complex64)
    for i in range(batch):
        ref = O.gemm_fp64(N, N, m, 2, 2, 1.0, a[i * 2 * m:], m, b[i * 4:], 2)
        assert O.residual(ref, got[i * 2 * m:(i + 1) * 2 * m], m, 2, m) < 4e-7
    # a unitary gate preserves the norm of every state vector
    for i in range(batch):
        x = a[i * 2 * m:(i + 1) * 2 * m].astype(np.complex128)
        y = got[i * 2 * m:(i + 1) * 2 * m].astype(np.complex128)
        assert abs(np.linalg.norm(y) / np.linalg.norm(x) - 1) < 1e-6
