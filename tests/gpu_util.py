"""Shared helpers of the GPU parity tests: build operands in column-major flat
buffers, run the library through its C ABI, run the oracle on the same data."""
import numpy as np

N, T, C = 111, 112, 113


def stored_shape(op, rows, cols):
    """Shape in memory of an operand whose op() has (rows, cols)."""
    return (rows, cols) if op == N else (cols, rows)


def make_operand(gen, seed, op, rows, cols, pad=0):
    r, c = stored_shape(op, rows, cols)
    ld = r + pad
    return gen(seed, ld * c), ld


def run_gemm(handle, dev, mode, opa, opb, m, n, k, alpha, a, lda, b, ldb, beta, c0, ldc, cplx,
             want_module_id=False):
    da, db, dc = dev.up(a), dev.up(b), dev.up(c0)
    out = handle.gemm(opa, opb, m, n, k, alpha, da, lda, db, ldb, beta, dc, ldc, mode, cplx=cplx,
                      want_module_id=want_module_id)
    c = dev.down(dc, np.complex64 if cplx else np.float32)
    return (c,) + (out if want_module_id else (out,))


def oracle_gemm(O, mode, opa, opb, m, n, k, alpha, a, lda, b, ldb, beta, c0, ldc):
    c = c0.copy()
    O.gemm(mode, opa, opb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc)
    return c


def rel_diff(x, y, m, n, ld):
    """Relative Frobenius difference of the logical m x n parts of two flat buffers."""
    xv = x.reshape(-1, ld)[:n, :m].astype(np.complex128)
    yv = y.reshape(-1, ld)[:n, :m].astype(np.complex128)
    return float(np.linalg.norm(xv - yv) / max(np.linalg.norm(yv), 1e-300))


def assert_same_up_to_summation_order(x, y, k):
    """x and y hold the same products added in a different order (kernels built on MFMAs of
    different K-depth): equal within a few FP32 roundings per partial sum, as a whole
    (Frobenius) and element by element -- a misplaced element would differ at order one."""
    if hasattr(x, "detach"):
        x, y = x.detach().cpu().numpy(), y.detach().cpu().numpy()
    xv = np.ascontiguousarray(x).view(np.float32).astype(np.float64).ravel()
    yv = np.ascontiguousarray(y).view(np.float32).astype(np.float64).ravel()
    assert xv.shape == yv.shape and np.isfinite(xv).all() and np.isfinite(yv).all()
    d = np.abs(xv - yv)
    bar = 2.0 ** -24 * np.sqrt(k)
    assert np.linalg.norm(d) <= 2.0 * bar * np.linalg.norm(yv), (np.linalg.norm(d) / np.linalg.norm(yv), bar)
    assert d.max() <= 16.0 * bar * np.abs(yv).max(), (d.max() / np.abs(yv).max(), bar)
