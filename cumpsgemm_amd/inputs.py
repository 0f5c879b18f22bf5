"""Seeded synthetic inputs shared by the tests and the benchmark.

Counter-based: element i of stream `seed` is a pure function of (seed, i)
(splitmix64 of seed * 2^40 + i), so the same matrices can be produced anywhere
without carrying data around.  All generators return flat float32 / complex64
numpy arrays in column-major order.
"""
import numpy as np

_MASK = np.uint64(0xFFFFFFFFFFFFFFFF)


def _splitmix64(x):
    x = (x + np.uint64(0x9E3779B97F4A7C15)) & _MASK
    z = x
    z = ((z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)) & _MASK
    z = ((z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)) & _MASK
    return z ^ (z >> np.uint64(31))


def _u01(seed, count, lane=0):
    """count doubles in [0, 1) with 24 random bits (exactly representable in FP32)."""
    with np.errstate(over="ignore"):
        idx = np.arange(count, dtype=np.uint64) + np.uint64((seed << 40) + (lane << 36))
        bits = _splitmix64(idx) >> np.uint64(40)
    return bits.astype(np.float64) * (1.0 / (1 << 24))


def uniform(seed, count, lo=-1.0, hi=1.0):
    """i.i.d. uniform[lo, hi) float32."""
    return (lo + (hi - lo) * _u01(seed, count)).astype(np.float32)


def normal(seed, count, sigma=1.0):
    """i.i.d. N(0, sigma^2) float32 (Box-Muller on two uniform streams)."""
    u1 = 1.0 - _u01(seed, count, lane=1)  # (0, 1]
    u2 = _u01(seed, count, lane=2)
    z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
    return (sigma * z).astype(np.float32)


def complex_normal(seed, count, sigma=1.0):
    """complex64 with independent N(0, sigma^2) real and imaginary parts."""
    out = np.empty(count, dtype=np.complex64)
    out.real = normal(seed, count, sigma)
    out.imag = normal(seed + 1000003, count, sigma)
    return out


def exponent_spread(seed, rows, cols, per_row, lo=-30, hi=30):
    """N(0,1) * 2^e with an integer exponent e ~ U[lo, hi] per row (per_row=True:
    A[i,k] = g * 2^{e_i}) or per column (B[k,j] = g * 2^{f_j}); column-major."""
    g = normal(seed, rows * cols).reshape(cols, rows)  # [col][row]
    n_e = rows if per_row else cols
    e = np.floor(lo + (hi - lo + 1) * _u01(seed + 77, n_e)).astype(np.int32)
    scale = np.ldexp(np.float32(1.0), e).astype(np.float32)
    out = g * (scale[None, :] if per_row else scale[:, None])
    return out.reshape(-1).astype(np.float32)


def random_unitary_2x2(seed):
    """2x2 unitary from the QR of a seeded complex Gaussian (FP64, rounded to FP32);
    column-major flat complex64 of length 4."""
    g = (normal(seed, 4).astype(np.float64) + 1j * normal(seed + 5, 4).astype(np.float64)).reshape(2, 2)
    q, r = np.linalg.qr(g)
    q = q * (np.diag(r) / np.abs(np.diag(r)))[None, :]
    return np.asfortranarray(q).reshape(-1, order="F").astype(np.complex64)
