"""ctypes front-end of the CPU oracle (oracle/tcec_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
cpu_baseline leg of the benchmark -- never by the product path.
Arrays are numpy, column-major is expressed through explicit (ld) arguments on
flat float32 buffers exactly like the C-ABI of the library under test.
"""
import ctypes
import os
import subprocess

import numpy as np

OP_N, OP_T, OP_C = 111, 112, 113
MODE_FP16TCEC, MODE_TF32TCEC, MODE_FP16TC, MODE_TF32TC, MODE_FP32 = 1, 2, 3, 4, 12
MODE_UNDEFINED, MODE_FP16TCEC_SCALING = 10, 11

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")


def build():
    """(Re)compile liboracle.so with the committed Makefile."""
    subprocess.check_call(["make", "-s", "-B", "-C", _HERE])


class ExpStats(ctypes.Structure):
    _fields_ = [
        ("max_exp_bits", ctypes.c_uint32),
        ("total", ctypes.c_uint64),
        ("underflow", ctypes.c_uint64),
        ("mode", ctypes.c_int),
        ("stage2_ran", ctypes.c_int),
    ]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        f32p = ctypes.POINTER(ctypes.c_float)
        f64p = ctypes.POINTER(ctypes.c_double)
        u16p = ctypes.POINTER(ctypes.c_uint16)
        sz = ctypes.c_size_t
        L.oracle_f32_to_f16_bits.restype = ctypes.c_uint16
        L.oracle_f32_to_f16_bits.argtypes = [ctypes.c_float]
        L.oracle_f16_bits_to_f32.restype = ctypes.c_float
        L.oracle_f16_bits_to_f32.argtypes = [ctypes.c_uint16]
        L.oracle_f32_to_bf16_bits.restype = ctypes.c_uint16
        L.oracle_f32_to_bf16_bits.argtypes = [ctypes.c_float]
        L.oracle_f32_to_f16_bits_array.argtypes = [f32p, u16p, sz]
        L.oracle_f32_to_bf16_bits_array.argtypes = [f32p, u16p, sz]
        L.oracle_split_fp16.argtypes = [f32p, f32p, f32p, sz]
        L.oracle_split_bf16x3.argtypes = [f32p, f32p, f32p, f32p, sz]
        L.oracle_sgemm.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, sz, sz, sz,
                                   ctypes.c_float, f32p, sz, f32p, sz, ctypes.c_float, f32p, sz]
        L.oracle_cgemm.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, sz, sz, sz,
                                   f32p, f32p, sz, f32p, sz, f32p, f32p, sz]
        L.oracle_gemm_fp64.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, sz, sz, sz,
                                       f64p, f32p, sz, f32p, sz, f64p, f32p, sz, f64p]
        L.oracle_residual.restype = ctypes.c_double
        L.oracle_residual.argtypes = [ctypes.c_int, sz, sz, f64p, f32p, sz]
        L.oracle_exp_stats.argtypes = [f32p, sz, sz, sz, sz, sz, ctypes.c_int, ctypes.c_float,
                                       ctypes.c_float, ctypes.c_float, ctypes.POINTER(ExpStats)]
        L.oracle_exp_max_bits.restype = ctypes.c_uint32
        L.oracle_exp_max_bits.argtypes = [f32p, sz, sz, sz, sz, sz, ctypes.c_int]
        L.oracle_scale_ab_coef.restype = ctypes.c_float
        L.oracle_scale_ab_coef.argtypes = [ctypes.c_float]
        L.oracle_reset_ab_coef.restype = ctypes.c_float
        L.oracle_reset_ab_coef.argtypes = [ctypes.c_float]
        L.oracle_scale_c_coef.restype = ctypes.c_float
        L.oracle_scale_c_coef.argtypes = [ctypes.c_float, ctypes.c_float, ctypes.c_int, ctypes.c_int]
        L.oracle_scale_matrix.argtypes = [f32p, sz, sz, sz, sz, sz, ctypes.c_int, ctypes.c_float]
        L.oracle_combine_flag.restype = ctypes.c_int
        L.oracle_combine_flag.argtypes = [ctypes.c_int, ctypes.c_int]
        L.oracle_next_ring_id.restype = ctypes.c_uint32
        L.oracle_next_ring_id.argtypes = [ctypes.c_uint32, ctypes.c_uint32]
        _lib = L
    return _lib


def _f32(a):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"] or a.flags["F_CONTIGUOUS"]
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def _flat32(a):
    """Flat float32 view of a float32 / complex64 buffer (no copy)."""
    a = np.ascontiguousarray(a) if not (a.flags["C_CONTIGUOUS"] or a.flags["F_CONTIGUOUS"]) else a
    if a.dtype == np.complex64:
        return a.reshape(-1, order="A").view(np.float32)
    assert a.dtype == np.float32
    return a.reshape(-1, order="A")


def f32_to_f16_bits(x):
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    out = np.empty(x.size, dtype=np.uint16)
    lib().oracle_f32_to_f16_bits_array(_f32(x), out.ctypes.data_as(ctypes.POINTER(ctypes.c_uint16)), x.size)
    return out


def f32_to_bf16_bits(x):
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    out = np.empty(x.size, dtype=np.uint16)
    lib().oracle_f32_to_bf16_bits_array(_f32(x), out.ctypes.data_as(ctypes.POINTER(ctypes.c_uint16)), x.size)
    return out


def split_fp16(x):
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    hi = np.empty_like(x)
    lo = np.empty_like(x)
    lib().oracle_split_fp16(_f32(x), _f32(hi), _f32(lo), x.size)
    return hi, lo


def split_bf16x3(x):
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    b = [np.empty_like(x) for _ in range(3)]
    lib().oracle_split_bf16x3(_f32(x), _f32(b[0]), _f32(b[1]), _f32(b[2]), x.size)
    return b


def gemm(mode, op_a, op_b, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc):
    """In-place C = alpha*op(A)op(B)+beta*C on flat buffers (float32 or complex64)."""
    if c.dtype == np.complex64:
        al = np.array([alpha.real, alpha.imag], dtype=np.float32)
        be = np.array([beta.real, beta.imag], dtype=np.float32)
        lib().oracle_cgemm(mode, op_a, op_b, m, n, k, _f32(al), _f32(_flat32(a)), lda,
                           _f32(_flat32(b)), ldb, _f32(be), _f32(_flat32(c)), ldc)
    else:
        lib().oracle_sgemm(mode, op_a, op_b, m, n, k, float(alpha), _f32(_flat32(a)), lda,
                           _f32(_flat32(b)), ldb, float(beta), _f32(_flat32(c)), ldc)
    return c


def gemm_fp64(op_a, op_b, m, n, k, alpha, a, lda, b, ldb, beta=0.0, c=None, ldc=0):
    """FP64 reference of the same FP32 inputs; returns dense (m*n) float64/complex128."""
    ncomp = 2 if a.dtype == np.complex64 else 1
    al = np.array([np.real(alpha), np.imag(alpha)], dtype=np.float64)
    be = np.array([np.real(beta), np.imag(beta)], dtype=np.float64)
    out = np.empty(m * n * ncomp, dtype=np.float64)
    f64p = ctypes.POINTER(ctypes.c_double)
    cptr = _f32(_flat32(c)) if c is not None else None
    lib().oracle_gemm_fp64(ncomp, op_a, op_b, m, n, k, al.ctypes.data_as(f64p), _f32(_flat32(a)), lda,
                           _f32(_flat32(b)), ldb, be.ctypes.data_as(f64p), cptr, ldc,
                           out.ctypes.data_as(f64p))
    return out.view(np.complex128) if ncomp == 2 else out


def residual(ref, c, m, n, ldc):
    """Relative Frobenius residual of c (flat, ldc) against dense FP64 ref."""
    ncomp = 2 if c.dtype == np.complex64 else 1
    r = ref.view(np.float64)
    return lib().oracle_residual(ncomp, m, n, r.ctypes.data_as(ctypes.POINTER(ctypes.c_double)),
                                 _f32(_flat32(c)), ldc)


def exp_stats(x, m, n, ld, batch=1, stride=0, ignore=0.0, underflow=2.0 ** -15, tol=0.0):
    ncomp = 2 if x.dtype == np.complex64 else 1
    out = ExpStats()
    lib().oracle_exp_stats(_f32(_flat32(x)), m, n, ld, batch, stride, ncomp, ignore, underflow, tol,
                           ctypes.byref(out))
    return out


def exp_max_bits(x, m, n, ld, batch=1, stride=0):
    ncomp = 2 if x.dtype == np.complex64 else 1
    return lib().oracle_exp_max_bits(_f32(_flat32(x)), m, n, ld, batch, stride, ncomp)


def scale_matrix(x, m, n, ld, coef, batch=1, stride=0):
    ncomp = 2 if x.dtype == np.complex64 else 1
    lib().oracle_scale_matrix(_f32(_flat32(x)), m, n, ld, batch, stride, ncomp, coef)
    return x
