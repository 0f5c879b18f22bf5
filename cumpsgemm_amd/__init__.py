"""Python binding of libcumpsgemm.so, the MI355X (gfx950) split-and-correct
SGEMM/CGEMM library.  Thin ctypes layer over the C ABI declared in
include/cumpsgemm/cumpsgemm.h and include/cumpsgemm/cumpsgemm_ext.h; device
memory is passed as raw pointers (ints) or as objects with ``data_ptr()``.

There is no CPU fallback: if the shared library is missing, loading raises.
"""
from ._lib import (  # noqa: F401
    OP_N, OP_T, OP_C,
    CUBLAS, FP16TCEC, TF32TCEC, FP16TC, TF32TC, CUBLAS_SIMT, CUBLAS_FP16TC, CUBLAS_TF32TC,
    DRY_RUN, AUTO, UNDEFINED, FP16TCEC_SCALING, FP32_SIMT,
    MODE_NAMES, STATUS_SUCCESS, STATUS_INVALID_VALUE,
    Handle, lib, lib_path, rule_lib_path, build, mode_string, hijack,
)
