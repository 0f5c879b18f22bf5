import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
# CUMPSGEMM_LIBRARY: another build of the library (a diagnostic one, say) instead of the in-tree file
_LIB = os.environ.get("CUMPSGEMM_LIBRARY") or os.path.join(_HERE, "libcumpsgemm.so")
_RULE_LIB = os.path.join(_HERE, "libcumpsgemm_rule.so")

# hipblasOperation_t
OP_N, OP_T, OP_C = 111, 112, 113
# cuMpSGEMM_compute_mode_t
(CUBLAS, FP16TCEC, TF32TCEC, FP16TC, TF32TC, CUBLAS_SIMT, CUBLAS_FP16TC, CUBLAS_TF32TC,
 DRY_RUN, AUTO, UNDEFINED, FP16TCEC_SCALING, FP32_SIMT) = range(13)
MODE_NAMES = ["CUBLAS", "FP16TCEC", "TF32TCEC", "FP16TC", "TF32TC", "CUBLAS_SIMT", "CUBLAS_FP16TC",
              "CUBLAS_TF32TC", "DRY_RUN", "AUTO", "UNDEFINED", "FP16TCEC_SCALING", "FP32_SIMT"]
# hipblasStatus_t
STATUS_SUCCESS, STATUS_INVALID_VALUE = 0, 3

_u64 = ctypes.c_uint64
_u32 = ctypes.c_uint
_ptr = ctypes.c_void_p
_int = ctypes.c_int


class _C2(ctypes.Structure):
    _fields_ = [("x", ctypes.c_float), ("y", ctypes.c_float)]


def lib_path():
    return _LIB


def rule_lib_path():
    return _RULE_LIB


def build(jobs=8):
    """Compile libcumpsgemm.so and libcumpsgemm_rule.so for gfx950 in-tree."""
    subprocess.check_call(["make", "-s", "-B", "-j", str(jobs), "-C", os.path.join(_HERE, "csrc")])


_lib = None


def lib():
    """The loaded shared library (raises if it has not been built)."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB):
            raise RuntimeError(
                f"{_LIB} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
                "(there is no CPU fallback)")
        # A process must end up with ONE HIP runtime.  PyTorch ships its own copy
        # of libamdhip64 (same SONAME as the system one): if it is going to be
        # used in this process, let it load first so that this library binds to
        # the runtime that owns the tensors' memory and streams.
        try:
            import torch  # noqa: F401
        except Exception:
            pass
        L = ctypes.CDLL(_LIB)
        _declare(L)
        _lib = L
    return _lib


def _declare(L):
    L.cuMpSGEMM_create.argtypes = [ctypes.POINTER(_ptr)]
    L.cuMpSGEMM_destroy.argtypes = [_ptr]
    L.cuMpSGEMM_set_stream.argtypes = [_ptr, _ptr]
    L.cuMpSGEMM_get_compute_mode_string.argtypes = [_int]
    L.cuMpSGEMM_get_compute_mode_string.restype = ctypes.c_char_p
    L.cuMpSGEMM_get_compute_mode.argtypes = [ctypes.c_char_p, _ptr, _int, _int, _u32, _u32, _u32]
    f32p = ctypes.POINTER(ctypes.c_float)
    c2p = ctypes.POINTER(_C2)
    gemm_tail = [_u64, _u64, _u64]
    L.cuMpSGEMM_sgemm.argtypes = [_ptr, _int, _int] + gemm_tail + [f32p, _ptr, _u64, _ptr, _u64, f32p, _ptr, _u64, _int]
    L.cuMpSGEMM_cgemm.argtypes = [_ptr, _int, _int] + gemm_tail + [c2p, _ptr, _u64, _ptr, _u64, c2p, _ptr, _u64, _int]
    L.cuMpSGEMM_sgemm_ex.argtypes = L.cuMpSGEMM_sgemm.argtypes + [ctypes.POINTER(_u32)]
    L.cuMpSGEMM_sgemm_no_alloc.argtypes = L.cuMpSGEMM_sgemm.argtypes
    L.cuMpSGEMM_set_walk_stamp_buffer.argtypes = [_ptr]
    L.cuMpSGEMM_get_static_scratch_size.argtypes = []
    L.cuMpSGEMM_get_static_scratch_size.restype = ctypes.c_size_t
    L.cuMpSGEMM_cgemm_ex.argtypes = L.cuMpSGEMM_cgemm.argtypes + [ctypes.POINTER(_u32)]
    L.cuMpSGEMM_sgemm_strided_batch.argtypes = [_ptr, _int, _int] + gemm_tail + [
        f32p, _ptr, _u64, _u64, _ptr, _u64, _u64, f32p, _ptr, _u64, _u64, _u64, _int]
    L.cuMpSGEMM_cgemm_strided_batch.argtypes = [_ptr, _int, _int] + gemm_tail + [
        c2p, _ptr, _u64, _u64, _ptr, _u64, _u64, c2p, _ptr, _u64, _u64, _u64, _int]
    L.cuMpSGEMM_sgemm_pipeline.argtypes = [_ptr, _int, _int] + gemm_tail + [
        f32p, _ptr, _u64, _u64, _ptr, _u64, _u64, f32p, _ptr, _u64, _u64, _u64, _int, _int,
        ctypes.POINTER(_u32)]
    L.cuMpSGEMM_cgemm_pipeline.argtypes = [_ptr, _int, _int] + gemm_tail + [
        c2p, _ptr, _u64, _u64, _ptr, _u64, _u64, c2p, _ptr, _u64, _u64, _u64, _int, _int,
        ctypes.POINTER(_u32)]
    for name, sp in (("cuMpSGEMM_sgemm_Mx2x2", f32p), ("cuMpSGEMM_cgemm_Mx2x2", c2p),
                     ("cuMpSGEMM_sgemm_2xNx2", f32p), ("cuMpSGEMM_cgemm_2xNx2", c2p)):
        getattr(L, name).argtypes = [_ptr, _int, _int, _u64, sp, _ptr, _u64, _u64, _ptr, _u64, _u64,
                                     sp, _ptr, _u64, _u64, _u64]
    L.cuMpSGEMM_get_workspace_size.argtypes = [_ptr]
    L.cuMpSGEMM_get_workspace_size.restype = ctypes.c_size_t
    L.cuMpSGEMM_get_workspace_pointer.argtypes = [_ptr]
    L.cuMpSGEMM_get_workspace_pointer.restype = _ptr
    L.cuMpSGEMM_reload_tuning_env.argtypes = []
    L.cuMpSGEMM_reload_tuning_env.restype = None
    L.cuMpSGEMM_describe_tile_config.argtypes = [_int, _int, _int, _int, _int, ctypes.c_char_p, ctypes.c_size_t]
    stats_args = [_ptr, _u32, _u32, _ptr, _u32, _u32, _u32]
    for name in ("cuMpSGEMM_exp_stats_ext_s", "cuMpSGEMM_exp_stats_ext_c",
                 "cuMpSGEMM_exp_max_ext_s", "cuMpSGEMM_exp_max_ext_c"):
        getattr(L, name).argtypes = stats_args
        getattr(L, name).restype = _u32
    L.cuMpSGEMM_exp_stats_pair_s.argtypes = [_ptr, _u32, _u32, _ptr, _u32, _u32, _u32, _ptr, _u32, _int,
                                             ctypes.POINTER(_u32)]
    L.cuMpSGEMM_exp_stats_pair_s.restype = None
    L.cuMpSGEMM_exp_max_pair_s.argtypes = [_ptr, _u32, _u32, _ptr, _u32, _u32, _u32, _ptr, _u32, ctypes.POINTER(_u32)]
    L.cuMpSGEMM_exp_max_pair_s.restype = None
    L.cuMpSGEMM_get_exp_stats.argtypes = [_ptr, _u32, ctypes.POINTER(_u64), ctypes.POINTER(_u64)]
    L.cuMpSGEMM_get_exp_stats.restype = None
    L.cuMpSGEMM_get_max_exp.argtypes = [_ptr, _u32]
    L.cuMpSGEMM_get_max_exp.restype = ctypes.c_float
    L.cuMpSGEMM_get_exp_stats_compute_mode_level.argtypes = [_ptr, _u32]
    L.cuMpSGEMM_set_exp_stats_params.argtypes = [_ptr, ctypes.c_float, ctypes.c_float, ctypes.c_float]
    L.cuMpSGEMM_set_exp_stats_params.restype = None
    L.cuMpSGEMM_get_current_exp_stats_buffer_id.argtypes = [_ptr]
    L.cuMpSGEMM_get_current_exp_stats_buffer_id.restype = _u32
    L.cuMpSGEMM_reset_exp_stats_buffer_id.argtypes = [_ptr]
    L.cuMpSGEMM_reset_exp_stats_buffer_id.restype = None
    L.cuMpSGEMM_enable_exp_stats.argtypes = [_ptr]
    L.cuMpSGEMM_disable_exp_stats.argtypes = [_ptr]
    for name in ("enable", "disable", "reset"):
        fn = getattr(L, f"cuMpSGEMM_{name}_exp_stats_profiling")
        fn.argtypes = [_ptr]
        fn.restype = None
    L.cuMpSGEMM_print_exp_stats_profiling.argtypes = [_ptr, _u32]
    L.cuMpSGEMM_print_exp_stats_profiling.restype = None
    L.cuMpSGEMM_get_exp_stats_profiling_entry.argtypes = [_ptr, ctypes.c_char_p, ctypes.POINTER(ctypes.c_double),
                                                          ctypes.POINTER(_u64)]
    scale_args = [_ptr, _u32, _u32, _u32, _u32, _ptr, _u32, _u32, _u32]
    for base in ("scale_A", "scale_B", "reset_scale_A", "reset_scale_B"):
        for sfx in ("s", "c"):
            fn = getattr(L, f"cuMpSGEMM_{base}_{sfx}")
            fn.argtypes = scale_args
            fn.restype = None
    for sfx in ("s", "c"):
        fn = getattr(L, f"cuMpSGEMM_scale_C_{sfx}")
        fn.argtypes = [_ptr, _u32, _u32, _u32, _u32, _u32, _ptr, _u32, _u32, _u32]
        fn.restype = None
    L.cuMpSGEMM_get_current_dynamic_launch_buffer_id.argtypes = [_ptr]
    L.cuMpSGEMM_get_current_dynamic_launch_buffer_id.restype = _u32
    L.cuMpSGEMM_get_next_dynamic_launch_buffer_id.argtypes = [_ptr]
    L.cuMpSGEMM_get_next_dynamic_launch_buffer_id.restype = _u32
    L.cuMpSGEMM_get_dynamic_launch_flag.argtypes = [_ptr, _u32]
    L.cuMpSGEMM_set_dynamic_launch_buffer_by_exp_stats.argtypes = [_ptr, _u32, _u32, _u32]
    L.cuMpSGEMM_set_dynamic_launch_buffer_by_exp_stats.restype = None
    L.cuMpSGEMM_set_dynamic_launch_flag_buffer_id.argtypes = [_ptr, _u32]
    L.cuMpSGEMM_set_dynamic_launch_flag_buffer_id.restype = None
    L.cuMpSGEMM_unset_dynamic_launch_flag_buffer_id.argtypes = [_ptr]
    L.cuMpSGEMM_unset_dynamic_launch_flag_buffer_id.restype = None
    L.cuMpSGEMM_hijack_get_internal_global_handle.restype = _ptr
    L.cuMpSGEMM_hijack_set_compute_mode.argtypes = [_int]
    L.cuMpSGEMM_hijack_set_restore_AB.argtypes = [_int]
    L.cuMpSGEMM_hijack_get_last_called_function_str.argtypes = [ctypes.c_char_p, ctypes.c_size_t]
    L.cuMpSGEMM_hijack_get_last_called_function_str.restype = ctypes.c_size_t
    L.cuMpSGEMM_hijack_query_compute_mode.argtypes = [ctypes.c_char_p, _int, _int, _u32, _u32, _u32]


def mode_string(mode):
    return lib().cuMpSGEMM_get_compute_mode_string(int(mode)).decode()


def _dptr(x):
    if x is None:
        return None
    if hasattr(x, "data_ptr"):
        return x.data_ptr()
    return int(x)


def _scalar(v, cplx):
    if cplx:
        v = complex(v)
        return ctypes.byref(_C2(v.real, v.imag))
    return ctypes.byref(ctypes.c_float(float(v)))


class Handle:
    """cuMpSGEMM_handle_t bound to the current HIP device.

    Method names, argument order and meaning follow the C++ API of
    include/cumpsgemm/cumpsgemm.hpp; ``cplx`` selects the hipComplex form."""

    def __init__(self, stream=None):
        self._L = lib()
        h = _ptr()
        st = self._L.cuMpSGEMM_create(ctypes.byref(h))
        if st != STATUS_SUCCESS:
            raise RuntimeError(f"cuMpSGEMM_create failed with hipblasStatus {st}")
        self._h = h
        if stream is not None:
            self.set_stream(stream)

    def close(self):
        if getattr(self, "_h", None):
            self._L.cuMpSGEMM_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def raw(self):
        return self._h

    def set_stream(self, stream):
        s = getattr(stream, "cuda_stream", stream)
        return self._L.cuMpSGEMM_set_stream(self._h, _ptr(int(s) if s else 0))

    def workspace_size(self):
        """Bytes of device memory held for pre-split operands."""
        return self._L.cuMpSGEMM_get_workspace_size(self._h)

    def workspace_pointer(self):
        """Device address of that workspace (0 until it exists)."""
        return self._L.cuMpSGEMM_get_workspace_pointer(self._h) or 0

    # ---- GEMM ----
    def gemm(self, op_a, op_b, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc, mode, cplx=False,
             want_module_id=False):
        fn = self._L.cuMpSGEMM_cgemm_ex if cplx else self._L.cuMpSGEMM_sgemm_ex
        mid = _u32(0)
        st = fn(self._h, op_a, op_b, m, n, k, _scalar(alpha, cplx), _dptr(a), lda, _dptr(b), ldb,
                _scalar(beta, cplx), _dptr(c), ldc, int(mode), ctypes.byref(mid))
        return (st, mid.value) if want_module_id else st

    def gemm_no_alloc(self, op_a, op_b, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc, mode):
        """cuMpSGEMM_sgemm_no_alloc: the pre-split path over the library's static scratch."""
        return self._L.cuMpSGEMM_sgemm_no_alloc(self._h, op_a, op_b, m, n, k, _scalar(alpha, False), _dptr(a),
                                                lda, _dptr(b), ldb, _scalar(beta, False), _dptr(c), ldc,
                                                int(mode))

    def gemm_strided_batch(self, op_a, op_b, m, n, k, alpha, a, lda, stridea, b, ldb, strideb, beta,
                           c, ldc, stridec, batch, mode, cplx=False):
        fn = self._L.cuMpSGEMM_cgemm_strided_batch if cplx else self._L.cuMpSGEMM_sgemm_strided_batch
        return fn(self._h, op_a, op_b, m, n, k, _scalar(alpha, cplx), _dptr(a), lda, stridea,
                  _dptr(b), ldb, strideb, _scalar(beta, cplx), _dptr(c), ldc, stridec, batch, int(mode))

    def gemm_pipeline(self, op_a, op_b, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc, mode,
                      cplx=False, stridea=0, strideb=0, stridec=0, batch=1, restore_ab=True):
        fn = self._L.cuMpSGEMM_cgemm_pipeline if cplx else self._L.cuMpSGEMM_sgemm_pipeline
        ids = (_u32 * 3)()
        st = fn(self._h, op_a, op_b, m, n, k, _scalar(alpha, cplx), _dptr(a), lda, stridea, _dptr(b),
                ldb, strideb, _scalar(beta, cplx), _dptr(c), ldc, stridec, batch, int(mode),
                1 if restore_ab else 0, ids)
        return st, tuple(ids)

    def gemm_Mx2x2(self, op_a, op_b, m, alpha, a, lda, b, ldb, beta, c, ldc, cplx=False,
                   stridea=0, strideb=0, stridec=0, batch=1):
        fn = self._L.cuMpSGEMM_cgemm_Mx2x2 if cplx else self._L.cuMpSGEMM_sgemm_Mx2x2
        return fn(self._h, op_a, op_b, m, _scalar(alpha, cplx), _dptr(a), lda, stridea, _dptr(b),
                  ldb, strideb, _scalar(beta, cplx), _dptr(c), ldc, stridec, batch)

    def gemm_2xNx2(self, op_a, op_b, n, alpha, a, lda, b, ldb, beta, c, ldc, cplx=False,
                   stridea=0, strideb=0, stridec=0, batch=1):
        fn = self._L.cuMpSGEMM_cgemm_2xNx2 if cplx else self._L.cuMpSGEMM_sgemm_2xNx2
        return fn(self._h, op_a, op_b, n, _scalar(alpha, cplx), _dptr(a), lda, stridea, _dptr(b),
                  ldb, strideb, _scalar(beta, cplx), _dptr(c), ldc, stridec, batch)

    # ---- exponent statistics ----
    def exp_stats_ext(self, m, n, ptr, ld, batch=1, stride=0, cplx=False):
        fn = self._L.cuMpSGEMM_exp_stats_ext_c if cplx else self._L.cuMpSGEMM_exp_stats_ext_s
        return fn(self._h, m, n, _dptr(ptr), ld, batch, stride)

    def exp_max_ext(self, m, n, ptr, ld, batch=1, stride=0, cplx=False):
        fn = self._L.cuMpSGEMM_exp_max_ext_c if cplx else self._L.cuMpSGEMM_exp_max_ext_s
        return fn(self._h, m, n, _dptr(ptr), ld, batch, stride)

    def exp_stats_pair(self, m_a, n_a, a, lda, m_b, n_b, b, ldb, flag_id=-1):
        """Full statistics of A and B with one launch per pass; returns their two slots."""
        ids = (_u32 * 2)()
        self._L.cuMpSGEMM_exp_stats_pair_s(self._h, m_a, n_a, _dptr(a), lda, m_b, n_b, _dptr(b), ldb, flag_id, ids)
        return ids[0], ids[1]

    def exp_max_pair(self, m_a, n_a, a, lda, m_b, n_b, b, ldb):
        """Maximum exponents of A and B with one launch; returns their two slots."""
        ids = (_u32 * 2)()
        self._L.cuMpSGEMM_exp_max_pair_s(self._h, m_a, n_a, _dptr(a), lda, m_b, n_b, _dptr(b), ldb, ids)
        return ids[0], ids[1]

    def get_exp_stats(self, buffer_id):
        """(underflow, total) like cumpsgemm::get_exp_stats."""
        u, t = _u64(0), _u64(0)
        self._L.cuMpSGEMM_get_exp_stats(self._h, buffer_id, ctypes.byref(u), ctypes.byref(t))
        return u.value, t.value

    def get_max_exp(self, buffer_id):
        return self._L.cuMpSGEMM_get_max_exp(self._h, buffer_id)

    def get_exp_stats_compute_mode_level(self, buffer_id):
        return self._L.cuMpSGEMM_get_exp_stats_compute_mode_level(self._h, buffer_id)

    def set_exp_stats_params(self, ignore_threshold, underflow_threshold, tolerance):
        self._L.cuMpSGEMM_set_exp_stats_params(self._h, ignore_threshold, underflow_threshold, tolerance)

    def get_current_exp_stats_buffer_id(self):
        return self._L.cuMpSGEMM_get_current_exp_stats_buffer_id(self._h)

    def reset_exp_stats_buffer_id(self):
        self._L.cuMpSGEMM_reset_exp_stats_buffer_id(self._h)

    # ---- wall-clock profiling of stats / scaling / GEMM launches ----
    def enable_exp_stats_profiling(self):
        self._L.cuMpSGEMM_enable_exp_stats_profiling(self._h)

    def disable_exp_stats_profiling(self):
        self._L.cuMpSGEMM_disable_exp_stats_profiling(self._h)

    def reset_exp_stats_profiling(self):
        self._L.cuMpSGEMM_reset_exp_stats_profiling(self._h)

    def print_exp_stats_profiling(self, csv=False):
        self._L.cuMpSGEMM_print_exp_stats_profiling(self._h, int(csv))

    def get_exp_stats_profiling_entry(self, name):
        """(seconds, count) recorded under a label, or None if the label never ran."""
        t, n = ctypes.c_double(0), _u64(0)
        if not self._L.cuMpSGEMM_get_exp_stats_profiling_entry(self._h, name.encode(), ctypes.byref(t),
                                                               ctypes.byref(n)):
            return None
        return t.value, n.value

    # ---- scaling ----
    def _scale(self, base, cplx, *args):
        getattr(self._L, f"cuMpSGEMM_{base}_{'c' if cplx else 's'}")(self._h, *args)

    def scale_A(self, stats_id, flag_id, m, n, ptr, ld, batch=1, stride=0, cplx=False):
        self._scale("scale_A", cplx, stats_id, flag_id, m, n, _dptr(ptr), ld, batch, stride)

    def scale_B(self, stats_id, flag_id, m, n, ptr, ld, batch=1, stride=0, cplx=False):
        self._scale("scale_B", cplx, stats_id, flag_id, m, n, _dptr(ptr), ld, batch, stride)

    def scale_C(self, stats_a, stats_b, flag_id, m, n, ptr, ld, batch=1, stride=0, cplx=False):
        self._scale("scale_C", cplx, stats_a, stats_b, flag_id, m, n, _dptr(ptr), ld, batch, stride)

    def reset_scale_A(self, stats_id, flag_id, m, n, ptr, ld, batch=1, stride=0, cplx=False):
        self._scale("reset_scale_A", cplx, stats_id, flag_id, m, n, _dptr(ptr), ld, batch, stride)

    def reset_scale_B(self, stats_id, flag_id, m, n, ptr, ld, batch=1, stride=0, cplx=False):
        self._scale("reset_scale_B", cplx, stats_id, flag_id, m, n, _dptr(ptr), ld, batch, stride)

    # ---- launch-flag ring ----
    def get_current_dynamic_launch_buffer_id(self):
        return self._L.cuMpSGEMM_get_current_dynamic_launch_buffer_id(self._h)

    def get_next_dynamic_launch_buffer_id(self):
        return self._L.cuMpSGEMM_get_next_dynamic_launch_buffer_id(self._h)

    def get_dynamic_launch_flag(self, buffer_id):
        return self._L.cuMpSGEMM_get_dynamic_launch_flag(self._h, buffer_id)

    def set_dynamic_launch_buffer_by_exp_stats(self, flag_id, a_id, b_id):
        self._L.cuMpSGEMM_set_dynamic_launch_buffer_by_exp_stats(self._h, flag_id, a_id, b_id)

    def set_dynamic_launch_flag_buffer_id(self, flag_id):
        self._L.cuMpSGEMM_set_dynamic_launch_flag_buffer_id(self._h, flag_id)

    def unset_dynamic_launch_flag_buffer_id(self):
        self._L.cuMpSGEMM_unset_dynamic_launch_flag_buffer_id(self._h)


class hijack:
    """cumpsgemm::hijack_control of the loaded library (host-side state only)."""

    @staticmethod
    def set_compute_mode(mode):
        if lib().cuMpSGEMM_hijack_set_compute_mode(int(mode)) != 0:
            raise RuntimeError("CUMPSGEMM_FP32_SIMT mode is currently not supported.")

    @staticmethod
    def unset_compute_mode():
        lib().cuMpSGEMM_hijack_unset_compute_mode()

    @staticmethod
    def query_compute_mode(func_name, op_a, op_b, m, n, k):
        return lib().cuMpSGEMM_hijack_query_compute_mode(func_name.encode(), op_a, op_b, m, n, k)

    @staticmethod
    def last_called_function_str():
        buf = ctypes.create_string_buffer(512)
        lib().cuMpSGEMM_hijack_get_last_called_function_str(buf, 512)
        return buf.value.decode()

    @staticmethod
    def is_library_loaded():
        return bool(lib().cuMpSGEMM_hijack_is_library_loaded())
