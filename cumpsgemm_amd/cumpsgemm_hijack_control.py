"""Run-time control of the hipBLAS interposer from Python: the counterpart of
the reference's pybind11 module of the same name (python/src/main.cpp:111-173).

Like that module it talks to the interposer only when libcumpsgemm.so has been
LD_PRELOADed into the interpreter; otherwise every call is a no-op and
is_library_loaded() is False (the reference links do-nothing stubs that the
preloaded library overrides, python/src/main.cpp:11-34).  The bookkeeping
switches that the reference keeps inside the module itself (auto kernel
selection, the two dimension thresholds, :7-9 and :91-109) live here too.

    LD_PRELOAD=.../libcumpsgemm.so python app.py
    >>> from cumpsgemm_amd import cumpsgemm_hijack_control as ctl
    >>> ctl.set_compute_mode(ctl.CUMPSGEMM_FP16TCEC)
"""
import ctypes
import enum


class compute_mode(enum.IntEnum):
    """Values of cuMpSGEMM_compute_mode_t (include/cumpsgemm/detail/common.h)."""
    CUMPSGEMM_CUBLAS = 0
    CUMPSGEMM_FP16TCEC = 1
    CUMPSGEMM_TF32TCEC = 2
    CUMPSGEMM_FP16TC = 3
    CUMPSGEMM_TF32TC = 4
    CUMPSGEMM_CUBLAS_SIMT = 5
    CUMPSGEMM_CUBLAS_FP16TC = 6
    CUMPSGEMM_CUBLAS_TF32TC = 7
    CUMPSGEMM_DRY_RUN = 8
    CUMPSGEMM_AUTO = 9
    CUMPSGEMM_FP16TCEC_SCALING = 11


globals().update(compute_mode.__members__)  # export_values()

_CONTROL_FN_T = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_uint, ctypes.c_uint,
                                 ctypes.c_uint)
_keepalive = {"control": None}
_state = {"auto_kernel_selection": False, "mn_threshold": 128, "k_threshold": 64}


def _process():
    """Symbols of the running process: finds the library only if it was preloaded."""
    return ctypes.CDLL(None)


def _sym(name, argtypes=(), restype=None):
    try:
        fn = getattr(_process(), name)
    except AttributeError:
        return None
    fn.argtypes = list(argtypes)
    fn.restype = restype
    return fn


def is_library_loaded():
    fn = _sym("cuMpSGEMM_hijack_is_library_loaded", restype=ctypes.c_int)
    return bool(fn()) if fn else False


def set_compute_mode(mode):
    fn = _sym("cuMpSGEMM_hijack_set_compute_mode", [ctypes.c_int], ctypes.c_int)
    if fn and fn(int(mode)) != 0:
        raise RuntimeError("this compute mode cannot be forced")


def unset_compute_mode():
    fn = _sym("cuMpSGEMM_hijack_unset_compute_mode")
    if fn:
        fn()


def enable_custom_gemm_Mx2x2():
    fn = _sym("cuMpSGEMM_hijack_enable_custom_gemm_Mx2x2")
    if fn:
        fn()


def disable_custom_gemm_Mx2x2():
    fn = _sym("cuMpSGEMM_hijack_disable_custom_gemm_Mx2x2")
    if fn:
        fn()


def set_exp_stats_params(ignore_threshold, underflow_threshold, underflow_tolerance_rate):
    fn = _sym("cuMpSGEMM_hijack_set_exp_stats_params", [ctypes.c_float] * 3)
    if fn:
        fn(ignore_threshold, underflow_threshold, underflow_tolerance_rate)


def get_last_called_function_str():
    fn = _sym("cuMpSGEMM_hijack_get_last_called_function_str", [ctypes.c_char_p, ctypes.c_size_t],
              ctypes.c_size_t)
    if not fn:
        return ""
    buf = ctypes.create_string_buffer(1024)
    fn(buf, len(buf))
    return buf.value.decode()


def set_last_called_function_str(func_str):
    fn = _sym("cuMpSGEMM_hijack_set_last_called_function_str", [ctypes.c_char_p])
    if fn:
        fn(func_str.encode())


def clear_last_called_function_str():
    fn = _sym("cuMpSGEMM_hijack_clear_last_called_function_str")
    if fn:
        fn()


def enable_restoring_AB_after_scaling():
    fn = _sym("cuMpSGEMM_hijack_set_restore_AB", [ctypes.c_int])
    if fn:
        fn(1)


def disable_restoring_AB_after_scaling():
    fn = _sym("cuMpSGEMM_hijack_set_restore_AB", [ctypes.c_int])
    if fn:
        fn(0)


def set_control_function(control_func):
    """control_func(op_A, op_B, m, n, k) -> compute_mode, asked at every
    intercepted GEMM before the rule library."""
    fn = _sym("cuMpSGEMM_hijack_set_control_function", [_CONTROL_FN_T])
    if not fn:
        return
    cb = _CONTROL_FN_T(lambda op_a, op_b, m, n, k: int(control_func(op_a, op_b, m, n, k)))
    fn(cb)
    _keepalive["control"] = cb  # the library keeps the pointer


def unset_control_function():
    fn = _sym("cuMpSGEMM_hijack_set_control_function", [ctypes.c_void_p])
    if fn:
        fn(None)
    _keepalive["control"] = None


def enable_auto_kernel_selection():
    _state["auto_kernel_selection"] = True


def disable_auto_kernel_selection():
    _state["auto_kernel_selection"] = False


def is_auto_kernel_selection_enabled():
    return _state["auto_kernel_selection"]


def set_global_cublas_dim_mn_threshold(dim):
    _state["mn_threshold"] = int(dim)


def get_global_cublas_dim_mn_threshold():
    return _state["mn_threshold"]


def set_global_cublas_dim_k_threshold(dim):
    _state["k_threshold"] = int(dim)


def get_global_cublas_dim_k_threshold():
    return _state["k_threshold"]
