"""Host-side behaviour of libcumpsgemm.so that needs no GPU: the library loads
and exports every symbol the public headers declare, mode names, the default
rule and its precedence chain, and the interposer's control switches
(reference behaviour: src/default_cumpsgemm_rule.cu:6-49,
src/cumpsgemm_cublas.cu:163-220, :1189-1271)."""
import os
import re
import subprocess
import sys
import textwrap

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INC = os.path.join(ROOT, "include", "cumpsgemm")


def _declared_c_symbols():
    names = set()
    for hdr in ("cumpsgemm.h", "cumpsgemm_ext.h"):
        text = open(os.path.join(INC, hdr)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(cuMpSGEMM_[A-Za-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_library_exports_every_declared_symbol(cg):
    L = cg.lib()
    declared = _declared_c_symbols()
    assert len(declared) >= 50
    missing = [n for n in declared if not hasattr(L, n)]
    assert not missing, missing


def test_interposed_hipblas_symbols_are_exported(cg):
    L = cg.lib()
    for n in ("hipblasSgemm", "hipblasCgemm", "hipblasSgemmStridedBatched",
              "hipblasCgemmStridedBatched", "hipblasGemmEx", "hipblasGemmStridedBatchedEx"):
        assert hasattr(L, n), n
    out = subprocess.check_output(["nm", "-D", "--defined-only", cg.lib_path()], text=True)
    # the ILP64 variants must be left to hipBLAS
    assert "hipblasSgemm_64" not in out and "hipblasGemmEx_64" not in out
    # C++ API symbols are exported too (drop-in for C++ callers)
    assert "cumpsgemm4gemmIf" in out.replace("_ZN9", "") or "gemmIfE" in out
    rule = subprocess.check_output(["nm", "-D", "--defined-only", cg.rule_lib_path()], text=True)
    assert "cuMpSGEMM_get_compute_mode" in rule


def test_mode_strings(cg):
    want = ["CUBLAS", "FP16TCEC", "TF32TCEC", "FP16TC", "TF32TC", "CUBLAS_SIMT", "CUBLAS_FP16TC",
            "CUBLAS_TF32TC", "DRY_RUN", "AUTO", "UNDEFINED", "FP16TCEC_SCALING", "FP32_SIMT"]
    assert [cg.mode_string(i) for i in range(13)] == want
    assert cg.mode_string(13) == "Unknown" and cg.mode_string(-1) == "Unknown"


def _run(code, env_extra=None):
    env = dict(os.environ)
    env.pop("CUMPSGEMM_COMPUTE_MODE", None)
    env.update(env_extra or {})
    env["PYTHONPATH"] = ROOT
    r = subprocess.run([sys.executable, "-c", textwrap.dedent(code)], env=env, text=True,
                       capture_output=True, timeout=120)
    assert r.returncode == 0, r.stderr
    return r.stdout


RULE_PROBE = """
    import cumpsgemm_amd as cg
    q = lambda m, n, k: cg.hijack.query_compute_mode("hipblasSgemm", 111, 112, m, n, k)
    print(q(2048, 2048, 2048), q(1024, 4096, 4096), q(4096, 1024, 4096), q(4096, 4096, 1024), q(1025, 1025, 1025))
"""


@pytest.mark.parametrize("env_value,mode", [
    ("FP16TCEC", 1), ("TF32TCEC", 2), ("FP16TC", 3), ("TF32TC", 4), ("CUBLAS_SIMT", 5),
    ("CUBLAS_FP16TC", 6), ("CUBLAS_TF32TC", 7), ("DRY_RUN", 8), ("AUTO", 9),
    ("FP16TCEC_SCALING", 11), ("CUBLAS", 0)])
def test_default_rule_env_values(env_value, mode):
    out = _run(RULE_PROBE, {"CUMPSGEMM_COMPUTE_MODE": env_value}).split()
    # any dimension <= 1024 forwards to hipBLAS before the environment is read
    assert out == [str(mode), "5", "5", "5", str(mode)]


def test_default_rule_unknown_and_unset_values():
    out = _run(RULE_PROBE, {"CUMPSGEMM_COMPUTE_MODE": "FP32_SIMT"})
    assert "[cuMpSGEMM ERROR] Unknown CUMPSGEMM_COMPUTE_MODE = FP32_SIMT. Ignored" in out
    assert out.strip().splitlines()[-1].split() == ["0", "5", "5", "5", "0"]
    quiet = _run(RULE_PROBE, {"CUMPSGEMM_COMPUTE_MODE": "bogus", "CUMPSGEMM_ERROR_LOG": "0"})
    assert "ERROR" not in quiet
    unset = _run(RULE_PROBE)
    assert unset.split() == ["0", "5", "5", "5", "0"] and "ERROR" not in unset


def test_static_mode_control_precedence_and_fp32_simt():
    out = _run("""
        import cumpsgemm_amd as cg
        q = lambda: cg.hijack.query_compute_mode("hipblasCgemm", 111, 111, 64, 64, 64)
        print(q())
        cg.hijack.set_compute_mode(cg.FP16TCEC); print(q())
        cg.hijack.set_compute_mode(cg.DRY_RUN); print(q())
        cg.hijack.unset_compute_mode(); print(q())
        try:
            cg.hijack.set_compute_mode(cg.FP32_SIMT); print("no error")
        except RuntimeError as e:
            print("raised", e)
        print(cg.hijack.is_library_loaded())
    """, {"CUMPSGEMM_COMPUTE_MODE": "TF32TCEC"})
    lines = out.strip().splitlines()
    assert lines[:4] == ["5", "1", "8", "5"]
    assert lines[4].startswith("raised") and "not supported" in lines[4]
    assert lines[5] == "True"


def test_user_rule_library_replaces_default(tmp_path):
    """A libcumpsgemm_rule.so earlier on the loader path that defines
    cuMpSGEMM_get_compute_mode wins over the built-in rule; with a rule library
    lacking the symbol the built-in rule stays in force (and a warning is logged
    when warnings are enabled)."""
    src = tmp_path / "rule.c"
    src.write_text("""
        int cuMpSGEMM_get_compute_mode(const char* f, void* h, int a, int b,
                                       unsigned m, unsigned n, unsigned k) {
          return (m == 7) ? 2 : 11;  /* TF32TCEC for m == 7, else FP16TCEC_SCALING */
        }""")
    so = tmp_path / "libcumpsgemm_rule.so"
    subprocess.check_call(["gcc", "-shared", "-fPIC", "-o", str(so), str(src)])
    probe = """
        import cumpsgemm_amd as cg
        print(cg.hijack.query_compute_mode("hipblasSgemm", 111, 111, 7, 9, 9),
              cg.hijack.query_compute_mode("hipblasSgemm", 111, 111, 8, 9, 9))
        cg.hijack.set_compute_mode(cg.FP16TC)
        print(cg.hijack.query_compute_mode("hipblasSgemm", 111, 111, 7, 9, 9))
    """
    ld = str(tmp_path) + ":" + os.environ.get("LD_LIBRARY_PATH", "")
    out = _run(probe, {"LD_LIBRARY_PATH": ld}).split()
    assert out == ["2", "11", "3"]
    # shipped rule library next to libcumpsgemm.so: same answers as the built-in rule
    out = _run(probe, {"CUMPSGEMM_COMPUTE_MODE": "AUTO"}).split()
    assert out == ["5", "5", "3"]
    empty = tmp_path / "empty"
    empty.mkdir()
    (empty / "e.c").write_text("int unrelated(void) { return 0; }")
    subprocess.check_call(["gcc", "-shared", "-fPIC", "-o", str(empty / "libcumpsgemm_rule.so"), str(empty / "e.c")])
    out = _run(probe, {"LD_LIBRARY_PATH": str(empty), "CUMPSGEMM_ERROR_LOG": "1",
                       "CUMPSGEMM_COMPUTE_MODE": "AUTO"})
    assert "[cuMpSGEMM WARNING] Failed to load a function cuMpSGEMM_get_compute_mode" in out
    assert out.strip().splitlines()[-2].split() == ["5", "5"]


def test_invalid_arguments_are_rejected_without_a_gpu(cg):
    """Zero dimensions / leading dimensions return INVALID_VALUE before any GPU
    work (reference src/cumpsgemm_cublas.cu:233-235, :607-610); DRY_RUN returns
    success without touching memory (:260-262)."""
    import ctypes
    L = cg.lib()
    one = ctypes.c_float(1.0)
    L.hipblasSgemm.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                               ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                               ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int]
    for dims in ((0, 4, 4, 4, 4, 4), (4, 0, 4, 4, 4, 4), (4, 4, 0, 4, 4, 4), (4, 4, 4, 0, 4, 4),
                 (4, 4, 4, 4, 0, 4), (4, 4, 4, 4, 4, 0)):
        m, n, k, lda, ldb, ldc = dims
        st = L.hipblasSgemm(None, 111, 111, m, n, k, ctypes.byref(one), None, lda, None, ldb,
                            ctypes.byref(one), None, ldc)
        assert st == cg.STATUS_INVALID_VALUE


def test_dry_run_touches_nothing():
    out = _run("""
        import ctypes, cumpsgemm_amd as cg
        L = cg.lib()
        cg.hijack.set_compute_mode(cg.DRY_RUN)
        one = ctypes.c_float(1.0)
        L.hipblasSgemm.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                   ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                                   ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int]
        st = L.hipblasSgemm(None, 111, 112, 5, 6, 7, ctypes.byref(one), None, 5, None, 6, ctypes.byref(one), None, 5)
        print(st)
        print(cg.hijack.last_called_function_str())
    """, {"CUMPSGEMM_INFO": "1"})
    assert "[cuMpSGEMM LOG] hipblasSgemm op=(N, T), shape=(5, 6, 7), mode=DRY_RUN[static][exp_stats:0]" in out
    lines = out.strip().splitlines()
    assert lines[-2] == "0" and lines[-1] == "hipblasSgemm,N,T,5,6,7,1,DRY_RUN"


def test_missing_library_fails_loudly(tmp_path):
    code = f"""
        import sys, importlib.util, os, shutil
        dst = r"{tmp_path}/pkg/cumpsgemm_amd"
        os.makedirs(dst)
        for f in ("__init__.py", "_lib.py", "inputs.py"):
            shutil.copy(os.path.join(r"{ROOT}", "cumpsgemm_amd", f), dst)
        sys.path.insert(0, r"{tmp_path}/pkg")
        sys.modules.pop("cumpsgemm_amd", None)
        import cumpsgemm_amd as cg
        assert cg.__file__.startswith(r"{tmp_path}")
        try:
            cg.lib(); print("loaded?!")
        except RuntimeError as e:
            print("raised:", "no CPU fallback" in str(e))
    """
    env = dict(os.environ)
    r = subprocess.run([sys.executable, "-c", textwrap.dedent(code)], env=env, text=True, capture_output=True)
    assert r.returncode == 0, r.stderr
    assert r.stdout.strip() == "raised: True"


# ---- Python control module (counterpart of the reference's pybind11 module,
# python/src/main.cpp:111-173) ------------------------------------------------
CTL_PROBE = """
    import ctypes
    from cumpsgemm_amd import cumpsgemm_hijack_control as ctl
    print(ctl.is_library_loaded())
    q = ctypes.CDLL(None)
    def query(m):
        try:
            f = q.cuMpSGEMM_hijack_query_compute_mode
        except AttributeError:
            return -1
        f.argtypes = [ctypes.c_char_p, ctypes.c_int, ctypes.c_int, ctypes.c_uint, ctypes.c_uint, ctypes.c_uint]
        return f(b"hipblasSgemm", 111, 111, m, 2048, 2048)
    print(query(2048))
    ctl.set_control_function(lambda op_a, op_b, m, n, k: ctl.CUMPSGEMM_TF32TCEC if m == 4096 else ctl.CUMPSGEMM_FP16TC)
    print(query(4096), query(2048))
    ctl.set_compute_mode(ctl.CUMPSGEMM_DRY_RUN); print(query(4096))
    ctl.unset_compute_mode(); ctl.unset_control_function(); print(query(4096))
    ctl.set_last_called_function_str("abc,N,N,1,2,3,1,FP16TCEC"); print(ctl.get_last_called_function_str())
    ctl.clear_last_called_function_str(); print(repr(ctl.get_last_called_function_str()))
    ctl.enable_custom_gemm_Mx2x2(); ctl.disable_custom_gemm_Mx2x2()
    ctl.disable_restoring_AB_after_scaling(); ctl.enable_restoring_AB_after_scaling()
    ctl.enable_auto_kernel_selection(); print(ctl.is_auto_kernel_selection_enabled())
    ctl.set_global_cublas_dim_mn_threshold(256); print(ctl.get_global_cublas_dim_mn_threshold(), ctl.get_global_cublas_dim_k_threshold())
    print(int(ctl.compute_mode.CUMPSGEMM_AUTO), int(ctl.CUMPSGEMM_CUBLAS_SIMT))
"""


def test_python_control_module_without_preload_is_inert():
    out = _run(CTL_PROBE, {"CUMPSGEMM_COMPUTE_MODE": "FP16TCEC"}).strip().splitlines()
    assert out[0] == "False" and out[1] == "-1"
    assert out[2] == "-1 -1" and out[5] == "" and out[6] == "''"
    assert out[7] == "True" and out[8] == "256 64" and out[9] == "9 5"


def test_python_control_module_drives_the_preloaded_library(cg):
    preload = cg.lib_path() + (":" + os.environ["LD_PRELOAD"] if os.environ.get("LD_PRELOAD") else "")
    out = _run(CTL_PROBE, {"CUMPSGEMM_COMPUTE_MODE": "FP16TCEC", "LD_PRELOAD": preload}).strip().splitlines()
    assert out[0] == "True"
    assert out[1] == "1"               # rule: env mode for dims > 1024
    assert out[2] == "2 3"             # control function consulted per call
    assert out[3] == "8"               # a forced mode outranks it
    assert out[4] == "1"               # both removed: back to the rule
    assert out[5] == "abc,N,N,1,2,3,1,FP16TCEC" and out[6] == "''"
    assert out[7] == "True" and out[8] == "256 64" and out[9] == "9 5"


def test_bench_refuses_more_than_one_gpu():
    """The benchmark is a one-GPU program: asking for more exits with a message and no JSON line."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0
    assert "ONE GPU" in (r.stderr + r.stdout)
    assert '"metric"' not in r.stdout
