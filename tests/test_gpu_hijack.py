"""LD_PRELOAD interception of hipBLAS by libcumpsgemm.so, exercised with a
stand-alone hipBLAS client (tests/native/hijack_probe, linked against the real
libhipblas.so).  What a drop-in user does: set CUMPSGEMM_COMPUTE_MODE and
LD_PRELOAD (reference README.md:27-31)."""
import os
import re
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROBE = os.path.join(ROOT, "tests", "native", "hijack_probe")
LIB = os.path.join(ROOT, "cumpsgemm_amd", "libcumpsgemm.so")


def _probe(env_extra, preload=True):
    assert os.path.exists(PROBE), "build tests/native/hijack_probe first (make -C tests/native)"
    env = dict(os.environ)
    for k in ("CUMPSGEMM_COMPUTE_MODE", "CUMPSGEMM_INFO", "CUMPSGEMM_CUSTOM_GEMM_MX2X2"):
        env.pop(k, None)
    env.update(env_extra)
    if preload:
        env["LD_PRELOAD"] = LIB + (":" + env["LD_PRELOAD"] if env.get("LD_PRELOAD") else "")
    r = subprocess.run([PROBE], env=env, text=True, capture_output=True, timeout=300)
    assert r.returncode == 0 and "DONE" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]
    res = {m.group(1): (int(m.group(2)), float(m.group(3)))
           for m in re.finditer(r"RESULT (\S+) status=(-?\d+) relerr=(\S+)", r.stdout)}
    logs = [l for l in r.stdout.splitlines() if l.startswith("[cuMpSGEMM")]
    return res, logs


FP32_CALLS = ["hipblasSgemm", "hipblasSgemm_TN", "hipblasSgemmStridedBatched", "hipblasGemmEx_f32",
              "hipblasGemmStridedBatchedEx_f32", "hipblasCgemm_CN"]


def test_without_preload_is_plain_hipblas():
    res, logs = _probe({"CUMPSGEMM_COMPUTE_MODE": "FP16TC", "CUMPSGEMM_INFO": "1"}, preload=False)
    assert not logs
    for name in FP32_CALLS:
        assert res[name][0] == 0 and res[name][1] < 2e-6
    assert res["zero_m"][0] == 0


def test_preload_fp16tcec_keeps_fp32_accuracy_and_logs_every_call():
    base, _ = _probe({}, preload=False)
    res, logs = _probe({"CUMPSGEMM_COMPUTE_MODE": "FP16TCEC", "CUMPSGEMM_INFO": "1"})
    for name in FP32_CALLS:
        assert res[name][0] == 0
        assert res[name][1] <= 2.0 * base[name][1] + 1e-9, (name, res[name], base[name])
    assert res["zero_m"][0] == 3  # HIPBLAS_STATUS_INVALID_VALUE from the interposer
    assert res["hipblasGemmEx_f16_in"] == (0, 0.0)  # forwarded untouched
    text = "\n".join(logs)
    assert "hipblasSgemm op=(N, N), shape=(1280, 1280, 1280), mode=FP16TCEC[dynamic][exp_stats:0]" in text
    assert "hipblasSgemm op=(T, N)" in text
    assert "hipblasSgemmStridedBatched op=(N, N), shape=(1280, 1280, 1280), batch=3, mode=FP16TCEC" in text
    assert "hipblasGemmEx op=(N, N)" in text and "hipblasGemmStridedBatchedEx op=(N, N)" in text
    # the complex call is 640^3: the default rule sends small problems to hipBLAS
    assert "hipblasCgemm op=(C, N), shape=(640, 640, 640), mode=CUBLAS_SIMT" in text


def test_preload_uncorrected_mode_is_really_in_the_path():
    res, _ = _probe({"CUMPSGEMM_COMPUTE_MODE": "FP16TC"})
    for name in ("hipblasSgemm", "hipblasSgemm_TN", "hipblasSgemmStridedBatched", "hipblasGemmEx_f32"):
        assert 1e-5 < res[name][1] < 2e-3  # fp16-level error: our kernel ran, not hipBLAS
    assert res["hipblasCgemm_CN"][1] < 2e-6  # small problem: forwarded


@pytest.mark.parametrize("mode", ["TF32TCEC", "FP16TCEC_SCALING", "AUTO"])
def test_preload_other_modes(mode):
    base, _ = _probe({}, preload=False)
    res, logs = _probe({"CUMPSGEMM_COMPUTE_MODE": mode, "CUMPSGEMM_INFO": "1"})
    for name in FP32_CALLS:
        assert res[name][0] == 0 and res[name][1] <= 2.0 * base[name][1] + 1e-9
    assert any(f"mode={mode}" in l for l in logs)


def test_device_pointer_mode_calls_are_forwarded():
    """alpha / beta in device memory (HIPBLAS_POINTER_MODE_DEVICE): the TCEC entry points read
    them on the host, so the interposer hands such a call to hipBLAS instead of faulting."""
    res, logs = _probe({"CUMPSGEMM_COMPUTE_MODE": "FP16TC", "CUMPSGEMM_INFO": "1", "CUMPSGEMM_ERROR_LOG": "1"})
    assert res["hipblasSgemm"][0] == 0 and res["hipblasSgemm"][1] > 1e-5       # our fp16 kernel
    st, err = res["hipblasSgemm_device_scalars"]
    assert st == 0 and err < 2e-6                                               # hipBLAS FP32
    text = "\n".join(logs)
    assert "[cuMpSGEMM WARNING] alpha / beta are in device memory" in text
    assert "forwarded to hipBLAS (device pointer mode)" in text


def test_preload_dry_run_leaves_c_untouched():
    res, logs = _probe({"CUMPSGEMM_COMPUTE_MODE": "DRY_RUN", "CUMPSGEMM_INFO": "1"})
    assert res["hipblasSgemm"] == (0, 1.0)  # C stayed zero: relative error exactly 1
    assert any("mode=DRY_RUN" in l for l in logs)


def test_culip_profiling_lines():
    """CUMPSGEMM_ENABLE_CULIP_PROFILING prints one '[CULiP Result][label] Nns'
    line per intercepted call, labels as in the reference
    (src/cumpsgemm_cublas.cu:430-441, :812-822, :393-398; src/culip.cu:19-33)."""
    assert os.path.exists(PROBE)
    env = dict(os.environ)
    env.update({"CUMPSGEMM_COMPUTE_MODE": "FP16TCEC", "CUMPSGEMM_ENABLE_CULIP_PROFILING": "1"})
    env["LD_PRELOAD"] = LIB + (":" + env["LD_PRELOAD"] if env.get("LD_PRELOAD") else "")
    r = subprocess.run([PROBE], env=env, text=True, capture_output=True, timeout=300)
    assert r.returncode == 0 and "DONE" in r.stdout
    lines = re.findall(r"^\[CULiP Result\]\[(\S+)\] (\d+)ns$", r.stdout, flags=re.M)
    labels = [l for l, _ in lines]
    assert "sgemm_FP16TCEC-NN-m1280-n1280-k1280" in labels
    assert "sgemm_FP16TCEC-TN-m1280-n1280-k1280" in labels
    assert "sgemm_stridedBatch_FP16TCEC-NN-m1280-n1280-k1280-batchCount3" in labels
    assert "hipblasCgemm-CN-m640-n640-k640" in labels  # forwarded call: the symbol's own name
    assert all(int(ns) > 0 for _, ns in lines)
    # off by default and with "0"
    env["CUMPSGEMM_ENABLE_CULIP_PROFILING"] = "0"
    r0 = subprocess.run([PROBE], env=env, text=True, capture_output=True, timeout=300)
    assert "[CULiP Result]" not in r0.stdout


def test_host_threads_with_their_own_streams_share_the_interposer():
    """Four host threads, each with its own hipBLAS handle and stream, call the intercepted
    hipblasSgemm at the same time (shapes large enough for the pre-split path and its shared
    workspace): every result equals the one computed alone."""
    res, _ = _probe({"CUMPSGEMM_COMPUTE_MODE": "FP16TCEC", "PROBE_THREADS": "4", "PROBE_N": "4096"})
    assert res["threads"] == (0, 0.0)


CPLX_CALLS = ["hipblasCgemm_CN", "hipblasCgemmStridedBatched", "hipblasGemmEx_c32", "hipblasGemmStridedBatchedEx_c32"]


def test_complex_entry_points_reach_the_tcec_kernels():
    """With 1100 x 1100 complex matrices (every dimension above the default rule's 1024) the four
    complex entry points are served by this library and keep complex64 accuracy."""
    base, _ = _probe({"PROBE_N": "2200"}, preload=False)
    res, logs = _probe({"CUMPSGEMM_COMPUTE_MODE": "FP16TCEC", "CUMPSGEMM_INFO": "1", "PROBE_N": "2200"})
    text = "\n".join(logs)
    for name in CPLX_CALLS:
        assert res[name][0] == 0 and base[name][0] == 0
        assert res[name][1] <= 2.0 * base[name][1] + 1e-9 and res[name][1] < 2.0 ** -23 * 1100 ** 0.5, (name, res[name])
    assert "hipblasCgemm op=(C, N), shape=(1100, 1100, 1100), mode=FP16TCEC" in text
    assert "hipblasCgemmStridedBatched op=(N, N), shape=(1100, 1100, 1100), batch=2, mode=FP16TCEC" in text
    assert text.count("hipblasGemmEx op=(N, N), shape=(1100, 1100, 1100), mode=FP16TCEC") == 1
    assert "hipblasGemmStridedBatchedEx op=(N, N), shape=(1100, 1100, 1100), batch=2, mode=FP16TCEC" in text


def test_gate_shapes_take_the_streaming_kernels_when_enabled():
    """M x 2 x 2 and 2 x N x 2 products (M, N powers of two) go to the dedicated streaming kernels
    when CUMPSGEMM_CUSTOM_GEMM_MX2X2 is set (reference src/cumpsgemm_cublas.cu:269-338), whatever
    the compute mode; otherwise the rule decides (small dimensions: hipBLAS)."""
    res, logs = _probe({"CUMPSGEMM_CUSTOM_GEMM_MX2X2": "1", "CUMPSGEMM_INFO": "1", "PROBE_MX2X2": "1"})
    text = "\n".join(logs)
    assert res["cgemm_Mx2x2"][0] == 0 and res["cgemm_Mx2x2"][1] < 2e-7
    assert res["sgemm_2xNx2"][0] == 0 and res["sgemm_2xNx2"][1] < 2e-7
    assert " +---> gemm_Mx2x2" in text and " +---> gemm_2xNx2" in text
    res, logs = _probe({"CUMPSGEMM_INFO": "1", "PROBE_MX2X2": "1"})
    text = "\n".join(logs)
    assert res["cgemm_Mx2x2"][0] == 0 and res["cgemm_Mx2x2"][1] < 2e-7 and res["sgemm_2xNx2"][1] < 2e-7
    assert "gemm_Mx2x2" not in text and "shape=(262144, 2, 2), mode=CUBLAS_SIMT" in text
