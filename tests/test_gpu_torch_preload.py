"""A PyTorch program run with the library preloaded: torch.matmul / bmm on
float32 and complex64 reach hipblasSgemm / hipblasSgemmStridedBatched /
hipblasCgemm, the interposer serves them in the mode chosen through the Python
control module, and the results are right.  Counterpart of the reference's
CuPy script (test/cupy/main.py) and of its Python module's use
(python/src/main.cpp:111-173) on ROCm.

The child is a separate process because LD_PRELOAD only acts at program start.
PyTorch ships its own copy of the HIP runtime; naming that copy first in
LD_PRELOAD makes the preloaded library bind to it, so the process has one
runtime."""
import importlib.util
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CHILD = r'''
import os, sys
sys.path.insert(0, os.getcwd())
import torch
torch.backends.cuda.preferred_blas_library("cublas")      # hipBLAS rather than hipBLASLt
from cumpsgemm_amd import cumpsgemm_hijack_control as ctl
assert ctl.is_library_loaded()
dev = torch.device("cuda:0")
torch.manual_seed(0)

def rel(c, ref):
    return (torch.linalg.norm(c.to(ref.dtype) - ref) / torch.linalg.norm(ref)).item()

n = 1536
a = torch.randn(n, n, device=dev); b = torch.randn(n, n, device=dev)
ref = a.double() @ b.double()
for name in ("FP16TCEC", "TF32TCEC", "FP16TC", "TF32TC", "CUBLAS"):
    ctl.set_compute_mode(getattr(ctl, "CUMPSGEMM_" + name))
    c = a @ b
    torch.cuda.synchronize()
    print("RESULT sgemm", name, "%.3e" % rel(c, ref), ctl.get_last_called_function_str(), flush=True)

# transposed operands arrive as op flags, not as copies
ctl.set_compute_mode(ctl.CUMPSGEMM_FP16TCEC)
c = a.t() @ b
torch.cuda.synchronize()
print("RESULT sgemm_t FP16TCEC", "%.3e" % rel(c, a.double().t() @ b.double()), ctl.get_last_called_function_str(), flush=True)

x = torch.randn(6, 1280, 1280, device=dev); y = torch.randn(6, 1280, 1280, device=dev)
z = torch.bmm(x, y)
torch.cuda.synchronize()
print("RESULT bmm FP16TCEC", "%.3e" % rel(z, x.double() @ y.double()), ctl.get_last_called_function_str(), flush=True)

ca = torch.randn(1100, 1100, device=dev, dtype=torch.complex64)
cb = torch.randn(1100, 1100, device=dev, dtype=torch.complex64)
cc = ca @ cb
torch.cuda.synchronize()
print("RESULT cgemm FP16TCEC", "%.3e" % rel(cc, ca.to(torch.complex128) @ cb.to(torch.complex128)),
      ctl.get_last_called_function_str(), flush=True)

# AUTO on operands far below fp16's range: plain FP16TCEC would lose them, AUTO must not
ctl.set_compute_mode(ctl.CUMPSGEMM_AUTO)
s = a * 1e-7
c = s @ b
torch.cuda.synchronize()
print("RESULT auto AUTO", "%.3e" % rel(c, s.double() @ b.double()), ctl.get_last_called_function_str(), flush=True)
assert torch.equal(s, a * 1e-7)                             # operands are left as they were

# a control function decides per call; small problems go to the vendor GEMM
ctl.unset_compute_mode()
ctl.set_control_function(lambda op_a, op_b, m, n, k: ctl.CUMPSGEMM_TF32TCEC if m >= 1024 else ctl.CUMPSGEMM_CUBLAS)
c = a @ b
torch.cuda.synchronize()
print("RESULT ctl_big -", "%.3e" % rel(c, ref), ctl.get_last_called_function_str(), flush=True)
t = a[:256, :256].contiguous() @ b[:256, :256].contiguous()
torch.cuda.synchronize()
print("RESULT ctl_small -", "%.3e" % rel(t, a[:256, :256].double() @ b[:256, :256].double()),
      ctl.get_last_called_function_str(), flush=True)
ctl.unset_control_function()

# statistics of the result of forwarded calls, switched on through the library's own handle
# (reference src/cumpsgemm_cublas.cu:420-425; hijack_control.hpp get_internal_global_handle)
import ctypes
P = ctypes.CDLL(None)
P.cuMpSGEMM_hijack_get_internal_global_handle.restype = ctypes.c_void_p
hd = ctypes.c_void_p(P.cuMpSGEMM_hijack_get_internal_global_handle())
P.cuMpSGEMM_enable_exp_stats.argtypes = [ctypes.c_void_p]
P.cuMpSGEMM_disable_exp_stats.argtypes = [ctypes.c_void_p]
P.cuMpSGEMM_get_current_exp_stats_buffer_id.argtypes = [ctypes.c_void_p]
P.cuMpSGEMM_get_current_exp_stats_buffer_id.restype = ctypes.c_uint
P.cuMpSGEMM_get_exp_stats.argtypes = [ctypes.c_void_p, ctypes.c_uint, ctypes.POINTER(ctypes.c_uint64),
                                      ctypes.POINTER(ctypes.c_uint64)]
P.cuMpSGEMM_get_max_exp.argtypes = [ctypes.c_void_p, ctypes.c_uint]
P.cuMpSGEMM_get_max_exp.restype = ctypes.c_float
P.cuMpSGEMM_enable_exp_stats(hd)
ctl.set_compute_mode(ctl.CUMPSGEMM_CUBLAS)
before = P.cuMpSGEMM_get_current_exp_stats_buffer_id(hd)
c = a @ b
torch.cuda.synchronize()
after = P.cuMpSGEMM_get_current_exp_stats_buffer_id(hd)
u, t = ctypes.c_uint64(0), ctypes.c_uint64(0)
P.cuMpSGEMM_get_exp_stats(hd, after, ctypes.byref(u), ctypes.byref(t))
mx = P.cuMpSGEMM_get_max_exp(hd, after)
want_max = 2.0 ** torch.floor(torch.log2(c.abs().max())).item()
small = int((c.abs() < 2.0 ** -15).sum().item())
if small > 0:   # zero tolerance: the second pass recounts against 2^-16 x the maximum exponent
    small = int((c.abs() < 2.0 ** -16 * want_max).sum().item())
print("RESULT cstats -", "%.3e" % 0.0, "%d %d %d %d %d %g %g" % (before, after, u.value, t.value, small, mx, want_max), flush=True)
P.cuMpSGEMM_disable_exp_stats(hd)
'''


@pytest.mark.gpu
def test_torch_matmul_is_served_by_the_preloaded_library(cg, torch_gpu):
    torch_lib = os.path.join(os.path.dirname(importlib.util.find_spec("torch").origin), "lib")
    preload = [os.path.join(torch_lib, "libamdhip64.so"), cg.lib_path()]
    env = dict(os.environ)
    if env.get("LD_PRELOAD"):
        preload.insert(0, env["LD_PRELOAD"])  # keep what the environment already preloads
    env["LD_PRELOAD"] = " ".join(preload)
    env["CUMPSGEMM_INFO"] = "1"
    env.pop("CUMPSGEMM_COMPUTE_MODE", None)
    r = subprocess.run([sys.executable, "-c", CHILD], env=env, cwd=ROOT, capture_output=True, text=True,
                       timeout=110)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    res = {}
    for ln in r.stdout.splitlines():
        m = re.match(r"RESULT (\w+) (\S+) (\S+) (.*)$", ln)
        if m:
            res[(m.group(1), m.group(2))] = (float(m.group(3)), m.group(4))
    out = r.stdout
    bar = 2.0 ** -23 * 1536 ** 0.5           # the reference's bar for the corrected modes
    for mode in ("FP16TCEC", "TF32TCEC"):
        err, last = res[("sgemm", mode)]
        assert err < bar and last == f"hipblasSgemm,N,N,1536,1536,1536,1,{mode}", out
    for mode in ("FP16TC", "TF32TC"):
        err, last = res[("sgemm", mode)]
        # no correction terms: clearly less accurate than the corrected modes, within the reference's bar
        assert 4 * res[("sgemm", "FP16TCEC")][0] < err < 2.0 ** -10 * 1536 ** 0.5 and last.endswith(mode), out
    assert res[("sgemm", "CUBLAS")][0] < 3e-6 and res[("sgemm", "CUBLAS")][1].endswith("CUBLAS"), out
    # a row-major torch matmul is the column-major product with the operands swapped, so a.t()
    # shows up as an op flag on the second operand
    err, last = res[("sgemm_t", "FP16TCEC")]
    assert err < bar and re.fullmatch(r"hipblasSgemm,[NT],[NT],1536,1536,1536,1,FP16TCEC", last) \
        and last != "hipblasSgemm,N,N,1536,1536,1536,1,FP16TCEC", out
    err, last = res[("bmm", "FP16TCEC")]
    assert err < 2.0 ** -23 * 1280 ** 0.5 and last == "hipblasSgemmStridedBatched,N,N,1280,1280,1280,6,FP16TCEC", out
    err, last = res[("cgemm", "FP16TCEC")]
    assert err < 2.0 ** -23 * 1100 ** 0.5 and last == "hipblasCgemm,N,N,1100,1100,1100,1,FP16TCEC", out
    err, last = res[("auto", "AUTO")]
    assert err < bar and last.startswith("hipblasSgemm,N,N,1536,1536,1536,1,"), out
    assert re.search(r"mode=AUTO\[static\]", out), out
    err, last = res[("ctl_big", "-")]
    assert err < bar and last.endswith("TF32TCEC"), out
    err, last = res[("ctl_small", "-")]
    assert err < 3e-6 and last == "hipblasSgemm,N,N,256,256,256,1,CUBLAS", out
    assert "[cuMpSGEMM LOG] hipblasSgemm op=(N, N), shape=(1536, 1536, 1536), mode=FP16TCEC[static]" in out, out
    # statistics of C after a forwarded call: one new slot, every element counted, the small ones found
    before, after, under, total, small, mx, want_max = res[("cstats", "-")][1].split()
    assert int(after) == int(before) + 1 and int(total) == 1536 * 1536 and int(under) == int(small)
    assert float(mx) == float(want_max)
    assert "mode=CUBLAS[static][exp_stats:1]" in out, out
