"""The C++ API as a C++ user sees it: tests/native/api_probe.cpp is compiled
against include/cumpsgemm/*.hpp and linked with libcumpsgemm.so (templates,
std::pair returns, optional module-id out-parameter), then run on the GPU."""
import os
import re
import subprocess

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROBE = os.path.join(ROOT, "tests", "native", "api_probe")


def test_cpp_api_client():
    assert os.path.exists(PROBE), "build tests/native/api_probe first (make -C tests/native)"
    r = subprocess.run([PROBE], text=True, capture_output=True, timeout=300)
    assert r.returncode == 0 and "DONE" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]
    res = dict(re.findall(r"RESULT (\S+) (\S+)", r.stdout))
    assert res["sgemm_status"] == "0" and float(res["sgemm_relerr"]) < 2.0 ** -23 * 170 ** 0.5
    assert res["sgemm_module"] in ("0", "1", "2")                 # a tile class, as in the reference
    assert res["cgemm_batch_status"] == "0" and float(res["cgemm_batch_relerr"]) < 2.0 ** -23 * 72 ** 0.5
    assert res["stats_max_ok"] == "1"
    # |x| <= 0.01 with a seventh of the entries near 1e-6: stage 1 sees underflow, stage 2
    # (relative thresholds) decides; either way every non-zero entry is counted
    assert res["stats_level"] in ("2", "11") and int(res["stats_total"]) > 0
    assert res["flag_mode"] in ("1", "2")
    assert res["scale_roundtrip"] == "1"
    assert (res["scale_applied"] == "1") == (res["flag_scale"][0] == "1")
