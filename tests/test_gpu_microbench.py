"""The micro-benchmarks under tests/native/microbench (the measurements behind the MFMA shape, the
LDS swizzle of the pre-split planes and the placement of the write-out's stores) build and run:
short runs, checked for a clean exit and plausible figures."""
import os
import re
import subprocess

import pytest

pytestmark = pytest.mark.gpu
DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "native", "microbench")


def _run(name, *args):
    exe = os.path.join(DIR, name)
    assert os.path.exists(exe), f"build {exe} first (make -C tests/native)"
    r = subprocess.run([exe, *args], text=True, capture_output=True, timeout=120)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    return r.stdout


def test_mfma_shapes_runs():
    out = _run("mfma_shapes", "200")
    rates = {(d, s): float(v) for d, s, v in re.findall(r"^(uniform\S*|zeros)\s+(\S+)\s+\S+ us\s+(\S+) TFLOP/s", out, re.M)}
    assert "status no error" in out and len(rates) == 4
    # no MFMA rate above the part's dense fp16 peak, none implausibly low
    assert all(100.0 < v < 2600.0 for v in rates.values()), rates


def test_lds_swizzle_runs():
    assert "status no error" in _run("lds_swizzle")


def test_stores_beside_mfma_runs():
    out = _run("stores_beside_mfma", "100", "4")
    assert "status ok" in out and out.count("mfma only") == 3
