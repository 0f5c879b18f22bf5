"""Known-answer fixtures of tests/golden/ (written by tests/golden/make_golden.py
from numpy's binary16 type, Python integer arithmetic and a scalar Python loop
-- no oracle, no library) against the oracle on the CPU and against the HIP
path on the GPU.  The reference itself holds no golden vectors for this path."""
import json
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
N, T = 111, 112
ALL_GEMM_MODES = [1, 2, 3, 4]  # FP16TCEC, TF32TCEC (bf16x3), FP16TC, TF32TC (bf16x2)


def _load(name):
    with open(os.path.join(GOLDEN, name)) as f:
        return json.load(f)


# ---- CPU: pins the oracle -------------------------------------------------------
def test_oracle_fp16_conversion_known_answers(O):
    g = _load("fp16_convert_kat.json")
    x = np.array(g["f32_bits"], dtype=np.uint32).view(np.float32)
    want = np.array(g["f16_bits"], dtype=np.uint16)
    got = O.f32_to_f16_bits(x)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all((got[nan] & 0x7c00) == 0x7c00) and np.all((got[nan] & 0x03ff) != 0)


def test_oracle_split_known_answers(O):
    g = _load("fp16_split_kat.json")
    a = np.array(g["a_bits"], dtype=np.uint32).view(np.float32)
    hi, lo = O.split_fp16(a)  # returned widened to fp32
    want_hi = np.array(g["hi_bits"], dtype=np.uint16).view(np.float16).astype(np.float32)
    want_lo = np.array(g["lo_bits"], dtype=np.uint16).view(np.float16).astype(np.float32)
    assert np.array_equal(hi.view(np.uint32), want_hi.view(np.uint32))
    assert np.array_equal(lo.view(np.uint32), want_lo.view(np.uint32))


def _exact_case_arrays(case):
    f = lambda v: np.array(v, dtype=np.float32)
    return f(case["a"]), f(case["b"]), f(case["c0"]), f(case["c"])


@pytest.mark.parametrize("mode", ALL_GEMM_MODES + [12])
def test_oracle_exact_gemms(O, mode):
    for case in _load("gemm_exact_kat.json")["cases"]:
        a, b, c0, want = _exact_case_arrays(case)
        opa, opb = (N if case["opa"] == "N" else T), (N if case["opb"] == "N" else T)
        c = c0.copy()
        O.gemm(mode, opa, opb, case["m"], case["n"], case["k"], float(case["alpha"]), a, case["lda"], b,
               case["ldb"], float(case["beta"]), c, case["m"])
        assert np.array_equal(c, want)


_OPS = {"N": 111, "T": 112, "C": 113}


def _exact_ccase_arrays(case):
    f = lambda v: np.array(v, dtype=np.float32).view(np.complex64)
    return f(case["a"]), f(case["b"]), f(case["c0"]), f(case["c"])


@pytest.mark.parametrize("mode", ALL_GEMM_MODES + [12])
def test_oracle_exact_complex_gemms(O, mode):
    """All nine op pairs with complex alpha and beta and padded leading dimensions: pins the
    oracle's complex epilogue (reference src/device_common.hpp:47-67) and its conjugation."""
    cases = _load("cgemm_exact_kat.json")["cases"]
    assert sorted(c["opa"] + c["opb"] for c in cases) == sorted(x + y for x in "NTC" for y in "NTC")
    for case in cases:
        a, b, c0, want = _exact_ccase_arrays(case)
        c = c0.copy()
        O.gemm(mode, _OPS[case["opa"]], _OPS[case["opb"]], case["m"], case["n"], case["k"], complex(*case["alpha"]),
               a, case["lda"], b, case["ldb"], complex(*case["beta"]), c, case["ldc"])
        assert np.array_equal(c.view(np.float32), want.view(np.float32)), (case["opa"], case["opb"])


def test_oracle_exp_stats_known_answers(O):
    for case in _load("exp_stats_kat.json")["cases"]:
        x = np.array(case["bits"], dtype=np.uint32).view(np.float32)
        got = O.exp_stats(x, len(x), 1, len(x), ignore=case["ignore_threshold"],
                          underflow=case["underflow_threshold"], tol=case["tolerance"])
        e = case["expect"]
        assert (got.max_exp_bits, got.total, got.underflow, got.mode, bool(got.stage2_ran)) == \
            (e["max_exp_bits"], e["total"], e["underflow"], e["mode"], e["stage2"]), case["name"]
        assert O.exp_max_bits(x, len(x), 1, len(x)) == e["max_exp_bits"]


# ---- GPU: the HIP path against the same fixtures -----------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("mode", ALL_GEMM_MODES)
def test_gpu_exact_gemms(handle, dev, mode):
    for case in _load("gemm_exact_kat.json")["cases"]:
        a, b, c0, want = _exact_case_arrays(case)
        opa, opb = (N if case["opa"] == "N" else T), (N if case["opb"] == "N" else T)
        da, db, dc = dev.up(a), dev.up(b), dev.up(c0)
        st = handle.gemm(opa, opb, case["m"], case["n"], case["k"], float(case["alpha"]), da, case["lda"], db,
                         case["ldb"], float(case["beta"]), dc, case["m"], mode)
        assert st == 0
        assert np.array_equal(dev.down(dc), want)


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ALL_GEMM_MODES)
def test_gpu_exact_complex_gemms(handle, dev, mode):
    for case in _load("cgemm_exact_kat.json")["cases"]:
        a, b, c0, want = _exact_ccase_arrays(case)
        da, db, dc = dev.up(a), dev.up(b), dev.up(c0)
        st = handle.gemm(_OPS[case["opa"]], _OPS[case["opb"]], case["m"], case["n"], case["k"],
                         complex(*case["alpha"]), da, case["lda"], db, case["ldb"], complex(*case["beta"]), dc,
                         case["ldc"], mode, cplx=True)
        assert st == 0
        got = dev.down(dc, np.complex64)
        assert np.array_equal(got.view(np.float32), want.view(np.float32)), (case["opa"], case["opb"])


@pytest.mark.gpu
def test_gpu_exp_stats_known_answers(handle, dev):
    try:
        for case in _load("exp_stats_kat.json")["cases"]:
            x = np.array(case["bits"], dtype=np.uint32).view(np.float32)
            handle.set_exp_stats_params(case["ignore_threshold"], case["underflow_threshold"], case["tolerance"])
            d = dev.up(x)
            sid = handle.exp_stats_ext(len(x), 1, d, len(x))
            under, total = handle.get_exp_stats(sid)
            e = case["expect"]
            bits = int(np.float32(handle.get_max_exp(sid)).view(np.uint32))
            assert (bits, total, under, handle.get_exp_stats_compute_mode_level(sid)) == \
                (e["max_exp_bits"], e["total"], e["underflow"], e["mode"]), case["name"]
            mid = handle.exp_max_ext(len(x), 1, d, len(x))
            assert int(np.float32(handle.get_max_exp(mid)).view(np.uint32)) == e["max_exp_bits"]
    finally:
        handle.set_exp_stats_params(0.0, 2.0 ** -15, 0.0)
