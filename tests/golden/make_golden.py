#!/usr/bin/env python3
"""Writes the known-answer fixtures of this directory.

The reference ships no golden vectors for this path (its tests generate data
at run time and compare against thresholds), so the fixtures pin the oracle
against independent implementations instead: numpy's IEEE binary16 type for the
conversions and the hi/lo split, plain Python integer arithmetic for GEMMs whose
result is exact, and a scalar Python loop over bit patterns for the exponent
statistics (counting rules of reference src/exp_stats.cu:32-62, decisions
:175-183 and :287-292).  Nothing here imports the oracle or the library.

    python tests/golden/make_golden.py        # rewrites the .json files
"""
import json
import os
import struct

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def f32_bits(x):
    return struct.unpack("<I", struct.pack("<f", x))[0]


def bits_f32(b):
    return struct.unpack("<f", struct.pack("<I", b & 0xffffffff))[0]


def edge_bit_patterns():
    pats = set()
    for e in list(range(0, 8)) + list(range(96, 146)) + [254, 255]:
        for m in (0, 1, 0x000fff, 0x001000, 0x001001, 0x002fff, 0x003000, 0x7fe000, 0x7fefff, 0x7ff000,
                  0x7ff001, 0x7fffff, 0x400000, 0x555555):
            for s in (0, 1):
                pats.add((s << 31) | (e << 23) | m)
    return sorted(pats)


def make_convert():
    pats = np.array(edge_bit_patterns(), dtype=np.uint32)
    with np.errstate(over="ignore"):
        h = pats.view(np.float32).astype(np.float16).view(np.uint16)
    return {"comment": "fp32 bit pattern -> fp16 bit pattern, round to nearest even (numpy float16); NaN entries "
                       "only require a NaN back",
            "f32_bits": [int(x) for x in pats], "f16_bits": [int(x) for x in h]}


def make_split():
    rng = np.random.default_rng(20240607)
    vals = np.concatenate([
        rng.uniform(-1, 1, 400).astype(np.float32),
        (rng.uniform(1, 2, 200) * 2.0 ** rng.integers(-24, 16, 200)).astype(np.float32),
        np.array([0.0, -0.0, 1.0, -1.0, 65504.0, 65519.996, 2.0 ** -14, 2.0 ** -24, 2.0 ** -25, 1.0 + 2.0 ** -11,
                  1.0 + 2.0 ** -10, 1.0 + 2.0 ** -12, 0.1, 1.0 / 3.0, 12345.678], dtype=np.float32)])
    hi = vals.astype(np.float16)
    r = (vals - hi.astype(np.float32)).astype(np.float32)          # exact in fp32
    lo = (r * np.float32(2048.0)).astype(np.float32).astype(np.float16)
    return {"comment": "hi = fp16(a); lo = fp16((a - fp32(hi)) * 2^11), evaluated with numpy float16/float32",
            "a_bits": [int(x) for x in vals.view(np.uint32)],
            "hi_bits": [int(x) for x in hi.view(np.uint16)],
            "lo_bits": [int(x) for x in lo.view(np.uint16)]}


def make_exact_gemm():
    """Operands with few significant bits and small exponents: every product and
    every partial sum is exactly representable, so any correct evaluation order in
    any of the emulation modes returns exactly the integer result."""
    rng = np.random.default_rng(7)
    cases = []
    for (m, n, k, opa, opb) in [(5, 4, 7, "N", "N"), (33, 17, 40, "T", "N"), (64, 64, 64, "N", "T"), (70, 3, 129, "T", "T")]:
        A = rng.integers(-8, 9, (m, k))
        B = rng.integers(-8, 9, (k, n))
        C0 = rng.integers(-4, 5, (m, n))
        alpha, beta = 2, -1
        C = alpha * (A @ B) + beta * C0
        a_mem = A if opa == "N" else A.T      # column-major storage of the stored operand
        b_mem = B if opb == "N" else B.T
        cases.append({"m": m, "n": n, "k": k, "opa": opa, "opb": opb, "alpha": alpha, "beta": beta,
                      "a": a_mem.flatten(order="F").tolist(), "lda": a_mem.shape[0],
                      "b": b_mem.flatten(order="F").tolist(), "ldb": b_mem.shape[0],
                      "c0": C0.flatten(order="F").tolist(), "c": C.flatten(order="F").tolist()})
    return {"comment": "small-integer GEMMs, column-major flat buffers, exact expected C = alpha*op(A)*op(B)+beta*C0",
            "cases": cases}


def make_exact_cgemm():
    """Gaussian-integer CGEMMs: every real product and partial sum is a small integer, so the
    result is exact in every emulation mode and in any order.  All nine (op A, op B) pairs,
    complex alpha and beta, leading dimensions larger than the matrices (and odd).  Computed
    with Python integers: re/im parts are kept apart, no floating point is involved."""
    rng = np.random.default_rng(11)
    shapes = [(5, 4, 7), (33, 17, 40), (64, 32, 64), (19, 70, 129), (40, 3, 33), (7, 9, 16), (65, 66, 35),
              (12, 12, 200), (31, 2, 64)]
    cases = []
    idx = 0
    for opa in "NTC":
        for opb in "NTC":
            m, n, k = shapes[idx]
            idx += 1
            Ar, Ai = rng.integers(-8, 9, (m, k)), rng.integers(-8, 9, (m, k))
            Br, Bi = rng.integers(-8, 9, (k, n)), rng.integers(-8, 9, (k, n))
            Cr, Ci = rng.integers(-4, 5, (m, n)), rng.integers(-4, 5, (m, n))
            (ar, ai), (br, bi) = [(2, -1), (-1, 2), (0, 3)][idx % 3], [(-1, 2), (3, 0), (1, 1)][idx % 3]
            # logical product with Python integers
            Pr = [[sum(int(Ar[i, p]) * int(Br[p, j]) - int(Ai[i, p]) * int(Bi[p, j]) for p in range(k))
                   for j in range(n)] for i in range(m)]
            Pi = [[sum(int(Ar[i, p]) * int(Bi[p, j]) + int(Ai[i, p]) * int(Br[p, j]) for p in range(k))
                   for j in range(n)] for i in range(m)]
            Er = [[ar * Pr[i][j] - ai * Pi[i][j] + br * int(Cr[i, j]) - bi * int(Ci[i, j]) for j in range(n)]
                  for i in range(m)]
            Ei = [[ar * Pi[i][j] + ai * Pr[i][j] + br * int(Ci[i, j]) + bi * int(Cr[i, j]) for j in range(n)]
                  for i in range(m)]

            def stored(Xr, Xi, op):
                # what sits in memory so that op(stored) is the logical operand
                if op == "N":
                    return Xr, Xi
                if op == "T":
                    return Xr.T, Xi.T
                return Xr.T, -Xi.T      # C: conjugate transpose

            def flat(Xr, Xi, ld):
                rows, cols = Xr.shape
                out = [0] * (2 * ld * cols)
                for j in range(cols):
                    for i in range(ld):
                        if i < rows:
                            out[2 * (i + j * ld)] = int(Xr[i, j])
                            out[2 * (i + j * ld) + 1] = int(Xi[i, j])
                        else:               # padding rows: a value that must never be used
                            out[2 * (i + j * ld)] = 99
                            out[2 * (i + j * ld) + 1] = -99
                return out
            sar, sai = stored(Ar, Ai, opa)
            sbr, sbi = stored(Br, Bi, opb)
            lda, ldb, ldc = sar.shape[0] + 3, sbr.shape[0] + 1, m + 1 + 2 * (m % 2)
            c0 = flat(Cr, Ci, ldc)
            c = flat(np.array(Er), np.array(Ei), ldc)
            cases.append({"m": m, "n": n, "k": k, "opa": opa, "opb": opb, "alpha": [ar, ai], "beta": [br, bi],
                          "a": flat(sar, sai, lda), "lda": lda, "b": flat(sbr, sbi, ldb), "ldb": ldb,
                          "c0": c0, "c": c, "ldc": ldc})
    return {"comment": "Gaussian-integer CGEMMs, column-major interleaved (re, im) flat buffers with padded leading "
                       "dimensions (padding rows hold 99 - 99i and must come back untouched in C); exact expected "
                       "C = alpha*op(A)*op(B) + beta*C0 from Python integer arithmetic",
            "cases": cases}


def stats_bruteforce(bits, ignore_thr, under_thr, tol):
    """Scalar restatement over bit patterns; returns the record a statistics
    pass leaves behind."""
    FP16TCEC, SCALING, TF32TCEC, UNDEFINED = 1, 11, 2, 0
    vals = [bits_f32(b) for b in bits]
    mx = 0.0
    for v in vals:
        av = abs(v)
        if av == av and av > mx:      # NaN is ignored by fmaxf
            mx = av
    max_bits = f32_bits(mx) & 0x7f800000
    max_exp = bits_f32(max_bits)

    def count(it, ut):
        total = under = 0
        for v in vals:
            av = abs(v)
            if av >= it:              # false for NaN
                total += 1
                if av < ut:
                    under += 1
        return total, under
    total, under = count(ignore_thr, under_thr)
    f = lambda x: float(np.float32(x))
    if f(under) > f(np.float32(total) * np.float32(tol)) or (max_exp > 0 and total == 0):
        it2 = float(np.float32(np.float32(ignore_thr / 2) * np.float32(max_exp)))
        ut2 = float(np.float32(np.float32(under_thr / 2) * np.float32(max_exp)))
        total, under = count(it2, ut2)
        mode = SCALING if f(under) <= f(np.float32(total) * np.float32(tol)) else TF32TCEC
        stage2 = True
    else:
        mode, stage2 = FP16TCEC, False
    return {"max_exp_bits": max_bits, "total": total, "underflow": under, "mode": mode, "stage2": stage2}


def make_stats():
    rng = np.random.default_rng(99)
    mats = {
        "zeros": [0] * 24,
        "unit_range": [f32_bits(x) for x in rng.uniform(0.25, 1.0, 60).astype(np.float32)],
        "tiny": [f32_bits(x) for x in (rng.uniform(0.5, 1.0, 60) * 2.0 ** -20).astype(np.float32)],
        "wide": [f32_bits(x) for x in (rng.uniform(1, 2, 80) * 2.0 ** rng.integers(-30, 31, 80)).astype(np.float32)],
        "one_huge": [f32_bits(1e30)] + [f32_bits(x) for x in rng.uniform(-1, 1, 40).astype(np.float32)],
        "denormals": [1, 2, 0x007fffff, 0x80000001, 0x00800000] * 5,
        "inf_nan": [0x7f800000, 0xff800000, 0x7fc00000, 0xffc00001] + [f32_bits(x) for x in rng.uniform(-1, 1, 20).astype(np.float32)],
        "mixed_sign_small": [f32_bits(x) for x in (rng.uniform(-1, 1, 64) * 2.0 ** -14).astype(np.float32)],
    }
    params = [(0.0, 2.0 ** -15, 0.0), (2.0 ** -24, 2.0 ** -15, 0.1), (0.0, 2.0 ** -15, 0.5)]
    cases = []
    for name, bits in mats.items():
        for (it, ut, tol) in params:
            cases.append({"name": name, "bits": bits, "ignore_threshold": it, "underflow_threshold": ut,
                          "tolerance": tol, "expect": stats_bruteforce(bits, it, ut, tol)})
    return {"comment": "fp32 matrices as bit patterns (one column, m = len); expected exp_stats record; mode ids "
                       "1 = FP16TCEC, 2 = TF32TCEC, 11 = FP16TCEC_SCALING", "cases": cases}


def main():
    for name, fn in (("fp16_convert_kat.json", make_convert), ("fp16_split_kat.json", make_split),
                     ("gemm_exact_kat.json", make_exact_gemm), ("cgemm_exact_kat.json", make_exact_cgemm),
                     ("exp_stats_kat.json", make_stats)):
        with open(os.path.join(HERE, name), "w") as f:
            json.dump(fn(), f, separators=(",", ":"))
        print("wrote", name, os.path.getsize(os.path.join(HERE, name)), "bytes")


if __name__ == "__main__":
    main()
