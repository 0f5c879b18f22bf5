#!/usr/bin/env python3
"""Replays the GEMMs recorded in an interposer log.

An application run with CUMPSGEMM_INFO=1 prints one line per intercepted call,

    [cuMpSGEMM LOG] hipblasSgemm op=(N, T), shape=(4, 128, 65536), mode=TF32TCEC[dynamic][exp_stats:0]

This tool reads such a log (the cuBLAS names of logs written by the reference
are accepted too), runs every recorded shape through the library with the
recorded mode on random inputs, checks the result against an FP64 GEMM with the
reference's threshold (2^-23 * sqrt(K) for the error-corrected modes, 2^-10 *
sqrt(K) for the others) and prints one line per shape in the reference
harness's CSV format -- the counterpart of its "log" command
(test/main.cu:820-1016, line format :404-410).

    python -m cumpsgemm_amd.replay_log app.log
"""
import re
import sys

LINE = re.compile(r"\[cuMpSGEMM LOG\] (\w+) op=\((.), (.)\), shape=\((\d+), (\d+), (\d+)\)"
                  r"(?:, batch=(\d+))?, mode=(\w+)")
COMPLEX_FUNCS = ("hipblasCgemm", "cublasCgemm_v2", "hipblasCgemmStridedBatched", "cublasCgemmStridedBatched")


def parse(path):
    calls = []
    with open(path) as f:
        for line in f:
            m = LINE.search(line)
            if not m:
                continue
            func, oa, ob, mm, nn, kk, batch, mode = m.groups()
            calls.append({"func": func, "op_a": oa, "op_b": ob, "m": int(mm), "n": int(nn), "k": int(kk),
                          "batch": int(batch) if batch else 1, "mode": mode,
                          "cplx": func in COMPLEX_FUNCS})
    return calls


def replay(calls, max_elements=1 << 28, out=sys.stdout):
    import torch

    import cumpsgemm_amd as cg
    dev = torch.device("cuda:0")
    h = cg.Handle()
    h.set_stream(torch.cuda.current_stream())
    ops = {"N": cg.OP_N, "T": cg.OP_T, "C": cg.OP_C}
    modes = {"FP16TCEC": cg.FP16TCEC, "TF32TCEC": cg.TF32TCEC, "FP16TC": cg.FP16TC, "TF32TC": cg.TF32TC,
             "FP16TCEC_SCALING": cg.FP16TCEC_SCALING, "AUTO": cg.AUTO}
    tested = passed = 0
    seen = set()
    for c in calls:
        key = tuple(sorted(c.items()))
        if key in seen or c["mode"] not in modes:
            continue  # forwarded modes (CUBLAS*) run hipBLAS itself; nothing of ours to test
        seen.add(key)
        m, n, k, batch, cplx = c["m"], c["n"], c["k"], c["batch"], c["cplx"]
        if max(m * k, k * n, m * n) * batch > max_elements:
            print(f"skip (too large) {c}", file=out)
            continue
        dt = torch.complex64 if cplx else torch.float32
        ar, ac = (m, k) if c["op_a"] == "N" else (k, m)
        br, bc = (k, n) if c["op_b"] == "N" else (n, k)
        # column-major storage = the transpose of a row-major torch tensor
        a = torch.randn(batch, ac, ar, device=dev, dtype=dt)
        b = torch.randn(batch, bc, br, device=dev, dtype=dt)
        cm = torch.zeros(batch, n, m, device=dev, dtype=dt)
        fa, fb, fc = (torch.view_as_real(t).reshape(-1) if cplx else t.reshape(-1) for t in (a, b, cm))

        def run():
            if c["mode"] in ("AUTO", "FP16TCEC_SCALING"):
                st, _ = h.gemm_pipeline(ops[c["op_a"]], ops[c["op_b"]], m, n, k, 1.0, fa, ar, fb, br, 0.0, fc, m,
                                        modes[c["mode"]], cplx=cplx, stridea=ar * ac, strideb=br * bc,
                                        stridec=m * n, batch=batch)
                return st
            return h.gemm_strided_batch(ops[c["op_a"]], ops[c["op_b"]], m, n, k, 1.0, fa, ar, ar * ac, fb, br,
                                        br * bc, 0.0, fc, m, m * n, batch, modes[c["mode"]], cplx=cplx)
        assert run() == 0
        torch.cuda.synchronize()
        module = 0
        if c["mode"] not in ("AUTO", "FP16TCEC_SCALING") and batch == 1:
            _, module = h.gemm(ops[c["op_a"]], ops[c["op_b"]], m, n, k, 1.0, fa, ar, fb, br, 0.0, fc, m,
                               modes[c["mode"]], cplx=cplx, want_module_id=True)

        def logical(t, op):
            x = t.transpose(1, 2).to(torch.complex128 if cplx else torch.float64)
            if op == "T":
                return x.transpose(1, 2)
            if op == "C":
                return x.transpose(1, 2).conj()
            return x
        ref = logical(a, c["op_a"]) @ logical(b, c["op_b"])
        got = cm.transpose(1, 2).to(ref.dtype)
        res = (torch.linalg.norm(got - ref) / torch.linalg.norm(ref)).item()
        corrected = c["mode"] in ("FP16TCEC", "TF32TCEC", "FP16TCEC_SCALING", "AUTO")
        bar = (2.0 ** -23 if corrected else 2.0 ** -10) * max(k, 1) ** 0.5
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(5):
            run()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / 5
        tflops = (8.0 if cplx else 2.0) * m * n * k * batch / ms / 1e9
        ok = res < bar
        tested += 1
        passed += ok
        # the result line of the reference harness (test/main.cu:404-410, batched :522-529):
        # gemm,MODE,opA,opB,m,n,k[,batch],TFlop/s,residual,OK|NG,module id
        kind = "cgemm" if cplx else "sgemm"
        shape = f"{m},{n},{k}" + (f",{batch}" if batch > 1 else "")
        print(f"{kind},{c['mode']},{c['op_a']},{c['op_b']},{shape},{tflops:e},{res:e},{'OK' if ok else 'NG'},{module}",
              file=out)
    h.close()
    print(f"{passed} / {tested} passed", file=out)
    return passed, tested


def main(argv):
    if len(argv) != 2:
        sys.exit(__doc__)
    passed, tested = replay(parse(argv[1]))
    sys.exit(0 if passed == tested else 1)


if __name__ == "__main__":
    main(sys.argv)
