#!/usr/bin/env python3
"""Accuracy / throughput harness with the commands and output lines of the
reference's test program (test/main.cu:1345-1510), driving the library through
its C ABI.

    python -m cumpsgemm_amd.harness sgemm [exp2|seq] min_N max_N interval MODE...
    python -m cumpsgemm_amd.harness cgemm [exp2|seq] min_N max_N interval MODE...
    python -m cumpsgemm_amd.harness sgemm_strided_batch [exp2|seq] min_N max_N interval batch MODE...
    python -m cumpsgemm_amd.harness cgemm_strided_batch [exp2|seq] min_N max_N interval batch MODE...
    python -m cumpsgemm_amd.harness sgemm_tall_skinny [exp2|seq] MN min_K max_K interval MODE...
    python -m cumpsgemm_amd.harness cgemm_tall_skinny [exp2|seq] MN min_K max_K interval MODE...
    python -m cumpsgemm_amd.harness sgemm_exp_stats N ignore_threshold underflow_threshold
    python -m cumpsgemm_amd.harness cgemm_exp_stats N ignore_threshold underflow_threshold
    python -m cumpsgemm_amd.harness sgemm_strided_batch_exp_stats N batch ignore_thr underflow_thr
    python -m cumpsgemm_amd.harness cgemm_strided_batch_exp_stats N batch ignore_thr underflow_thr
    python -m cumpsgemm_amd.harness sgemm_exp_stats_bw min_log_N max_log_N batch
    python -m cumpsgemm_amd.harness cgemm_exp_stats_bw min_log_N max_log_N batch
    python -m cumpsgemm_amd.harness log /path/to/log

MODE is any of FP16TCEC, TF32TCEC, FP16TC, TF32TC, FP16TCEC_SCALING, CUBLAS.
With "exp2" the size arguments are base-2 logarithms.  What each command does:

* the gemm commands run every op pair (N,T for real; N,T,C for complex) at
  every size: one checked launch whose relative Frobenius residual against an
  FP64 product must be below 2^-23*sqrt(K) (2^-10*sqrt(K) for FP16TC / TF32TC)
  (test/main.cu:68-74,153-234), then 32 timed launches bracketed by device
  synchronisation, reported as 2mnk (x4 for complex) per second
  (test/main.cu:383-398); one CSV line per case in the reference's format
  (test/main.cu:404-410, batched :522-529).  FP16TCEC_SCALING is FP16TCEC
  between exp_stats/scale_A/scale_B and scale_C/reset (test/main.cu:325-361).
  CUBLAS is the vendor FP32 GEMM.
* the exp_stats commands run the AUTO sequence by hand (statistics of A and B,
  launch flag, scaling, GEMM, scaling of C, statistics of C) on N(0, 2^-16)
  inputs and print the counts, decisions and residual (test/main.cu:1018-1267).
* the exp_stats_bw commands report the statistics and scaling passes in GB/s
  with the reference's byte accounting: one read per statistics pass, one read
  and one write per scaling pass (test/main.cu:1269-1342).
* log replays a CUMPSGEMM_INFO=1 log (see replay_log).

Inputs are normal random numbers from torch's generator with seed 0 (the
reference draws from cuRAND Philox with seed 0; the streams differ, the
distribution does not).
"""
import ctypes
import sys
import time

OPS_REAL = ("N", "T")
OPS_CPLX = ("N", "T", "C")
TEST_COUNT = 32  # timed launches per case (test/main.cu:17)
IMPLEMENTATIONS = ("FP16TCEC", "TF32TCEC", "FP16TC", "TF32TC", "FP16TCEC_SCALING", "CUBLAS")


def error_threshold(mode_name, n):
    """test/main.cu:68-74."""
    if mode_name in ("FP16TC", "TF32TC"):
        return 2.0 ** -10 * n ** 0.5
    return 2.0 ** -23 * n ** 0.5


class _Vendor:
    """The vendor FP32 / complex64 GEMM, bound directly so the interposer is not involved."""

    def __init__(self, stream):
        self.hb = ctypes.CDLL("libhipblas.so")
        self.h = ctypes.c_void_p()
        if self.hb.hipblasCreate(ctypes.byref(self.h)) != 0:
            raise RuntimeError("hipblasCreate failed")
        self.hb.hipblasSetStream(self.h, ctypes.c_void_p(stream))
        i, p, ll = ctypes.c_int, ctypes.c_void_p, ctypes.c_longlong
        gemm = [p, i, i, i, i, i, p, p, i, p, i, p, p, i]
        batched = [p, i, i, i, i, i, p, p, i, ll, p, i, ll, p, p, i, ll, i]
        self.hb.hipblasSgemm.argtypes = gemm
        self.hb.hipblasCgemm.argtypes = gemm
        self.hb.hipblasSgemmStridedBatched.argtypes = batched
        self.hb.hipblasCgemmStridedBatched.argtypes = batched

    def gemm(self, cplx, op_a, op_b, m, n, k, a, lda, sa, b, ldb, sb, c, ldc, sc, batch):
        one = (ctypes.c_float * 2)(1.0, 0.0)
        zero = (ctypes.c_float * 2)(0.0, 0.0)
        if batch == 1:
            fn = self.hb.hipblasCgemm if cplx else self.hb.hipblasSgemm
            return fn(self.h, op_a, op_b, m, n, k, one, a, lda, b, ldb, zero, c, ldc)
        fn = self.hb.hipblasCgemmStridedBatched if cplx else self.hb.hipblasSgemmStridedBatched
        return fn(self.h, op_a, op_b, m, n, k, one, a, lda, sa, b, ldb, sb, zero, c, ldc, sc, batch)

    def close(self):
        self.hb.hipblasDestroy(self.h)


class Harness:
    def __init__(self, out=sys.stdout):
        import torch

        import cumpsgemm_amd as cg
        self.torch, self.cg, self.out = torch, cg, out
        self.dev = torch.device("cuda:0")
        self.h = cg.Handle()
        self.h.set_stream(torch.cuda.current_stream())
        self.vendor = _Vendor(torch.cuda.current_stream().cuda_stream)
        self.ops = {"N": cg.OP_N, "T": cg.OP_T, "C": cg.OP_C}
        # one generator with seed 0 serves every draw, as in the reference (test/main.cu:543-558)
        self.gen = torch.Generator(device=self.dev)
        self.gen.manual_seed(0)
        self.modes = {"FP16TCEC": cg.FP16TCEC, "TF32TCEC": cg.TF32TCEC, "FP16TC": cg.FP16TC,
                      "TF32TC": cg.TF32TC, "FP16TCEC_SCALING": cg.FP16TCEC, "CUBLAS": cg.CUBLAS,
                      "AUTO": cg.AUTO}

    def close(self):
        self.vendor.close()
        self.h.close()

    def p(self, *a):
        print(*a, file=self.out, flush=True)

    def randn(self, count, cplx, std=1.0):
        x = self.torch.randn(count * (2 if cplx else 1), device=self.dev, generator=self.gen)
        return x * std if std != 1.0 else x

    # column-major matrix (rows x cols, leading dimension ld) number `b` of a flat float buffer
    def matrix(self, flat, rows, cols, ld, cplx, stride=0, b=0):
        t = self.torch.view_as_complex(flat.view(-1, 2)) if cplx else flat
        return t[b * stride:b * stride + ld * cols].view(cols, ld)[:, :rows].transpose(0, 1)

    def residual(self, cplx, op_a, op_b, m, n, k, a, lda, sa, b, ldb, sb, c, ldc, sc, batch):
        """Mean over the batch of sqrt(sum |ref - c|^2 / sum |ref|^2) in FP64 (test/main.cu:153-234)."""
        wide = self.torch.complex128 if cplx else self.torch.float64
        total = 0.0
        for i in range(batch):
            am = self.matrix(a, *((m, k) if op_a == "N" else (k, m)), lda, cplx, sa, i).to(wide)
            bm = self.matrix(b, *((k, n) if op_b == "N" else (n, k)), ldb, cplx, sb, i).to(wide)
            am = am if op_a == "N" else (am.transpose(0, 1).conj() if op_a == "C" else am.transpose(0, 1))
            bm = bm if op_b == "N" else (bm.transpose(0, 1).conj() if op_b == "C" else bm.transpose(0, 1))
            ref = am @ bm
            got = self.matrix(c, m, n, ldc, cplx, sc, i).to(wide)
            total += (self.torch.linalg.norm(got - ref) / self.torch.linalg.norm(ref)).item()
        return total / batch

    def case(self, cplx, imp, op_a, op_b, m, n, k, a, lda, b, ldb, c, ldc, batch=None, stride=0):
        """One CSV line: a checked launch, then TEST_COUNT timed ones (test/main.cu:308-417, 420-535)."""
        h, mode = self.h, self.modes[imp]
        scaling = imp == "FP16TCEC_SCALING"
        nb = batch or 1
        sa = sb = sc = stride
        ar, ac = (m, k) if op_a == "N" else (k, m)
        br, bc = (k, n) if op_b == "N" else (n, k)
        module = [0]

        def run(reset=False):
            if imp == "CUBLAS":
                st = self.vendor.gemm(cplx, self.ops[op_a], self.ops[op_b], m, n, k, a.data_ptr(), lda, sa,
                                      b.data_ptr(), ldb, sb, c.data_ptr(), ldc, sc, nb)
                assert st == 0
                return
            if scaling:
                ida = h.exp_stats_ext(ar, ac, a, lda, nb, sa, cplx=cplx)
                h.scale_A(ida, 1, ar, ac, a, lda, nb, sa, cplx=cplx)
                idb = h.exp_stats_ext(br, bc, b, ldb, nb, sb, cplx=cplx)
                h.scale_B(idb, 1, br, bc, b, ldb, nb, sb, cplx=cplx)
            if batch is None:
                st, module[0] = h.gemm(self.ops[op_a], self.ops[op_b], m, n, k, 1.0, a, lda, b, ldb, 0.0, c, ldc,
                                       mode, cplx=cplx, want_module_id=True)
            else:
                st = h.gemm_strided_batch(self.ops[op_a], self.ops[op_b], m, n, k, 1.0, a, lda, sa, b, ldb, sb,
                                          0.0, c, ldc, sc, nb, mode, cplx=cplx)
            assert st == 0
            if scaling:
                h.scale_C(ida, idb, 1, m, n, c, ldc, nb, sc, cplx=cplx)
                if reset:
                    h.reset_scale_A(ida, 1, ar, ac, a, lda, nb, sa, cplx=cplx)
                    h.reset_scale_B(idb, 1, br, bc, b, ldb, nb, sb, cplx=cplx)

        run(True)
        self.torch.cuda.synchronize()
        res = self.residual(cplx, op_a, op_b, m, n, k, a, lda, sa, b, ldb, sb, c, ldc, sc, nb)
        ok = res < error_threshold(imp, k if batch is None else m)
        self.torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(TEST_COUNT):
            run()
        self.torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / TEST_COUNT
        tflops = 2.0 * m * n * k * nb * (4 if cplx else 1) / dt * 1e-12
        shape = f"{m},{n},{k}" + ("" if batch is None else f",{nb}")
        self.p(f"{'cgemm' if cplx else 'sgemm'},{self.cg.mode_string(mode)},{op_a},{op_b},{shape},"
               f"{tflops:e},{res:e},{'OK' if ok else 'NG'},{module[0]}")
        return ok

    @staticmethod
    def sizes(is_seq, lo, hi, interval):
        return [v if is_seq else 1 << v for v in range(lo, hi + 1, interval)]

    def gemm_test(self, cplx, is_seq, lo, hi, interval, imps, batch=None):
        """test/main.cu:539-630 (batch None) and :715-820."""
        ns = self.sizes(is_seq, lo, hi, interval)
        stride = max(ns) ** 2 if ns else 0
        count = stride * (batch or 1)
        a, b = self.randn(count, cplx), self.randn(count, cplx)
        c = self.torch.zeros_like(a)
        self.p("## gemm_test" if batch is None else "## gemm_strided_batch_test")
        self.p("type,mode,op_A,op_B,m,n,k," + ("" if batch is None else "batch_count,")
               + "throughput_in_tflops,residual,check,module_stage")
        tests = passed = 0
        ops = OPS_CPLX if cplx else OPS_REAL
        for imp in imps:
            for op_a in ops:
                for op_b in ops:
                    for n in ns:
                        passed += self.case(cplx, imp, op_a, op_b, n, n, n, a, n, b, n, c, n, batch, stride)
                        tests += 1
        self.p(f"Result : {passed} / {tests} passed")
        return passed == tests

    def tall_skinny_test(self, cplx, is_seq, mn, lo, hi, interval, imps):
        """test/main.cu:632-713."""
        ks = self.sizes(is_seq, lo, hi, interval)
        count = mn * max(ks) if ks else 0
        a, b = self.randn(count, cplx), self.randn(count, cplx)
        c = self.torch.zeros(mn * mn * (2 if cplx else 1), device=self.dev)
        self.p("## gemm_tall_skinny_test")
        self.p("type,mode,op_A,op_B,m,n,k,throughput_in_tflops,residual,check,module_stage")
        tests = passed = 0
        ops = OPS_CPLX if cplx else OPS_REAL
        for imp in imps:
            for op_a in ops:
                for op_b in ops:
                    for k in ks:
                        passed += self.case(cplx, imp, op_a, op_b, mn, mn, k, a, mn if op_a == "N" else k,
                                            b, k if op_b == "N" else mn, c, mn)
                        tests += 1
        self.p(f"Result : {passed} / {tests} passed")
        return passed == tests

    def exp_stats_test(self, cplx, n, ignore_thr, underflow_thr, batch=1):
        """The AUTO sequence step by step on small-valued inputs (test/main.cu:1018-1267)."""
        h, cg = self.h, self.cg
        count = n * n * batch
        a = self.randn(count, cplx, 1.0 / 65536)
        b = self.randn(count, cplx, 1.0 / 65536)
        a_org, b_org = a.clone(), b.clone()
        c = self.torch.zeros_like(a)
        self.p("## gemm_exp_stats_test")
        h.set_exp_stats_params(ignore_thr, underflow_thr, 0.1)
        h.reset_exp_stats_profiling()
        h.enable_exp_stats_profiling()
        ida = h.exp_stats_ext(n, n, a, n, batch, n * n, cplx=cplx)
        idb = h.exp_stats_ext(n, n, b, n, batch, n * n, cplx=cplx)
        stats_a, stats_b = h.get_exp_stats(ida), h.get_exp_stats(idb)
        flag_id = h.get_next_dynamic_launch_buffer_id()
        h.set_dynamic_launch_buffer_by_exp_stats(flag_id, ida, idb)
        flag = h.get_dynamic_launch_flag(flag_id)
        h.scale_A(ida, flag_id, n, n, a, n, batch, n * n, cplx=cplx)
        h.scale_B(idb, flag_id, n, n, b, n, batch, n * n, cplx=cplx)
        h.set_dynamic_launch_flag_buffer_id(flag_id)
        if batch == 1:
            st = h.gemm(cg.OP_N, cg.OP_N, n, n, n, 1.0, a, n, b, n, 0.0, c, n, cg.AUTO, cplx=cplx)
        else:
            st = h.gemm_strided_batch(cg.OP_N, cg.OP_N, n, n, n, 1.0, a, n, n * n, b, n, n * n, 0.0, c, n, n * n,
                                      batch, cg.AUTO, cplx=cplx)
        assert st == 0
        h.unset_dynamic_launch_flag_buffer_id()
        h.scale_C(ida, idb, flag_id, n, n, c, n, batch, n * n, cplx=cplx)
        h.disable_exp_stats_profiling()
        idc = h.exp_stats_ext(n, n, c, n, batch, n * n, cplx=cplx)
        stats_c = h.get_exp_stats(idc)
        res = self.residual(cplx, "N", "N", n, n, n, a_org, n, n * n, b_org, n, n * n, c, n, n * n, batch)
        ok = res < error_threshold("AUTO", n)

        def line(name, stats, sid, with_mode):
            under, total = stats
            rate = under / total if total else 0.0
            s = (f"  {name} = [underflow: {under:10d} / {total:10d} ({rate:6.2f}), "
                 f"max_exp={h.get_max_exp(sid):e}, buffer_id = {sid}")
            if with_mode:
                s += f" -> mode={cg.mode_string(h.get_exp_stats_compute_mode_level(sid))}"
            return s + "]"
        self.p(f"# [{'cgemm' if cplx else 'sgemm'}:{'AUTO':>8s}, N={n}, batch_size={batch}, "
               f"u={underflow_thr:e}, i={ignore_thr:e}]")
        self.p(line("A", stats_a, ida, True))
        self.p(line("B", stats_b, idb, True))
        self.p(line("C", stats_c, idc, False))
        self.p(f"  Compute mode = [{cg.mode_string(flag & 0x1f)}, SCALE_A={(flag >> 6) & 1}, "
               f"SCALE_B={(flag >> 5) & 1}]")
        self.p(f"  Error = [{res:e}, {'OK' if ok else 'NG'}]")
        self.out.flush()
        h.print_exp_stats_profiling()
        return ok

    def exp_stats_bw_test(self, cplx, min_log_n, max_log_n, batch=1):
        """Statistics and scaling passes in GB/s (test/main.cu:1269-1342)."""
        h = self.h
        count = (1 << (2 * max_log_n)) * batch
        a_org = self.randn(count, cplx, 1.0 / 65536)
        a = a_org.clone()
        self.p("## exp_stats_bw_test")
        # ignore nothing, count everything below 1 as underflow, tolerate none: both passes run
        h.set_exp_stats_params(0.0, 1.0, 0.0)
        h.enable_exp_stats_profiling()
        self.p("gemm,N,exp_stats_1_bw_in_gbps,exp_stats_2_bw_in_gbps,scale_bw_in_gbps")
        for log_n in range(min_log_n, max_log_n + 1):
            h.reset_exp_stats_profiling()
            n = 1 << log_n
            elems = n * n * (2 if cplx else 1) * batch
            a[:elems].copy_(a_org[:elems])
            for _ in range(100):
                sid = h.exp_stats_ext(n, n, a, n, batch, n * n, cplx=cplx)
                h.scale_A(sid, 1, n, n, a, n, batch, n * n, cplx=cplx)
            bw = {}
            for label, passes in (("exp_stats_1", 1), ("exp_stats_2", 1), ("scaling_AB", 2)):
                e = h.get_exp_stats_profiling_entry(label)
                bw[label] = passes * elems * 4 * e[1] / e[0] * 1e-9 if e and e[0] > 0 else 0.0
            self.p(f"{'C' if cplx else 'S'},{n},{bw['exp_stats_1']:e},{bw['exp_stats_2']:e},{bw['scaling_AB']:e}")
        h.disable_exp_stats_profiling()
        return True


def _imps(names):
    imps = []
    for nm in names:
        if nm in IMPLEMENTATIONS:
            imps.append(nm)
        else:
            print(f"Unknown compute mode : {nm}")
    print("Testing implementations: " + " ".join(imps) + " ", flush=True)
    return imps


def main(argv, out=sys.stdout):
    if len(argv) < 2:
        sys.exit(__doc__)
    cmd = argv[1]
    cplx = cmd.startswith("cgemm")
    kind = cmd[5:] if cmd[:5] in ("sgemm", "cgemm") else cmd
    if cmd == "log":
        if len(argv) != 3:
            sys.exit(__doc__)
        from .replay_log import parse, replay
        passed, tested = replay(parse(argv[2]), out=out)
        return passed == tested
    try:
        if kind == "_exp_stats":
            n, ignore, under = int(argv[2]), float(argv[3]), float(argv[4])
            job = lambda t: t.exp_stats_test(cplx, n, ignore, under)  # noqa: E731
        elif kind == "_strided_batch_exp_stats":
            n, batch, ignore, under = int(argv[2]), int(argv[3]), float(argv[4]), float(argv[5])
            job = lambda t: t.exp_stats_test(cplx, n, ignore, under, batch)  # noqa: E731
        elif kind == "_exp_stats_bw":
            lo, hi, batch = int(argv[2]), int(argv[3]), int(argv[4])
            job = lambda t: t.exp_stats_bw_test(cplx, lo, hi, batch)  # noqa: E731
        elif kind in ("", "_tall_skinny", "_strided_batch") and argv[2] in ("exp2", "seq"):
            is_seq = argv[2] == "seq"
            if kind == "":
                lo, hi, step = (int(v) for v in argv[3:6])
                imps = _imps(argv[6:])
                job = lambda t: t.gemm_test(cplx, is_seq, lo, hi, step, imps)  # noqa: E731
            elif kind == "_tall_skinny":
                mn, lo, hi, step = (int(v) for v in argv[3:7])
                imps = _imps(argv[7:])
                job = lambda t: t.tall_skinny_test(cplx, is_seq, mn, lo, hi, step, imps)  # noqa: E731
            else:
                lo, hi, step, batch = (int(v) for v in argv[3:7])
                imps = _imps(argv[7:])
                job = lambda t: t.gemm_test(cplx, is_seq, lo, hi, step, imps, batch)  # noqa: E731
        else:
            sys.exit(__doc__)
    except (IndexError, ValueError):
        sys.exit(__doc__)
    t = Harness(out)
    try:
        return job(t)
    finally:
        t.close()


if __name__ == "__main__":
    sys.exit(0 if main(sys.argv) else 1)
