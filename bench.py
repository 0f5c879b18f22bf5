#!/usr/bin/env python3
"""Headline benchmark: effective FP32 TFLOP/s (2MNK/t) of FP16TCEC SGEMM at
M=N=K=8192 (NN, uniform[-1,1], alpha=1, beta=0) on one MI355X, with the relative
Frobenius error against an FP64 GEMM of the same inputs, next to hipBLAS native
FP32 SGEMM on the same GPU and to the split-and-correct algorithm on host cores.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--headline-only]

One "step" is one GEMM call through the C ABI (cuMpSGEMM_sgemm) with operands
resident in HBM.  Prints ONE JSON line.  After the headline's timed region the
other benchmark configurations run as well (C1 on the host cores, C2 layouts and
bf16x3, C3 batched CGEMM, C4 scaling pipeline, C5a tall-skinny, C5b Mx2x2) and
are reported under "extra", each with its own roofline, its error against FP64
and the vendor FP32 routine on the same inputs; --headline-only skips them.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

FP16_MFMA_PEAK_TFLOPS = 2500.0  # MI355X dense fp16 MFMA
HBM_PEAK_GBS = 8000.0
# HBM bytes per 8192^3 FP16TCEC launch of the GEMM kernel from the rocprofv3
# FETCH_SIZE + WRITE_SIZE counters, scaled by what the same counters read for a
# plain copy of known size (profiles/gemm_fp16tcec_8192_nn.md).  This is L2-miss
# traffic on the fabric (Infinity Cache or HBM); the algorithmic minimum is
# 3 * 8192^2 * 4 B = 0.805e9.  The call's two pre-split passes add 1.07e9.
GEMM_TRAFFIC_BYTES = 5.70e9


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def host_cores():
    """Threads of the host-core legs: the share of the host this job was given (OMP_NUM_THREADS when the
    environment sets it -- a GPU box hands a one-GPU job part of its cores --, else every core)."""
    env = int(os.environ.get("OMP_NUM_THREADS", "0") or 0)
    if env > 0:
        return env, f"{env} threads = OMP_NUM_THREADS as set by the environment, of {os.cpu_count()} cores visible"
    n = os.cpu_count() or 1
    return n, f"all {n} cores"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=32)   # the reference times 32 calls (test/main.cu:15)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--size", type=int, default=8192)
    ap.add_argument("--full", action="store_true", help="(default now: kept so that old command lines work)")
    ap.add_argument("--headline-only", action="store_true", help="skip the other configurations")
    ap.add_argument("--no-cpu", action="store_true", help="skip the host-core baseline")
    ap.add_argument("--kernel-only", action="store_true",
                    help="time the FP16TCEC GEMM only (no FP64 check, hipBLAS or CPU legs): for profilers")
    ap.add_argument("--kernel", default="gemm", choices=["gemm", "copy", "exp_stats", "exp_max", "scale", "mx2x2"],
                    help="with --kernel-only: which kernel to run (copy = a plain device copy of the "
                         "same bytes, the reference point for the HBM traffic counters)")
    ap.add_argument("--shape", default=None,
                    help="with --kernel-only: M,N,K[,BATCH] instead of a square --size (BATCH > 1: strided batch)")
    ap.add_argument("--cplx", action="store_true", help="with --kernel-only --shape: complex64 operands (CGEMM)")
    ap.add_argument("--stamps", action="store_true",
                    help="with --kernel-only --shape and a library built with -DCUMPSGEMM_WALK_STAMPS=1 "
                         "(CUMPSGEMM_LIBRARY=...): print the in-kernel clock stamps of one call of the "
                         "tile-walking pre-split kernel, tile by tile")
    ap.add_argument("--op", default="NN", choices=["NN", "TN", "NT", "TT"])
    ap.add_argument("--data", default="uniform", choices=["uniform", "zeros", "ones", "ints", "fp16"],
                    help="with --kernel-only: operand values (the part is power-limited and the MFMAs' "
                         "draw depends on how many operand bits toggle)")
    ap.add_argument("--mode", default="FP16TCEC", choices=["FP16TCEC", "TF32TCEC", "FP16TC", "TF32TC"])
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (no collectives, no sharding); use --gpus 1")

    import torch
    import cumpsgemm_amd as cg
    from cumpsgemm_amd import inputs

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    cg.lib()  # fails loudly if the HIP library has not been built
    dev = torch.device("cuda:0")
    stream = torch.cuda.current_stream()
    h = cg.Handle()
    h.set_stream(stream)

    n = args.size
    m = k = n
    if args.kernel_only and args.kernel != "gemm":
        hbm_kernel_only(args, torch, cg, inputs, h, dev, stream)
        h.close()
        return
    if args.kernel_only and args.shape:
        shape_kernel_only(args, torch, cg, h, dev, stream)
        h.close()
        return
    log(f"[bench] generating {n}x{n} inputs (seeds 1, 2)")
    a_host = inputs.uniform(1, m * k)
    b_host = inputs.uniform(2, k * n)
    a = torch.from_numpy(a_host).to(dev)
    b = torch.from_numpy(b_host).to(dev)
    c = torch.zeros(m * n, device=dev)
    if args.kernel_only and args.data != "uniform":
        if args.data == "zeros":
            a.zero_(), b.zero_()
        elif args.data == "ones":
            a.fill_(1.0), b.fill_(1.0)
        elif args.data == "ints":
            a, b = torch.round(a * 8), torch.round(b * 8)
        else:  # values an fp16 holds exactly: the lo planes of the split are zero
            a, b = a.half().float(), b.half().float()

    def timed(fn, steps, warmup, settle_ms=float(os.environ.get("BENCH_SETTLE_MS", "100"))):
        # The part lowers its clocks within milliseconds of going idle (every leg
        # below starts with host-side set-up) and takes tens of milliseconds of
        # load to raise them again: calls made before that are up to 25 % slow.
        # So the GPU is kept busy with the same call for `settle_ms` first; the
        # `warmup` untimed calls and the `steps` timed ones follow back to back.
        t_settle = time.perf_counter()
        while (time.perf_counter() - t_settle) * 1e3 < settle_ms:
            fn()
            torch.cuda.synchronize()
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record(stream)
        for _ in range(steps):
            fn()
        e1.record(stream)
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3 / steps
        return wall_ms, e0.elapsed_time(e1) / steps

    flops = 2.0 * m * n * k

    def tcec(mode, opa=cg.OP_N, opb=cg.OP_N):
        def fn():
            st = h.gemm(opa, opb, m, n, k, 1.0, a, n, b, n, 0.0, c, n, mode)
            assert st == 0
        return fn

    log("[bench] FP16TCEC timed region")
    if args.kernel_only:
        opa = cg.OP_T if args.op[0] == "T" else cg.OP_N
        opb = cg.OP_T if args.op[1] == "T" else cg.OP_N
        wall_ms, ev_ms = timed(tcec(getattr(cg, args.mode), opa, opb), args.steps, args.warmup)
        print(json.dumps({"kernel_only": True, "op": args.op, "mode": args.mode, "size": n, "data": args.data,
                          "ms_per_step": round(wall_ms, 4), "kernel_ms": round(ev_ms, 4),
                          "tflops": round(flops / (ev_ms * 1e-3) / 1e12, 2)}), flush=True)
        h.close()
        return
    wall_ms, ev_ms = timed(tcec(cg.FP16TCEC), args.steps, args.warmup)
    # which path served the call: 200 = pre-split operands, else the tile class of the in-loop kernel
    _, module_id = h.gemm(cg.OP_N, cg.OP_N, m, n, k, 1.0, a, n, b, n, 0.0, c, n, cg.FP16TCEC, want_module_id=True)
    value = flops / (wall_ms * 1e-3) / 1e12
    kernel_tflops = flops / (ev_ms * 1e-3) / 1e12

    # ---- error against FP64 (rocBLAS DGEMM on widened inputs), same inputs ----
    log("[bench] FP64 reference")
    A64 = a.view(n, n).t().double()  # column-major buffer -> logical matrix
    B64 = b.view(n, n).t().double()
    ref = A64 @ B64
    ref_norm = torch.linalg.norm(ref).item()

    def rel_err():
        got = c.view(n, n).t().double()
        return (torch.linalg.norm(got - ref) / ref_norm).item()

    tcec(cg.FP16TCEC)()
    err_tcec = rel_err()

    # ---- hipBLAS native FP32 SGEMM on the same GPU ----
    log("[bench] hipBLAS SGEMM")
    hb_tflops, err_sgemm = None, None
    try:
        hb = ctypes.CDLL("libhipblas.so")
        hbh = ctypes.c_void_p()
        assert hb.hipblasCreate(ctypes.byref(hbh)) == 0
        hb.hipblasSetStream(hbh, ctypes.c_void_p(stream.cuda_stream))
        one, zero = ctypes.c_float(1.0), ctypes.c_float(0.0)
        hb.hipblasSgemm.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                    ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                                    ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int]

        def sgemm():
            st = hb.hipblasSgemm(hbh, 111, 111, m, n, k, ctypes.byref(one), a.data_ptr(), n, b.data_ptr(), n,
                                 ctypes.byref(zero), c.data_ptr(), n)
            assert st == 0
        hb_wall, _ = timed(sgemm, max(4, args.steps // 2), 2)
        hb_tflops = flops / (hb_wall * 1e-3) / 1e12
        sgemm()
        err_sgemm = rel_err()
        hb.hipblasDestroy(hbh)
    except Exception as e:  # pragma: no cover
        log(f"[bench] hipBLAS comparison unavailable: {e}")

    extra = {}
    if not args.headline_only and n == 8192:
        del ref, A64, B64
        torch.cuda.empty_cache()
        extra = full_suite(torch, cg, inputs, h, dev, stream, timed, log, a, b, c, not args.no_cpu)

    # ---- CPU baseline: the same algorithm on the host cores (oracle, bounded sample) ----
    cpu = None
    if not args.no_cpu:
        log("[bench] CPU baseline (oracle)")
        from oracle import oracle as O
        O.lib()
        cores, cores_why = host_cores()
        os.environ["OMP_NUM_THREADS"] = str(cores)

        def cpu_run(cn):
            ca, cb = inputs.uniform(1, cn * cn), inputs.uniform(2, cn * cn)
            cc = np.zeros(cn * cn, np.float32)
            t0 = time.perf_counter()
            O.gemm(O.MODE_FP16TCEC, O.OP_N, O.OP_N, cn, cn, cn, 1.0, ca, cn, cb, cn, 0.0, cc, cn)
            return time.perf_counter() - t0

        # bounded sample: 1/8 of the step first; the whole step only when the
        # host cores are fast enough to finish it in about half a minute
        cn = min(n, 4096)
        dt = cpu_run(cn)
        if cn < n and dt * (n // cn) ** 3 < 30.0:
            cn = n
            dt = cpu_run(cn)
        frac = "the whole" if cn == n else f"1/{(n // cn) ** 3} of the"
        cpu = {"value": round(2.0 * cn ** 3 / dt / 1e12, 5), "unit": "TFLOP/s", "cores": cores, "kind": "port",
               "sample": f"one FP16TCEC SGEMM NN {cn}^3 (same generator, seeds 1,2) = {frac} "
                         f"{n}^3 step, split included, {dt:.1f} s; {cores_why}"}

    out = {
        "metric": "effective FP32 TFLOP/s (2MNK/t) at 8192^3 FP16TCEC + rel. error vs FP64",
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        # every timed region is preceded by 100 ms of the same call (the part's clocks need that long to
        # come up after host-side set-up), then the `warmup` untimed calls, then the `steps` timed ones
        "settle_ms": 100,
        "ms_per_step": round(wall_ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16 (hi/lo split of f32, 3 MFMA products, f32 accumulate)",
        "data": "synthetic",
        "config": {"workload": f"C2: SGEMM NN M=N=K={n}, A,B uniform[-1,1] seeds (1,2), alpha=1, beta=0, mode FP16TCEC",
                   "layout": "NN", "mode": "FP16TCEC"},
        "rel_error_vs_fp64": err_tcec,
        "rel_error_hipblas_sgemm_vs_fp64": err_sgemm,
        "error_ratio_vs_sgemm": (err_tcec / err_sgemm) if err_sgemm else None,
        "hipblas_sgemm_tflops": round(hb_tflops, 2) if hb_tflops else None,
        "speedup_vs_hipblas_sgemm": round(value / hb_tflops, 3) if hb_tflops else None,
        # frac = the fraction of the emulation roofline (fp16 MFMA peak / products): `achieved` is the fp16 MFMA
        # work the kernel issues -- 3 products per real multiply-add of the algorithm, i.e. 3 x the algorithmic
        # 2MNK flops of one launch -- over the launch's average duration between HIP events on its stream
        "roofline": headline_roofline(flops, ev_ms, module_id, n),
        "cpu_baseline": cpu,
    }
    if extra:
        out["extra"] = extra
    print(json.dumps(out), flush=True)
    h.close()


def shape_kernel_only(args, torch, cg, h, dev, stream):
    """One GEMM call of any shape in a loop, for profilers (operands made on the device: uniform[-1,1) or --data)."""
    dims = [int(x) for x in args.shape.split(",")]
    m, n, k = dims[:3]
    batch = dims[3] if len(dims) > 3 else 1
    es = 2 if args.cplx else 1
    opa = cg.OP_T if args.op[0] == "T" else cg.OP_N
    opb = cg.OP_T if args.op[1] == "T" else cg.OP_N
    lda, ldb = (m if opa == cg.OP_N else k), (k if opb == cg.OP_N else n)
    a = torch.rand(batch * m * k * es, device=dev) * 2 - 1
    b = torch.rand(batch * k * n * es, device=dev) * 2 - 1
    if args.data == "zeros":
        a.zero_(), b.zero_()
    elif args.data == "ones":
        a.fill_(1.0), b.fill_(1.0)
    elif args.data == "ints":
        a, b = torch.round(a * 8), torch.round(b * 8)
    elif args.data == "fp16":
        a, b = a.half().float(), b.half().float()
    c = torch.zeros(batch * m * n * es, device=dev)
    mode = getattr(cg, args.mode)
    if batch > 1:
        fn = lambda: h.gemm_strided_batch(opa, opb, m, n, k, 1.0, a, lda, m * k, b, ldb, k * n, 0.0, c, m, m * n, batch,
                                          mode, cplx=args.cplx)
    else:
        fn = lambda: h.gemm(opa, opb, m, n, k, 1.0, a, lda, b, ldb, 0.0, c, m, mode, cplx=args.cplx)
    settle = float(os.environ.get("BENCH_SETTLE_MS", "100"))
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < settle:
        fn()
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for _ in range(args.steps):
        fn()
    e1.record(stream)
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / args.steps
    flops = (8.0 if args.cplx else 2.0) * m * n * k * batch
    print(json.dumps({"kernel_only": True, "shape": [m, n, k, batch], "cplx": args.cplx, "op": args.op, "mode": args.mode,
                      "data": args.data, "kernel_ms": round(ms, 4), "tflops": round(flops / ms / 1e9, 2)}), flush=True)
    if args.stamps:
        walk_stamps(torch, cg, dev, fn, k)


def walk_stamps(torch, cg, dev, fn, k):
    """One more call with the stamp buffer installed; per tile of the two traced workgroups: clocks from the
    previous event to `this wave is done with the step` and from there to `past the barrier`, for every
    K-step, and the clocks the write-out took to issue."""
    L = cg.lib()
    buf = torch.zeros(1024, dtype=torch.int64, device=dev)
    if L.cuMpSGEMM_set_walk_stamp_buffer(buf.data_ptr()) != 0:
        sys.exit("bench.py --stamps: this library was not built with -DCUMPSGEMM_WALK_STAMPS=1")
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    fn()
    e1.record()
    torch.cuda.synchronize()
    L.cuMpSGEMM_set_walk_stamp_buffer(None)
    us = e0.elapsed_time(e1) * 1e3
    t = buf.cpu().numpy()
    nk = (k + 31) // 32
    per = 2 * nk + 1
    for wg, base in ((0, 0), (101, 512)):
        cnt = int(t[base])
        ev = [int(x) % (1 << 64) for x in t[base + 1: base + 1 + cnt]]
        clk = [e & ((1 << 60) - 1) for e in ev]
        if cnt < 2 * per:
            print(f"workgroup {wg}: {cnt} stamps (the call did not run the tile-walking pre-split kernel?)")
            continue
        print(f"workgroup {wg}: call {us:.0f} us, {cnt} stamps over {clk[-1] - clk[0]} clocks "
              f"({(clk[-1] - clk[0]) / us:.0f} clocks per us)")
        for ti in range(1, min(cnt // per, 6)):
            seg = clk[ti * per - 1: (ti + 1) * per]
            d = [seg[i + 1] - seg[i] for i in range(len(seg) - 1)]
            print(f"  tile {ti}: own work + wait {[d[2 * i] for i in range(nk)]} at the barrier "
                  f"{[d[2 * i + 1] for i in range(nk)]} write-out {d[-1]}")


def hbm_kernel_only(args, torch, cg, inputs, h, dev, stream):
    """One HBM-bound kernel of the path in a loop, for profilers: --size is the
    matrix order (mx2x2: log2 of M)."""
    n = args.size
    if args.kernel == "mx2x2":
        M = 1 << n
        x = torch.randn(M * 4, device=dev)
        u = torch.from_numpy(inputs.random_unitary_2x2(9).view(np.float32)).to(dev)
        y = torch.zeros(M * 4, device=dev)
        nbytes = 2.0 * M * 2 * 8
        fn = lambda: h.gemm_Mx2x2(cg.OP_N, cg.OP_N, M, 1.0, x, M, u, 2, 0.0, y, M, cplx=True)
    else:
        a = torch.from_numpy(inputs.exponent_spread(3, n, n, per_row=True)).to(dev)
        nbytes = 4.0 * n * n
        if args.kernel == "copy":
            d = torch.empty_like(a)
            nbytes *= 2
            fn = lambda: d.copy_(a)
        elif args.kernel == "exp_stats":
            fn = lambda: h.exp_stats_ext(n, n, a, n)
        elif args.kernel == "exp_max":
            fn = lambda: h.exp_max_ext(n, n, a, n)
        else:
            sid = h.exp_max_ext(n, n, a, n)
            nbytes *= 2
            state = [0]

            def fn():
                (h.reset_scale_A if state[0] & 1 else h.scale_A)(sid, 1, n, n, a, n)
                state[0] += 1
    for _ in range(args.warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for _ in range(args.steps):
        fn()
    e1.record(stream)
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / args.steps
    print(json.dumps({"kernel_only": True, "kernel": args.kernel, "size": n, "bytes_per_call": nbytes,
                      "ms_per_call": round(ms, 5), "GBs": round(nbytes / ms / 1e6, 1)}), flush=True)


def mfma_roofline(flops, ev_ms, products, kernels):
    """Roofline entry of an MFMA-bound configuration.  `flops`: algorithmic flops of one call (2MNK, 8MNK
    complex); `ev_ms`: its duration between HIP events on the launch stream; `products`: MFMA products issued
    per real multiply-add of the algorithm.  achieved = products x flops / t, the fp16 / bf16 MFMA work
    issued, against the dense MFMA peak -- so frac is the fraction of the emulation roofline (peak / products)."""
    eff = flops / (ev_ms * 1e-3) / 1e12
    return {"bound": "mfma", "achieved": round(products * eff, 2), "peak": FP16_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": round(products * eff / FP16_MFMA_PEAK_TFLOPS, 4), "kernel_ms": round(ev_ms, 4),
            "mfma_products_per_real_mac": products, "effective_tflops": round(eff, 2),
            "emulation_roofline_tflops": round(FP16_MFMA_PEAK_TFLOPS / products, 1),
            "effective_over_raw_peak": round(eff / FP16_MFMA_PEAK_TFLOPS, 4), "kernels": kernels}


def headline_roofline(flops, ev_ms, module_id, n):
    r = mfma_roofline(flops, ev_ms, 3,
                      "pack_split_pair_kernel + gemm_tcec_kernel (persistent, packed)" if module_id == 200
                      else "gemm_tcec_kernel")
    # one call = one pre-split launch for both operands (about 0.2 ms) + the GEMM kernel: all inside kernel_ms
    r["traffic"] = GEMM_TRAFFIC_BYTES if n == 8192 else None
    r["traffic_source"] = ("constant from the committed rocprofv3 counter runs (profiles/gemm_fp16tcec_8192_nn.md), "
                           "not measured in this run")
    return r


def hbm_roofline(nbytes, ev_ms, kernels):
    g = nbytes / (ev_ms * 1e-3) / 1e9
    return {"bound": "hbm", "achieved": round(g, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(g / HBM_PEAK_GBS, 4), "kernel_ms": round(ev_ms, 5), "bytes_per_call": nbytes,
            "kernels": kernels}


def full_suite(torch, cg, inputs, h, dev, stream, timed, log, a, b, c, with_cpu):
    """The other benchmark configurations (C1, C2 layouts and bf16x3, C3, C4, C5a, C5b), reported
    under "extra".  a, b, c: the headline's 8192^2 device buffers (uniform, seeds 1 and 2)."""
    res = {}

    def rel_err(got, ref):
        return (torch.linalg.norm(got - ref) / torch.linalg.norm(ref)).item()

    # C1: the split-and-correct arithmetic on the host cores at 1024^3 (oracle), against FP64
    if with_cpu:
        from oracle import oracle as O
        O.lib()
        cores, _ = host_cores()
        s1 = 1024
        ca, cb = inputs.uniform(1, s1 * s1), inputs.uniform(2, s1 * s1)
        cc, c32 = np.zeros(s1 * s1, np.float32), np.zeros(s1 * s1, np.float32)
        log("[bench] C1 host cores 1024^3")
        O.gemm(O.MODE_FP16TCEC, O.OP_N, O.OP_N, s1, s1, s1, 1.0, ca, s1, cb, s1, 0.0, cc, s1)   # warm-up
        t0 = time.perf_counter()
        O.gemm(O.MODE_FP16TCEC, O.OP_N, O.OP_N, s1, s1, s1, 1.0, ca, s1, cb, s1, 0.0, cc, s1)
        dt = time.perf_counter() - t0
        O.gemm(O.MODE_FP32, O.OP_N, O.OP_N, s1, s1, s1, 1.0, ca, s1, cb, s1, 0.0, c32, s1)
        ref1 = O.gemm_fp64(O.OP_N, O.OP_N, s1, s1, s1, 1.0, ca, s1, cb, s1)
        # the same problem through the GPU library, for the record
        da, db, dc = torch.from_numpy(ca).to(dev), torch.from_numpy(cb).to(dev), torch.zeros(s1 * s1, device=dev)
        h.gemm(cg.OP_N, cg.OP_N, s1, s1, s1, 1.0, da, s1, db, s1, 0.0, dc, s1, cg.FP16TCEC)
        _, gev = timed(lambda: h.gemm(cg.OP_N, cg.OP_N, s1, s1, s1, 1.0, da, s1, db, s1, 0.0, dc, s1, cg.FP16TCEC),
                       20, 3)
        res["C1_sgemm_NN_1024_host_cores"] = {
            "host_gflops": round(2.0 * s1 ** 3 / dt / 1e9, 1), "cores": cores,
            "rel_error_fp16tcec_cpu": O.residual(ref1, cc, s1, s1, s1),
            "rel_error_fp32_cpu": O.residual(ref1, c32, s1, s1, s1),
            "rel_error_fp16tcec_gpu": O.residual(ref1, dc.cpu().numpy(), s1, s1, s1),
            "gpu_tflops": round(2.0 * s1 ** 3 / gev / 1e9, 2), "dtype": "f16 hi/lo split of f32 emulated in f32 on the host"}

    # C2 layouts and modes at 8192^3 (the headline's buffers)
    n = 8192
    A, B = a.view(n, n).t().double(), b.view(n, n).t().double()
    A32, B32 = a.view(n, n).t(), b.view(n, n).t()
    for name, opa, opb in (("NN", cg.OP_N, cg.OP_N), ("TN", cg.OP_T, cg.OP_N), ("NT", cg.OP_N, cg.OP_T)):
        ref = (A.t() if opa == cg.OP_T else A) @ (B.t() if opb == cg.OP_T else B)
        x32, y32 = (A32.t() if opa == cg.OP_T else A32), (B32.t() if opb == cg.OP_T else B32)
        vwall, _ = timed(lambda: torch.matmul(x32, y32), 6, 2)
        verr = rel_err(torch.matmul(x32, y32).double(), ref)
        modes = [("FP16TCEC", cg.FP16TCEC, 3), ("bf16x3", cg.TF32TCEC, 6)]
        if name == "NN":                     # the modes without correction terms, for scale (one layout)
            modes += [("FP16TC", cg.FP16TC, 1), ("bf16x2", cg.TF32TC, 3)]
        for mode_name, mode, prods in modes:
            if name == "NN" and mode_name == "FP16TCEC":
                continue                     # the headline itself
            log(f"[bench] C2 {name} {mode_name}")
            fn = lambda: h.gemm(opa, opb, n, n, n, 1.0, a, n, b, n, 0.0, c, n, mode)
            wall, ev = timed(fn, 10, 2)
            res[f"C2_{name}_{mode_name}"] = {
                "tflops": round(2.0 * n ** 3 / wall / 1e9, 2), "rel_error": rel_err(c.view(n, n).t().double(), ref),
                "vendor_fp32_matmul_tflops": round(2.0 * n ** 3 / vwall / 1e9, 2), "rel_error_vendor_fp32": verr,
                "dtype": {"FP16TCEC": "f16 hi/lo", "bf16x3": "bf16 three-term split (stands in for TF32TCEC)",
                          "FP16TC": "f16, no correction terms (FP16TC)",
                          "bf16x2": "bf16 two-term split (stands in for TF32TC)"}[mode_name],
                "roofline": mfma_roofline(2.0 * n ** 3, ev, prods, "pack_split_pair_kernel + gemm_tcec_kernel " +
                                          ("(packed, one tile per workgroup)" if mode_name == "FP16TC"
                                           else "(persistent, packed)"))}
        del ref
    del A, B, A32, B32
    torch.cuda.empty_cache()

    # C3: strided-batched CGEMM, batch 64 x 512^3
    bs, s = 64, 512
    za = torch.from_numpy(inputs.complex_normal(1, bs * s * s, (1.0 / (2 * s)) ** 0.5).view(np.float32)).to(dev)
    zb = torch.from_numpy(inputs.complex_normal(2, bs * s * s, (1.0 / (2 * s)) ** 0.5).view(np.float32)).to(dev)
    zc = torch.zeros(bs * s * s * 2, device=dev)
    fn = lambda: h.gemm_strided_batch(cg.OP_N, cg.OP_N, s, s, s, 1.0, za, s, s * s, zb, s, s * s, 0.0, zc, s, s * s,
                                      bs, cg.FP16TCEC, cplx=True)
    log("[bench] C3 batched CGEMM")
    wall, ev = timed(fn, 20, 3)
    ZA = torch.view_as_complex(za.view(bs, s, s, 2)).transpose(1, 2).to(torch.complex128)
    ZB = torch.view_as_complex(zb.view(bs, s, s, 2)).transpose(1, 2).to(torch.complex128)
    ZC = torch.view_as_complex(zc.view(bs, s, s, 2)).transpose(1, 2).to(torch.complex128)
    za32 = torch.view_as_complex(za.view(bs, s, s, 2)).transpose(1, 2)
    zb32 = torch.view_as_complex(zb.view(bs, s, s, 2)).transpose(1, 2)
    vwall, _ = timed(lambda: torch.matmul(za32, zb32), 20, 2)
    zref = ZA @ ZB
    res["C3_cgemm_batch64_512"] = {
        "tflops": round(8.0 * s ** 3 * bs / wall / 1e9, 2), "rel_error": rel_err(ZC, zref),
        "vendor_complex64_matmul_tflops": round(8.0 * s ** 3 * bs / vwall / 1e9, 2),
        "rel_error_vendor_complex64": rel_err(torch.matmul(za32, zb32).to(torch.complex128), zref),
        "dtype": "f16 hi/lo, four real products per complex product (12 MFMA products per complex multiply-add)",
        "roofline": mfma_roofline(8.0 * s ** 3 * bs, ev, 3, "gemm_tcec_kernel (complex)")}
    del za, zb, zc, ZA, ZB, ZC, zref
    torch.cuda.empty_cache()

    # C4: FP16TCEC_SCALING pipeline at 4096^3 with 2^{+-30} row/column exponents
    n = 4096
    ea = inputs.exponent_spread(3, n, n, per_row=True)
    eb = inputs.exponent_spread(4, n, n, per_row=False)
    a4, b4 = torch.from_numpy(ea).to(dev), torch.from_numpy(eb).to(dev)
    c4 = torch.zeros(n * n, device=dev)
    ref = a4.view(n, n).t().double() @ b4.view(n, n).t().double()
    log("[bench] C4 scaling pipeline")
    fn = lambda: h.gemm_pipeline(cg.OP_N, cg.OP_N, n, n, n, 1.0, a4, n, b4, n, 0.0, c4, n, cg.FP16TCEC_SCALING)
    wall, ev = timed(fn, 10, 2)
    err_scaled = rel_err(c4.view(n, n).t().double(), ref)
    awall, aev = timed(lambda: h.gemm_pipeline(cg.OP_N, cg.OP_N, n, n, n, 1.0, a4, n, b4, n, 0.0, c4, n, cg.AUTO), 10, 2)
    err_auto = rel_err(c4.view(n, n).t().double(), ref)
    vwall, _ = timed(lambda: torch.matmul(a4.view(n, n).t(), b4.view(n, n).t()), 10, 2)
    err_fp32 = rel_err((a4.view(n, n).t() @ b4.view(n, n).t()).double(), ref)
    st_ms = timed(lambda: h.exp_stats_ext(n, n, a4, n), 20, 3)[1]
    mx_ms = timed(lambda: h.exp_max_ext(n, n, a4, n), 20, 3)[1]
    # what the pipelines launch: A and B scanned by one launch per pass
    stp_ms = timed(lambda: h.exp_stats_pair(n, n, a4, n, n, n, b4, n), 20, 3)[1]
    mxp_ms = timed(lambda: h.exp_max_pair(n, n, a4, n, n, n, b4, n), 20, 3)[1]
    sid = h.exp_max_ext(n, n, a4, n)
    sc_ms = timed(lambda: (h.scale_A(sid, 1, n, n, a4, n), h.reset_scale_A(sid, 1, n, n, a4, n)), 20, 3)[1] / 2
    nbytes = 4.0 * n * n
    res["C4_scaling_4096"] = {
        "pipeline_tflops": round(2.0 * n ** 3 / wall / 1e9, 2), "auto_pipeline_tflops": round(2.0 * n ** 3 / awall / 1e9, 2),
        "rel_error_scaling": err_scaled, "rel_error_auto": err_auto, "rel_error_vendor_fp32": err_fp32,
        "vendor_fp32_matmul_tflops": round(2.0 * n ** 3 / vwall / 1e9, 2),
        "dtype": "f16 hi/lo after one power-of-two scaling per matrix (AUTO decides for bf16x3 on these inputs)",
        # the whole pipeline of one call: exp_max of A and B (one launch), pre-split with scaling, GEMM
        "roofline": mfma_roofline(2.0 * n ** 3, ev, 3, "exp_stats_kernel<max> + pack_split_pair_kernel + gemm_tcec_kernel (packed, scaled)"),
        # two passes (stage 1 + stage 2) over one 64 MiB matrix / one pass / read + write
        "roofline_exp_stats": hbm_roofline(2 * nbytes, st_ms, "exp_stats_kernel<0> + exp_stats_kernel<1>"),
        "roofline_exp_max": hbm_roofline(nbytes, mx_ms, "exp_stats_kernel<2>"),
        # A and B (2 x 64 MiB) in one launch per pass, as the FP16TCEC_SCALING / AUTO pipelines scan them
        "roofline_exp_stats_pair": hbm_roofline(4 * nbytes, stp_ms, "exp_stats_kernel<0> + exp_stats_kernel<1>, A and B per launch"),
        "roofline_exp_max_pair": hbm_roofline(2 * nbytes, mxp_ms, "exp_stats_kernel<2>, A and B in one launch"),
        "roofline_scaling": hbm_roofline(2 * nbytes, sc_ms, "scaling_kernel")}
    del a4, b4, c4, ref
    torch.cuda.empty_cache()

    # C5a: tall-skinny 16384 x 16384 x 256
    mm, kk = 16384, 256
    a5 = torch.from_numpy(inputs.uniform(1, mm * kk)).to(dev)
    b5 = torch.from_numpy(inputs.uniform(2, kk * mm)).to(dev)
    c5 = torch.zeros(mm * mm, device=dev)
    log("[bench] C5a tall-skinny")
    fn = lambda: h.gemm(cg.OP_N, cg.OP_N, mm, mm, kk, 1.0, a5, mm, b5, kk, 0.0, c5, mm, cg.FP16TCEC)
    wall, ev = timed(fn, 10, 2)
    _, mid5 = h.gemm(cg.OP_N, cg.OP_N, mm, mm, kk, 1.0, a5, mm, b5, kk, 0.0, c5, mm, cg.FP16TCEC, want_module_id=True)
    ref = a5.view(kk, mm).t().double() @ b5.view(mm, kk).t().double()
    A32, B32 = a5.view(kk, mm).t(), b5.view(mm, kk).t()
    vwall, _ = timed(lambda: torch.matmul(A32, B32), 10, 2)
    res["C5a_16384x16384x256"] = {
        "tflops": round(2.0 * mm * mm * kk / wall / 1e9, 2), "rel_error": rel_err(c5.view(mm, mm).t().double(), ref),
        "vendor_fp32_matmul_tflops": round(2.0 * mm * mm * kk / vwall / 1e9, 2),
        "rel_error_vendor_fp32": rel_err(torch.matmul(A32, B32).double(), ref), "dtype": "f16 hi/lo",
        "c_write_floor_ms": round(4.0 * mm * mm / (HBM_PEAK_GBS * 1e9) * 1e3, 4),
        "roofline": mfma_roofline(2.0 * mm * mm * kk, ev, 3,
                                  "pack_split_pair_kernel + gemm_tcec_kernel (persistent, packed)" if mid5 == 200
                                  else "gemm_tcec_kernel (in-loop split, persistent)")}
    del a5, b5, c5, ref
    torch.cuda.empty_cache()

    # C5b: Mx2x2 CGEMM, M = 2^27 (state vector x 2x2 unitary), HBM-bound
    M = 1 << 27
    log("[bench] C5b Mx2x2")
    x = torch.randn(M * 2 * 2, device=dev) * (0.5 ** 0.5)
    u = torch.from_numpy(inputs.random_unitary_2x2(9).view(np.float32)).to(dev)
    y = torch.zeros(M * 2 * 2, device=dev)
    fn = lambda: h.gemm_Mx2x2(cg.OP_N, cg.OP_N, M, 1.0, x, M, u, 2, 0.0, y, M, cplx=True)
    wall, ev = timed(fn, 10, 2)
    X = torch.view_as_complex(x.view(2, M, 2)[:, : 1 << 20].contiguous()).t().to(torch.complex128)
    Y = torch.view_as_complex(y.view(2, M, 2)[:, : 1 << 20].contiguous()).t().to(torch.complex128)
    U = torch.view_as_complex(u.view(2, 2, 2)).t().to(torch.complex128)
    res["C5b_cgemm_2^27x2x2"] = {
        "GBs": round(2.0 * M * 2 * 8 / ev / 1e6, 1), "rel_error_first_2^20_rows": rel_err(Y, X @ U),
        "dtype": "f32 (plain FMA streaming kernel: wider than FP16TCEC, as the reference's external Mx2x2 kernels)",
        "roofline": hbm_roofline(2.0 * M * 2 * 8, ev, "long2x2_kernel")}
    return res


if __name__ == "__main__":
    main()
