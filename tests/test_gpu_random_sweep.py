"""Seeded random problems at sizes the CPU oracle would take minutes for: large
shapes around the thresholds of the pre-split paths, every op, odd leading
dimensions, alpha / beta, the scaling pipelines, real and complex.  The
reference is the FP64 product of the same operands on the GPU (the vendor's
DGEMM / ZGEMM through torch), the bar the reference harness's: relative
Frobenius residual below 2^-23 * sqrt(K) for the corrected modes, 2^-10 *
sqrt(K) for FP16TC (test/main.cu:68-74); with beta != 0 the bar is widened by
the FP32 rounding of beta * C."""
import random

import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", [3, 11])
def test_random_large_problems(cg, torch_gpu, seed):
    torch = torch_gpu
    dev = torch.device("cuda:0")
    h = cg.Handle()
    h.set_stream(torch.cuda.current_stream())
    h.set_exp_stats_params(0.0, 2.0 ** -15, 0.1)  # AUTO may decide for scaled FP16TCEC
    rng = random.Random(seed)
    ops = {"N": cg.OP_N, "T": cg.OP_T, "C": cg.OP_C}
    failures = []
    try:
        for case in range(40):
            cplx = rng.random() < 0.3
            if rng.random() < 0.6:
                m, n = rng.randint(2000, 5200), rng.randint(2000, 5200)
                k = rng.choice([rng.randint(128, 2100), 256, 512, 1024, 300])
            else:
                m, n, k = rng.randint(1, 700), rng.randint(1, 700), rng.randint(1, 3000)
            oa = rng.choice("NTC" if cplx else "NT")
            ob = rng.choice("NTC" if cplx else "NT")
            mode_name = rng.choice(["FP16TCEC", "TF32TCEC", "FP16TCEC_SCALING", "AUTO", "FP16TC"])
            mode = getattr(cg, mode_name)
            dt = torch.complex64 if cplx else torch.float32
            ar, ac = (m, k) if oa == "N" else (k, m)
            br, bc = (k, n) if ob == "N" else (n, k)
            lda, ldb, ldc = ar + rng.choice([0, 0, 1, 7]), br + rng.choice([0, 0, 3]), m + rng.choice([0, 0, 5])
            scale = rng.choice([1.0, 1.0, 2.0 ** -20, 2.0 ** 6])
            gen = torch.Generator(device=dev)
            gen.manual_seed(1000 * seed + case)
            a = torch.randn(ac, lda, device=dev, dtype=dt, generator=gen) * scale   # column-major ar x ac
            b = torch.randn(bc, ldb, device=dev, dtype=dt, generator=gen)
            c0 = torch.randn(n, ldc, device=dev, dtype=dt, generator=gen)
            alpha = rng.choice([1.0, 1.0, -0.5, 2.0])
            beta = rng.choice([0.0, 0.0, 1.0, -0.25])
            pipeline = mode_name in ("FP16TCEC_SCALING", "AUTO")
            if pipeline:
                beta = 0.0
            c = c0.clone()
            fa, fb, fc = (torch.view_as_real(t).reshape(-1) if cplx else t.reshape(-1) for t in (a, b, c))
            what = (f"case {case}: {'c' if cplx else 's'} {mode_name} {oa}{ob} m={m} n={n} k={k} "
                    f"ld=({lda},{ldb},{ldc}) alpha={alpha} beta={beta} scale={scale}")
            print(what, flush=True)
            if pipeline:
                st, _ = h.gemm_pipeline(ops[oa], ops[ob], m, n, k, alpha, fa, lda, fb, ldb, beta, fc, ldc, mode,
                                        cplx=cplx)
            else:
                st = h.gemm(ops[oa], ops[ob], m, n, k, alpha, fa, lda, fb, ldb, beta, fc, ldc, mode, cplx=cplx)
            assert st == 0, what
            torch.cuda.synchronize()
            wide = torch.complex128 if cplx else torch.float64

            def logical(t, rows, op):
                x = t[:, :rows].transpose(0, 1).to(wide)
                return x if op == "N" else (x.transpose(0, 1).conj() if op == "C" else x.transpose(0, 1))
            ref = alpha * (logical(a, ar, oa) @ logical(b, br, ob)) + beta * c0[:, :m].transpose(0, 1).to(wide)
            got = c[:, :m].transpose(0, 1).to(wide)
            res = (torch.linalg.norm(got - ref) / torch.linalg.norm(ref)).item()
            bar = (2.0 ** -10 if mode_name == "FP16TC" else 2.0 ** -23) * max(k, 1) ** 0.5 * (4 if beta != 0 else 1)
            if mode_name in ("FP16TCEC", "FP16TC") and scale < 1e-3:
                bar = 1.0  # unscaled fp16 loses inputs this small by design; only the other checks apply
            if not res < bar:
                failures.append(f"{what}: residual {res:.3e} >= {bar:.3e}")
            if not torch.equal(c[:, m:], c0[:, m:]):
                failures.append(f"{what}: padding rows of C were written")
            if pipeline and float(a.abs().max()) > 8 * scale:   # (a scaled operand would peak near 2^14)
                failures.append(f"{what}: operand A was left scaled")
    finally:
        torch.cuda.synchronize()
        h.close()
    assert not failures, "\n".join(failures)
