"""Every benchmark configuration at its real size, through the C ABI, against an FP64 product of the
same inputs (torch DGEMM / ZGEMM on the device, in blocks).  Bars: relative Frobenius residual at most
twice that of the vendor FP32 GEMM on the same inputs, and below 2^-23 * sqrt(K), the bar of the
reference's own test program (test/main.cu:68-74).  Inputs are made on the device with the
distribution each configuration names; A and B must come back unchanged."""
import numpy as np
import pytest

from cumpsgemm_amd import inputs

pytestmark = pytest.mark.gpu
N_OP, T_OP = 111, 112
FP16TCEC, TF32TCEC, AUTO, SCALING = 1, 2, 9, 11


def _residuals(torch, c_rows, ref_rows_fn, fp32_rows_fn, total_rows, step):
    """Relative Frobenius residuals of the result and of the FP32 comparator, accumulated over
    row blocks of the (row-major) result so that the FP64 copies stay small."""
    num = num32 = den = 0.0
    for r0 in range(0, total_rows, step):
        r1 = min(total_rows, r0 + step)
        ref = ref_rows_fn(r0, r1)
        num += float(((c_rows(r0, r1).double() - ref).abs() ** 2).sum())
        num32 += float(((fp32_rows_fn(r0, r1).double() - ref).abs() ** 2).sum())
        den += float((ref.abs() ** 2).sum())
        del ref
    return (num / den) ** 0.5, (num32 / den) ** 0.5


@pytest.mark.parametrize("mode", [FP16TCEC, TF32TCEC])
@pytest.mark.parametrize("layout", ["NN", "TN", "NT"])
def test_c2_sgemm_8192_cubed(cg, torch_gpu, handle, mode, layout):
    torch = torch_gpu
    dev = torch.device("cuda:0")
    s = 8192
    g = torch.Generator(device=dev).manual_seed(1)
    a = torch.rand((s, s), generator=g, device=dev) * 2 - 1      # the stored (column-major) square matrices
    b = torch.rand((s, s), generator=g, device=dev) * 2 - 1
    a0, b0 = a.clone(), b.clone()
    c = torch.full((s, s), float("nan"), device=dev)             # beta = 0 must not read C
    opa = T_OP if layout[0] == "T" else N_OP
    opb = T_OP if layout[1] == "T" else N_OP
    st, mid = handle.gemm(opa, opb, s, s, s, 1.0, a, s, b, s, 0.0, c, s, mode, want_module_id=True)
    torch.cuda.synchronize()
    assert st == 0 and mid == 200                                # the pre-split path, as in the benchmark
    # row-major views: a column-major m x k matrix is the (k, m) tensor; C^T = op(B)^T op(A)^T
    at = a if opa == N_OP else a.t()                             # (k, m)
    bt = b if opb == N_OP else b.t()                             # (n, k)
    r, r32 = _residuals(torch, lambda r0, r1: c[r0:r1],
                        lambda r0, r1: bt[r0:r1].double() @ at.double(),
                        lambda r0, r1: bt[r0:r1] @ at, s, 2048)
    assert r <= 2.0 * r32 and r < 2.0 ** -23 * s ** 0.5, (r, r32)
    assert torch.equal(a, a0) and torch.equal(b, b0)


def test_c3_cgemm_batch64_512_cubed(cg, torch_gpu, handle):
    torch = torch_gpu
    dev = torch.device("cuda:0")
    s, batch = 512, 64
    g = torch.Generator(device=dev).manual_seed(3)
    sigma = (1.0 / (2 * s)) ** 0.5
    a = torch.view_as_complex(torch.randn((batch, s, s, 2), generator=g, device=dev) * sigma)
    b = torch.view_as_complex(torch.randn((batch, s, s, 2), generator=g, device=dev) * sigma)
    c = torch.view_as_complex(torch.full((batch, s, s, 2), float("nan"), device=dev))
    st = handle.gemm_strided_batch(N_OP, N_OP, s, s, s, 1.0, torch.view_as_real(a), s, s * s,
                                   torch.view_as_real(b), s, s * s, 0.0, torch.view_as_real(c), s, s * s,
                                   batch, FP16TCEC, cplx=True)
    torch.cuda.synchronize()
    assert st == 0
    ref = b.to(torch.complex128) @ a.to(torch.complex128)        # per matrix: C^T = B^T A^T
    r = (torch.linalg.norm(c.to(torch.complex128) - ref) / torch.linalg.norm(ref)).item()
    r32 = (torch.linalg.norm((b @ a).to(torch.complex128) - ref) / torch.linalg.norm(ref)).item()
    assert r <= 2.0 * r32 and r < 2.0 ** -23 * s ** 0.5, (r, r32)
    # every matrix of the batch on its own
    per = torch.linalg.norm((c.to(torch.complex128) - ref).reshape(batch, -1), dim=1) / \
        torch.linalg.norm(ref.reshape(batch, -1), dim=1)
    assert float(per.max()) < 2.0 ** -23 * s ** 0.5


@pytest.mark.parametrize("mode", [SCALING, AUTO])
@pytest.mark.parametrize("restore", [True, False])
def test_c4_scaling_stress_4096_cubed(O, cg, torch_gpu, handle, mode, restore):
    """A[i,k] = N(0,1) * 2^e_i, B[k,j] = N(0,1) * 2^f_j, e, f uniform in [-30, 30]: values far outside
    fp16's range.  The statistics are bit-exact with the oracle's scalar count; the GEMM of the
    pipeline (after one power-of-two scaling per matrix) keeps FP32-level accuracy."""
    torch = torch_gpu
    dev = torch.device("cuda:0")
    s = 4096
    a_np = inputs.exponent_spread(3, s, s, per_row=True)
    b_np = inputs.exponent_spread(4, s, s, per_row=False)
    a = torch.from_numpy(a_np).to(dev).view(s, s)                # (k, m) row-major = column-major m x k
    b = torch.from_numpy(b_np).to(dev).view(s, s)                # (n, k)
    a0, b0 = a.clone(), b.clone()
    c = torch.full((s, s), float("nan"), device=dev)
    st, ids = handle.gemm_pipeline(N_OP, N_OP, s, s, s, 1.0, a, s, b, s, 0.0, c, s, mode, restore_ab=restore)
    torch.cuda.synchronize()
    assert st == 0
    sa, sb = O.exp_stats(a_np, s, s, s), O.exp_stats(b_np, s, s, s)
    for sid, want in ((ids[0], sa), (ids[1], sb)):
        assert int(np.float32(handle.get_max_exp(sid)).view(np.uint32)) == want.max_exp_bits
        if mode == AUTO:
            assert handle.get_exp_stats(sid) == (want.underflow, want.total)
            assert handle.get_exp_stats_compute_mode_level(sid) == want.mode
    if mode == AUTO:
        assert handle.get_dynamic_launch_flag(ids[2]) == O.lib().oracle_combine_flag(sa.mode, sb.mode)
    r, r32 = _residuals(torch, lambda r0, r1: c[r0:r1],
                        lambda r0, r1: b0[r0:r1].double() @ a0.double(),
                        lambda r0, r1: b0[r0:r1] @ a0, s, 2048)
    assert r <= 2.0 * r32 and r < 2.0 ** -23 * s ** 0.5, (mode, r, r32)
    if restore:
        assert torch.equal(a, a0) and torch.equal(b, b0)
    elif mode == SCALING:
        # left scaled: one power of two per matrix, 2^14 / 2^floor(log2 max|x|)
        fa = 2.0 ** 14 / float(np.uint32(sa.max_exp_bits).view(np.float32))
        fb = 2.0 ** 14 / float(np.uint32(sb.max_exp_bits).view(np.float32))
        assert torch.equal(a, a0 * fa) and torch.equal(b, b0 * fb)


def test_c5a_tall_skinny_16384x16384x256(cg, torch_gpu, handle):
    torch = torch_gpu
    dev = torch.device("cuda:0")
    m = n = 16384
    k = 256
    g = torch.Generator(device=dev).manual_seed(5)
    a = torch.rand((k, m), generator=g, device=dev) * 2 - 1      # column-major m x k
    b = torch.rand((n, k), generator=g, device=dev) * 2 - 1      # column-major k x n
    a0, b0 = a.clone(), b.clone()
    c = torch.full((n, m), float("nan"), device=dev)
    st = handle.gemm(N_OP, N_OP, m, n, k, 1.0, a, m, b, k, 0.0, c, m, FP16TCEC)
    torch.cuda.synchronize()
    assert st == 0
    r, r32 = _residuals(torch, lambda r0, r1: c[r0:r1], lambda r0, r1: b[r0:r1].double() @ a.double(),
                        lambda r0, r1: b[r0:r1] @ a, n, 2048)
    assert r <= 2.0 * r32 and r < 2.0 ** -23 * k ** 0.5, (r, r32)
    assert torch.equal(a, a0) and torch.equal(b, b0)
    del c
    torch.cuda.empty_cache()


def test_c5b_gate_application_2_to_27(cg, torch_gpu, handle):
    """A state vector of 2^27 x 2 complex64 amplitudes times a random 2 x 2 unitary (QR of a seeded
    complex Gaussian), through the streaming kernel.  That kernel computes in plain FP32 (wider than
    FP16TCEC): its bar is the FP32 one, 2^-23 * sqrt(K) with K = 2."""
    torch = torch_gpu
    dev = torch.device("cuda:0")
    m = 1 << 27
    g = torch.Generator(device=dev).manual_seed(6)
    a = torch.view_as_complex(torch.randn((2, m, 2), generator=g, device=dev) * 0.5 ** 0.5)  # column-major m x 2
    u_np = inputs.random_unitary_2x2(9)                            # column-major: u[i + 2 j]
    u = torch.from_numpy(u_np).to(dev)
    c = torch.view_as_complex(torch.full((2, m, 2), float("nan"), device=dev))
    st = handle.gemm_Mx2x2(N_OP, N_OP, m, 1.0, torch.view_as_real(a), m, torch.view_as_real(u), 2, 0.0,
                           torch.view_as_real(c), m, cplx=True)
    torch.cuda.synchronize()
    assert st == 0
    u64 = torch.from_numpy(u_np.astype(np.complex128)).to(dev)
    num = den = 0.0
    step = 1 << 24
    for r0 in range(0, m, step):
        x0, x1 = a[0, r0:r0 + step].to(torch.complex128), a[1, r0:r0 + step].to(torch.complex128)
        for q in range(2):
            ref = x0 * u64[2 * q] + x1 * u64[2 * q + 1]
            num += float(((c[q, r0:r0 + step].to(torch.complex128) - ref).abs() ** 2).sum())
            den += float((ref.abs() ** 2).sum())
    r = (num / den) ** 0.5
    assert r < 2.0 ** -23 * 2 ** 0.5, r
    # a unitary keeps the norm of the state
    n_in = float(torch.linalg.vector_norm(a.to(torch.complex128)))
    n_out = float(torch.linalg.vector_norm(c.to(torch.complex128)))
    assert abs(n_out / n_in - 1.0) < 1e-6
    del a, c
    torch.cuda.empty_cache()
