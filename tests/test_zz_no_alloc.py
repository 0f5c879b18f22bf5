"""cuMpSGEMM_sgemm_no_alloc -- the variant of cuMpSGEMM_sgemm that keeps the pre-split planes in
the library's static device array -- against cuMpSGEMM_sgemm itself, through the C ABI: two calls
in a row, the second with a smaller input (the array keeps the first call's contents), plus the
size limit.  Bar: bit-identical where the existing entry point takes its pre-split path too (the
same kernels on the same planes); where it splits in the K loop (MFMAs that add 16 K-values
where the pre-split kernels' add 32) or splits K (float atomics without a fixed order),
agreement to the summation-order tolerance 4 * 2^-24 * sqrt(K) (relative Frobenius)."""
import numpy as np
import pytest

from cumpsgemm_amd import inputs

pytestmark = pytest.mark.gpu
N_OP, T_OP = 111, 112
FP16TCEC, TF32TCEC, FP16TC = 1, 2, 3


def _pair(cg, torch, h, mode, opa, opb, m, n, k, alpha, beta, seed, fp64_bar=False):
    dev = torch.device("cuda:0")
    pad = 3
    lda = (m if opa == N_OP else k) + pad
    ldb = (k if opb == N_OP else n) + pad
    ldc = m + pad
    a = torch.from_numpy(inputs.uniform(seed, lda * (k if opa == N_OP else m))).to(dev)
    b = torch.from_numpy(inputs.uniform(seed + 1, ldb * (n if opb == N_OP else k))).to(dev)
    c0 = torch.from_numpy(inputs.uniform(seed + 2, ldc * n)).to(dev)
    c_ref, c_new = c0.clone(), c0.clone()
    st, mid = h.gemm(opa, opb, m, n, k, alpha, a, lda, b, ldb, beta, c_ref, ldc, mode, want_module_id=True)
    assert st == 0
    torch.cuda.synchronize()
    ws_before = h.workspace_size()
    free_before = torch.cuda.mem_get_info()[0]
    st = h.gemm_no_alloc(opa, opb, m, n, k, alpha, a, lda, b, ldb, beta, c_new, ldc, mode)
    assert st == 0
    torch.cuda.synchronize()
    assert h.workspace_size() == ws_before and torch.cuda.mem_get_info()[0] == free_before
    if mid == 200:
        assert torch.equal(c_new, c_ref), (mode, opa, opb, m, n, k, mid)
    else:
        x, y = c_new.double(), c_ref.double()
        assert float((x - y).norm() / y.norm()) <= 4 * 2.0 ** -24 * np.sqrt(k), (m, n, k, mid)
    # the padding of C (rows m .. ldc) is untouched
    assert torch.equal(c_new.view(n, ldc)[:, m:], c0.view(n, ldc)[:, m:])
    if fp64_bar:   # small problems: against FP64 as well, within the reference's bar 2^-23 sqrt(K)
        A = a.view(-1, lda)[:, :(m if opa == N_OP else k)].double()
        A = A.t() if opa == N_OP else A                 # logical m x k
        B = b.view(-1, ldb)[:, :(k if opb == N_OP else n)].double()
        B = B.t() if opb == N_OP else B                 # logical k x n
        ref = alpha * (A @ B) + beta * c0.view(n, ldc)[:, :m].t().double()
        got = c_new.view(n, ldc)[:, :m].t().double()
        assert float((got - ref).norm() / ref.norm()) <= 2.0 ** -23 * np.sqrt(k), (m, n, k)


@pytest.mark.parametrize("mode", [FP16TCEC, TF32TCEC])
def test_no_alloc_matches_sgemm_on_two_calls_in_a_row(cg, torch_gpu, mode):
    h = cg.Handle()
    h.set_stream(torch_gpu.cuda.current_stream())
    try:
        # (4096 + 4096) * 1024 * 4 (6) bytes = 32 (48) MiB of the 64 MiB array ...
        _pair(cg, torch_gpu, h, mode, N_OP, N_OP, 4096, 4096, 1024, 1.0, 0.0, 100)
        # ... then smaller, ragged problems over the same array: other layouts, beta != 0
        _pair(cg, torch_gpu, h, mode, T_OP, N_OP, 1000, 777, 520, 0.5, 0.25, 110)
        _pair(cg, torch_gpu, h, mode, N_OP, T_OP, 300, 2500, 131, -1.0, 1.0, 120)
    finally:
        torch_gpu.cuda.synchronize()
        h.close()


@pytest.mark.parametrize("mode", [FP16TCEC, TF32TCEC])
def test_no_alloc_on_problems_smaller_than_one_tile(cg, torch_gpu, mode, monkeypatch):
    """The call takes the pre-split path whatever the shape: results narrower or lower than the
    256 x 128 (128 x 128) tile of its kernels, down to a single row or column -- and whatever
    the variables say that steer cuMpSGEMM_sgemm away from that path."""
    h = cg.Handle()
    h.set_stream(torch_gpu.cuda.current_stream())
    try:
        _pair(cg, torch_gpu, h, mode, N_OP, N_OP, 70, 33, 130, 1.0, 0.0, 130, fp64_bar=True)
        _pair(cg, torch_gpu, h, mode, T_OP, N_OP, 1, 4096, 256, 1.5, -0.5, 140, fp64_bar=True)
        _pair(cg, torch_gpu, h, mode, N_OP, T_OP, 4100, 1, 160, 1.0, 1.0, 150, fp64_bar=True)
        monkeypatch.setenv("CUMPSGEMM_PACKED", "0")
        monkeypatch.setenv("CUMPSGEMM_FORCE_TILE_CLASS", "2")
        monkeypatch.setenv("CUMPSGEMM_FORCE_KSPLIT", "4")
        _pair(cg, torch_gpu, h, mode, N_OP, N_OP, 300, 200, 256, 1.0, 0.0, 160, fp64_bar=True)
    finally:
        torch_gpu.cuda.synchronize()
        h.close()


def test_no_alloc_refuses_what_it_cannot_hold(cg, torch_gpu):
    torch = torch_gpu
    dev = torch.device("cuda:0")
    h = cg.Handle()
    h.set_stream(torch.cuda.current_stream())
    try:
        assert cg.lib().cuMpSGEMM_get_static_scratch_size() == 64 << 20
        m = n = 4096
        k = 2048 + 32                                  # one K-step over the limit
        a = torch.zeros(m * k, device=dev)
        b = torch.zeros(k * n, device=dev)
        c = torch.full((m * n,), 3.0, device=dev)
        assert h.gemm_no_alloc(N_OP, N_OP, m, n, k, 1.0, a, m, b, k, 0.0, c, m, FP16TCEC) == 3
        assert h.gemm_no_alloc(N_OP, N_OP, m, n, 2048, 1.0, a, m, b, 2048, 0.0, c, m, TF32TCEC) == 3
        assert h.gemm_no_alloc(N_OP, N_OP, m, n, 64, 1.0, a, m, b, 64, 0.0, c, m, FP16TCEC) == 3
        assert h.gemm_no_alloc(N_OP, N_OP, m, n, 1024, 1.0, a, m, b, 1024, 0.0, c, m, FP16TC) == 3
        torch.cuda.synchronize()
        assert float(c.min()) == 3.0 and float(c.max()) == 3.0   # refused calls write nothing
        assert h.gemm_no_alloc(N_OP, N_OP, m, n, 2048, 1.0, a, m, b, 2048, 0.0, c, m, FP16TCEC) == 0
        torch.cuda.synchronize()
        assert float(c.abs().max()) == 0.0
    finally:
        torch.cuda.synchronize()
        h.close()
