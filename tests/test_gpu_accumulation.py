"""Long sums of same-sign products.  The kernels keep the leading (hi * hi) sum in the MFMA
accumulator for the whole K range instead of starting every K-slice from zero and adding the
slices in FP32 outside the matrix unit, which is what the reference's arithmetic library does to
get round a truncating tensor-core accumulate.  Zero-mean data would hide such a truncation inside
the 2^-23 * sqrt(K) bar (the errors cancel); operands that are all positive do not: a truncating
accumulate loses about half an ulp of the running sum per addition, always in the same direction,
i.e. a relative error near K/16 * 2^-25 (K = 32768: 6e-5 against a bar of 2.2e-5, and against
about 1e-6 for round-to-nearest)."""
import numpy as np
import pytest

from cumpsgemm_amd import inputs
from gpu_util import N, T, assert_same_up_to_summation_order, oracle_gemm, rel_diff

pytestmark = pytest.mark.gpu
FP16TCEC, TF32TCEC, FP32 = 1, 2, 12


def _positive(seed, count):
    return inputs.uniform(seed, count, 0.5, 1.0)


@pytest.mark.parametrize("mode", [FP16TCEC, TF32TCEC])
@pytest.mark.parametrize("form,m,n,k", [
    ("one_chain", 256, 192, 8192),      # one workgroup per tile sums all of K in one accumulator
    ("one_chain", 256, 192, 32768),
    ("split_k", 256, 192, 32768),       # the planner's own choice for a small C: K split, float atomics
    ("walk", 1024, 768, 1024),          # persistent kernel (32 K-steps per tile)
])
def test_same_sign_operands_in_loop_kernels(O, handle, dev, monkeypatch, mode, form, m, n, k):
    monkeypatch.setenv("CUMPSGEMM_PACKED", "0")
    if form != "split_k":
        monkeypatch.setenv("CUMPSGEMM_FORCE_KSPLIT", "1")
    a, b = _positive(51, m * k), _positive(52, k * n)
    da, db, dc = dev.up(a), dev.up(b), dev.up(np.zeros(m * n, np.float32))
    st, mid = handle.gemm(T, N, m, n, k, 1.0, da, k, db, k, 0.0, dc, m, mode, want_module_id=True)
    assert st == 0
    assert (mid >= 100) == (form == "split_k"), mid
    c = dev.down(dc)
    ref = O.gemm_fp64(T, N, m, n, k, 1.0, a, k, b, k)
    zero = np.zeros(m * n, np.float32)
    c_or = oracle_gemm(O, mode, T, N, m, n, k, 1.0, a, k, b, k, 0.0, zero, m)
    c32 = oracle_gemm(O, FP32, T, N, m, n, k, 1.0, a, k, b, k, 0.0, zero, m)
    r, r_or, r32 = O.residual(ref, c, m, n, m), O.residual(ref, c_or, m, n, m), O.residual(ref, c32, m, n, m)
    assert r < 2.0 ** -23 * np.sqrt(k), (r, r_or, r32)
    assert r <= 2.0 * r32, (r, r32)
    assert rel_diff(c, c_or, m, n, m) <= 4 * 2.0 ** -24 * np.sqrt(k)


@pytest.mark.parametrize("mode", [FP16TCEC, TF32TCEC])
def test_same_sign_operands_pre_split_kernels(cg, torch_gpu, monkeypatch, mode):
    """The pre-split kernels at K = 8192 (one tile per workgroup, 256 K-steps in one accumulator):
    the in-loop kernels' result up to the order of summation (their MFMAs add 16 K-values, the
    pre-split kernels' 32), and within the bars against an FP64 product."""
    torch = torch_gpu
    dev = torch.device("cuda:0")
    m, n, k = 4096, 2048, 8192
    g = torch.Generator(device=dev).manual_seed(53)
    a = torch.rand((m, k), generator=g, device=dev) * 0.5 + 0.5     # column-major k x m: op_A = T
    b = torch.rand((n, k), generator=g, device=dev) * 0.5 + 0.5     # column-major k x n
    h = cg.Handle()
    h.set_stream(torch.cuda.current_stream())
    try:
        outs = []
        monkeypatch.setenv("CUMPSGEMM_NO_COLUMN_SPLIT", "1")   # one launch, K unsplit: a fixed summation order
        monkeypatch.setenv("CUMPSGEMM_FORCE_KSPLIT", "1")
        for packed in ("1", "0"):
            monkeypatch.setenv("CUMPSGEMM_PACKED", packed)
            c = torch.zeros((n, m), device=dev)
            st, mid = h.gemm(T, N, m, n, k, 1.0, a, k, b, k, 0.0, c, m, mode, want_module_id=True)
            torch.cuda.synchronize()
            assert st == 0 and (mid == 200) == (packed == "1"), mid
            outs.append(c)
        assert_same_up_to_summation_order(outs[0], outs[1], k)
        ref = b.double() @ a.double().t()
        r = (torch.linalg.norm(outs[0].double() - ref) / torch.linalg.norm(ref)).item()
        r32 = (torch.linalg.norm((b @ a.t()).double() - ref) / torch.linalg.norm(ref)).item()
        assert r < 2.0 ** -23 * k ** 0.5 and r <= 2.0 * r32, (r, r32)
    finally:
        torch.cuda.synchronize()
        h.close()
