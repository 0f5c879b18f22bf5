"""Operands whose byte offsets do not fit 32 bits (more than 4 GiB in one
matrix): every kernel addresses with 64-bit arithmetic.  The inputs are made on
the device and the FP64 product of the same operands is the reference, with the
rows / columns that live beyond the 4 GiB mark also checked on their own."""
import pytest

pytestmark = pytest.mark.gpu
N_OP, T_OP = 111, 112
FP16TCEC, TF32TCEC, SCALING = 1, 2, 11
GIB4_ELEMS = 1 << 30                     # floats in 4 GiB


def _rel(torch, c, ref):
    return (torch.linalg.norm(c.double() - ref) / torch.linalg.norm(ref)).item()


@pytest.mark.parametrize("op_a", [N_OP, T_OP])
@pytest.mark.parametrize("mode", [FP16TCEC, TF32TCEC])
def test_tall_operand_beyond_4gib(cg, torch_gpu, handle, op_a, mode):
    torch = torch_gpu
    dev = torch.device("cuda:0")
    m, n, k = (1 << 20) + 192, 96, 1056
    assert m * k > GIB4_ELEMS
    g = torch.Generator(device=dev).manual_seed(5)
    # column-major m x k (N) is a row-major k x m tensor; T stores k x m column-major
    a = torch.rand((k, m) if op_a == N_OP else (m, k), generator=g, device=dev) - 0.5
    b = torch.rand((n, k), generator=g, device=dev) - 0.5        # column-major k x n
    c = torch.zeros((n, m), device=dev)                            # column-major m x n
    lda = m if op_a == N_OP else k
    st = handle.gemm(op_a, N_OP, m, n, k, 1.0, a, lda, b, k, 0.0, c, m, mode)
    assert st == 0
    torch.cuda.synchronize()
    bar = 2.0 ** -23 * k ** 0.5
    a_log = a if op_a == N_OP else a.t()                           # (k, m) view: A^T
    # reference by blocks of rows of C, so that the FP64 copy of A stays small
    worst = 0.0
    for r0 in range(0, m, 1 << 18):
        r1 = min(m, r0 + (1 << 18))
        ref = b.double() @ a_log[:, r0:r1].double()                # (n, rows) = C^T block
        worst = max(worst, _rel(torch, c[:, r0:r1], ref))
    assert worst < bar, worst
    del a, c
    torch.cuda.empty_cache()


def test_result_beyond_4gib(cg, torch_gpu, handle):
    torch = torch_gpu
    dev = torch.device("cuda:0")
    m, n, k = (1 << 20) + 64, 1040, 64
    assert m * n > GIB4_ELEMS
    g = torch.Generator(device=dev).manual_seed(6)
    a = torch.rand((k, m), generator=g, device=dev) - 0.5          # column-major m x k
    b = torch.rand((n, k), generator=g, device=dev) - 0.5
    c = torch.full((n, m), 0.25, device=dev)
    st = handle.gemm(N_OP, N_OP, m, n, k, 2.0, a, m, b, k, -1.0, c, m, FP16TCEC)
    assert st == 0
    torch.cuda.synchronize()
    bar = 2.0 ** -23 * k ** 0.5
    worst = 0.0
    for c0 in range(0, n, 130):
        c1 = min(n, c0 + 130)
        ref = 2.0 * (b[c0:c1].double() @ a.double()) - 0.25
        worst = max(worst, _rel(torch, c[c0:c1], ref))
    assert worst < bar, worst
    del a, c
    torch.cuda.empty_cache()


def test_pre_split_operand_beyond_4gib(cg, torch_gpu, handle):
    """32768 x 32768 A: its fp16 planes, like the source, span more than 4 GiB."""
    torch = torch_gpu
    dev = torch.device("cuda:0")
    m, n, k = 32768, 4096, 32768 + 32
    assert m * k > GIB4_ELEMS
    g = torch.Generator(device=dev).manual_seed(7)
    a = torch.rand((k, m), generator=g, device=dev) - 0.5
    b = torch.rand((n, k), generator=g, device=dev) - 0.5
    c = torch.zeros((n, m), device=dev)
    st, mid = handle.gemm(N_OP, N_OP, m, n, k, 1.0, a, m, b, k, 0.0, c, m, FP16TCEC, want_module_id=True)
    assert st == 0 and mid == 200
    torch.cuda.synchronize()
    assert handle.workspace_size() >= (m + n) * k * 4
    bar = 2.0 ** -23 * k ** 0.5
    worst = 0.0
    for r0 in range(0, m, 8192):
        ref = b.double() @ a[:, r0:r0 + 8192].double()
        worst = max(worst, _rel(torch, c[:, r0:r0 + 8192], ref))
        del ref
    assert worst < bar, worst
    del a, b, c
    torch.cuda.empty_cache()


def test_statistics_and_scaling_beyond_4gib(cg, torch_gpu, handle):
    torch = torch_gpu
    dev = torch.device("cuda:0")
    m, n = (1 << 20) + 320, 1030
    ld = m + 8
    assert m * n > GIB4_ELEMS
    x = torch.full((n, ld), 0.5, device=dev)
    x[:, m:] = 7e4                                  # padding rows are not part of the matrix
    x[n - 3:, :m] = 2.0 ** -20                      # under the threshold, in the last columns only
    x[n - 1, m - 1] = 3.0                           # the maximum sits in the very last element
    handle.set_exp_stats_params(2.0 ** -40, 2.0 ** -15, 0.1)
    try:
        sid = handle.exp_stats_ext(m, n, x, ld)
        under, total = handle.get_exp_stats(sid)
        assert (under, total) == (3 * m - 1, m * n)
        assert handle.get_max_exp(sid) == 2.0
        assert handle.get_exp_stats_compute_mode_level(sid) == FP16TCEC
        mid = handle.exp_max_ext(m, n, x, ld)
        assert handle.get_max_exp(mid) == 2.0
        # preset flag slot 1 asks for scaling: times 2^14 / 2^1, the padding is left alone
        handle.scale_A(mid, 1, m, n, x, ld)
        torch.cuda.synchronize()
        f = 8192.0
        assert x[0, 0].item() == 0.5 * f and x[n - 1, m - 1].item() == 3.0 * f
        assert x[n - 2, m - 5].item() == 2.0 ** -20 * f
        assert x[n - 1, m].item() == 7e4 and x[5, m + 7].item() == 7e4
        assert torch.count_nonzero(x[:, :m] == 0.5 * f).item() == (n - 3) * m
        assert torch.count_nonzero(x[:, m:] == 7e4).item() == 8 * n
    finally:
        handle.set_exp_stats_params(0.0, 2.0 ** -15, 0.0)
    del x
    torch.cuda.empty_cache()


def test_statistics_count_beyond_32_bits(cg, torch_gpu, handle):
    """A dense matrix of more than 2^32 elements: the counters are 64 bits wide."""
    torch = torch_gpu
    dev = torch.device("cuda:0")
    m, n = 1 << 20, 4100
    assert m * n > 1 << 32
    x = torch.full((n, m), 2.0 ** -18, device=dev)
    x[n - 1, m - 7:] = 40.0
    try:
        sid = handle.exp_stats_ext(m, n, x, m)
        under, total = handle.get_exp_stats(sid)
        # first pass: nearly everything is under 2^-15, so the second pass recounts against
        # thresholds relative to the maximum (2^5): 2^-18 < 2^-16 * 2^5 still counts as lost
        assert (under, total) == (m * n - 7, m * n)
        assert handle.get_max_exp(sid) == 32.0
        assert handle.get_exp_stats_compute_mode_level(sid) == TF32TCEC
    finally:
        handle.set_exp_stats_params(0.0, 2.0 ** -15, 0.0)
    del x
    torch.cuda.empty_cache()
