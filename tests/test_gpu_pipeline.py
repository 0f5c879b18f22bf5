"""The mode pipelines (FP16TCEC_SCALING, AUTO) end to end on the GPU: the
statistics and flags they record, restoration of A and B, and the error of the
result against an FP64 GEMM, next to plain FP16TCEC and plain FP32."""
import numpy as np
import pytest

from cumpsgemm_amd import inputs
from gpu_util import N, T, assert_same_up_to_summation_order, oracle_gemm

pytestmark = pytest.mark.gpu
FP16TCEC, TF32TCEC, AUTO, SCALING, FP32 = 1, 2, 9, 11, 12


def _pipeline(handle, dev, mode, opa, opb, m, n, k, a, b, cplx=False, restore=True):
    lda = m if opa == N else k
    ldb = k if opb == N else n
    da, db = dev.up(a), dev.up(b)
    dc = dev.up(np.zeros(m * n, a.dtype))
    st, ids = handle.gemm_pipeline(opa, opb, m, n, k, 1.0, da, lda, db, ldb, 0.0, dc, m, mode, cplx=cplx,
                                   restore_ab=restore)
    assert st == 0
    dt = np.complex64 if cplx else np.float32
    return dev.down(dc, dt), dev.down(da, dt), dev.down(db, dt), ids


def test_scaling_rescues_tiny_inputs(O, handle, dev):
    """Inputs ~2^-20: plain FP16TCEC loses the lo term to fp16 underflow; after
    power-of-two scaling the result is as accurate as FP32."""
    m = n = k = 384
    a = (inputs.uniform(1, m * k) * np.float32(2.0 ** -20)).astype(np.float32)
    b = (inputs.uniform(2, k * n) * np.float32(2.0 ** -18)).astype(np.float32)
    ref = O.gemm_fp64(N, N, m, n, k, 1.0, a, m, b, k)
    r_fp32 = O.residual(ref, oracle_gemm(O, FP32, N, N, m, n, k, 1.0, a, m, b, k, 0.0, np.zeros(m * n, np.float32), m), m, n, m)
    c_plain, _, _, _ = _pipeline(handle, dev, FP16TCEC, N, N, m, n, k, a, b)
    c_scaled, a_after, b_after, ids = _pipeline(handle, dev, SCALING, N, N, m, n, k, a, b)
    r_plain, r_scaled = O.residual(ref, c_plain, m, n, m), O.residual(ref, c_scaled, m, n, m)
    assert r_scaled <= 2.0 * r_fp32
    assert r_plain > 50 * r_scaled  # the unscaled path visibly degrades
    # A and B are restored bit-exactly
    assert np.array_equal(a_after.view(np.uint32), a.view(np.uint32))
    assert np.array_equal(b_after.view(np.uint32), b.view(np.uint32))
    assert ids[2] == 1  # forced flag slot
    assert int(np.float32(handle.get_max_exp(ids[0])).view(np.uint32)) == O.exp_max_bits(a, m, k, m)
    assert int(np.float32(handle.get_max_exp(ids[1])).view(np.uint32)) == O.exp_max_bits(b, k, n, k)
    # parity with the oracle's pipeline: scale, TCEC GEMM, unscale
    L = O.lib()
    ma, mb = handle.get_max_exp(ids[0]), handle.get_max_exp(ids[1])
    sa = O.scale_matrix(a.copy(), m, k, m, L.oracle_scale_ab_coef(ma))
    sb = O.scale_matrix(b.copy(), k, n, k, L.oracle_scale_ab_coef(mb))
    co = oracle_gemm(O, FP16TCEC, N, N, m, n, k, 1.0, sa, m, sb, k, 0.0, np.zeros(m * n, np.float32), m)
    O.scale_matrix(co, m, n, m, L.oracle_scale_c_coef(ma, mb, 0, 0))
    assert np.linalg.norm(co.astype(np.float64) - c_scaled) / np.linalg.norm(co.astype(np.float64)) < 2.0 ** -21 * np.sqrt(k)


def test_scaling_without_restore_leaves_scaled_operands(O, handle, dev):
    m = n = k = 128
    a = (inputs.uniform(3, m * k) * np.float32(2.0 ** -10)).astype(np.float32)
    b = inputs.uniform(4, k * n)
    _, a_after, b_after, ids = _pipeline(handle, dev, SCALING, T, T, m, n, k, a, b, restore=False)
    ma = handle.get_max_exp(ids[0])
    assert np.array_equal(a_after, O.scale_matrix(a.copy(), k, m, k, O.lib().oracle_scale_ab_coef(ma)))
    assert 2.0 ** 14 <= np.abs(b_after).max() < 2.0 ** 15


@pytest.mark.parametrize("case", ["unit", "tiny", "wide"])
def test_auto_mode_decision_and_accuracy(O, handle, dev, case):
    m = n = k = 320
    if case == "unit":
        a, b = inputs.uniform(5, m * k, 0.25, 1.0), inputs.uniform(6, k * n, 0.25, 1.0)
        want_mode, want_scale = FP16TCEC, (0, 0)
    elif case == "tiny":
        a = (inputs.uniform(5, m * k, 0.5, 1.0) * np.float32(2.0 ** -20)).astype(np.float32)
        b = inputs.uniform(6, k * n, 0.25, 1.0)
        want_mode, want_scale = FP16TCEC, (1, 0)
    else:
        a = inputs.exponent_spread(5, m, k, per_row=True)
        b = inputs.exponent_spread(6, k, n, per_row=False)
        want_mode, want_scale = TF32TCEC, (0, 0)
    c, a_after, b_after, ids = _pipeline(handle, dev, AUTO, N, N, m, n, k, a, b)
    flag = handle.get_dynamic_launch_flag(ids[2])
    assert flag & 0x1f == want_mode
    assert (bool(flag & 0x40), bool(flag & 0x20)) == tuple(bool(x) for x in want_scale)
    sa, sb = O.exp_stats(a, m, k, m), O.exp_stats(b, k, n, k)
    assert flag == O.lib().oracle_combine_flag(sa.mode, sb.mode)
    assert handle.get_exp_stats(ids[0]) == (sa.underflow, sa.total)
    assert handle.get_exp_stats(ids[1]) == (sb.underflow, sb.total)
    assert np.array_equal(a_after.view(np.uint32), a.view(np.uint32))
    assert np.array_equal(b_after.view(np.uint32), b.view(np.uint32))
    ref = O.gemm_fp64(N, N, m, n, k, 1.0, a, m, b, k)
    r_fp32 = O.residual(ref, oracle_gemm(O, FP32, N, N, m, n, k, 1.0, a, m, b, k, 0.0, np.zeros(m * n, np.float32), m), m, n, m)
    assert O.residual(ref, c, m, n, m) <= 2.0 * r_fp32


def _auto_operand(kind, seed, rows, cols, per_row):
    if kind == "unit":      # decided by the first statistics pass: FP16TCEC
        return inputs.uniform(seed, rows * cols, 0.25, 1.0)
    if kind == "tiny":      # second pass: FP16TCEC with scaling
        return (inputs.uniform(seed, rows * cols, 0.5, 1.0) * np.float32(2.0 ** -20)).astype(np.float32)
    return inputs.exponent_spread(seed, rows, cols, per_row=per_row)  # second pass: TF32TCEC


@pytest.mark.parametrize("size", [96, 1024])
def test_auto_launch_flag_for_every_pair_of_decisions(O, handle, dev, size):
    """The launch flag is written by the second statistics pass itself, by
    whichever of the two matrices' scans finishes last -- or leaves at once
    because the first pass had already decided.  All nine pairs of decisions,
    with one and with many workgroups per matrix, twice on the same handle (the
    arrival counter of the pair resets itself)."""
    m = n = k = size
    want = {"unit": FP16TCEC, "tiny": SCALING, "wide": TF32TCEC}
    for rep in range(2):
        for ka in ("unit", "tiny", "wide"):
            for kb in ("unit", "tiny", "wide"):
                a = _auto_operand(ka, 21 + rep, m, k, True)
                b = _auto_operand(kb, 31 + rep, k, n, False)
                _, _, _, ids = _pipeline(handle, dev, AUTO, N, N, m, n, k, a, b)
                assert handle.get_exp_stats_compute_mode_level(ids[0]) == want[ka], (ka, kb, rep)
                assert handle.get_exp_stats_compute_mode_level(ids[1]) == want[kb], (ka, kb, rep)
                flag = handle.get_dynamic_launch_flag(ids[2])
                assert flag == O.lib().oracle_combine_flag(want[ka], want[kb]), (ka, kb, rep)


def test_auto_complex_batched(O, handle, dev):
    m, n, k, batch = 64, 48, 80, 3
    a = inputs.complex_normal(7, m * k * batch, 2.0 ** -19)
    b = inputs.complex_normal(8, k * n * batch, 1.0)
    da, db, dc = dev.up(a), dev.up(b), dev.up(np.zeros(m * n * batch, np.complex64))
    st, ids = handle.gemm_pipeline(N, N, m, n, k, 1.0, da, m, db, k, 0.0, dc, m, AUTO, cplx=True,
                                   stridea=m * k, strideb=k * n, stridec=m * n, batch=batch)
    assert st == 0
    c = dev.down(dc, np.complex64)
    flag = handle.get_dynamic_launch_flag(ids[2])
    sa = O.exp_stats(a, m, k, m, batch=batch, stride=m * k)
    sb = O.exp_stats(b, k, n, k, batch=batch, stride=k * n)
    assert flag == O.lib().oracle_combine_flag(sa.mode, sb.mode)
    assert np.array_equal(dev.down(da, np.complex64), a)
    for i in range(batch):
        ref = O.gemm_fp64(N, N, m, n, k, 1.0, a[i * m * k:], m, b[i * k * n:], k)
        cf = oracle_gemm(O, FP32, N, N, m, n, k, 1.0, a[i * m * k:], m, b[i * k * n:], k, 0.0, np.zeros(m * n, np.complex64), m)
        assert O.residual(ref, c[i * m * n:(i + 1) * m * n], m, n, m) <= 2.0 * O.residual(ref, cf, m, n, m)


@pytest.mark.parametrize("mode", [SCALING, AUTO])
@pytest.mark.parametrize("cplx,opa,opb,m,n,k", [
    (False, N, N, 512, 384, 256),    # interior tiles: persistent fused kernels
    (False, T, N, 200, 130, 100),    # edge tiles
    (False, N, T, 256, 256, 4096),   # split-K
    (True, N, N, 256, 128, 192),
    (True, T, T, 70, 90, 50),
])
def test_fused_scaling_matches_in_place_scaling(O, handle, dev, monkeypatch, mode, cplx, opa, opb, m, n, k):
    """The pipelines scale A, B and C inside the GEMM kernel; the stand-alone
    passes (scale A, B in place, GEMM, scale C, undo) must give the same bits:
    every factor is a power of two."""
    gen = (lambda s, c: inputs.complex_normal(s, c, 1.0)) if cplx else inputs.uniform
    a = (gen(31, m * k) * np.float32(2.0 ** -21)).astype(np.complex64 if cplx else np.float32)
    b = (gen(32, k * n) * np.float32(2.0 ** -3)).astype(np.complex64 if cplx else np.float32)
    outs = []
    for fused in (True, False):
        if fused:
            monkeypatch.delenv("CUMPSGEMM_NO_FUSED_SCALING", raising=False)
        else:
            monkeypatch.setenv("CUMPSGEMM_NO_FUSED_SCALING", "1")
        c, a_after, b_after, ids = _pipeline(handle, dev, mode, opa, opb, m, n, k, a, b, cplx=cplx)
        assert np.array_equal(a_after.view(np.uint32), a.view(np.uint32))
        assert np.array_equal(b_after.view(np.uint32), b.view(np.uint32))
        outs.append(c)
    if k <= 2048:  # split-K accumulates with atomics: order, hence bits, vary
        assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))
    ref = O.gemm_fp64(opa, opb, m, n, k, 1.0, a, m if opa == N else k, b, k if opb == N else n)
    cf = oracle_gemm(O, FP32, opa, opb, m, n, k, 1.0, a, m if opa == N else k, b, k if opb == N else n, 0.0,
                     np.zeros(m * n, a.dtype), m)
    for c in outs:
        assert O.residual(ref, c, m, n, m) <= 2.0 * O.residual(ref, cf, m, n, m)


# Large real problems in FP16TCEC_SCALING take the pre-split path: A and B are
# scaled and split once into fp16 planes (workspace of the handle) and the GEMM
# kernel only folds the inverse scaling of C into alpha.  Same scaling, same
# split, same products as the two other forms (which agree bit for bit); the
# pre-split kernels' MFMAs add 32 K-values where the in-loop kernels' add 16, so
# they agree with those up to the order of summation.
def test_complex_scaled_pre_split_path_matches_in_loop(cg, torch_gpu, dev, monkeypatch):
    """FP16TCEC_SCALING on a large complex problem: the pre-pass scales, splits and
    de-interleaves; the in-loop fused form's result up to the order of summation."""
    m, n, k = 3800, 3700, 288
    C_OP = 113
    a = (inputs.complex_normal(75, m * k, 1.0) * np.float32(2.0 ** -21)).astype(np.complex64)
    b = (inputs.complex_normal(76, n * k, 1.0) * np.float32(2.0 ** 4)).astype(np.complex64)
    h = cg.Handle()
    h.set_stream(torch_gpu.cuda.current_stream())
    try:
        outs = []
        for packed in ("0", None):
            if packed is None:
                monkeypatch.delenv("CUMPSGEMM_PACKED", raising=False)
            else:
                monkeypatch.setenv("CUMPSGEMM_PACKED", packed)
            c, a_after, b_after, _ = _pipeline(h, dev, SCALING, N, C_OP, m, n, k, a, b, cplx=True)
            assert (h.workspace_size() >= (m + n) * k * 8) == (packed is None)
            assert np.array_equal(a_after.view(np.uint32), a.view(np.uint32))
            outs.append(c)
        assert_same_up_to_summation_order(outs[0], outs[1], k)
        assert float(np.abs(outs[0]).max()) > 0
    finally:
        torch_gpu.cuda.synchronize()
        h.close()


@pytest.mark.parametrize("opa,opb,m,n,k", [
    (N, N, 4096, 4096, 256),      # (the path is taken from m*n/(m+n) >= 1800 on)
    (T, N, 4000, 3700, 300),      # ragged M, N and K
    (N, T, 3800, 4100, 288),
    (T, T, 3712, 4096, 256),
])
@pytest.mark.parametrize("mode", [SCALING, AUTO])
def test_scaled_pre_split_path_matches_the_other_forms(O, cg, torch_gpu, dev, monkeypatch, mode, opa, opb, m, n, k):
    a = (inputs.uniform(71, m * k) * np.float32(2.0 ** -22)).astype(np.float32)
    b = (inputs.uniform(72, k * n) * np.float32(2.0 ** 5)).astype(np.float32)
    h = cg.Handle()                      # a fresh handle owns no workspace yet
    h.set_stream(torch_gpu.cuda.current_stream())
    # AUTO: with a tenth of the elements allowed below the threshold A is found to need scaling
    # and B to be fine as it is, so the FP16TCEC candidate runs, scaling A only
    h.set_exp_stats_params(0.0, 2.0 ** -15, 0.1)
    try:
        outs = {}
        for form in ("in_loop", "in_place", "pre_split"):
            monkeypatch.delenv("CUMPSGEMM_NO_FUSED_SCALING", raising=False)
            monkeypatch.delenv("CUMPSGEMM_PACKED", raising=False)
            if form == "in_loop":
                monkeypatch.setenv("CUMPSGEMM_PACKED", "0")
            elif form == "in_place":
                monkeypatch.setenv("CUMPSGEMM_NO_FUSED_SCALING", "1")
                monkeypatch.setenv("CUMPSGEMM_PACKED", "0")   # (the unscaled pre-split path serves NT layouts)
            c, a_after, b_after, ids = _pipeline(h, dev, mode, opa, opb, m, n, k, a, b)
            if mode == AUTO:
                assert h.get_dynamic_launch_flag(ids[2]) == (FP16TCEC | 0x40)
            # only the pre-split form holds a workspace: fp16 hi + lo planes of A and B
            assert (h.workspace_size() >= (m + n) * k * 4) == (form == "pre_split")
            assert np.array_equal(a_after.view(np.uint32), a.view(np.uint32))
            assert np.array_equal(b_after.view(np.uint32), b.view(np.uint32))
            outs[form] = c
        assert np.array_equal(outs["in_loop"].view(np.uint32), outs["in_place"].view(np.uint32))
        assert_same_up_to_summation_order(outs["pre_split"], outs["in_loop"], k)
    finally:
        torch_gpu.cuda.synchronize()
        h.close()
    if opa == T and opb == N:            # the other forms are checked against FP64 elsewhere; once here
        ref = O.gemm_fp64(opa, opb, m, n, k, 1.0, a, k, b, k)
        cf = oracle_gemm(O, FP32, opa, opb, m, n, k, 1.0, a, k, b, k, 0.0, np.zeros(m * n, np.float32), m)
        assert O.residual(ref, outs["pre_split"], m, n, m) <= 2.0 * O.residual(ref, cf, m, n, m)


@pytest.mark.parametrize("k", [256, 512])
def test_auto_pre_split_path_steps_aside_for_bf16x3(O, cg, torch_gpu, dev, monkeypatch, k):
    """Same shape class, but AUTO decides for TF32TCEC (no underflow tolerated):
    the gated pre-pass and the gated FP16TCEC kernel do nothing, the bf16x3
    kernel (k = 256: the in-loop one; k = 512: its own gated pre-split form)
    produces C -- the same result, up to the order of summation for the pre-split
    form, as with the pre-split path forbidden."""
    m, n = 4096, 4096
    a = (inputs.uniform(81, m * k) * np.float32(2.0 ** -22)).astype(np.float32)
    b = (inputs.uniform(82, k * n) * np.float32(2.0 ** 5)).astype(np.float32)
    h = cg.Handle()
    h.set_stream(torch_gpu.cuda.current_stream())
    try:
        outs = []
        for packed in ("0", None):
            if packed is None:
                monkeypatch.delenv("CUMPSGEMM_PACKED", raising=False)
            else:
                monkeypatch.setenv("CUMPSGEMM_PACKED", packed)
            c, _, _, ids = _pipeline(h, dev, AUTO, N, N, m, n, k, a, b)
            assert h.get_dynamic_launch_flag(ids[2]) & 0x1f == TF32TCEC
            outs.append(c)
        if k == 256:
            assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))
        else:
            assert_same_up_to_summation_order(outs[0], outs[1], k)
    finally:
        torch_gpu.cuda.synchronize()
        h.close()
    ref = O.gemm_fp64(N, N, m, n, k, 1.0, a, m, b, k)
    cf = oracle_gemm(O, FP32, N, N, m, n, k, 1.0, a, m, b, k, 0.0, np.zeros(m * n, np.float32), m)
    assert O.residual(ref, outs[1], m, n, m) <= 2.0 * O.residual(ref, cf, m, n, m)


@pytest.mark.parametrize("mode", [SCALING, AUTO])
def test_pipeline_rejects_what_the_statistics_cannot_address(handle, dev, mode):
    """The statistics and scaling passes take 32-bit leading dimensions and strides (as in the
    reference); a scaled call that needs more is refused before anything is launched."""
    x = dev.up(np.ones(64, np.float32))
    big = (1 << 32) + 8
    # batched, stride of A beyond 32 bits (nothing is read: the call returns at once)
    st, _ = handle.gemm_pipeline(N, N, 4, 4, 4, 1.0, x, 4, x, 4, 0.0, x, 4, mode, stridea=big, strideb=16,
                                 stridec=16, batch=2)
    assert st == 3                       # HIPBLAS_STATUS_INVALID_VALUE
    st, _ = handle.gemm_pipeline(N, N, 4, 4, 4, 1.0, x, big, x, 4, 0.0, x, 4, mode)
    assert st == 3
    # the plain modes address with 64 bits and take the same arguments
    c = dev.up(np.zeros(16, np.float32))
    st, _ = handle.gemm_pipeline(N, N, 4, 4, 1, 1.0, x, big, x, 4, 0.0, c, 4, FP16TCEC)
    assert st == 0 and np.array_equal(dev.down(c), np.ones(16, np.float32))


@pytest.mark.parametrize("mode", [SCALING, AUTO])
@pytest.mark.parametrize("cplx", [False, True])
@pytest.mark.parametrize("restore,fused", [(True, True), (True, False), (False, False), (False, True)])
def test_scaled_pipelines_with_beta(O, handle, dev, monkeypatch, mode, cplx, restore, fused):
    """alpha * op(A) * op(B) + beta * C in the scaled modes, beta != 0, against FP64: the fused form
    (A, B untouched), the stand-alone passes with restoration and the two forms that leave A and B
    scaled (stand-alone passes; fused GEMM with A and B scaled afterwards)
    all keep beta * C_old out of the rescaling of C.  (Rescaling the finished C, as the reference's
    sequence does, src/cumpsgemm_cublas.cu:549-559, would multiply beta * C_old by 2^-17 here.)"""
    m, n, k = 200, 136, 160
    dt = np.complex64 if cplx else np.float32
    gen = (lambda s, c: inputs.complex_normal(s, c, 1.0)) if cplx else inputs.uniform
    a = (gen(91, m * k) * np.float32(2.0 ** -21)).astype(dt)     # needs scaling (by 2^34 or so)
    b = (gen(92, k * n) * np.float32(2.0 ** 3)).astype(dt)
    c0 = (gen(93, (m + 5) * n) * np.float32(2.0 ** -16)).astype(dt)  # same magnitude as alpha*A*B
    alpha, beta = ((0.75 - 0.5j), (-1.25 + 0.5j)) if cplx else (0.75, -1.25)
    ldc = m + 5
    if fused:
        monkeypatch.delenv("CUMPSGEMM_NO_FUSED_SCALING", raising=False)
    else:
        monkeypatch.setenv("CUMPSGEMM_NO_FUSED_SCALING", "1")
    if mode == AUTO:
        handle.set_exp_stats_params(0.0, 2.0 ** -15, 0.1)
    try:
        da, db, dc = dev.up(a), dev.up(b), dev.up(c0)
        st, ids = handle.gemm_pipeline(T, N, m, n, k, alpha, da, k, db, k, beta, dc, ldc, mode, cplx=cplx,
                                       restore_ab=restore)
        assert st == 0
        c = dev.down(dc, dt)
        a_after = dev.down(da, dt)
    finally:
        handle.set_exp_stats_params(0.0, 2.0 ** -15, 0.0)
    if mode == AUTO:
        assert handle.get_dynamic_launch_flag(ids[2]) == (FP16TCEC | 0x40)
    assert np.array_equal(a_after, a) == restore
    if not restore:   # A is left multiplied by 2^14 / 2^floor(log2 max|A|), whichever form ran
        ma = handle.get_max_exp(ids[0])
        want = O.scale_matrix(a.view(np.float32).copy(), (2 if cplx else 1) * k, m, (2 if cplx else 1) * k,
                              O.lib().oracle_scale_ab_coef(ma))
        assert np.array_equal(a_after.view(np.float32), want)
    ref = O.gemm_fp64(T, N, m, n, k, alpha, a, k, b, k, beta, c0, ldc)
    cf = oracle_gemm(O, FP32, T, N, m, n, k, alpha, a, k, b, k, beta, c0, ldc)
    r, r32 = O.residual(ref, c, m, n, ldc), O.residual(ref, cf, m, n, ldc)
    assert r <= 2.0 * r32 + 2.0 ** -24, (r, r32)
    # rows m .. ldc of every column are not part of C
    assert np.array_equal(c.reshape(n, ldc)[:, m:], c0.reshape(n, ldc)[:, m:])


@pytest.mark.parametrize("mode", [SCALING, AUTO])
@pytest.mark.parametrize("restore", [True, False])
def test_scaled_pipeline_keeps_a_large_c_with_tiny_operands(handle, dev, mode, restore):
    """A and B near 2^-30 are scaled up by 2^44 each, so the product of the two inverse factors is
    2^-88; with beta != 0 and C_old near 2^45 nothing on the way may divide C_old by that product
    (2^133 is outside FP32).  alpha * A * B (about 2^-55) vanishes next to beta * C_old here, so the
    result is beta * C_old exactly."""
    m = n = k = 128
    a = (inputs.uniform(71, m * k) * np.float32(2.0 ** -30)).astype(np.float32)
    b = (inputs.uniform(72, k * n) * np.float32(2.0 ** -30)).astype(np.float32)
    c0 = (inputs.uniform(73, m * n) * np.float32(2.0 ** 45)).astype(np.float32)
    if mode == AUTO:
        handle.set_exp_stats_params(0.0, 2.0 ** -15, 0.1)
    try:
        da, db, dc = dev.up(a), dev.up(b), dev.up(c0)
        st, ids = handle.gemm_pipeline(N, N, m, n, k, 1.0, da, m, db, k, 0.5, dc, m, mode, restore_ab=restore)
        assert st == 0
        c = dev.down(dc)
        a_after = dev.down(da)
    finally:
        handle.set_exp_stats_params(0.0, 2.0 ** -15, 0.0)
    assert np.isfinite(c).all()
    assert np.array_equal(c, np.float32(0.5) * c0)
    assert np.array_equal(a_after, a) == restore
    if not restore:
        assert 2.0 ** 14 <= np.abs(a_after).max() < 2.0 ** 15


@pytest.mark.parametrize("mode", [SCALING, AUTO])
@pytest.mark.parametrize("missing", ["a", "b", "c"])
def test_scaled_pipeline_refuses_a_null_matrix_before_any_launch(handle, dev, mode, missing):
    """A null operand leaves the statistics nothing to scan; the call is refused before the scaling
    passes and the GEMM could run on whatever the slot and flag rings held: C and the operands stay
    as they were and no slot or flag is taken from the rings."""
    m = n = k = 96
    a, b = inputs.uniform(74, m * k), inputs.uniform(75, k * n)
    c0 = inputs.uniform(76, m * n)
    da, db, dc = dev.up(a), dev.up(b), dev.up(c0)
    slot_before = handle.get_current_exp_stats_buffer_id()
    args = {"a": da, "b": db, "c": dc}
    args[missing] = None
    st, _ = handle.gemm_pipeline(N, N, m, n, k, 1.0, args["a"], m, args["b"], k, 0.0, args["c"], m, mode,
                                 restore_ab=False)
    assert st == 3                       # HIPBLAS_STATUS_INVALID_VALUE
    assert handle.get_current_exp_stats_buffer_id() == slot_before
    assert np.array_equal(dev.down(dc), c0) and np.array_equal(dev.down(da), a) and np.array_equal(dev.down(db), b)
