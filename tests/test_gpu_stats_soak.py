"""Soak of the single-launch statistics reduction: the hand-over of the per-workgroup partial
records to the last workgroup is ordered by properties of the hardware rather than by fences, so it
is exercised here many thousand times over views of every size (1 .. 2^26 elements, i.e. 1 .. 256
publishing workgroups) and every result is compared bit-exactly with an independent count of the
same view (torch reductions on the device; the CPU oracle on a sample).  Stops at the first
mismatch."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
UNDEFINED, FP16TCEC, TF32TCEC, SCALING = 10, 1, 2, 11
LAUNCHES = 10000


def _expected(torch, x, ignore, under, tol):
    """(max_exp_bits, mode, underflow, total) as the two-stage algorithm defines them."""
    ax = x.abs()
    mx_bits = int(ax.max().view(torch.int32)) & 0x7f800000
    mx = float(np.uint32(mx_bits).view(np.float32))

    def counts(ig, un):
        total = int((ax >= ig).sum())
        underflow = int(((ax >= ig) & (ax < un)).sum())
        return underflow, total

    u, t = counts(ignore, under)
    if np.float32(u) > np.float32(np.float32(t) * np.float32(tol)) or (mx > 0 and t == 0):
        # second pass: thresholds relative to the maximum, (threshold / 2) * 2^floor(log2 max)
        u, t = counts(float(np.float32(np.float32(ignore) / np.float32(2)) * np.float32(mx)),
                      float(np.float32(np.float32(under) / np.float32(2)) * np.float32(mx)))
        mode = SCALING if np.float32(u) <= np.float32(np.float32(t) * np.float32(tol)) else TF32TCEC
    else:
        mode = FP16TCEC
    return mx_bits, mode, u, t


def test_ten_thousand_launches_of_every_size(O, cg, torch_gpu, handle):
    torch = torch_gpu
    dev = torch.device("cuda:0")
    cap = 1 << 26
    g = torch.Generator(device=dev).manual_seed(20)
    # magnitudes from 2^-40 to 2^10, so that both thresholds and the maximum depend on the view
    pool = torch.randn(cap, generator=g, device=dev) * torch.exp2(
        torch.randint(-40, 11, (cap,), generator=g, device=dev).float())
    pool[::4097] = 0.0
    rng = np.random.default_rng(21)
    ignore, under, tol = 2.0 ** -38, 2.0 ** -15, 0.05
    handle.set_exp_stats_params(ignore, under, tol)
    try:
        for it in range(LAUNCHES):
            count = int(2.0 ** rng.uniform(0.0, 26.0))
            count = min(max(count, 1), cap)
            if it % 50 == 0:                         # all 256 workgroups publishing
                count = int(rng.integers(cap // 2, cap + 1))
            off = int(rng.integers(0, cap - count + 1))
            x = pool[off:off + count]
            sid = handle.exp_stats_ext(count, 1, x, count)
            mid = handle.exp_max_ext(count, 1, x, count)
            want = _expected(torch, x, ignore, under, tol)
            got = (int(np.float32(handle.get_max_exp(sid)).view(np.uint32)),
                   handle.get_exp_stats_compute_mode_level(sid)) + handle.get_exp_stats(sid)
            assert got == want, (it, off, count, got, want)
            assert int(np.float32(handle.get_max_exp(mid)).view(np.uint32)) == want[0], (it, off, count)
            if it % 500 == 0 and count <= 1 << 22:   # and the CPU oracle on a sample
                o = O.exp_stats(x.cpu().numpy(), count, 1, count, ignore=ignore, underflow=under, tol=tol)
                assert (o.max_exp_bits, o.mode, o.underflow, o.total) == want, (it, off, count)
    finally:
        handle.set_exp_stats_params(0.0, 2.0 ** -15, 0.0)
