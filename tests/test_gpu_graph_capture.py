"""The GEMM entry points and the FP16TCEC_SCALING / AUTO pipelines only launch
kernels on the handle's stream (no allocation, memset, copy or synchronisation
once the handle exists), so a caller can capture them into a HIP graph.  Each
replay is checked against an eager call on the same inputs, with the inputs
changed and eager work run between replays."""
import numpy as np
import pytest

from cumpsgemm_amd import inputs
from gpu_util import assert_same_up_to_summation_order

pytestmark = pytest.mark.gpu
N_OP = 111
FP16TCEC, TF32TCEC, AUTO, SCALING = 1, 2, 9, 11


@pytest.mark.parametrize("mode,cplx", [(FP16TCEC, False), (TF32TCEC, False), (FP16TCEC, True),
                                       (SCALING, False), (AUTO, False)])
def test_captured_calls_replay_like_eager_calls(cg, torch_gpu, mode, cplx):
    torch = torch_gpu
    m, n, k = 640, 384, 512
    es = 2 if cplx else 1
    dev = torch.device("cuda:0")
    h = cg.Handle()
    side = torch.cuda.Stream()
    a = torch.empty(m * k * es, device=dev)
    b = torch.empty(k * n * es, device=dev)
    c_graph = torch.zeros(m * n * es, device=dev)
    c_eager = torch.zeros(m * n * es, device=dev)

    def call(c_out):
        if mode in (SCALING, AUTO):
            st, _ = h.gemm_pipeline(N_OP, N_OP, m, n, k, 1.0, a, m, b, k, 0.0, c_out, m, mode, cplx=cplx)
        else:
            st = h.gemm(N_OP, N_OP, m, n, k, 1.0, a, m, b, k, 0.0, c_out, m, mode, cplx=cplx)
        assert st == 0

    def fill(seed, scale):
        a.copy_(torch.from_numpy(inputs.uniform(seed, m * k * es) * np.float32(scale)).to(dev))
        b.copy_(torch.from_numpy(inputs.uniform(seed + 1, k * n * es)).to(dev))

    try:
        fill(1, 1.0)
        h.set_stream(side)
        with torch.cuda.stream(side):
            call(c_graph)                       # warm-up outside the capture (lazy kernel loading)
            # (a call whose K is split adds its chunks with float atomics, in no fixed order:
            # such a replay equals the eager call up to the order of summation, the others bit for bit)
            probe = FP16TCEC if mode in (SCALING, AUTO) else mode
            st, mid = h.gemm(N_OP, N_OP, m, n, k, 1.0, a, m, b, k, 0.0, c_eager, m, probe, cplx=cplx,
                             want_module_id=True)
            assert st == 0
        k_is_split = 100 <= mid < 200
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            h.set_stream(torch.cuda.current_stream())
            call(c_graph)
        for rep, scale in enumerate((1.0, 2.0 ** -18, 3.0)):
            fill(10 + 2 * rep, scale)
            c_graph.zero_()
            torch.cuda.synchronize()
            g.replay()
            torch.cuda.synchronize()
            h.set_stream(torch.cuda.current_stream())
            call(c_eager)                       # eager work between the replays
            torch.cuda.synchronize()
            if k_is_split:
                assert_same_up_to_summation_order(c_graph, c_eager, k)
            else:
                assert torch.equal(c_graph, c_eager), (mode, cplx, rep)
            assert float(c_eager.abs().max()) > 0
    finally:
        torch.cuda.synchronize()
        h.close()


def test_capture_never_grows_the_workspace(cg, torch_gpu, monkeypatch):
    """A call that would take the pre-split path while its workspace is still missing must not
    allocate or synchronise under capture: it runs the in-loop kernels instead (the same result up
    to the order of summation)."""
    torch = torch_gpu
    m, n, k = 4096, 3840, 768
    dev = torch.device("cuda:0")
    h = cg.Handle()
    side = torch.cuda.Stream()
    a = torch.from_numpy(inputs.uniform(31, m * k)).to(dev)
    b = torch.from_numpy(inputs.uniform(32, k * n)).to(dev)
    c_graph = torch.zeros(m * n, device=dev)
    c_eager = torch.zeros(m * n, device=dev)

    def call(c_out):
        # op_A = N, op_B = T: both operands M/N-contiguous, the layout that pre-splits from K = 256 on
        return h.gemm(N_OP, 112, m, n, k, 1.0, a, m, b, n, 0.0, c_out, m, FP16TCEC, want_module_id=True)

    try:
        h.set_stream(side)
        monkeypatch.setenv("CUMPSGEMM_PACKED", "0")
        with torch.cuda.stream(side):
            assert call(c_graph)[0] == 0        # loads the in-loop kernels, leaves the workspace alone
        torch.cuda.synchronize()
        monkeypatch.delenv("CUMPSGEMM_PACKED")
        assert h.workspace_size() == 0
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            h.set_stream(torch.cuda.current_stream())
            st, mid = call(c_graph)
        assert st == 0 and mid != 200 and h.workspace_size() == 0
        c_graph.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        h.set_stream(torch.cuda.current_stream())
        st, mid = call(c_eager)                 # eager: allocates and takes the pre-split path
        torch.cuda.synchronize()
        assert st == 0 and mid == 200 and h.workspace_size() >= (m + n) * k * 4
        assert_same_up_to_summation_order(c_graph, c_eager, k)
    finally:
        torch.cuda.synchronize()
        h.close()


def test_captured_workspace_outlives_a_larger_eager_call(cg, torch_gpu):
    """A graph captured on the pre-split path holds the address of the handle's workspace.  A
    later, larger eager call makes the handle take a new workspace; the captured one must stay
    allocated so that replays of the graph keep working on memory they own."""
    torch = torch_gpu
    m, n, k = 4096, 3840, 768
    dev = torch.device("cuda:0")
    h = cg.Handle()
    side = torch.cuda.Stream()
    a = torch.from_numpy(inputs.uniform(41, m * k)).to(dev)
    b = torch.from_numpy(inputs.uniform(42, k * n)).to(dev)
    c_graph = torch.zeros(m * n, device=dev)
    c_eager = torch.zeros(m * n, device=dev)

    def call(c_out):
        return h.gemm(N_OP, 112, m, n, k, 1.0, a, m, b, n, 0.0, c_out, m, FP16TCEC, want_module_id=True)

    try:
        h.set_stream(side)
        with torch.cuda.stream(side):
            st, mid = call(c_eager)             # outside the capture: allocates the workspace
        torch.cuda.synchronize()
        assert st == 0 and mid == 200
        ws_captured, size_captured = h.workspace_pointer(), h.workspace_size()
        assert ws_captured != 0
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            h.set_stream(torch.cuda.current_stream())
            st, mid = call(c_graph)
        assert st == 0 and mid == 200 and h.workspace_pointer() == ws_captured
        # a larger eager call on the same handle: new workspace, the old one is kept
        m2 = n2 = 4096
        k2 = 2048
        a2 = torch.from_numpy(inputs.uniform(43, m2 * k2)).to(dev)
        b2 = torch.from_numpy(inputs.uniform(44, k2 * n2)).to(dev)
        c2 = torch.zeros(m2 * n2, device=dev)
        h.set_stream(torch.cuda.current_stream())
        st, mid = h.gemm(N_OP, 112, m2, n2, k2, 1.0, a2, m2, b2, n2, 0.0, c2, m2, FP16TCEC, want_module_id=True)
        torch.cuda.synchronize()
        assert st == 0 and mid == 200 and h.workspace_size() > size_captured
        ws_new = h.workspace_pointer()
        assert ws_new != ws_captured
        # memory allocated now must not land on the captured workspace (it would if it had been freed)
        filler = torch.full((size_captured // 4,), 7.0, device=dev)
        assert not (ws_captured <= filler.data_ptr() < ws_captured + size_captured)
        for _ in range(2):
            c_graph.zero_()
            torch.cuda.synchronize()
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(c_graph, c_eager)
            assert float(filler.min()) == 7.0 and float(filler.max()) == 7.0
    finally:
        torch.cuda.synchronize()
        h.close()
