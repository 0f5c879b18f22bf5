"""Two handles on two streams with their calls interleaved: each handle owns its
rings, flags and pre-split workspace, so the results are those of running each
sequence alone (bit for bit: none of the calls splits K)."""
import numpy as np
import pytest

from cumpsgemm_amd import inputs

pytestmark = pytest.mark.gpu
N_OP, T_OP = 111, 112
FP16TCEC, TF32TCEC, SCALING = 1, 2, 11


def test_interleaved_calls_on_two_handles(cg, torch_gpu):
    torch = torch_gpu
    dev = torch.device("cuda:0")
    shapes = [(4096, 3600, 640, FP16TCEC, N_OP, T_OP),    # pre-split path (NT)
              (1024, 768, 512, TF32TCEC, T_OP, N_OP),
              (4096, 4096, 288, SCALING, N_OP, N_OP)]     # pipeline, pre-split with fused scaling
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    handles = [cg.Handle(), cg.Handle()]
    for h, s in zip(handles, streams):
        h.set_stream(s)
    try:
        data = []
        for i, (m, n, k, mode, oa, ob) in enumerate(shapes):
            a = torch.from_numpy(inputs.uniform(100 + i, m * k)).to(dev)
            b = torch.from_numpy(inputs.uniform(200 + i, k * n)).to(dev)
            data.append((a, b))
        torch.cuda.synchronize()

        def call(h, i, c):
            m, n, k, mode, oa, ob = shapes[i]
            a, b = data[i]
            lda = m if oa == N_OP else k
            ldb = k if ob == N_OP else n
            if mode == SCALING:
                st, _ = h.gemm_pipeline(oa, ob, m, n, k, 1.0, a, lda, b, ldb, 0.0, c, m, mode)
            else:
                st = h.gemm(oa, ob, m, n, k, 1.0, a, lda, b, ldb, 0.0, c, m, mode)
            assert st == 0

        # reference: every call alone
        ref = []
        for i, (m, n, *_rest) in enumerate(shapes):
            c = torch.zeros(m * n, device=dev)
            with torch.cuda.stream(streams[0]):
                call(handles[0], i, c)
            torch.cuda.synchronize()
            ref.append(c)
        # interleaved: handle 0 runs 0,1,2,0,1,2..., handle 1 runs 2,1,0,... on the other stream
        outs = [[torch.zeros_like(r) for r in ref] for _ in range(2)]
        for rep in range(3):
            for j in range(len(shapes)):
                with torch.cuda.stream(streams[0]):
                    call(handles[0], j, outs[0][j])
                with torch.cuda.stream(streams[1]):
                    call(handles[1], len(shapes) - 1 - j, outs[1][len(shapes) - 1 - j])
        torch.cuda.synchronize()
        for which in range(2):
            for i in range(len(shapes)):
                assert torch.equal(outs[which][i], ref[i]), (which, i)
        assert handles[0].workspace_size() > 0 and handles[1].workspace_size() > 0
    finally:
        torch.cuda.synchronize()
        for h in handles:
            h.close()


def test_one_handle_alternating_between_two_streams(cg, torch_gpu):
    """A handle's workspaces and rings are shared by all its calls: when its stream changes,
    the new stream is ordered behind the work queued on the old one, so calls issued back to
    back on alternating streams give what each gives alone."""
    torch = torch_gpu
    dev = torch.device("cuda:0")
    shapes = [(4096, 3600, 640, FP16TCEC, N_OP, T_OP),    # pre-split path: the workspace is reused
              (3840, 3840, 512, FP16TCEC, N_OP, T_OP),
              (4096, 4096, 288, SCALING, N_OP, N_OP)]     # statistics slots, flags, fused scaling
    s0, s1 = torch.cuda.Stream(), torch.cuda.Stream()
    h = cg.Handle()
    try:
        data = []
        for i, (m, n, k, mode, oa, ob) in enumerate(shapes):
            a = torch.from_numpy(inputs.uniform(300 + i, m * k)).to(dev)
            b = torch.from_numpy(inputs.uniform(400 + i, k * n)).to(dev)
            data.append((a, b))
        torch.cuda.synchronize()

        def call(i, c):
            m, n, k, mode, oa, ob = shapes[i]
            a, b = data[i]
            lda = m if oa == N_OP else k
            ldb = k if ob == N_OP else n
            if mode == SCALING:
                st, _ = h.gemm_pipeline(oa, ob, m, n, k, 1.0, a, lda, b, ldb, 0.0, c, m, mode)
            else:
                st = h.gemm(oa, ob, m, n, k, 1.0, a, lda, b, ldb, 0.0, c, m, mode)
            assert st == 0

        ref = []
        h.set_stream(s0)
        for i, (m, n, *_rest) in enumerate(shapes):
            c = torch.zeros(m * n, device=dev)
            call(i, c)
            torch.cuda.synchronize()
            ref.append(c)
        outs = [[torch.zeros_like(r) for r in ref] for _ in range(4)]
        for rep in range(4):
            for i in range(len(shapes)):
                h.set_stream(s0 if (rep + i) % 2 == 0 else s1)   # no synchronisation in between
                call(i, outs[rep][i])
        torch.cuda.synchronize()
        for rep in range(4):
            for i in range(len(shapes)):
                assert torch.equal(outs[rep][i], ref[i]), (rep, i)
    finally:
        torch.cuda.synchronize()
        h.close()
