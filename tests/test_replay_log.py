"""The log-replay tool (counterpart of the reference harness's "log" command,
test/main.cu:820-1016): parsing on the CPU, replay on the GPU."""
import io

import pytest

LOG = """\
some application output
[cuMpSGEMM LOG] hipblasSgemm op=(N, N), shape=(1280, 1280, 1280), mode=FP16TCEC[dynamic][exp_stats:0]
[cuMpSGEMM LOG] hipblasSgemm op=(N, N), shape=(1280, 1280, 1280), mode=FP16TCEC[dynamic][exp_stats:0]
[cuMpSGEMM LOG] cublasCgemm_v2 op=(N, T), shape=(4, 128, 65536), mode=TF32TCEC
[cuMpSGEMM LOG] hipblasSgemmStridedBatched op=(T, N), shape=(300, 200, 96), batch=3, mode=FP16TC[static][exp_stats:0]
[cuMpSGEMM LOG] hipblasCgemm op=(C, N), shape=(640, 640, 640), mode=CUBLAS_SIMT[dynamic][exp_stats:0]
[cuMpSGEMM LOG] hipblasGemmEx op=(N, C), shape=(257, 129, 100), mode=AUTO[dynamic][exp_stats:1]
[cuMpSGEMM LOG]  +---> gemm_Mx2x2
"""


def test_parse(tmp_path):
    from cumpsgemm_amd import replay_log
    p = tmp_path / "app.log"
    p.write_text(LOG)
    calls = replay_log.parse(str(p))
    assert len(calls) == 6
    assert calls[0] == {"func": "hipblasSgemm", "op_a": "N", "op_b": "N", "m": 1280, "n": 1280, "k": 1280,
                        "batch": 1, "mode": "FP16TCEC", "cplx": False}
    assert calls[2]["cplx"] and calls[2]["mode"] == "TF32TCEC" and calls[2]["k"] == 65536
    assert calls[3]["batch"] == 3 and calls[3]["op_a"] == "T"
    assert calls[4]["mode"] == "CUBLAS_SIMT"


@pytest.mark.gpu
def test_replay(tmp_path, cg, torch_gpu):
    from cumpsgemm_amd import replay_log
    p = tmp_path / "app.log"
    p.write_text(LOG)
    out = io.StringIO()
    passed, tested = replay_log.replay(replay_log.parse(str(p)), out=out)
    text = out.getvalue()
    # duplicates collapse, forwarded (CUBLAS_*) calls are not ours to replay
    assert (passed, tested) == (4, 4), text
    import re
    assert re.search(r"^sgemm,FP16TCEC,N,N,1280,1280,1280,\d\.\d+e[+-]\d+,\d\.\d+e-\d+,OK,\d+$", text, re.M), text
    assert re.search(r"^sgemm,FP16TC,T,N,300,200,96,3,", text, re.M) and "4 / 4 passed" in text
