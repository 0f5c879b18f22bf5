"""The command-line harness (counterpart of the reference's test program,
test/main.cu:1345-1510): argument handling on the CPU, every command at small
sizes on the GPU with its output lines checked against the reference's formats
(test/main.cu:404-410, :522-529, :1217-1229, :1300-1340)."""
import io
import re

import pytest

NUM = r"\d\.\d+e[+-]\d+"


def test_error_threshold():
    from cumpsgemm_amd import harness
    # test/main.cu:68-74
    assert harness.error_threshold("FP16TCEC", 4096) == 2.0 ** -23 * 64
    assert harness.error_threshold("TF32TCEC", 1024) == 2.0 ** -23 * 32
    assert harness.error_threshold("FP16TC", 1024) == 2.0 ** -10 * 32
    assert harness.error_threshold("TF32TC", 256) == 2.0 ** -10 * 16
    assert harness.error_threshold("CUBLAS", 256) == 2.0 ** -23 * 16


def test_sizes():
    from cumpsgemm_amd.harness import Harness
    assert Harness.sizes(True, 256, 1024, 256) == [256, 512, 768, 1024]
    assert Harness.sizes(False, 8, 12, 2) == [256, 1024, 4096]


@pytest.mark.parametrize("argv", [
    ["prog"], ["prog", "sgemm"], ["prog", "sgemm", "linear", "1", "2", "1", "FP16TCEC"],
    ["prog", "sgemm", "seq", "x", "2", "1"], ["prog", "log"], ["prog", "nonsense", "seq", "1", "2", "1"],
    ["prog", "sgemm_exp_stats", "128"], ["prog", "cgemm_exp_stats_bw", "5"],
])
def test_bad_arguments_print_usage(argv):
    from cumpsgemm_amd import harness
    with pytest.raises(SystemExit) as e:
        harness.main(argv)
    assert "sgemm_tall_skinny" in str(e.value.code)  # the usage text, no GPU touched


def _run(argv):
    from cumpsgemm_amd import harness
    out = io.StringIO()
    ok = harness.main(["prog"] + argv, out=out)
    return ok, out.getvalue()


@pytest.mark.gpu
def test_sgemm_sweep(cg, torch_gpu):
    ok, text = _run(["sgemm", "seq", "192", "448", "256", "FP16TCEC", "TF32TCEC", "FP16TC", "TF32TC",
                     "FP16TCEC_SCALING", "CUBLAS"])
    assert ok, text
    assert "type,mode,op_A,op_B,m,n,k,throughput_in_tflops,residual,check,module_stage" in text
    lines = [ln for ln in text.splitlines() if ln.startswith("sgemm,")]
    assert len(lines) == 6 * 4 * 2  # modes x op pairs x sizes
    for ln in lines:
        assert re.fullmatch(rf"sgemm,\w+,[NT],[NT],(\d+),\1,\1,{NUM},{NUM},OK,\d+", ln), ln
    # FP16TCEC_SCALING reports the mode it runs the GEMM in, as the reference does
    assert sum(ln.startswith("sgemm,FP16TCEC,") for ln in lines) == 16
    assert "Result : 48 / 48 passed" in text


@pytest.mark.gpu
def test_cgemm_exp2_sweep(cg, torch_gpu):
    ok, text = _run(["cgemm", "exp2", "7", "8", "1", "FP16TCEC", "TF32TCEC"])
    assert ok, text
    lines = [ln for ln in text.splitlines() if ln.startswith("cgemm,")]
    assert len(lines) == 2 * 9 * 2
    assert {ln.split(",")[4] for ln in lines} == {"128", "256"}
    assert {(ln.split(",")[2], ln.split(",")[3]) for ln in lines} == {(a, b) for a in "NTC" for b in "NTC"}
    assert "Result : 36 / 36 passed" in text


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["sgemm", "cgemm"])
def test_strided_batch_sweep(cg, torch_gpu, kind):
    ok, text = _run([f"{kind}_strided_batch", "seq", "96", "160", "64", "5", "FP16TCEC", "FP16TCEC_SCALING"])
    assert ok, text
    assert "type,mode,op_A,op_B,m,n,k,batch_count,throughput_in_tflops,residual,check,module_stage" in text
    lines = [ln for ln in text.splitlines() if ln.startswith(kind + ",")]
    assert len(lines) == 2 * (4 if kind == "sgemm" else 9) * 2
    for ln in lines:
        assert re.fullmatch(rf"{kind},FP16TCEC,[NTC],[NTC],(\d+),\1,\1,5,{NUM},{NUM},OK,\d+", ln), ln


@pytest.mark.gpu
def test_tall_skinny_sweep(cg, torch_gpu):
    ok, text = _run(["sgemm_tall_skinny", "exp2", "64", "10", "14", "4", "FP16TCEC", "TF32TCEC"])
    assert ok, text
    lines = [ln for ln in text.splitlines() if ln.startswith("sgemm,")]
    assert len(lines) == 2 * 4 * 2
    assert {ln.split(",")[6] for ln in lines} == {"1024", "16384"}
    assert all(ln.split(",")[4:6] == ["64", "64"] for ln in lines)
    ok, text = _run(["cgemm_tall_skinny", "seq", "48", "1000", "1000", "1", "FP16TCEC"])
    assert ok and "Result : 9 / 9 passed" in text, text


@pytest.mark.gpu
@pytest.mark.parametrize("argv", [["sgemm_exp_stats", "512", "0", "1.52587890625e-05"],
                                  ["cgemm_exp_stats", "256", "1e-30", "1.52587890625e-05"],
                                  ["sgemm_strided_batch_exp_stats", "128", "4", "0", "1.52587890625e-05"]])
def test_exp_stats_command(cg, torch_gpu, argv):
    ok, text = _run(argv)
    assert ok, text
    kind = argv[0][:5]
    n = int(argv[1])
    batch = int(argv[2]) if "batch" in argv[0] else 1
    assert re.search(rf"^# \[{kind}:    AUTO, N={n}, batch_size={batch}, u={NUM}, i={NUM}\]$", text, re.M), text
    counted = n * n * batch * (2 if kind == "cgemm" else 1)
    # N(0, 2^-16) inputs: a large share is below 2^-15, so the first decision cannot be
    # FP16TCEC; the maximum is far above it, so scaling rescues fp16
    for name in "AB":
        m = re.search(rf"^  {name} = \[underflow: +(\d+) / +(\d+) \( *(\d\.\d\d)\), max_exp=({NUM}), "
                      rf"buffer_id = \d+ -> mode=(\w+)\]$", text, re.M)
        assert m, text
        assert int(m.group(2)) <= counted and m.group(5) == "FP16TCEC_SCALING", text
        # printed with seven digits; about 4 to 5 sigma is the largest of so many samples
        assert any(abs(float(m.group(4)) / 2.0 ** e - 1) < 1e-6 for e in (-15, -14, -13)), text
    assert re.search(r"^  C = \[underflow: +\d+ / +\d+ \( *\d\.\d\d\), max_exp=\S+, buffer_id = \d+\]$", text, re.M)
    assert "  Compute mode = [FP16TCEC, SCALE_A=1, SCALE_B=1]" in text, text
    assert re.search(rf"^  Error = \[{NUM}, OK\]$", text, re.M), text


@pytest.mark.gpu
def test_exp_stats_bw_command(cg, torch_gpu):
    ok, text = _run(["sgemm_exp_stats_bw", "8", "10", "1"])
    assert ok and "gemm,N,exp_stats_1_bw_in_gbps,exp_stats_2_bw_in_gbps,scale_bw_in_gbps" in text, text
    rows = [ln.split(",") for ln in text.splitlines() if ln.startswith("S,")]
    assert [r[1] for r in rows] == ["256", "512", "1024"]
    # with thresholds (0, 1, 0) and inputs far below 1 both statistics passes run every time
    assert all(float(v) > 0 for r in rows for v in r[2:]), text
    ok, text = _run(["cgemm_exp_stats_bw", "7", "7", "2"])
    assert ok and re.search(rf"^C,128,{NUM},{NUM},{NUM}$", text, re.M), text
