"""The benchmark's command-line contract, as far as it can be checked without a GPU, and (on a
GPU) the shape of the JSON line it prints."""
import json
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message(monkeypatch, capsys):
    sys.path.insert(0, ROOT)
    import bench
    monkeypatch.setattr(sys, "argv", ["bench.py", "--gpus", "2"])
    with pytest.raises(SystemExit) as e:
        bench.main()
    assert e.value.code not in (0, None)
    cap = capsys.readouterr()
    assert "one GPU" in cap.err and cap.out.strip() == ""


def test_product_code_never_touches_the_oracle():
    """Only tests, the smoke check and the benchmark's cpu_baseline leg may use oracle/."""
    pkg = os.path.join(ROOT, "sliced_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".cpp", ".h")):
                text = open(os.path.join(dirpath, f), errors="replace").read()
                assert "import oracle" not in text and "from oracle" not in text and "orc_" not in text, f


CONTRACT_KEYS = ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                 "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline")


def check_line(out, steps, warmup):
    lines = [l for l in out.splitlines() if l.strip()]
    assert len(lines) == 1, "stdout must carry the result line and nothing else"
    assert len(lines[0]) < 4096, len(lines[0])
    j = json.loads(lines[0])
    for k in CONTRACT_KEYS:
        assert k in j, k
    assert j["n_gpus"] == 1 and j["steps"] == steps and j["warmup"] == warmup and j["dtype"] == "f32" and j["vs_baseline"] is None
    assert "workload" in j["config"] and "model" not in j["config"]
    assert j["config"]["spin_up_s"] > 0 and "gemm_wide_kernel<false,false,true>" in j["config"]["kernel"]
    rf = j["roofline"]
    assert rf["bound"] == "mfma" and rf["unit"] == "TFLOP/s" and rf["peak"] == 157.3
    assert abs(rf["frac"] - rf["achieved"] / rf["peak"]) < 1e-9
    assert 0.3 < rf["frac"] < 1.0
    assert "traffic" in rf
    return j


@pytest.mark.gpu
def test_json_line_has_the_contract_fields(monkeypatch, capsys, tmp_path):
    # in-process: a process that has initialised the GPU must not start another program
    sys.path.insert(0, ROOT)
    import bench
    monkeypatch.setattr(sys, "argv", ["bench.py", "--no-suite", "--no-cpu", "--steps", "5", "--warmup", "2",
                                      "--detail", str(tmp_path / "d.json")])
    bench.main()
    check_line(capsys.readouterr().out, 5, 2)
    assert "headline" in json.load(open(tmp_path / "d.json"))


@pytest.mark.gpu
def test_default_run_prints_one_short_line_with_roofline_and_cpu_baseline(monkeypatch, capsys, tmp_path):
    """The arguments the benchmark runs with when none are given: the whole suite and the CPU side.
    The one stdout line must stay short enough for a reader that keeps only the tail of the output."""
    sys.path.insert(0, ROOT)
    import bench
    detail = tmp_path / "detail.json"
    monkeypatch.setattr(sys, "argv", ["bench.py", "--detail", str(detail)])
    bench.main()
    j = check_line(capsys.readouterr().out, 20, 5)
    rf, cpu = j["roofline"], j["cpu_baseline"]
    for key in ("achieved_median", "TFLOPs A*B", "TFLOPs A*Bt", "TFLOPs At*B", "GBps sum_rows 16384^2", "GBps sum_cols 16384^2",
                "GBps max_rows 16384^2", "GBps max_cols 16384^2", "GBps mean 2^28", "GBps transpose 16384^2",
                "GBps softmax fwd 32768x4096", "GBps softmax bwd 32768x4096", "GBps ew chain 2^28", "steps/s C1", "steps/s C5"):
        assert key in rf, key
    for key in ("value", "unit", "cores", "kind", "sample", "cblas_TFLOPs"):
        assert key in cpu, key
    assert cpu["kind"] == "port" and cpu["cores"] >= 1 and cpu["value"] > 0
    assert any(k.startswith("C1 steps_per_s") for k in cpu) and any(k.startswith("C5 steps_per_s") for k in cpu)
    full = json.load(open(detail))
    for part in ("headline", "gemm_forms", "gemm_sweep", "ops", "tape_chain", "mlp", "cpu_baseline", "line"):
        assert part in full, part
    assert full["line"] == j
