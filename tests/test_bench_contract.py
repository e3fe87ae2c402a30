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


@pytest.mark.gpu
def test_json_line_has_the_contract_fields(monkeypatch, capsys):
    # in-process: a process that has initialised the GPU must not start another program
    sys.path.insert(0, ROOT)
    import bench
    monkeypatch.setattr(sys, "argv", ["bench.py", "--no-suite", "--no-cpu", "--steps", "5", "--warmup", "2"])
    bench.main()
    out = capsys.readouterr().out
    lines = [l for l in out.splitlines() if l.strip()]
    assert len(lines) == 1
    j = json.loads(lines[0])
    for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
              "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert k in j, k
    assert j["n_gpus"] == 1 and j["steps"] == 5 and j["warmup"] == 2 and j["dtype"] == "f32" and j["vs_baseline"] is None
    assert "workload" in j["config"]
    rf = j["roofline"]
    assert rf["bound"] == "mfma" and rf["unit"] == "TFLOP/s" and rf["peak"] == 157.3
    assert abs(rf["frac"] - rf["achieved"] / rf["peak"]) < 1e-9
    assert 0.3 < rf["frac"] < 1.0
