"""bench.py's command-line contract (CPU side) and, on a GPU, the shape of the
JSON line it prints."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused_with_a_message():
    proc = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True,
                          timeout=120)
    assert proc.returncode != 0
    assert "one GPU" in proc.stderr
    assert proc.stdout.strip() == ""


def test_cpu_path_table_runs_without_a_gpu():
    sys.path.insert(0, ROOT)
    import bench

    rows = bench.cpu_path_table([], budget_s=0.2)
    kinds = {(r["kernel"], r["config"]) for r in rows}
    assert ("softmax_causal fwd+bwd", "cfg1") in kinds and ("bias_gelu fwd+bwd", "cfg5") in kinds
    for r in rows:
        assert r["cpu_GBps"] > 0 and r["gpu_GBps"] is None and r["cores"] >= 1


@pytest.mark.gpu
def test_json_line_carries_the_contract_keys(device, capsys, monkeypatch):
    # in this process: a GPU process starts no other program
    sys.path.insert(0, ROOT)
    import bench

    monkeypatch.setattr(sys, "argv", [BENCH, "--steps", "5", "--warmup", "2", "--table-iters", "0",
                                      "--no-cpu-baseline"])
    bench.main()
    lines = [l for l in capsys.readouterr().out.splitlines() if l.strip()]
    assert len(lines) == 1, "exactly one line on stdout"
    out = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step",
                "higher_is_better", "scaling", "vs_baseline", "dtype", "data", "config", "roofline"):
        assert key in out, key
    assert out["n_gpus"] == 1 and out["steps"] == 5 and out["warmup"] == 2
    assert out["unit"] == "GB/s" and out["vs_baseline"] is None and out["higher_is_better"] is True
    assert "workload" in out["config"] and "model" not in out["config"]
    rf = out["roofline"]
    assert rf["bound"] == "hbm" and rf["peak"] == 8000.0
    assert abs(rf["frac"] - rf["achieved"] / rf["peak"]) < 1e-3
    assert 0.3 < rf["frac"] < 0.85
