"""bench.py's output contract: exactly one JSON line on stdout carrying the agreed keys; the model-building helpers of
the secondary workloads keep their progress messages off stdout."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_bench_prints_one_json_line():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--steps", "2", "--warmup", "1", "--no-extra",
                        "--no-cpu-baseline"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1, r.stdout[:2000]
    out = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline"):
        assert key in out, key
    assert out["n_gpus"] == 1 and out["steps"] == 2 and out["unit"] == "GB/s" and out["vs_baseline"] is None
    roof = out["roofline"]
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and 0.05 < roof["frac"] < 1.0
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert "workload" in out["config"] and "model" not in out["config"]


def test_model_builders_keep_stdout_clean(capsys):
    import torch
    sys.path.insert(0, ROOT)
    import bench
    gen = torch.Generator(device="cuda").manual_seed(1)
    model = bench._random_llama7b(gen, n_layers=1)
    assert capsys.readouterr().out == ""
    del model
    torch.cuda.empty_cache()
