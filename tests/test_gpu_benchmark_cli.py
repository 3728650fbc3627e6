"""The reference-style benchmark runs from its command line and writes the reference's JSON document
(benchmarks/bench_all_to_all.py:501-515, flags :569-594)."""

import json
import subprocess
import sys
from pathlib import Path

import pytest

pytestmark = pytest.mark.gpu

SCRIPT = Path(__file__).resolve().parent.parent / "pplx-garden_amd" / "benchmarks" / "bench_all_to_all.py"
STAT_KEYS = {"mean", "stddev", "min", "p01", "p25", "p50", "p75", "p95", "p99", "max"}   # utils/math.py:42-53


@pytest.mark.parametrize("extra", [[], ["--quantize"], ["--sources", "all", "--max-num-tokens", "64"]],
                         ids=["caller_quantised", "quantise_inside", "all_ranks_send"])
def test_benchmark_cli(tmp_path, extra):
    out = tmp_path / "result.json"
    cmd = [sys.executable, str(SCRIPT), "--world-size", "4", "--num-experts", "32", "--hidden-dim", "2048",
           "--hidden-dim-scale", "16", "--num-experts-per-token", "4", "--num-warmup", "3", "--num-repeats", "12",
           "--output", str(out)] + extra
    print(" ".join(cmd), flush=True)
    done = subprocess.run(cmd, capture_output=True, text=True, timeout=110)
    assert done.returncode == 0, done.stderr[-2000:]
    doc = json.loads(out.read_text())
    assert set(doc) == {"dispatch", "combine"}
    for phase in ("dispatch", "combine"):
        assert set(doc[phase]) == {"both", "send", "recv"}
        for part in ("both", "send", "recv"):
            stats = doc[phase][part]
            assert set(stats) == STAT_KEYS, sorted(stats)
            assert 0 < stats["min"] <= stats["p50"] <= stats["max"]


def test_bench_py_prints_one_line_with_the_agreed_fields():
    """`python bench.py --steps K --warmup W`: one JSON line; the step metric, the roofline of the dominant
    kernel from at least 50 kernel-own samples whatever K is, the CPU baseline, and the other baseline shapes."""
    repo = Path(__file__).resolve().parent.parent
    cmd = [sys.executable, str(repo / "bench.py"), "--steps", "8", "--warmup", "2", "--cpu-reps", "1"]
    print(" ".join(cmd), flush=True)
    done = subprocess.run(cmd, capture_output=True, text=True, timeout=115)
    assert done.returncode == 0, done.stderr[-2000:]
    lines = [l for l in done.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    line = json.loads(lines[0])
    for key, want in (("unit", "GB/s"), ("n_gpus", 1), ("steps", 8), ("warmup", 2), ("higher_is_better", True),
                      ("vs_baseline", None), ("data", "synthetic")):
        assert line[key] == want, key
    assert "workload" in line["config"] and "model" not in line["config"]
    assert abs(line["value"] - 829_816_832 / (line["ms_per_step"] * 1e-3) / 1e9) < 1.0
    roof = line["roofline"]
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and roof["unit"] == "GB/s"
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert roof["samples"] >= 50
    assert roof["traffic"] is None or roof["traffic"] >= roof["bytes_per_launch"]
    cpu = line["cpu_baseline"]
    assert cpu["kind"] == "port" and cpu["cores"] == 1 and cpu["value"] > 0 and cpu["sample"]
    assert line["cpu_baseline_more"]["numpy_oracle"]["value"] > 0
    assert line["cpu_baseline_more"]["torch_oracle_all_cores"]["value"] > 0
    whole = line["prefill_4096_all_ranks_send"]
    assert whole["algorithmic_bytes"] == 8 * (301072384 + 528744448) and whole["step_us_wall"] > 0
    assert line["cpu_baseline_more"]["torch_oracle_all_cores"]["cores"] >= 1
    for shape in ("decode_128", "qwen3_decode_128", "kimi_1024"):
        assert line[shape]["step_us_wall"] > 0 and line[shape]["kernel_samples"] >= 50
    assert line["prefill_4096"]["graph_replay"]["step_us_wall"] > 0
    assert line["kimi_1024"]["bar_us_for_70pct"] == 37.0
