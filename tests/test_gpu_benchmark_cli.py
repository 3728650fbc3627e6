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
