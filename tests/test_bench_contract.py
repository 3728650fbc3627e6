"""What the benchmark and the entry points promise without a GPU."""

import subprocess
import sys
from pathlib import Path

REPO = Path(__file__).resolve().parent.parent


def test_bench_refuses_more_than_one_gpu():
    """Every logical rank lives in one GPU's memory: a run on several GPUs is refused with a message."""
    done = subprocess.run([sys.executable, str(REPO / "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                          timeout=120)
    assert done.returncode != 0
    assert "one GPU" in done.stdout + done.stderr
    assert not done.stdout.strip().startswith("{")      # no result line


def test_algorithmic_bytes_per_token():
    """Bytes per token of the DeepSeek-V3 shape: dispatch 2H + 4K + K(H + 4H/128), combine 2HK + 8K + 2H."""
    sys.path.insert(0, str(REPO))
    import bench
    d, c = bench.algorithmic_bytes(1, 7168, 8)
    assert (d, c) == (73_504, 129_088)
    d, c = bench.algorithmic_bytes(4096, 7168, 8)
    assert d + c == 4096 * 202_592


def test_entry_points_exist():
    sys.path.insert(0, str(REPO))
    import __graft_entry__ as entry
    assert callable(entry.build) and callable(entry.smoke)
