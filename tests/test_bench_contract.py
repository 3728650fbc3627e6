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


def test_traffic_is_reported_only_for_the_sources_it_was_measured_on(tmp_path, monkeypatch):
    """`roofline.traffic` comes from a counter summary under profiles/ that records the fingerprint of the
    kernel sources it was measured on; with other sources the benchmark reports no traffic at all."""
    sys.path.insert(0, str(REPO))
    import bench
    fingerprint = bench.kernel_sources_sha256()
    assert len(fingerprint) == 64 and fingerprint == bench.kernel_sources_sha256()
    # comments and blank lines do not count, code does
    assert bench.code_only("int a = 1;  // one\n\n/* two\n lines */ int b;\n") == "int a = 1;\nint b;"
    assert bench.code_only("int a = 2;") != bench.code_only("int a = 1;")
    traffic, note = bench.measured_traffic()
    if traffic:      # the committed summary belongs to the committed sources
        assert 0.99 * 528_744_448 < traffic["combine_gather_kernel"] < 1.05 * 528_744_448
        assert 0.99 * 301_072_384 < traffic["dispatch_resolve_kernel"] < 1.05 * 301_072_384
    else:
        assert "other kernel sources" in note
    summary = tmp_path / "summary.md"
    monkeypatch.setattr(bench, "TRAFFIC_PROFILE", summary)
    assert bench.measured_traffic()[0] == {}                                   # no summary
    summary.write_text("csrc_sha256: " + "0" * 64 + "\ntraffic_bytes: combine_gather_kernel=7\n")
    assert bench.measured_traffic()[0] == {}                                   # other sources
    summary.write_text(f"text\ncsrc_sha256: {fingerprint}\ntraffic_bytes: combine_gather_kernel=7\n"
                       "traffic_bytes: dispatch_resolve_kernel=9\n")
    assert bench.measured_traffic()[0] == {"combine_gather_kernel": 7, "dispatch_resolve_kernel": 9}
