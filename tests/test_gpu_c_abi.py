"""The C ABI driven by a C++ program with nothing but the HIP runtime around it (no Python, no torch):
one step through the group calls, one through the split calls and one through the dispatch that
allocates nothing, checked on the host by the program
itself (expert counts against a host histogram, the reference's round-trip identity)."""

import subprocess
import sys
from pathlib import Path

import pytest

pytestmark = pytest.mark.gpu


def test_cpp_caller_of_the_c_abi():
    repo = Path(__file__).resolve().parent.parent
    sys.path.insert(0, str(repo / "pplx-garden_amd"))
    exe = repo / "pplx-garden_amd" / "pplx_garden_amd" / "lib" / "a2a_selftest"
    assert exe.exists(), "run pplx-garden_amd/build.py first"
    print("running", exe, flush=True)
    done = subprocess.run([str(exe)], capture_output=True, text=True, timeout=100)
    print(done.stdout, done.stderr, flush=True)
    assert done.returncode == 0, done.stderr
    assert "selftest passed" in done.stdout
    assert "group calls" in done.stdout and "split calls" in done.stdout
    assert "static dispatch: identical to a2a_dispatch" in done.stdout
    # a first call under stream capture is refused; a refused call leaves no node in the caller's graph
    assert "first call under capture: refused" in done.stdout
    assert "refused call recorded nothing, accepted call recorded" in done.stdout


def test_memory_ceilings_program_runs():
    """The yardstick of the roofline figures (plain kernels of the step's access shapes) runs and reports
    every line; its numbers are read by people, not asserted here."""
    repo = Path(__file__).resolve().parent.parent
    exe = repo / "pplx-garden_amd" / "pplx_garden_amd" / "lib" / "a2a_ceilings"
    assert exe.exists(), "run pplx-garden_amd/build.py first"
    print("running", exe, flush=True)
    done = subprocess.run([str(exe)], capture_output=True, text=True, timeout=100)
    print(done.stdout, done.stderr, flush=True)
    assert done.returncode == 0, done.stderr
    lines = [l for l in done.stdout.splitlines() if "GB/s" in l]
    # the yardstick lines that the summaries under profiles/ quote as ceilings
    for name in ("read-only sweep, 512 MiB", "write-only sweep, 512 MiB, 512 workgroups",
                 "128 workgroups x 64 KiB streams", "copy, 512 MiB read + 512 MiB written",
                 "push (pack's shape), random payload", "push (pack's shape), all-zero rows written",
                 "gather (combine's shape)", "gather, reads only", "the gather's output alone",
                 "rows of 7392 bytes, read and written", "rows of 14336 bytes, read and written",
                 "push, 1024 tokens", "gather, 1024 tokens"):
        hits = [l for l in lines if name in l]
        assert hits, name
        for l in hits:                     # "<name>   <us> us   <GB/s> GB/s": two positive numbers
            us, gbs = float(l.split()[-4]), float(l.split()[-2])
            assert 0.5 < us < 1e4 and 100 < gbs < 8000, l
    # what a launch costs by itself
    launches = [l for l in done.stdout.splitlines() if "us per launch" in l]
    assert len(launches) == 5 and all(0.3 < float(l.split()[-4]) < 100 for l in launches), launches
    assert any("own start and stop events" in l for l in done.stdout.splitlines())
