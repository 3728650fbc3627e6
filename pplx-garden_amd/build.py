"""Build the HIP library for gfx950, in-tree.

    python pplx-garden_amd/build.py

Compiles every file under csrc/ with hipcc into
pplx_garden_amd/lib/liba2a_mi355.so, examples/selftest.cpp (a C++ caller of
the C ABI) into pplx_garden_amd/lib/a2a_selftest and examples/ceilings.hip (what
the memory system sustains for the step's access shapes, without the library)
into pplx_garden_amd/lib/a2a_ceilings.  hipcc cross-compiles without a GPU.
"""

from __future__ import annotations

import os
import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent
REPO = ROOT.parent
CSRC = ROOT / "csrc"
OUT_DIR = ROOT / "pplx_garden_amd" / "lib"
LIB_NAME = "liba2a_mi355.so"

SOURCES = ["a2a_route.hip", "a2a_dispatch.hip", "a2a_combine.hip", "a2a_staged.hip", "a2a_context.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    # packed fp32 instructions are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wextra", "-Wno-unused-parameter", "-Wno-unknown-warning-option",
]


def library_path() -> Path:
    return OUT_DIR / LIB_NAME


def selftest_path() -> Path:
    return OUT_DIR / "a2a_selftest"


def ceilings_path() -> Path:
    return OUT_DIR / "a2a_ceilings"


def build(verbose: bool = True) -> Path:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    OUT_DIR.mkdir(parents=True, exist_ok=True)
    obj_dir = ROOT / "build"
    obj_dir.mkdir(exist_ok=True)
    includes = ["-I", str(REPO / "include"), "-I", str(CSRC)]
    procs = []
    objects = []
    for src in SOURCES:
        obj = obj_dir / (src + ".o")
        objects.append(str(obj))
        cmd = [hipcc, *HIPCC_FLAGS, *includes, "-c", str(CSRC / src), "-o", str(obj)]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    failed = False
    for src, proc in procs:
        out, _ = proc.communicate()
        # hipcc's host pass does not know the packed-fp32 feature name; that warning is harmless
        lines = [l for l in out.splitlines() if "packed-fp32-ops" not in l and l.strip()]
        if lines and verbose:
            print("\n".join(lines), flush=True)
        if proc.returncode != 0:
            print(f"hipcc failed on {src}", file=sys.stderr)
            if not verbose:
                print(out, file=sys.stderr)
            failed = True
    if failed:
        raise RuntimeError("hipcc failed")
    link = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objects, "-o", str(library_path()), "-ldl"]
    if verbose:
        print(" ".join(link), flush=True)
    subprocess.run(link, check=True)
    # A caller of the C ABI with nothing but the HIP runtime around it (no Python, no torch).
    selftest = [hipcc, "-O2", "-std=c++17", "-I", str(REPO / "include"), str(ROOT / "examples" / "selftest.cpp"),
                "-o", str(selftest_path()), "-L", str(OUT_DIR), "-la2a_mi355", "-Wl,-rpath,$ORIGIN"]
    if verbose:
        print(" ".join(selftest), flush=True)
    subprocess.run(selftest, check=True)
    # The yardstick of the roofline figures: plain kernels of the step's access shapes.
    ceilings = [hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
                "-packed-fp32-ops", str(ROOT / "examples" / "ceilings.hip"), "-o", str(ceilings_path())]
    if verbose:
        print(" ".join(ceilings), flush=True)
    out = subprocess.run(ceilings, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    lines = [l for l in out.stdout.splitlines() if "packed-fp32-ops" not in l and l.strip()]
    if lines and verbose:
        print("\n".join(lines), flush=True)
    if out.returncode != 0:
        raise RuntimeError("hipcc failed on ceilings.hip")
    return library_path()


if __name__ == "__main__":
    print(build())
