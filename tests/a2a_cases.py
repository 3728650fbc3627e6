"""The workloads of the parity tests are the benchmark's: pplx-garden_amd/benchmarks/workloads.py."""

from workloads import *  # noqa: F401,F403
from workloads import _generator  # noqa: F401
