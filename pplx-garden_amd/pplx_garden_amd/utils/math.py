"""Integer helpers and the latency statistics the benchmark reports.

Same definitions as the reference's python/pplx_garden/utils/math.py:5-109
(round_up, ceil_div, and the percentile rule of `Statistics`), restated.
"""

from __future__ import annotations

import math
from dataclasses import dataclass, fields


def round_up(n: int, m: int) -> int:
    return -(-n // m) * m


def ceil_div(n: int, m: int) -> int:
    return -(-n // m)


def _percentile(ordered: list[float], p: float) -> float:
    # utils/math.py:75-79: the sample at int(n*p); when n*p is fractional and a
    # next sample exists, the midpoint of the two.
    n = len(ordered)
    index = int(n * p)
    if n * p == index or index + 1 >= n:
        return ordered[index]
    return (ordered[index] + ordered[index + 1]) / 2


@dataclass
class Statistics:
    mean: float = 0.0
    stddev: float = 0.0
    min: float = 0.0
    p01: float = 0.0
    p25: float = 0.0
    p50: float = 0.0
    p75: float = 0.0
    p95: float = 0.0
    p99: float = 0.0
    max: float = 0.0

    @classmethod
    def create(cls, xs: list[float]) -> "Statistics":
        if not xs:
            return cls()
        ordered = sorted(xs)
        n = len(xs)
        mean = math.fsum(xs) / n
        var = math.fsum((x - mean) ** 2 for x in xs) / (n - 1) if n > 1 else 0.0
        return cls(
            mean=mean, stddev=math.sqrt(var), min=ordered[0],
            p01=_percentile(ordered, 0.01), p25=_percentile(ordered, 0.25),
            p50=_percentile(ordered, 0.5), p75=_percentile(ordered, 0.75),
            p95=_percentile(ordered, 0.95), p99=_percentile(ordered, 0.99),
            max=ordered[-1])

    def as_dict(self) -> dict:
        return {f.name: getattr(self, f.name) for f in fields(self)}

    def __str__(self) -> str:
        parts = [f"mean={self.mean:.1f}±{self.stddev:.1f} μs"]
        for name in ("min", "p01", "p25", "p50", "p75", "p95", "p99", "max"):
            parts.append(f"{name}={getattr(self, name):.1f} μs")
        return ", ".join(parts)
