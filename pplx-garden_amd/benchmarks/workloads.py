"""Workloads of the benchmarks and the parity tests, generated on the CPU.

Every tensor comes from `torch.Generator('cpu')` seeded per (case, rank), so the
oracle and the GPU see identical bits.  The routing generators restate the
reference's (tests/p2p_all_to_all/data.py:7-22: K distinct experts per token)
and add the skewed ones the benchmark configurations ask for.
"""

from __future__ import annotations

from dataclasses import dataclass, replace
from typing import List, Optional

import numpy as np
import torch


@dataclass(frozen=True)
class Case:
    name: str
    num_tokens: int          # T per sending rank
    hidden_dim: int          # H
    num_experts: int         # E
    world_size: int          # N logical ranks
    topk: int                # K
    seed: int
    routing: str = "uniform"     # "uniform" | "zipf" | "reference"
    zipf_s: float = 0.0
    expert_padding: int = 1
    outliers: bool = False       # 1 % of the elements multiplied by 50
    node_size: Optional[int] = None
    weights: str = "softmax"     # "softmax" | "normalized" (rand / sum, as the reference)

    @property
    def experts_per_rank(self) -> int:
        return -(-self.num_experts // self.world_size)

    @property
    def hidden_dim_scale(self) -> int:
        return self.hidden_dim // 128


# The five configurations of the baseline (C0..C4).
C0 = Case("c0_plumbing", 64, 2048, 32, 4, 4, 1000)
C1 = Case("c1_qwen3_decode", 128, 2048, 128, 8, 8, 1001)
C2 = Case("c2_dsv3_decode", 128, 7168, 256, 8, 8, 1002, outliers=True)
C3 = Case("c3_dsv3_prefill", 4096, 7168, 256, 8, 8, 1003, routing="zipf", zipf_s=1.2)
C4 = Case("c4_kimi_mixed", 1024, 7168, 384, 16, 8, 1004, routing="zipf", zipf_s=1.0,
          expert_padding=128)
BASELINE_CASES = [C0, C1, C2, C3, C4]


def scaled(case: Case, num_tokens: int) -> Case:
    return replace(case, name=f"{case.name}_t{num_tokens}", num_tokens=num_tokens)


def _generator(case: Case, rank: int) -> torch.Generator:
    g = torch.Generator(device="cpu")
    g.manual_seed(case.seed + 7919 * rank)
    return g


def make_indices(case: Case, rank: int, num_tokens: Optional[int] = None) -> torch.Tensor:
    """[T, K] expert ids, K distinct per token, as int32 (viewed as uint32 by the operator)."""
    T = case.num_tokens if num_tokens is None else num_tokens
    g = _generator(case, rank)
    E, K = case.num_experts, case.topk
    if T == 0:
        return torch.zeros((0, K), dtype=torch.int32)
    if case.routing == "uniform":
        idx = torch.rand((T, E), generator=g).topk(K, dim=-1).indices
    elif case.routing == "reference":
        # tests/p2p_all_to_all/data.py:14-22
        scores = torch.randn((T, E), generator=g).abs() + 1
        idx = torch.topk(scores, K, dim=-1, largest=True, sorted=True).indices
    elif case.routing == "zipf":
        perm_gen = torch.Generator(device="cpu")
        perm_gen.manual_seed(case.seed)          # same popularity on every rank
        perm = torch.randperm(E, generator=perm_gen)
        p = torch.empty(E, dtype=torch.float64)
        p[perm] = torch.arange(1, E + 1, dtype=torch.float64) ** (-case.zipf_s)
        idx = torch.multinomial(p.expand(T, E), K, replacement=False, generator=g)
    else:
        raise ValueError(case.routing)
    return idx.to(torch.int32)


@dataclass
class RankData:
    x: torch.Tensor          # [T, H] bfloat16
    indices: torch.Tensor    # [T, K] int32 (non-negative)
    weights: torch.Tensor    # [T, K] float32

    @property
    def indices_u32(self) -> torch.Tensor:
        return self.indices.view(torch.uint32)


def make_rank(case: Case, rank: int, num_tokens: Optional[int] = None) -> RankData:
    T = case.num_tokens if num_tokens is None else num_tokens
    indices = make_indices(case, rank, T)
    g = _generator(case, rank)
    g.manual_seed(case.seed + 7919 * rank + 1)
    x = torch.randn((T, case.hidden_dim), generator=g)
    if case.outliers:
        mask = torch.rand((T, case.hidden_dim), generator=g) < 0.01
        x = torch.where(mask, x * 50.0, x)
    x = x.to(torch.bfloat16)
    if case.weights == "softmax":
        w = torch.softmax(torch.randn((T, case.topk), generator=g), dim=-1)
    else:
        # tests/p2p_all_to_all/data.py:93-99
        w = torch.rand((T, case.topk), generator=g)
        w = w / w.sum(dim=-1, keepdim=True)
    return RankData(x=x, indices=indices, weights=w.to(torch.float32).contiguous())


def make_world(case: Case, sources: str = "all") -> List[RankData]:
    """Inputs of every rank.  sources="one": only rank 0 has tokens (the share of
    work of one GPU); "all": every rank sends `num_tokens`; "ragged": rank r
    sends a different number of tokens, some none."""
    out = []
    for r in range(case.world_size):
        if sources == "all":
            T = case.num_tokens
        elif sources == "one":
            T = case.num_tokens if r == 0 else 0
        elif sources == "ragged":
            T = [case.num_tokens, 0, max(case.num_tokens // 3, 1), 1][r % 4]
        else:
            raise ValueError(sources)
        out.append(make_rank(case, r, T))
    return out


def bf16_codes(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def rows_needed(case: Case, world) -> int:
    """Rows a receive buffer needs so that no rank overflows (with padding)."""
    Le = case.experts_per_rank
    counts = np.zeros(case.num_experts, dtype=np.int64)
    for rd in world:
        counts += np.bincount(rd.indices.numpy().reshape(-1), minlength=case.num_experts)
    pad = case.expert_padding
    padded = (counts + pad - 1) // pad * pad
    per_rank = [padded[r * Le:(r + 1) * Le].sum() for r in range(case.world_size)]
    return int(max(max(per_rank), 1))
