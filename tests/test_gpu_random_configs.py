"""Seeded random configurations: group sizes, expert counts that do not divide, top-k, hidden sizes,
paddings, node sizes and ragged token counts drawn at random, each run through the group calls and the
split calls, with and without the one-launch paths of small steps, against the oracle."""

import numpy as np
import pytest
import torch

from a2a_cases import Case, make_rank
from a2a_harness import assert_combine_close, assert_dispatch_equal, rows_needed, run_gpu, run_oracle

pytestmark = pytest.mark.gpu


def draw(seed: int):
    rng = np.random.default_rng(40_000 + seed)
    world = int(rng.choice([1, 2, 3, 4, 6, 8, 12, 16]))
    node_sizes = [d for d in range(1, world + 1) if world % d == 0]
    node_size = int(rng.choice(node_sizes))
    experts_per_rank = int(rng.integers(1, 10))
    num_experts = max(1, world * experts_per_rank - int(rng.integers(0, experts_per_rank)))
    topk = int(rng.integers(1, min(num_experts, 9) + 1))
    hidden = int(rng.choice([128, 256, 384, 1024, 2048, 4096, 7168]))
    case = Case(f"random_{seed}", int(rng.integers(1, 200)), hidden, num_experts, world, topk, 50_000 + seed,
                routing=str(rng.choice(["uniform", "zipf"])), zipf_s=1.1,
                expert_padding=int(rng.choice([1, 1, 4, 16])), outliers=bool(rng.integers(0, 2)),
                node_size=node_size)
    tokens = [int(rng.integers(0, case.num_tokens + 1)) if rng.random() < 0.8 else 0 for _ in range(world)]
    tokens[int(rng.integers(0, world))] = case.num_tokens   # one rank sends the maximum
    return case, tokens


@pytest.mark.parametrize("seed", range(16))
def test_random_configuration(seed):
    from pplx_garden_amd.native.p2p_all_to_all import FLAG_SEPARATE_ROUTING
    case, tokens = draw(seed)
    print(f"seed={seed} case={case} tokens={tokens}", flush=True)
    device = torch.device("cuda:0")
    world = [make_rank(case, r, t) for r, t in enumerate(tokens)]
    rows = rows_needed(case, world)
    want = run_oracle(case, world, rows)
    for split in (False, True):
        for flags in (0, FLAG_SEPARATE_ROUTING):
            print(f"  split={split} flags={flags}", flush=True)
            got = run_gpu(case, world, rows, device, split=split, context_flags=flags)
            assert_dispatch_equal(case, got, want)
            assert_combine_close(case, got, want)
