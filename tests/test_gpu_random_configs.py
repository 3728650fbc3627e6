"""Seeded random configurations: group sizes, expert counts that do not divide, top-k, hidden sizes,
paddings, node sizes and ragged token counts drawn at random, each run through the group calls and the
split calls, with and without the one-launch paths of small steps, against the oracle; and sequences of
steps of varying size (empty ones, one sender, all senders) on one context, group and split calls mixed."""

from dataclasses import replace

import numpy as np
import pytest
import torch

from a2a_cases import Case, make_rank
from a2a_harness import assert_combine_close, assert_dispatch_equal, make_ops, rows_needed, run_gpu, run_oracle

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


def draw_sequence(seed: int):
    rng = np.random.default_rng(190_000 + seed)
    world = int(rng.choice([1, 2, 4, 8, 16]))
    node_size = int(rng.choice([d for d in range(1, world + 1) if world % d == 0]))
    experts_per_rank = int(rng.integers(1, 34))
    num_experts = max(1, world * experts_per_rank - int(rng.integers(0, experts_per_rank)))
    topk = int(rng.integers(1, min(num_experts, 9) + 1))
    hidden = int(rng.choice([256, 1024, 2048]))
    T = int(rng.integers(300, 1200)) if rng.random() < 0.4 else int(rng.integers(1, 200))   # both dispatch paths
    case = Case(f"sequence_{seed}", T, hidden, num_experts, world, topk, 170_000 + seed,
                routing=str(rng.choice(["uniform", "zipf"])), zipf_s=1.2,
                expert_padding=int(rng.choice([1, 4, 16])), node_size=node_size)
    steps = []
    for _ in range(6):
        mode = rng.random()
        if mode < 0.5:
            tokens = [int(rng.integers(0, T + 1)) if rng.random() < 0.7 else 0 for _ in range(world)]
        elif mode < 0.65:
            tokens = [0] * world
        elif mode < 0.8:
            tokens = [0] * world
            tokens[int(rng.integers(0, world))] = int(rng.integers(1, T + 1))
        else:
            tokens = [T] * world
        steps.append((tokens, bool(rng.integers(0, 2))))
    return case, steps, int(rng.choice([0, 0, 2]))   # 2 = A2A_FLAG_SEPARATE_ROUTING


@pytest.mark.parametrize("seed", range(8))
def test_random_sequence_of_steps_on_one_context(seed):
    """What one step leaves behind in the context (the two copies of the step totals and whose turn it is,
    the marks of empty senders, staged rows of a larger step) must not show in the next."""
    case, steps, flags = draw_sequence(seed)
    print(f"seed={seed} case={case} flags={flags}", flush=True)
    device = torch.device("cuda:0")
    _, ops = make_ops(case, device, context_flags=flags)
    try:
        for i, (tokens, split) in enumerate(steps):
            step_case = replace(case, seed=case.seed + 1000 * i)
            print(f"  step {i} split={split} tokens={tokens}", flush=True)
            world = [make_rank(step_case, r, t) for r, t in enumerate(tokens)]
            rows = max(rows_needed(step_case, world), 1)
            want = run_oracle(step_case, world, rows)
            got = run_gpu(step_case, world, rows, device, split=split, ops=ops)
            assert_dispatch_equal(step_case, got, want)
            assert_combine_close(step_case, got, want)
    finally:
        for op in ops:
            op.destroy()
