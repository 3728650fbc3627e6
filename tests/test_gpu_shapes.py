"""Shapes off the beaten path: experts that do not divide evenly over the ranks, top-k other than 8
(including more routes than one scale-store round covers), hidden sizes that are not a multiple of a
wavefront's slab, the largest group, repeated experts inside a token."""

import pytest
import torch

from a2a_cases import Case, make_world
from a2a_harness import assert_combine_close, assert_dispatch_equal, rows_needed, run_gpu, run_oracle

pytestmark = pytest.mark.gpu

SHAPES = [
    Case("uneven_experts", 40, 256, 10, 4, 3, 7001),                       # Le = 3, last rank owns 1 expert
    Case("rank_without_experts", 24, 128, 5, 4, 2, 7002),                  # Le = 2, rank 3 owns none
    Case("top1", 33, 384, 6, 2, 1, 7003),
    Case("top12", 50, 1536, 48, 4, 12, 7004),                              # two rounds of scale stores
    Case("top64", 9, 128, 64, 2, 64, 7005),                                # every expert, K = 64
    Case("hidden_128", 70, 128, 16, 4, 4, 7006),                           # one scale group per token
    Case("hidden_9216", 20, 9216, 32, 4, 8, 7007, outliers=True),          # 9 slabs
    Case("world_32", 64, 256, 64, 32, 4, 7008, expert_padding=8, node_size=8),
    Case("world_1", 100, 512, 7, 1, 3, 7009, expert_padding=16),
    Case("several_chunks", 700, 256, 24, 4, 8, 7010, routing="zipf", zipf_s=1.5),   # 5600 entries: 6 chunks
    Case("many_chunks", 600, 128, 64, 2, 64, 7012),                        # 38 400 entries of one source: 38 chunks
    Case("wide_ranks", 900, 128, 90, 2, 8, 7013, expert_padding=4),        # Le = 45 experts per rank, two-launch dispatch
    Case("largest_group", 400, 128, 1024, 32, 6, 7014, expert_padding=128, node_size=16),   # 32 ranks x 1024 experts
]


@pytest.mark.parametrize("split", [False, True], ids=["group", "split"])
@pytest.mark.parametrize("case", SHAPES, ids=lambda c: c.name)
def test_shapes(case, split):
    print(f"case={case.name} split={split}", flush=True)
    device = torch.device("cuda:0")
    world = make_world(case, "ragged" if case.world_size > 1 else "all")
    rows = rows_needed(case, world)
    want = run_oracle(case, world, rows)
    got = run_gpu(case, world, rows, device, split=split)
    assert_dispatch_equal(case, got, want)
    assert_combine_close(case, got, want)


@pytest.mark.parametrize("split", [False, True], ids=["group", "split"])
def test_repeated_experts_inside_a_token(split):
    """The kernels do not require the K experts of a token to be distinct
    (a2a_dispatch_send.cu:183-190 counts entries, not tokens)."""
    case = Case("repeats", 37, 256, 6, 2, 4, 7011)
    world = make_world(case, "all")
    gen = torch.Generator().manual_seed(5)
    for rd in world:
        rd.indices.copy_(torch.randint(0, case.num_experts, rd.indices.shape, generator=gen, dtype=torch.int32))
    rows = rows_needed(case, world)
    want = run_oracle(case, world, rows)
    got = run_gpu(case, world, rows, torch.device("cuda:0"), split=split)
    assert_dispatch_equal(case, got, want)
    assert_combine_close(case, got, want)
