"""Groups of ranks that hold the same tokens (dp_size > 1) beyond the reference's two tiny cases:
several nodes, several groups per node, padding, scales."""

import pytest
import torch

from a2a_dp import check_dp, run_gpu_dp
from a2a_transport import RefConfig, make_ref_rank

pytestmark = pytest.mark.gpu

BF16, F32, FP8 = torch.bfloat16, torch.float32, torch.float8_e4m3fn

CONFIGS = [
    RefConfig("dp2_two_nodes", 8, 2, 64, 32, 256, None, 4, BF16, BF16, None, expert_padding=4, node_size=4),
    RefConfig("dp4_one_node", 8, 4, 40, 16, 128, None, 3, F32, F32, None),
    RefConfig("dp2_fp8_scales", 4, 2, 96, 32, 1024, 8, 8, FP8, BF16, F32, node_size=2),
    RefConfig("dp8_single_group", 8, 8, 33, 24, 256, None, 6, BF16, BF16, None),
    # large enough for the two-launch dispatch (4 groups x 700 tokens x 8 = 22 400 entries)
    RefConfig("dp2_two_launch", 8, 2, 700, 32, 256, None, 8, BF16, BF16, None, expert_padding=4, node_size=4),
    RefConfig("dp4_two_launch_fp8", 8, 4, 1300, 48, 512, 4, 8, FP8, BF16, F32, node_size=8),
    # one group of 600 tokens x 6: the one-launch dispatch of a larger single source, rows copied as bytes
    RefConfig("dp8_single_group_larger", 8, 8, 600, 24, 256, None, 6, BF16, BF16, None, expert_padding=3),
    # no dp groups, the caller's scales, 800 tokens a rank: the one-launch send of the split calls copies scale rows
    RefConfig("dp1_fp8_scales_800", 4, 1, 800, 32, 1024, 8, 8, FP8, BF16, F32, node_size=2),
]


@pytest.mark.parametrize("split", [False, True], ids=["group", "split"])
@pytest.mark.parametrize("cfg", CONFIGS, ids=lambda c: c.name)
def test_dp_groups(cfg, split):
    print(f"cfg={cfg.name} split={split}", flush=True)
    groups = [make_ref_rank(cfg, g) for g in range(cfg.world_size // cfg.dp_size)]
    got, rows = run_gpu_dp(cfg, groups, torch.device("cuda:0"), split)
    check_dp(cfg, groups, rows, got)


ONE_GROUP_SENDS = [
    (RefConfig("dp2_one_group_sends", 8, 2, 96, 64, 1024, 8, 8, FP8, BF16, F32, node_size=4), 96, 2),
    (RefConfig("dp4_one_group_sends_bf16", 8, 4, 50, 16, 512, None, 4, BF16, BF16, None, expert_padding=4), 50, 1),
    (RefConfig("dp2_one_group_sends_700", 4, 2, 700, 32, 1024, 8, 8, FP8, BF16, F32, node_size=2), 700, 0),
]


@pytest.mark.parametrize("split", [False, True], ids=["group", "split"])
@pytest.mark.parametrize("cfg,tokens,sender", ONE_GROUP_SENDS, ids=lambda v: v.name if isinstance(v, RefConfig) else str(v))
def test_one_dp_group_sends(cfg, tokens, sender, split):
    """Of several dp groups one alone has tokens (the others hold none this step): the one-launch kernels
    of a single source serve the step, and every rank of every group still receives its experts' rows
    and the sending group's ranks their combined tokens."""
    print(f"cfg={cfg.name} split={split}", flush=True)
    groups = [make_ref_rank(cfg, g, tokens if g == sender else 0) for g in range(cfg.world_size // cfg.dp_size)]
    got, rows = run_gpu_dp(cfg, groups, torch.device("cuda:0"), split)
    check_dp(cfg, groups, rows, got)


def test_accumulate_is_refused_with_dp_groups():
    """python/pplx_garden/kernels/p2p_all_to_all.py:457-458"""
    from pplx_garden_amd.distributed.loopback import LoopbackWorld
    from pplx_garden_amd.kernels.p2p_all_to_all import P2PAllToAll

    lw = LoopbackWorld(2)
    dev = torch.device("cuda:0")
    op = P2PAllToAll(max_num_tokens=4, num_experts=4, expert_padding=1, hidden_dim=16, hidden_dim_scale=None,
                     in_dtype=BF16, out_dtype=BF16, scale_dtype=None, num_experts_per_token=1, nets_per_gpu=1,
                     max_private_tokens=None, device=dev, dp_group=lw.dp_group(0, 2), node_group=None,
                     global_group=lw.group(0))
    try:
        with pytest.raises(AssertionError):
            op.combine(out_tokens=torch.zeros((1, 16), dtype=BF16, device=dev),
                       indices=torch.zeros((1, 1), dtype=torch.int32, device=dev).view(torch.uint32),
                       weights=torch.ones((1, 1), device=dev), expert_y=torch.zeros((4, 16), dtype=BF16, device=dev),
                       accumulate=True)
    finally:
        op.destroy()
