"""The reference's own parameter list (tests/p2p_all_to_all/test_p2p_all_to_all.py:243-550),
replayed with all ranks on one GPU, through both the group calls and the split calls."""

import pytest
import torch

from a2a_transport import RefConfig, check, make_ref_rank, rows_for, run_gpu

pytestmark = pytest.mark.gpu

F32, BF16, FP8 = torch.float32, torch.bfloat16, torch.float8_e4m3fn

MATRIX = [
    RefConfig("TP2-NIC1-FP32", 2, 1, 128, 16, 128, None, 2, F32, F32, None),
    RefConfig("TP2-NIC1-FP32-MIXED", 2, 1, 128, 16, 128, None, 2, F32, F32, None, max_private_tokens=8),
    RefConfig("TP2-NIC1-FP32-NVL", 2, 1, 128, 16, 128, None, 2, F32, F32, None, max_private_tokens=8, node_size=2),
    RefConfig("TP2-NIC1-BF16", 2, 1, 128, 16, 128, None, 2, BF16, BF16, None),
    RefConfig("TP2-NIC1-BF16-PADDED", 2, 1, 8, 16, 16, None, 2, BF16, BF16, None, expert_padding=16),
    RefConfig("TP2-NIC1-FP8", 2, 1, 2, 16, 128, 16, 2, BF16, BF16, F32),
    RefConfig("TP4-NIC1-FP32", 4, 1, 128, 128, 128, None, 8, F32, F32, None),
    RefConfig("TP4-NIC2-BF16", 4, 1, 128, 256, 7168, None, 8, BF16, BF16, None),
    RefConfig("TP8-BF16", 8, 1, 128, 128, 7168, None, 8, BF16, BF16, None),
    RefConfig("TP8-FP8", 8, 1, 256, 128, 7168, 56, 8, FP8, BF16, F32),
    RefConfig("TP4-FP8-NVL2", 4, 1, 128, 128, 7168, 56, 8, FP8, BF16, F32, node_size=2),
    RefConfig("TP2-EMPTY", 2, 1, 1, 2, 4, None, 1, F32, F32, None, max_private_tokens=32),
]

DP2 = [
    RefConfig("TP4-DP2-NIC1-BF16", 4, 2, 1, 4, 8, None, 1, BF16, BF16, None),
    RefConfig("TP4-DP2-NVL2", 4, 2, 8, 4, 4, None, 4, F32, F32, None),
]


@pytest.mark.parametrize("split", [False, True], ids=["group", "split"])
@pytest.mark.parametrize("cfg", MATRIX, ids=lambda c: c.name)
def test_reference_matrix(cfg, split):
    print(f"cfg={cfg.name} split={split}", flush=True)
    device = torch.device("cuda:0")
    world = [make_ref_rank(cfg, r) for r in range(cfg.world_size)]
    rows = rows_for(cfg, world)
    got = run_gpu(cfg, world, rows, device, split)
    check(cfg, world, rows, got)


@pytest.mark.parametrize("split", [False, True], ids=["group", "split"])
@pytest.mark.parametrize("cfg", DP2, ids=lambda c: c.name)
def test_reference_matrix_dp2(cfg, split):
    """The two configurations with ranks that share tokens (dp_size 2): ranks of a group pass the
    same data, every rank receives its experts' rows and every rank gets the combined tokens."""
    from a2a_dp import check_dp, run_gpu_dp

    print(f"cfg={cfg.name} split={split}", flush=True)
    groups = [make_ref_rank(cfg, g) for g in range(cfg.world_size // cfg.dp_size)]
    got, rows = run_gpu_dp(cfg, groups, torch.device("cuda:0"), split)
    check_dp(cfg, groups, rows, got)


def test_transposed_scale_output():
    """out_expert_x_scale may have any (token, element) strides (a2a_dispatch_recv.cu:141,153)."""
    cfg = MATRIX[9]
    device = torch.device("cuda:0")
    world = [make_ref_rank(cfg, r, 64) for r in range(cfg.world_size)]
    rows = rows_for(cfg, world)
    for split in (False, True):
        got = run_gpu(cfg, world, rows, device, split, scale_layout="col")
        check(cfg, world, rows, got)
