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


SINGLE = [
    (RefConfig("ONE-SENDER-FP8", 8, 1, 128, 256, 7168, 56, 8, FP8, BF16, F32), 128, 3),
    (RefConfig("ONE-SENDER-FP8-COL", 8, 1, 128, 128, 2048, 16, 8, FP8, BF16, F32, expert_padding=16), 100, 0),
    (RefConfig("ONE-SENDER-BF16", 4, 1, 64, 64, 7168, None, 6, BF16, BF16, None), 37, 2),
    (RefConfig("ONE-SENDER-F32-3-TOKENS", 16, 1, 8, 48, 256, None, 3, F32, F32, None, node_size=4), 3, 9),
    (RefConfig("ONE-SENDER-FP8-700", 8, 1, 700, 256, 7168, 56, 8, FP8, BF16, F32), 700, 5),
    (RefConfig("ONE-SENDER-BF16-900", 16, 1, 900, 96, 2048, None, 8, BF16, BF16, None, expert_padding=8), 900, 1),
    (RefConfig("ONE-SENDER-FP8-1000-TOP3", 4, 1, 1000, 64, 1024, 8, 3, FP8, F32, F32), 1000, 0),
]


@pytest.mark.parametrize("cfg,tokens,sender", SINGLE, ids=lambda v: v.name if isinstance(v, RefConfig) else str(v))
def test_one_sender_in_transport_mode(cfg, tokens, sender):
    """One rank has tokens (one GPU's share of a decode step) and the rows travel as the caller's bytes
    with the caller's scales: the small step of one source takes the kernel with a spare wavefront per
    token (or per four tokens, from 448 tokens on) also when it does not quantise.  fp8 rows with 56, 16
    and 8 scales a row (row-major and transposed output), bf16 and float rows without scales, fewer tokens
    than tables to write, mid-size steps of one and of two rounds."""
    device = torch.device("cuda:0")
    world = [make_ref_rank(cfg, r, tokens if r == sender else 0) for r in range(cfg.world_size)]
    rows = rows_for(cfg, world)
    for layout in (("row", "col") if cfg.hidden_dim_scale else ("row",)):
        got = run_gpu(cfg, world, rows, device, False, scale_layout=layout)
        check(cfg, world, rows, got)

