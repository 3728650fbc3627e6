"""The baseline's full-size configurations: the GPU sends one rank's batch and holds the
receive buffers of every logical rank.  Checked row by row against the oracle and through
properties that do not depend on the size."""

import numpy as np
import pytest
import torch

import a2a_oracle as oracle
import c_oracle
from a2a_cases import C3, C4, bf16_codes, make_world
from a2a_harness import assert_combine_close, assert_dispatch_equal, rows_needed, run_gpu, run_oracle

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("case", [C3, C4], ids=lambda c: c.name)
def test_full_size_one_source(case):
    print(f"case={case.name}", flush=True)
    device = torch.device("cuda:0")
    world = make_world(case, "one")
    rows = rows_needed(case, world)
    want = run_oracle(case, world, rows)
    got = run_gpu(case, world, rows, device)
    assert_dispatch_equal(case, got, want)
    assert_combine_close(case, got, want)

    N, Le, K = case.world_size, case.experts_per_rank, case.topk
    idx = world[0].indices.numpy().astype(np.int64)
    # counts are the bincount of the routing (tests/p2p_all_to_all/data.py:50-53)
    counts = np.bincount(idx.reshape(-1), minlength=case.num_experts)
    for r in range(N):
        np.testing.assert_array_equal(got.num_tokens[r][: len(counts[r * Le:(r + 1) * Le])], counts[r * Le:(r + 1) * Le])
    # expert ranges start at multiples of the padding and hold tokens in ascending order
    q, s = oracle.quantize_block128(bf16_codes(world[0].x))
    slots = want.slots[0]
    for r in range(N):
        start = 0
        for le in range(Le):
            e = r * Le + le
            if e >= case.num_experts:
                break
            assert start % case.expert_padding == 0
            toks = np.flatnonzero((idx == e).any(axis=1))          # ascending tokens routed to e
            np.testing.assert_array_equal(got.x[r][start:start + len(toks)], q[toks])
            start = oracle.round_up(start + len(toks), case.expert_padding)
    # a checksum of checksums: every token's bytes appear exactly K times over all receivers
    total = sum(int(got.x[r][want.written[r]].astype(np.uint64).sum()) for r in range(N))
    assert total == K * int(q.astype(np.uint64).sum())
    # the reference's round trip: combine(2 * dequant(dispatch(x))) ~ 2 x (weights sum to 1)
    x = oracle.bf16_to_f32(bf16_codes(world[0].x)).astype(np.float64)
    out = oracle.bf16_to_f32(got.out_tokens[0]).astype(np.float64)
    amax = np.abs(x).reshape(x.shape[0], -1, 128).max(axis=2, keepdims=True)
    bound = np.repeat(2 * amax / 448 * 16 + 2 ** -7 * 2 * amax, 128, axis=2).reshape(x.shape)
    assert (np.abs(out - 2 * x) <= bound).all()
    del slots, s


def test_full_size_combine_is_bit_exact_with_true_fma():
    """The kernel's float fused multiply-add chain, k ascending, against the C restatement."""
    case = C3
    device = torch.device("cuda:0")
    world = make_world(case, "one")
    rows = rows_needed(case, world)
    got = run_gpu(case, world, rows, device)
    N = case.world_size
    cw = c_oracle.CWorld(case.num_experts, N, N, case.expert_padding, case.hidden_dim, case.topk, rows)
    cw.route_all([rd.indices.numpy() for rd in world])
    cw.dispatch([bf16_codes(rd.x) for rd in world])
    cw.act()
    outs = cw.combine([rd.weights.numpy() for rd in world])
    np.testing.assert_array_equal(got.out_tokens[0], outs[0])


@pytest.mark.parametrize("split", [False, True], ids=["group", "split"])
def test_full_size_all_sources(split):
    """The prefill shape with ALL 8 logical ranks sending 4096 tokens (32 768 tokens, 262 144 copies): the
    group calls, and the four split calls, against the C restatement, dispatch and combine bit for bit."""
    case = C3
    device = torch.device("cuda:0")
    world = make_world(case, "all")
    rows = rows_needed(case, world)
    N = case.world_size
    rng = np.random.default_rng(1)
    ys = [rng.integers(0x3C00, 0x4000, size=(rows, case.hidden_dim), dtype=np.uint16) for _ in range(N)]
    got = run_gpu(case, world, rows, device, expert_y_override=ys, split=split)
    c_oracle.set_threads(16)
    try:
        cw = c_oracle.CWorld(case.num_experts, N, N, case.expert_padding, case.hidden_dim, case.topk, rows)
        cw.route_all([rd.indices.numpy() for rd in world])
        cw.dispatch([bf16_codes(rd.x) for rd in world])
        for r in range(N):
            cw.y[r][:] = ys[r]
        outs = cw.combine([rd.weights.numpy() for rd in world])
    finally:
        c_oracle.set_threads(1)
    for r in range(N):
        per_expert = cw.tpe[r * cw.Le:(r + 1) * cw.Le]
        n = int(per_expert.sum())                      # padding 1: the rows are dense
        np.testing.assert_array_equal(got.num_tokens[r], per_expert.astype(np.int32))
        np.testing.assert_array_equal(got.x[r][:n], cw.out_x[r][:n])
        np.testing.assert_array_equal(got.x_scale[r][:n].view(np.uint32), cw.out_s[r][:n].view(np.uint32))
        assert (got.x[r][n:] == 0xA5).all()
        np.testing.assert_array_equal(got.out_tokens[r], outs[r])
