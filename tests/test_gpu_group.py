"""Parity of the group calls (every rank calls dispatch()/combine() with send and recv)."""

import pytest
import torch

from a2a_cases import C0, C1, C2, C3, C4, make_world, scaled
from a2a_harness import assert_combine_close, assert_dispatch_equal, rows_needed, run_gpu, run_oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def device():
    return torch.device("cuda:0")


@pytest.mark.parametrize("case,sources", [
    (C0, "all"), (C0, "one"), (C0, "ragged"),
    (C1, "all"), (C1, "one"),
    (C2, "all"), (C2, "one"),
    (scaled(C3, 512), "all"),
    (scaled(C4, 256), "all"), (scaled(C4, 256), "ragged"),
], ids=lambda v: v.name if hasattr(v, "name") else v)
def test_group_parity(case, sources, device):
    print(f"case={case.name} sources={sources}", flush=True)
    world = make_world(case, sources)
    rows = rows_needed(case, world)
    want = run_oracle(case, world, rows)
    got = run_gpu(case, world, rows, device)
    assert_dispatch_equal(case, got, want)
    assert_combine_close(case, got, want)
    # the fused multiply-add chain is deterministic: expect (almost) every element bit-equal
    same = sum(int((g == w).sum()) for g, w in zip(got.out_tokens, want.out_tokens))
    total = sum(g.size for g in got.out_tokens)
    assert same >= total * 0.9999, (same, total)


@pytest.mark.parametrize("split", [False, True], ids=["group", "split"])
@pytest.mark.parametrize("case,sources", [(C0, "ragged"), (C2, "all"), (C2, "one")],
                         ids=lambda v: v.name if hasattr(v, "name") else v)
def test_small_steps_with_separate_routing_kernels(case, sources, split, device):
    """Small steps normally count their routing inside the dispatch (or send) kernel; with
    A2A_FLAG_SEPARATE_ROUTING they run the routing kernels first.  Both must match the oracle, hence
    each other, bit for bit."""
    from pplx_garden_amd.native.p2p_all_to_all import FLAG_SEPARATE_ROUTING
    print(f"case={case.name} sources={sources} split={split}", flush=True)
    world = make_world(case, sources)
    rows = rows_needed(case, world)
    want = run_oracle(case, world, rows)
    for flags in (0, FLAG_SEPARATE_ROUTING):
        got = run_gpu(case, world, rows, device, split=split, context_flags=flags)
        assert_dispatch_equal(case, got, want)
        assert_combine_close(case, got, want)


def test_steps_of_different_sizes_on_one_context(device):
    """One set of operators, a sequence of steps that take the one-launch dispatch, the two-launch
    dispatch (whose step totals alternate between two copies on the device) and the split calls in
    turn: every step must match the oracle, whatever ran before it."""
    from a2a_cases import Case, make_rank
    from a2a_harness import make_ops
    case = Case("mixed_steps", 1500, 256, 32, 8, 8, 8100, expert_padding=4)
    _, ops = make_ops(case, device)
    try:
        steps = [([40, 0, 13, 1, 0, 0, 40, 7], False), ([1500, 0, 0, 0, 0, 0, 0, 0], False),
                 ([1500, 300, 0, 1, 90, 0, 0, 1200], False), ([128] * 8, True), ([600] * 8, False),
                 ([0] * 8, False), ([64] * 8, False), ([1100, 0, 0, 0, 0, 0, 0, 5], True),
                 ([1100, 0, 0, 0, 0, 0, 0, 5], False), ([700] * 8, False)]
        for i, (tokens, split) in enumerate(steps):
            print(f"step {i}: tokens={tokens} split={split}", flush=True)
            step_case = scaled(case, max(tokens))
            world = [make_rank(step_case, r, t) for r, t in enumerate(tokens)]
            rows = rows_needed(step_case, world)
            want = run_oracle(step_case, world, rows)
            got = run_gpu(step_case, world, rows, device, split=split, ops=ops)
            assert_dispatch_equal(step_case, got, want)
            assert_combine_close(step_case, got, want)
    finally:
        for op in ops:
            op.destroy()
