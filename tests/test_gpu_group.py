"""Parity of the group calls (every rank calls dispatch()/combine() with send and recv)."""

import numpy as np
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
