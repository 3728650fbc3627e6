"""The torch restatement of the path (the many-threaded CPU baseline of the benchmark) against the
numpy oracle: counts, slots, fp8 bytes and scales bit for bit; combine within the baseline's tolerance
(torch multiplies and adds in two rounded steps where the oracle fuses them)."""

from dataclasses import replace

import numpy as np
import pytest
import torch

import a2a_oracle as oracle
import a2a_oracle_torch as torch_oracle
from a2a_cases import C0, C1, bf16_codes, make_rank, rows_needed, scaled


def _world(case, tokens):
    return [make_rank(case, r, t) for r, t in enumerate(tokens)]


@pytest.mark.parametrize("case,tokens", [
    (C0, [64, 64, 64, 64]),
    (replace(C0, name="ragged_two_nodes", node_size=2, expert_padding=4), [64, 0, 17, 1]),
    (replace(scaled(C1, 96), name="zipf_one_source", routing="zipf", zipf_s=1.2, expert_padding=16),
     [96, 0, 0, 0, 0, 0, 0, 0]),
    (replace(C0, name="odd_experts", num_experts=30, topk=3), [5, 64, 0, 33]),
], ids=lambda v: v.name if hasattr(v, "name") else None)
def test_torch_restatement_equals_the_numpy_oracle(case, tokens):
    world = _world(case, tokens)
    N = case.world_size
    rows = rows_needed(case, world)
    inputs = [oracle.RankInput(x=bf16_codes(rd.x), indices=rd.indices.numpy()) for rd in world]
    want = oracle.dispatch_world(inputs, num_experts=case.num_experts, world_size=N,
                                 node_size=case.node_size or N, expert_padding=case.expert_padding,
                                 out_rows=rows, quantize=True)
    n, ox, os_, slots = torch_oracle.dispatch_world(
        [rd.x for rd in world], [rd.indices for rd in world], num_experts=case.num_experts, world_size=N,
        node_size=case.node_size or N, expert_padding=case.expert_padding, out_rows=rows)
    for r in range(N):
        np.testing.assert_array_equal(n[r].numpy(), want[r].num_tokens)
        w = want[r].written
        np.testing.assert_array_equal(ox[r].numpy()[w], want[r].x[w])
        np.testing.assert_array_equal(os_[r].numpy()[w].view(np.uint32), want[r].x_scale[w].view(np.uint32))
        assert not ox[r].numpy()[~w].any()
        np.testing.assert_array_equal(slots[r].numpy(), want[0].slots[r])

    gen = torch.Generator().manual_seed(5)
    ys = [torch.randn((rows, case.hidden_dim), generator=gen).to(torch.bfloat16) for _ in range(N)]
    want_out = oracle.combine_world([bf16_codes(y) for y in ys], [rd.indices.numpy() for rd in world],
                                    [rd.weights.numpy() for rd in world], want[0].slots,
                                    num_experts=case.num_experts, world_size=N)
    got_out = torch_oracle.combine_world(ys, [rd.indices for rd in world], [rd.weights for rd in world], slots,
                                         num_experts=case.num_experts, world_size=N)
    for r in range(N):
        g = got_out[r].to(torch.float32).numpy()
        w = oracle.bf16_to_f32(want_out[r])
        assert g.shape == w.shape
        if g.size:
            np.testing.assert_allclose(g, w, rtol=1e-2, atol=1e-2 * float(np.abs(w).max()) * 1e-2)


def test_route_matches_bincount_and_a_stable_sort():
    gen = torch.Generator().manual_seed(11)
    idx = torch.randint(0, 37, (200, 5), generator=gen)
    count, toff, incl = torch_oracle.route(idx, 37)
    np.testing.assert_array_equal(count.numpy(), np.bincount(idx.numpy().reshape(-1), minlength=37))
    np.testing.assert_array_equal(incl.numpy(), np.cumsum(count.numpy()))
    flat = idx.numpy().reshape(-1)
    seen = np.zeros(37, dtype=np.int64)
    for i, e in enumerate(flat):                      # brute force: rank among equal experts, in order
        assert toff.reshape(-1)[i] == seen[e]
        seen[e] += 1
