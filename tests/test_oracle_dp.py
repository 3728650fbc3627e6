"""Pins the oracle's dp-group branch (ranks of a group hold the same tokens) and the row-by-row
formulation of the dispatch (`world_by_rows`) that the GPU tests of dp groups are checked against.

`process_routing_info(dp_size > 1)` is compared with an enumeration written from the rules, not from its
loops: which group a rank receives from and through which member (a2a_worker.rs:633), in what order the
groups are laid out (a2a_worker.rs:681-694), where an expert's rows start (a2a_worker.rs:598-606) and
where a copy sits in the sender's expert-sorted order (a2a_dispatch_send.cu:54).  `world_by_rows` with
dp_size = 1 must reproduce `dispatch_world`, which is pinned by closed forms elsewhere."""

import numpy as np
import pytest

import a2a_oracle as oracle
from a2a_cases import C0, C1, C4, bf16_codes, make_world, scaled
from a2a_harness import rows_needed


def _enumerate_receiver(num_routed, r, N, node, D, pad):
    """Rows receiver r gets, in arrival order, from the rules: (group, expert, j-th copy of that pair)."""
    G, E = num_routed.shape
    Le = -(-E // N)
    fe, le_end = r * Le, min((r + 1) * Le, E)
    groups_per_node, nodes = node // D, N // node
    my_node, my_group = r // node, r // D
    order = []
    for step in range(1, nodes):                      # other nodes, starting at the next one
        n = (my_node + step) % nodes
        order += [n * groups_per_node + j for j in range(groups_per_node)]
    for step in range(1, groups_per_node):            # the other groups of my node, after mine, wrapping
        order.append(my_node * groups_per_node + (my_group % groups_per_node + step) % groups_per_node)
    order.append(my_group)
    rows = []
    for g in order:
        for e in range(fe, le_end):
            rows += [(g, e, j) for j in range(int(num_routed[g, e]))]
    remote = sum(int(num_routed[g, fe:le_end].sum()) for g in order[: (nodes - 1) * groups_per_node])
    return order, rows, remote


@pytest.mark.parametrize("N,E,node,D,pad", [(4, 8, 4, 2, 1), (4, 4, 4, 2, 1), (8, 16, 4, 2, 4), (8, 24, 8, 4, 1),
                                            (8, 16, 4, 4, 3), (4, 6, 2, 2, 2), (8, 8, 2, 1, 1)])
def test_process_routing_info_with_dp_groups_against_an_enumeration(N, E, node, D, pad):
    rng = np.random.default_rng(N * 100 + E * 10 + D + pad)
    G = N // D
    Le = -(-E // N)
    num_routed = rng.integers(0, 5, (G, E)).astype(np.uint32)
    if G > 1:
        num_routed[rng.integers(0, G)] = 0              # a group that sends nothing
    excl = np.c_[np.zeros(G, np.int64), np.cumsum(num_routed.astype(np.int64), axis=1)[:, :-1]]
    seen_copies = set()
    for r in range(N):
        lay = oracle.process_routing_info(num_routed, r, N, node, D, pad, 0)
        order, rows, remote = _enumerate_receiver(num_routed, r, N, node, D, pad)
        assert order == oracle.source_order(r, N, node, D)
        assert sorted(order) == list(range(G))
        fe, le_end = r * Le, min((r + 1) * Le, E)
        tpe = num_routed[:, fe:le_end].astype(np.int64).sum(axis=0)
        np.testing.assert_array_equal(lay.tokens_per_expert[: le_end - fe], tpe)
        assert lay.num_recv_tokens == len(rows) == int(tpe.sum())
        assert lay.num_efa_tokens == remote
        padded = (tpe + pad - 1) // pad * pad
        start = np.cumsum(padded) - padded          # empty for a rank that owns no expert
        np.testing.assert_array_equal(lay.padded_offset, start)
        filled = np.zeros(le_end - fe, dtype=np.int64)
        for i, (g, e, j) in enumerate(rows):
            # the member of the group with my dp rank is the one that sends to me (a2a_worker.rs:633)
            assert lay.source_rank[i] == g * D + r % D
            assert lay.source_rank[i] // D == g
            # j-th copy of (g, e) in the sender's order sorted by expert (a2a_dispatch_send.cu:54)
            assert lay.source_position[i] == excl[g, e] + j
            # rows of an expert fill its range in arrival order
            assert lay.padded_index[i] == start[e - fe] + filled[e - fe]
            filled[e - fe] += 1
            assert (g, e, j) not in seen_copies
            seen_copies.add((g, e, j))
        np.testing.assert_array_equal(filled, tpe)
        # every destination row once, inside its expert's range
        assert len(set(lay.padded_index.tolist())) == lay.num_recv_tokens
    # every copy of every group is received by exactly one rank: the owner of its expert
    assert len(seen_copies) == int(num_routed.sum())


def test_dp_peers_receive_through_their_own_member_and_share_the_groups_rows():
    """Two receivers with the same dp rank read from the same member of a source group; the rows a
    group sends to an expert do not depend on which member sends them."""
    N, E, node, D = 8, 16, 8, 2
    rng = np.random.default_rng(77)
    num_routed = rng.integers(0, 4, (N // D, E)).astype(np.uint32)
    lays = [oracle.process_routing_info(num_routed, r, N, node, D, 1, 0) for r in range(N)]
    for r in range(N):
        assert set((lays[r].source_rank % D).tolist()) <= {r % D}
    # receivers r and r^1 are dp peers: each gets its OWN experts' rows, and together the group's
    # counts for those experts
    Le = E // N
    for r in range(0, N, 2):
        both = lays[r].num_recv_tokens + lays[r + 1].num_recv_tokens
        assert both == int(num_routed[:, r * Le:(r + 2) * Le].sum())


@pytest.mark.parametrize("case,sources", [(C0, "all"), (C1, "all"), (C0, "ragged"),
                                          (scaled(C4, 96), "ragged")],
                         ids=lambda v: v.name if hasattr(v, "name") else v)
def test_world_by_rows_without_dp_groups_is_dispatch_world(case, sources):
    world = make_world(case, sources)
    rows = rows_needed(case, world)
    N = case.world_size
    node = case.node_size or N
    inputs = [oracle.RankInput(x=bf16_codes(rd.x), indices=rd.indices.numpy()) for rd in world]
    want = oracle.dispatch_world(inputs, num_experts=case.num_experts, world_size=N, node_size=node,
                                 expert_padding=case.expert_padding, out_rows=rows, quantize=True)
    payloads, scales = [], []
    for rd in world:
        if rd.x.shape[0]:
            q, s = oracle.quantize_block128(bf16_codes(rd.x))
        else:
            q = np.zeros((0, case.hidden_dim), np.uint8)
            s = np.zeros((0, case.hidden_dim_scale), np.float32)
        payloads.append(q)
        scales.append(s)
    got, (slot_rank, slot_row) = oracle.world_by_rows(
        [rd.indices.numpy() for rd in world], payloads, scales, num_experts=case.num_experts, world_size=N,
        node_size=node, dp_size=1, expert_padding=case.expert_padding, out_rows=rows)
    Le = case.experts_per_rank
    for r in range(N):
        np.testing.assert_array_equal(got[r].num_tokens, want[r].num_tokens)
        np.testing.assert_array_equal(got[r].written, want[r].written)
        np.testing.assert_array_equal(got[r].x, want[r].x)
        np.testing.assert_array_equal(got[r].x_scale.view(np.uint32), want[r].x_scale.view(np.uint32))
    for g, rd in enumerate(world):
        idx = rd.indices.numpy().astype(np.int64)
        np.testing.assert_array_equal(slot_rank[g], idx // Le)
        np.testing.assert_array_equal(slot_row[g], want[0].slots[g])
