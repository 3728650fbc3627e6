"""Pins the routing pass and the receiver layout of the oracle: library routines
(bincount, cumsum), brute-force loops on small inputs, the invariants the
reference's own test checks, and numpy against the C restatement."""

import numpy as np
import pytest

import a2a_oracle as oracle
import c_oracle
from a2a_cases import C0, C1, C4, make_indices, scaled


def _brute_token_offset(idx, E):
    seen = [0] * E
    out = []
    for e in idx.reshape(-1).tolist():
        out.append(seen[e])
        seen[e] += 1
    return np.array(out, dtype=np.uint32)


@pytest.mark.parametrize("case", [C0, C1, scaled(C4, 96)], ids=lambda c: c.name)
def test_route_counts_offsets_and_stable_rank(case):
    idx = make_indices(case, 0).numpy()
    count, toff, eoff = oracle.route(idx, case.num_experts)
    # the reference's own check: bincount (tests/p2p_all_to_all/data.py:50-53)
    np.testing.assert_array_equal(count, np.bincount(idx.reshape(-1), minlength=case.num_experts))
    np.testing.assert_array_equal(eoff, np.cumsum(count))          # inclusive, a2a_dispatch_send.cu:236-242
    np.testing.assert_array_equal(toff, _brute_token_offset(idx, case.num_experts))
    c2, t2, e2 = c_oracle.route(idx, case.num_experts)
    np.testing.assert_array_equal(c2, count)
    np.testing.assert_array_equal(t2, toff)
    np.testing.assert_array_equal(e2, eoff)


def test_route_handles_repeats_empty_and_rejects_bad_ids():
    idx = np.array([[3, 3, 3], [0, 3, 0]], dtype=np.int32)     # the kernels do not require distinct experts
    count, toff, eoff = oracle.route(idx, 4)
    assert count.tolist() == [2, 0, 0, 4] and toff.tolist() == [0, 1, 2, 0, 3, 1] and eoff.tolist() == [2, 2, 2, 6]
    c, t, e = oracle.route(np.zeros((0, 4), np.int32), 8)
    assert c.sum() == 0 and t.size == 0 and e.tolist() == [0] * 8
    with pytest.raises(ValueError):
        oracle.route(np.array([[8]], np.int32), 8)
    with pytest.raises(ValueError):
        c_oracle.route(np.array([[8]], np.int32), 8)


def test_positions_are_a_sort_by_expert():
    case = C0
    idx = make_indices(case, 1).numpy()
    count, toff, eoff = oracle.route(idx, case.num_experts)
    pos, off = oracle.positions(idx, toff, eoff, case.experts_per_rank)
    flat = idx.reshape(-1)
    # positions enumerate the entries sorted by (expert, token, k): a stable sort
    np.testing.assert_array_equal(np.argsort(flat, kind="stable"), np.argsort(pos.reshape(-1)))
    assert sorted(pos.reshape(-1).tolist()) == list(range(flat.size))
    # offset is relative to the first expert of the destination rank (a2a_dispatch_send.cu:55-57)
    Le = case.experts_per_rank
    rank_start = np.r_[0, np.cumsum(count)][(flat // Le) * Le]
    np.testing.assert_array_equal(off.reshape(-1), pos.reshape(-1) - rank_start)


@pytest.mark.parametrize("world,node,rank,expected", [
    (4, 4, 0, [1, 2, 3, 0]), (4, 4, 2, [3, 0, 1, 2]), (8, 8, 7, [0, 1, 2, 3, 4, 5, 6, 7]),
    # two nodes of two: the other node first, then the node neighbour, then self (a2a_worker.rs:681-694)
    (4, 2, 0, [2, 3, 1, 0]), (4, 2, 3, [0, 1, 2, 3]),
    (8, 4, 5, [0, 1, 2, 3, 6, 7, 4, 5]), (6, 2, 2, [4, 5, 0, 1, 3, 2]), (1, 1, 0, [0]),
])
def test_source_order_known_answers(world, node, rank, expected):
    assert oracle.source_order(rank, world, node) == expected
    assert sorted(expected) == list(range(world))


@pytest.mark.parametrize("world,node,dp,rank,expected", [
    # Worked by hand through the three loops of a2a_worker.rs:681-694 (groups, not ranks, are visited).
    # 2 nodes of 4 ranks, groups of 2: rank 5 is on node 1 in group 2; node 0's groups 0, 1 first,
    # then the other group of its node (3), then its own.
    (8, 4, 2, 5, [0, 1, 3, 2]),
    (8, 4, 2, 2, [2, 3, 0, 1]),
    # one node, four groups of two: rank 2 is in group 1; the groups after it, wrapping, then its own
    (8, 8, 2, 2, [2, 3, 0, 1]),
    # a group is a whole node: only the other node's group, then the own
    (8, 4, 4, 6, [0, 1]),
    # three nodes: nodes 1 and 2 in turn, then the node neighbour, then the own group
    (12, 4, 2, 1, [2, 3, 4, 5, 1, 0]),
    (12, 4, 2, 10, [0, 1, 2, 3, 4, 5]),
])
def test_source_order_known_answers_with_dp_groups(world, node, dp, rank, expected):
    assert oracle.source_order(rank, world, node, dp) == expected
    assert sorted(expected) == list(range(world // dp))


@pytest.mark.parametrize("N,E,node,pad,maxpriv", [(4, 32, 4, 1, 3), (4, 32, 2, 4, 0), (8, 64, 4, 16, 5),
                                                  (2, 16, 2, 1, 8), (3, 10, 3, 2, 1)])
def test_receiver_layout_invariants_and_closed_form(N, E, node, pad, maxpriv):
    rng = np.random.default_rng(N * 1000 + E + pad)
    num_routed = rng.integers(0, 7, (N, E)).astype(np.uint32)
    num_routed[rng.integers(0, N), :] = 0                      # a source with nothing to send
    Le = -(-E // N)
    base = oracle.slot_base(num_routed, N, node, pad).astype(np.int64)
    tpe_c, poff_c, base_c = c_oracle.layout(num_routed, node, pad)
    np.testing.assert_array_equal(base_c, base)
    for r in range(N):
        lay = oracle.process_routing_info(num_routed, r, N, node, 1, pad, maxpriv)
        fe, le_end = r * Le, min((r + 1) * Le, E)
        n_local = max(le_end - fe, 0)
        tpe = num_routed[:, fe:le_end].sum(axis=0)
        # counts: what the reference's test checks first (test_p2p_all_to_all.py:192-194)
        np.testing.assert_array_equal(lay.tokens_per_expert[:n_local], tpe)
        np.testing.assert_array_equal(tpe_c[fe:le_end], tpe)
        assert lay.num_recv_tokens == tpe.sum() == len(lay.padded_index)
        # slot ranges: expert le occupies [padded_offset, padded_offset + tpe), ranges advance by
        # round_up(., pad) (test_p2p_all_to_all.py:200-206), no slot is used twice
        start = 0
        slots = sorted(lay.padded_index.tolist())
        expect = []
        for le in range(n_local):
            assert lay.padded_offset[le] == start == poff_c[fe + le]
            expect += list(range(start, start + int(tpe[le])))
            start = oracle.round_up(start + int(tpe[le]), pad)
        assert slots == expect
        # closed form: the run of source g in expert e starts at base[g, e]
        got = []
        for g in oracle.source_order(r, N, node):
            for e in range(fe, le_end):
                got += [base[g, e] + j for j in range(num_routed[g, e])]
        np.testing.assert_array_equal(lay.padded_index, np.array(got, dtype=np.uint32))
        # source rank and position of every received row
        ranks, poss = [], []
        excl = np.c_[np.zeros(N, np.int64), np.cumsum(num_routed, axis=1)[:, :-1]]
        for g in oracle.source_order(r, N, node):
            for e in range(fe, le_end):
                ranks += [g] * int(num_routed[g, e])
                poss += [excl[g, e] + j for j in range(num_routed[g, e])]
        np.testing.assert_array_equal(lay.source_rank, np.array(ranks, dtype=np.uint32))
        np.testing.assert_array_equal(lay.source_position, np.array(poss, dtype=np.uint32))
        # rows from other nodes come first (num_efa_tokens, a2a_worker.rs:681-687)
        other = [g for g in range(N) if g // node != r // node]
        assert lay.num_efa_tokens == num_routed[other][:, fe:le_end].sum()


def test_source_dispatch_offset_variants_name_the_same_row():
    """With no private region and one node, the reference's offsets are the sender's position
    (bit 31 marks 'read from the peer's send buffer', a2a_worker.rs:649-651)."""
    rng = np.random.default_rng(5)
    N, E = 4, 16
    num_routed = rng.integers(0, 5, (N, E)).astype(np.uint32)
    for r in range(N):
        lay = oracle.process_routing_info(num_routed, r, N, N, 1, 1, 0)
        own = lay.source_rank == r
        np.testing.assert_array_equal(lay.source_dispatch_offset[own], lay.source_position[own])
        np.testing.assert_array_equal(lay.source_dispatch_offset[~own] & 0x7FFFFFFF, lay.source_position[~own])
        assert ((lay.source_dispatch_offset[~own] >> 31) == 1).all()
        # combine sends every row back to the sender's own position (a2a_worker.rs:659-667)
        np.testing.assert_array_equal(lay.combine_send_offset, lay.source_position)
    # with a private region the first max_private rows of a peer are addressed inside it
    lay = oracle.process_routing_info(num_routed, 0, N, N, 1, 1, 3)
    for g in range(1, N):
        rows = np.flatnonzero(lay.source_rank == g)
        k = min(3, len(rows))
        np.testing.assert_array_equal(lay.source_dispatch_offset[rows[:k]], 3 * g + np.arange(k))


@pytest.mark.parametrize("N,node,D,private", [(4, 2, 1, 2), (8, 4, 1, 0), (8, 2, 2, 3), (6, 2, 1, 100), (8, 4, 2, 1)])
def test_dispatch_offsets_name_distinct_rows_of_the_three_regions(N, node, D, private):
    """`source_dispatch_offset` addresses a receive region of G private parts of `private` rows each,
    followed by the overflow part (a2a_worker.rs:636-656).  Whatever the counts: a row of another
    rank is in its source's private part while that lasts, then in the sender's own buffer (bit 31,
    same node) or in the overflow part (other nodes); no two rows share an address of one buffer; the overflow part
    is filled source by source in rank order, each source's rows in arrival order."""
    rng = np.random.default_rng(N * 7 + node + private)
    G, E = N // D, 2 * N
    Le = E // N
    num_routed = rng.integers(0, 6, (G, E)).astype(np.uint32)
    for r in range(N):
        lay = oracle.process_routing_info(num_routed, r, N, node, D, 1, private)
        fe = r * Le
        per_group = num_routed[:, fe:fe + Le].astype(np.int64).sum(axis=1)
        below = np.r_[0, np.cumsum(per_group)[:-1]]
        seen_of_group = np.zeros(G, dtype=np.int64)
        addresses = set()
        for i in range(lay.num_recv_tokens):
            peer = int(lay.source_rank[i])
            g = peer // D
            assert peer % D == r % D
            sdo = int(lay.source_dispatch_offset[i])
            if peer == r:
                assert sdo == lay.source_position[i] == lay.combine_send_offset[i] or D > 1
                assert sdo == lay.source_position[i]
                continue
            j = int(seen_of_group[g])
            seen_of_group[g] += 1
            if j < private:
                assert sdo == private * g + j and sdo < private * G
            elif peer // node == r // node:
                assert sdo == (int(lay.source_position[i]) | 1 << 31)
            else:
                assert sdo == private * G + (below[g] + j - private)
                assert sdo >= private * G
            where = (peer, sdo) if sdo >> 31 else sdo      # bit 31: a row of THAT peer's send buffer
            assert where not in addresses
            addresses.add(where)
            # the way back: the sender's own position on the same node, else the row's place among
            # all rows this rank got, source by source in rank order (a2a_worker.rs:659-667)
            want_cso = int(lay.source_position[i]) if peer // node == r // node else below[g] + j
            assert lay.combine_send_offset[i] == want_cso


def test_strides_and_capacities_known_answers():
    # a2a_dispatch_send.cu:586-588: fp8 H=7168 with 56 scales -> 7168 + 224 + 16
    assert oracle.dispatch_token_stride(7168, 1, 56, 4) == 7408
    assert oracle.dispatch_token_stride(2048, 1, 16, 4) == 2128
    assert oracle.dispatch_token_stride(128, 4, 0, 0) == 528
    assert oracle.dispatch_token_stride(4, 4, 0, 0) == 32
    assert oracle.combine_token_stride(7168, 2) == 14336
    assert oracle.combine_token_stride(4, 4) == 16
    # p2p_all_to_all.py:92-114 for the DeepSeek decode shape: Le=32, avg=int(4*1.2)=4
    assert oracle.buffer_capacity(128, 256, 8, 8, 1, 1) == (32, 128, 128 * 8 + 8192)
    # the 1-token case of the reference's tests (E=2, N=2, K=1, max_private 32)
    assert oracle.buffer_capacity(1, 2, 1, 2, 1, 1, 32) == (1, 32, 32 * 2 + 2)
    # avg = int(ceil(16/16) * 1.2) = 1, private = 8, recv = 8*2 + round_up(max(min(32+120, 128), 128), 16)
    assert oracle.buffer_capacity(8, 16, 2, 2, 1, 16) == (8, 8, 144)
