"""Parity of the four split calls (all sends, then all recvs) and of the routing tables they
leave behind, against the oracle's restatement of the reference's host worker."""

from dataclasses import replace

import numpy as np
import pytest
import torch

import a2a_oracle as oracle
from a2a_cases import C0, C1, C2, C4, Case, make_world, scaled
from a2a_harness import (assert_combine_close, assert_dispatch_equal, make_ops, rows_needed, run_gpu,
                         run_oracle, SENTINEL)
from pplx_garden_amd.native import p2p_all_to_all as native

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def device():
    return torch.device("cuda:0")


@pytest.mark.parametrize("case,sources", [
    (C0, "all"), (C0, "ragged"), (C1, "all"), (C2, "one"), (scaled(C4, 128), "ragged"),
    (replace(C0, name="c0_two_nodes", node_size=2), "all"),
    # sends of 448 to 1024 tokens count their routing inside the staging launch, a workgroup for several tokens
    (scaled(C4, 700), "one"), (scaled(C0, 900), "ragged"), (scaled(C1, 1024), "all"),
], ids=lambda v: v.name if hasattr(v, "name") else v)
def test_split_parity(case, sources, device):
    print(f"case={case.name} sources={sources}", flush=True)
    world = make_world(case, sources)
    rows = rows_needed(case, world)
    want = run_oracle(case, world, rows)
    got = run_gpu(case, world, rows, device, split=True)
    assert_dispatch_equal(case, got, want)
    assert_combine_close(case, got, want)


QUICK_SENDS = [
    # (tokens, hidden, experts, ranks, top-k, padding, sources, experts may repeat inside a token)
    (1, 2048, 128, 8, 8, 1, "one", False),
    (3, 2048, 128, 8, 8, 16, "all", True),
    (128, 7168, 250, 8, 5, 8, "ragged", False),       # experts that do not fill 64-lane passes, nor divide among the ranks
    (200, 2048, 1024, 8, 2, 1, "all", True),          # sixteen passes of the resolver's scan
    (100, 2048, 128, 8, 12, 1, "ragged", True),       # more than eight routes a token
    (64, 1024, 8, 8, 1, 1, "all", False),
    (96, 15360, 64, 4, 4, 1, "ragged", False),        # 960 pieces a row: sixteen wavefronts, the resolver is the last
    (40, 16384, 64, 4, 4, 1, "ragged", False),        # a piece too many for a spare wavefront: the kernel without one
    (300, 512, 96, 2, 6, 4, "all", True),             # entries beyond what the threads ask for at the head
    # steps of 448 to 1024 tokens: a workgroup per two to four tokens, teams of wavefronts and a spare one
    (700, 7168, 384, 16, 8, 128, "one", False),       # three tokens a workgroup, two teams, two rounds
    (1024, 2048, 128, 8, 8, 1, "all", True),          # four teams, one round
    (600, 7168, 250, 8, 5, 8, "ragged", True),
    (512, 15360, 64, 4, 4, 1, "ragged", False),       # one team of fifteen wavefronts, two rounds
    (600, 512, 96, 2, 12, 4, "all", True),            # 48 routes a workgroup
    (1000, 256, 40, 1, 3, 1, "all", False),           # one rank
]


@pytest.mark.parametrize("tokens,hidden,experts,ranks,topk,pad,sources,repeats", QUICK_SENDS,
                         ids=[f"{t}x{h}_e{e}_n{n}_k{k}_pad{p}_{s}{'_repeats' if rep else ''}"
                              for t, h, e, n, k, p, s, rep in QUICK_SENDS])
def test_quick_send_of_small_steps(tokens, hidden, experts, ranks, topk, pad, sources, repeats, device):
    """The send of a small step with dense index rows takes a kernel in which a spare wavefront per token
    scans the counts and writes the token's positions while the others quantise and stage the row (a
    step of 448 to 1024 tokens: a spare wavefront per workgroup of two to four tokens).  One
    token, experts that do not fill the scan's passes, many passes, more routes than a wavefront's
    eighth, rows of sixteen wavefronts, entries beyond the first batch, tokens that name an expert
    twice: rows, scales and the routing tables are the oracle's, bit for bit."""
    case = Case(f"quick_send_{tokens}x{hidden}", tokens, hidden, experts, ranks, topk, 4242 + tokens,
                expert_padding=pad)
    world = make_world(case, sources)
    if repeats:
        gen = torch.Generator().manual_seed(tokens)
        for rd in world:
            if rd.indices.shape[0] > 0:
                rd.indices[::3, topk - 1] = rd.indices[::3, 0]      # every third token names its first expert twice
                rd.indices.copy_(rd.indices[torch.randperm(rd.indices.shape[0], generator=gen)])
    rows = rows_needed(case, world)
    want = run_oracle(case, world, rows)
    _, ops = make_ops(case, device)
    try:
        got = run_gpu(case, world, rows, device, split=True, ops=ops)
        assert_dispatch_equal(case, got, want)
        assert_combine_close(case, got, want)
        ctx = ops[0].context
        for g, rd in enumerate(world):
            T = rd.indices.shape[0]
            if T == 0:
                continue
            count, toff, eoff = oracle.route(rd.indices.numpy(), experts)
            np.testing.assert_array_equal(ctx.read_table(g, native.TABLE_NUM_ROUTED, experts).numpy(), count)
            np.testing.assert_array_equal(ctx.read_table(g, native.TABLE_EXPERT_OFFSETS, experts).numpy(), eoff)
            np.testing.assert_array_equal(ctx.read_table(g, native.TABLE_TOKEN_OFFSET, T * topk).numpy(), toff)
    finally:
        for op in ops:
            op.destroy()


@pytest.mark.parametrize("max_private", [0, 3, 8, None], ids=lambda v: f"private_{v}")
@pytest.mark.parametrize("node_size", [4, 2, 1])
def test_routing_tables_match_the_host_worker(node_size, max_private, device):
    """num_routed, expert_offsets, token_offset per sender; padded_index, source_rank, source
    position, the two offset tables with their private / same-node (bit 31) / overflow encoding
    and the received-row counts per receiver (a2a_worker.rs:526-703)."""
    case = replace(C0, name=f"c0_node{node_size}", node_size=node_size, expert_padding=4)
    world = make_world(case, "ragged")
    rows = rows_needed(case, world)
    N, E, K, Le = case.world_size, case.num_experts, case.topk, case.experts_per_rank
    _, ops = make_ops(case, device, max_private_tokens=max_private)
    try:
        ctx = ops[0].context
        private = ops[0].max_private_tokens
        assert private == (max_private if max_private is not None else 72)   # int(ceil(64*4/32) * 1.2) * 8
        dev = [dict(x=rd.x.to(device), idx=rd.indices_u32.to(device), w=rd.weights.to(device)) for rd in world]
        outs = [dict(n=torch.zeros(Le, dtype=torch.int32, device=device),
                     x=torch.zeros((rows, case.hidden_dim), dtype=torch.uint8, device=device).view(torch.float8_e4m3fn),
                     s=torch.zeros((rows, case.hidden_dim_scale), dtype=torch.float32, device=device))
                for _ in range(N)]
        for phase in (dict(do_send=True, do_recv=False), dict(do_send=False, do_recv=True)):
            for r in range(N):
                ops[r].dispatch(out_expert_num_tokens=outs[r]["n"], out_expert_x=outs[r]["x"],
                                out_expert_x_scale=outs[r]["s"], dp_x=dev[r]["x"], dp_x_scale=None,
                                indices=dev[r]["idx"], weights=dev[r]["w"], **phase)
        torch.cuda.synchronize(device)
        assert ctx.status() == 0
        num_routed = np.zeros((N, E), dtype=np.uint32)
        for g, rd in enumerate(world):
            count, toff, eoff = oracle.route(rd.indices.numpy(), E)
            num_routed[g] = count
            T = rd.indices.shape[0]
            np.testing.assert_array_equal(ctx.read_table(g, native.TABLE_NUM_ROUTED, E).numpy(), count)
            np.testing.assert_array_equal(ctx.read_table(g, native.TABLE_EXPERT_OFFSETS, E).numpy(), eoff)
            np.testing.assert_array_equal(ctx.read_table(g, native.TABLE_TOKEN_OFFSET, T * K).numpy(), toff)
        for r in range(N):
            lay = oracle.process_routing_info(num_routed, r, N, node_size, 1, case.expert_padding, private)
            nrecv = ctx.read_table(r, native.TABLE_NUM_RECV_TOKENS, 2).numpy()
            assert nrecv.tolist() == [lay.num_recv_tokens, lay.num_efa_tokens]
            n = lay.num_recv_tokens
            np.testing.assert_array_equal(ctx.read_table(r, native.TABLE_PADDED_INDEX, n).numpy(), lay.padded_index)
            np.testing.assert_array_equal(ctx.read_table(r, native.TABLE_SOURCE_RANK, n).numpy(), lay.source_rank)
            np.testing.assert_array_equal(ctx.read_table(r, native.TABLE_SOURCE_POSITION, n).numpy(), lay.source_position)
            np.testing.assert_array_equal(ctx.read_table(r, native.TABLE_SOURCE_DISPATCH_OFFSET, n).numpy(),
                                          lay.source_dispatch_offset)
            np.testing.assert_array_equal(ctx.read_table(r, native.TABLE_COMBINE_SEND_OFFSET, n).numpy(),
                                          lay.combine_send_offset)
            np.testing.assert_array_equal(outs[r]["n"].cpu().numpy(), lay.tokens_per_expert)
    finally:
        for op in ops:
            op.destroy()


def test_group_call_tables_and_slots(device):
    """The group call leaves the same sender tables and the receiver row of every copy."""
    case = C1
    world = make_world(case, "all")
    rows = rows_needed(case, world)
    N, E, K, Le = case.world_size, case.num_experts, case.topk, case.experts_per_rank
    _, ops = make_ops(case, device)
    try:
        ctx = ops[0].context
        keep = []
        for r, rd in enumerate(world):
            t = dict(x=rd.x.to(device), idx=rd.indices_u32.to(device), w=rd.weights.to(device),
                     n=torch.zeros(Le, dtype=torch.int32, device=device),
                     ox=torch.zeros((rows, case.hidden_dim), dtype=torch.uint8, device=device).view(torch.float8_e4m3fn),
                     os=torch.zeros((rows, case.hidden_dim_scale), dtype=torch.float32, device=device))
            keep.append(t)
            ops[r].dispatch(out_expert_num_tokens=t["n"], out_expert_x=t["ox"], out_expert_x_scale=t["os"],
                            dp_x=t["x"], dp_x_scale=None, indices=t["idx"], weights=t["w"])
        torch.cuda.synchronize(device)
        assert ctx.status() == 0
        _, toffs, eoffs, slots = oracle.world_routing([rd.indices.numpy() for rd in world], E, N, N, 1)
        for g, rd in enumerate(world):
            T = rd.indices.shape[0]
            np.testing.assert_array_equal(ctx.read_table(g, native.TABLE_TOKEN_OFFSET, T * K).numpy(), toffs[g])
            np.testing.assert_array_equal(ctx.read_table(g, native.TABLE_EXPERT_OFFSETS, E).numpy(), eoffs[g])
            np.testing.assert_array_equal(ctx.read_table(g, native.TABLE_SLOT, T * K).numpy(), slots[g].reshape(-1))
    finally:
        for op in ops:
            op.destroy()


def test_a_second_step_reuses_the_context(device):
    """Two steps in a row on the same operators, the second with fewer tokens and other routing:
    nothing of the first step may leak into the second."""
    case = C0
    first = make_world(case, "all")
    second = make_world(replace(case, seed=case.seed + 1), "ragged")
    rows = max(rows_needed(case, first), rows_needed(case, second))
    N, Le = case.world_size, case.experts_per_rank
    for split in (False, True):
        _, ops = make_ops(case, device)
        try:
            for world in (first, second):
                want = run_oracle(case, world, rows)
                outs = []
                for r, rd in enumerate(world):
                    outs.append(dict(
                        x=rd.x.to(device), idx=rd.indices_u32.to(device), w=rd.weights.to(device),
                        n=torch.full((Le,), -1, dtype=torch.int32, device=device),
                        ox=torch.full((rows, case.hidden_dim), SENTINEL, dtype=torch.uint8, device=device).view(torch.float8_e4m3fn),
                        os=torch.full((rows, case.hidden_dim_scale), -7.0, dtype=torch.float32, device=device)))
                phases = [dict(do_send=True, do_recv=False), dict(do_send=False, do_recv=True)] if split else [dict()]
                for phase in phases:
                    for r in range(N):
                        o = outs[r]
                        ops[r].dispatch(out_expert_num_tokens=o["n"], out_expert_x=o["ox"], out_expert_x_scale=o["os"],
                                        dp_x=o["x"], dp_x_scale=None, indices=o["idx"], weights=o["w"], **phase)
                torch.cuda.synchronize(device)
                assert ops[0].context.status() == 0
                for r in range(N):
                    np.testing.assert_array_equal(outs[r]["n"].cpu().numpy(), want.num_tokens[r])
                    w = want.written[r]
                    np.testing.assert_array_equal(outs[r]["ox"].view(torch.uint8).cpu().numpy()[w], want.x[r][w])
                    assert (outs[r]["ox"].view(torch.uint8).cpu().numpy()[~w] == SENTINEL).all()
        finally:
            for op in ops:
                op.destroy()
