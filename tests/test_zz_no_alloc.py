"""`a2a_dispatch_static` (the group dispatch without a context and without any allocation: its routing
tables live in a fixed array inside the library) against `a2a_dispatch` on a context, through the C ABI.

Bar: bit-exact, every byte of every output buffer including the untouched padding rows, and bit-exact
against the oracle.  Several calls in a row on the same array, larger and smaller in turn, taking the
two-launch path (whose step totals must start from zero) and the one-launch path of small steps."""

import ctypes

import numpy as np
import pytest
import torch

from a2a_cases import Case, bf16_codes, make_rank
from a2a_harness import SENTINEL, WorldResult, assert_dispatch_equal, rows_needed
import a2a_oracle as oracle
from pplx_garden_amd.native import p2p_all_to_all as native

pytestmark = pytest.mark.gpu

DEV = torch.device("cuda:0")


def _config(case: Case, max_tokens: int) -> native.A2AConfig:
    return native.A2AConfig(
        struct_size=ctypes.sizeof(native.A2AConfig), hidden_dim=case.hidden_dim,
        hidden_dim_scale=case.hidden_dim_scale, in_elemsize=1, out_elemsize=2,
        out_dtype=native.SCALAR_TYPE[torch.bfloat16], scale_elemsize=4, max_num_tokens=max_tokens,
        max_recv_tokens=max_tokens * case.topk * case.world_size, max_private_tokens=0,
        num_experts=case.num_experts, expert_padding=case.expert_padding,
        num_experts_per_token=case.topk, dp_size=1, node_size=case.node_size or case.world_size,
        world_size=case.world_size, device=0, flags=0)


class _Buffers:
    """Inputs on the device and sentinel-filled outputs of one step."""

    def __init__(self, case: Case, world, rows: int):
        N, H, Hs, Le, K = case.world_size, case.hidden_dim, case.hidden_dim_scale, case.experts_per_rank, case.topk
        self.keep = [dict(x=rd.x.to(DEV), idx=rd.indices.to(DEV)) for rd in world]
        self.n = [torch.full((Le,), -1, dtype=torch.int32, device=DEV) for _ in range(N)]
        self.x = [torch.full((rows, H), SENTINEL, dtype=torch.uint8, device=DEV) for _ in range(N)]
        self.s = [torch.full((rows, Hs), -7.0, dtype=torch.float32, device=DEV) for _ in range(N)]
        self.args = []
        for r, rd in enumerate(world):
            T = rd.x.shape[0]
            self.args.append(native.A2ADispatchArgs(
                num_tokens=T, x_ptr=self.keep[r]["x"].data_ptr() if T else None, x_stride=2 * H,
                x_scale_ptr=None, x_scale_stride_elem=0, x_scale_stride_token=0,
                indices=self.keep[r]["idx"].data_ptr() if T else None, indices_stride=K,
                weights=None, weights_stride=K, bound_m=None,
                out_num_tokens=self.n[r].data_ptr(), out_x=self.x[r].data_ptr(), out_x_stride=H,
                out_x_rows=rows, out_x_scale=self.s[r].data_ptr(), out_x_scale_stride_elem=1,
                out_x_scale_stride_token=Hs))

    def result(self) -> WorldResult:
        torch.cuda.synchronize(DEV)
        return WorldResult([t.cpu().numpy() for t in self.n], [t.cpu().numpy() for t in self.x],
                           [t.cpu().numpy() for t in self.s], [])


def _oracle(case: Case, world, rows: int) -> WorldResult:
    inputs = [oracle.RankInput(x=bf16_codes(rd.x), indices=rd.indices.numpy()) for rd in world]
    outs = oracle.dispatch_world(inputs, num_experts=case.num_experts, world_size=case.world_size,
                                 node_size=case.node_size or case.world_size,
                                 expert_padding=case.expert_padding, out_rows=rows, quantize=True)
    res = WorldResult([o.num_tokens for o in outs], [o.x for o in outs], [o.x_scale for o in outs], [])
    res.written = [o.written for o in outs]
    return res


def test_static_dispatch_matches_the_context_dispatch():
    case = Case("static_steps", 640, 512, 64, 4, 8, 9100, expert_padding=4)
    # tokens per rank of consecutive calls: large (two launches), smaller (one launch), large again but
    # smaller than the first (the step totals of the first call must not leak), tiny, empty, one larger
    # source alone (one launch whose workgroups take several tokens each), large
    steps = [[640, 600, 0, 512], [100, 0, 7, 64], [300, 310, 290, 5], [1, 0, 0, 0], [0, 0, 0, 0],
             [0, 640, 0, 0], [640, 640, 640, 640]]
    stream = torch.cuda.current_stream(DEV).cuda_stream
    cfg = _config(case, case.num_tokens)
    ctx = native.AllToAllContext.create(
        hidden_dim=case.hidden_dim, hidden_dim_scale=case.hidden_dim_scale, in_elemsize=1, out_elemsize=2,
        out_dtype=torch.bfloat16, scale_elemsize=4, max_num_tokens=case.num_tokens,
        max_recv_tokens=cfg.max_recv_tokens, max_private_tokens=0, num_experts=case.num_experts,
        expert_padding=case.expert_padding, num_experts_per_token=case.topk, dp_size=1,
        node_size=case.world_size, world_size=case.world_size, device=0)
    flags = torch.zeros(1, dtype=torch.int32, device=DEV)
    try:
        for i, tokens in enumerate(steps):
            print(f"step {i}: tokens={tokens}", flush=True)
            world = [make_rank(case, r, t) for r, t in enumerate(tokens)]
            rows = rows_needed(case, world)
            want = _oracle(case, world, rows)

            a = _Buffers(case, world, rows)
            ctx.dispatch(a.args, True, stream)
            via_context = a.result()
            assert ctx.status(stream) == 0

            b = _Buffers(case, world, rows)
            native.dispatch_static(cfg, b.args, True, flags.data_ptr(), stream)
            via_static = b.result()
            assert int(flags.item()) == 0

            for r in range(case.world_size):
                np.testing.assert_array_equal(via_static.num_tokens[r], via_context.num_tokens[r])
                np.testing.assert_array_equal(via_static.x[r], via_context.x[r])
                np.testing.assert_array_equal(via_static.x_scale[r].view(np.uint32),
                                              via_context.x_scale[r].view(np.uint32))
            assert_dispatch_equal(case, via_static, want)
    finally:
        ctx.destroy()


def test_static_dispatch_reports_bad_input_through_the_callers_flag_word():
    case = Case("static_flags", 16, 256, 16, 2, 2, 9200)
    world = [make_rank(case, r, 16) for r in range(2)]
    world[1].indices[3, 1] = 99                       # not an expert
    rows = 64
    cfg = _config(case, 16)
    stream = torch.cuda.current_stream(DEV).cuda_stream
    flags = torch.zeros(1, dtype=torch.int32, device=DEV)
    b = _Buffers(case, world, rows)
    native.dispatch_static(cfg, b.args, True, flags.data_ptr(), stream)
    torch.cuda.synchronize(DEV)
    assert int(flags.item()) == native.DEV_BAD_EXPERT_ID
    # without a flag word the same call drops the copy silently and still completes
    native.dispatch_static(cfg, _Buffers(case, world, rows).args, True, None, stream)
    torch.cuda.synchronize(DEV)


def test_static_dispatch_can_be_captured_in_a_hip_graph():
    """What the entry point is for: a caller under stream capture.  After one eager call (which looks up the
    address of the fixed array on this GPU), a call is captured and replayed three times with eager work and
    another, different static call in between (it overwrites the shared tables): every replay must write
    what the oracle says."""
    case = Case("static_graph", 600, 256, 32, 4, 8, 9300, expert_padding=2)
    stream = torch.cuda.current_stream(DEV).cuda_stream
    cfg = _config(case, case.num_tokens)
    world = [make_rank(case, r, t) for r, t in enumerate([600, 0, 333, 590])]      # two-launch path
    other = [make_rank(case, r, t) for r, t in enumerate([9, 50, 0, 1])]           # one-launch path
    rows = max(rows_needed(case, world), rows_needed(case, other))
    want = _oracle(case, world, rows)
    b = _Buffers(case, world, rows)
    o = _Buffers(case, other, rows)
    native.dispatch_static(cfg, b.args, True, None, stream)                        # eager: also the set-up call
    assert_dispatch_equal(case, b.result(), want)
    args = (native.A2ADispatchArgs * case.world_size)(*b.args)
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream(device=DEV)
    side.wait_stream(torch.cuda.current_stream(DEV))
    with torch.cuda.stream(side):
        native.dispatch_static(cfg, args, True, None, side.cuda_stream)
    torch.cuda.current_stream(DEV).wait_stream(side)
    torch.cuda.synchronize(DEV)
    with torch.cuda.graph(graph):
        native.dispatch_static(cfg, args, True, None, torch.cuda.current_stream(DEV).cuda_stream)
    for i in range(3):
        for t in b.n + b.x + b.s:
            t.fill_(0)
        for t in b.x:
            t.fill_(SENTINEL)
        for t in b.s:
            t.fill_(-7.0)
        native.dispatch_static(cfg, o.args, True, None, stream)                    # leaves other tables behind
        scratch = torch.randn(1 << 20, device=DEV).sum()
        torch.cuda.synchronize(DEV)
        graph.replay()
        assert_dispatch_equal(case, b.result(), want)
        del scratch


def _raw_step(N, H, Hs, K, E, Le, tokens, rows, *, in_elemsize, seed, dp_size=1, scale_transposed=False):
    """Inputs and sentinel-filled outputs of one step without quantisation (rows travel as bytes,
    scales are the caller's): returns (keep-alive list, args, output tensors)."""
    keep, args, outs = [], [], []
    for r in range(N):
        g = r // dp_size                                     # the members of a dp group pass the same tokens
        gg = torch.Generator().manual_seed(seed + 31 * g)
        T = tokens[g]
        x = torch.randn((T, H), generator=gg).to(torch.bfloat16 if in_elemsize == 2 else torch.float32).to(DEV)
        idx = torch.rand((T, E), generator=gg).topk(K, dim=-1).indices.to(torch.int32).to(DEV)
        xs = None
        if Hs:
            xs = torch.randn((Hs, T) if scale_transposed else (T, Hs), generator=gg).to(DEV)
        n = torch.full((Le,), -1, dtype=torch.int32, device=DEV)
        ox = torch.full((rows, H * in_elemsize), SENTINEL, dtype=torch.uint8, device=DEV)
        os_ = torch.full((rows, max(Hs, 1)), -7.0, dtype=torch.float32, device=DEV)
        keep.append((x, idx, xs))
        outs.append((n, ox, os_))
        args.append(native.A2ADispatchArgs(
            num_tokens=T, x_ptr=x.data_ptr() if T else None, x_stride=H * in_elemsize,
            x_scale_ptr=xs.data_ptr() if Hs and T else None,
            x_scale_stride_elem=(T if scale_transposed else 1) if Hs else 0,
            x_scale_stride_token=(1 if scale_transposed else Hs) if Hs else 0,
            indices=idx.data_ptr() if T else None, indices_stride=K, weights=None, weights_stride=K, bound_m=None,
            out_num_tokens=n.data_ptr(), out_x=ox.data_ptr(), out_x_stride=H * in_elemsize, out_x_rows=rows,
            out_x_scale=os_.data_ptr() if Hs else None, out_x_scale_stride_elem=1 if Hs else 0,
            out_x_scale_stride_token=Hs))
    return keep, args, outs


@pytest.mark.parametrize("name,N,node,dp,H,Hs,in_elemsize,steps", [
    # rows that travel as bytes with the caller's scales (the x_scale copy of the kernels), scales transposed
    ("bf16_with_scales", 4, 4, 1, 384, 3, 2, [[300, 0, 41, 299], [5, 6, 0, 1], [0, 1400, 0, 0]]),
    # dp groups of two on two nodes of two: the on-device source order and the masks of the sources laid
    # out earlier are only computed by this entry point's own prepare kernel
    ("dp2_two_nodes", 4, 2, 2, 256, 0, 4, [[700, 650], [3, 9], [1300, 0]]),
    ("dp2_three_nodes", 12, 4, 2, 128, 0, 2, [[40, 0, 33, 1, 60, 17], [600, 580, 0, 640, 1, 333]]),
], ids=lambda v: v if isinstance(v, str) else None)
def test_static_dispatch_without_quantisation_and_with_dp_groups(name, N, node, dp, H, Hs, in_elemsize, steps):
    """Byte for byte what a2a_dispatch on a context writes (that path is checked against the oracle by
    the reference-matrix and dp-group tests), over consecutive steps of different sizes."""
    E, K, pad = 24, 3, 2
    Le = -(-E // N)
    max_tokens = max(max(s) for s in steps)
    stream = torch.cuda.current_stream(DEV).cuda_stream
    common = dict(hidden_dim=H, hidden_dim_scale=Hs, in_elemsize=in_elemsize, out_elemsize=2,
                  scale_elemsize=4 if Hs else 0, max_num_tokens=max_tokens, max_recv_tokens=max_tokens * K * N,
                  max_private_tokens=0, num_experts=E, expert_padding=pad, num_experts_per_token=K, dp_size=dp,
                  node_size=node, world_size=N, device=0)
    cfg = native.A2AConfig(struct_size=ctypes.sizeof(native.A2AConfig), out_dtype=native.SCALAR_TYPE[torch.bfloat16],
                           flags=0, **common)
    ctx = native.AllToAllContext.create(out_dtype=torch.bfloat16, **common)
    flags = torch.zeros(1, dtype=torch.int32, device=DEV)
    try:
        for i, tokens in enumerate(steps):
            print(f"{name} step {i}: tokens per group={tokens}", flush=True)
            rows = max(sum(tokens) * K + pad * Le, 1)
            ka, a, out_a = _raw_step(N, H, Hs, K, E, Le, tokens, rows, in_elemsize=in_elemsize, seed=70 + i,
                                     dp_size=dp, scale_transposed=True)
            kb, b, out_b = _raw_step(N, H, Hs, K, E, Le, tokens, rows, in_elemsize=in_elemsize, seed=70 + i,
                                     dp_size=dp, scale_transposed=True)
            ctx.dispatch(a, False, stream)
            assert ctx.status(stream) == 0
            native.dispatch_static(cfg, b, False, flags.data_ptr(), stream)
            torch.cuda.synchronize(DEV)
            assert int(flags.item()) == 0
            wrote = 0
            for r in range(N):
                for ta, tb in zip(out_a[r], out_b[r]):
                    assert torch.equal(ta.view(torch.uint8), tb.view(torch.uint8)), f"rank {r}"
                wrote += int((out_a[r][0].clamp_min(0)).sum().item())
            assert wrote == sum(tokens) * K                    # every copy arrived: nothing compared is vacuous
            del ka, kb
    finally:
        ctx.destroy()


def test_static_dispatch_refusals_enqueue_nothing():
    """Steps whose tables do not fit the fixed array, more tokens than max_num_tokens, and flags are refused
    on the host with the status and a text that names the sizes; a refused call records no node when a
    stream is being captured (the C++ self-test counts the nodes of such a graph)."""
    case = Case("static_refusals", 16, 256, 256, 8, 8, 9400)
    world = [make_rank(case, r, 16) for r in range(8)]
    b = _Buffers(case, world, 256)
    stream = torch.cuda.current_stream(DEV).cuda_stream
    big = _config(case, 40000)                                   # 8 ranks x 40000 tokens x 8 routes: tables beyond 8 MiB
    args = list(b.args)
    args[0] = native.A2ADispatchArgs.from_buffer_copy(args[0])
    args[0].num_tokens = 40000
    with pytest.raises(RuntimeError, match="bytes of routing tables"):
        native.dispatch_static(big, args, True, None, stream)
    with pytest.raises(RuntimeError, match="exceeds maximum"):
        native.dispatch_static(_config(case, 16), args, True, None, stream)
    flagged = _config(case, 16)
    flagged.flags = native.FLAG_SEPARATE_ROUTING
    with pytest.raises(RuntimeError, match="takes no flags"):
        native.dispatch_static(flagged, b.args, True, None, stream)
    # the refused calls left the outputs alone, and the same buffers still take an accepted call
    torch.cuda.synchronize(DEV)
    assert all((t == SENTINEL).all() for t in b.x)
    native.dispatch_static(_config(case, 16), b.args, True, None, stream)
    want = _oracle(case, world, 256)
    assert_dispatch_equal(case, b.result(), want)
