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
