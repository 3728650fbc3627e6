"""bound_m, accumulate, element types, error reporting and the quantiser on every bf16 value."""

from dataclasses import replace

import numpy as np
import pytest
import torch

import a2a_oracle as oracle
from a2a_cases import C0, C1, C2, bf16_codes, make_world, scaled
from a2a_harness import (SENTINEL, WorldResult, assert_combine_close, assert_dispatch_equal, make_ops, rows_needed,
                         run_gpu, run_oracle)
from a2a_transport import RefConfig, make_ref_rank, oracle_combine, oracle_dispatch, rows_for
from a2a_transport import make_ops as make_transport_ops
from pplx_garden_amd.native import p2p_all_to_all as native

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def test_quantiser_on_every_bf16_value_and_many_scales():
    """Each group of 128 holds a run of consecutive bf16 codes plus one element that sets the
    group maximum, so every finite bf16 value meets many different scales."""
    H = 2048
    codes = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    finite = codes[np.isfinite(oracle.bf16_to_f32(codes))]
    rng = np.random.default_rng(17)
    groups = []
    for rep, top in enumerate([1e-3, 0.11, 1.0, 7.5, 300.0, 3e4, 1e9, 3e38]):
        vals = finite.copy()
        rng.shuffle(vals)
        vals = vals[: len(vals) // 127 * 127].reshape(-1, 127)
        top_code = oracle.f32_to_bf16(np.full((vals.shape[0], 1), top, dtype=np.float32))
        groups.append(np.concatenate([vals, top_code], axis=1))
    g = np.concatenate(groups, axis=0)
    g = g[: g.shape[0] // (H // 128) * (H // 128)]
    x_codes = g.reshape(-1, H)
    T = x_codes.shape[0]
    case = replace(C0, name="quant_all", num_tokens=T, topk=1, num_experts=4, world_size=1)
    x = torch.from_numpy(x_codes.view(np.int16).copy()).view(torch.bfloat16)
    idx = torch.zeros((T, 1), dtype=torch.int32)
    w = torch.ones((T, 1), dtype=torch.float32)
    _, ops = make_ops(case, DEV, max_num_tokens=T)
    try:
        n = torch.zeros(4, dtype=torch.int32, device=DEV)
        ox = torch.zeros((T, H), dtype=torch.uint8, device=DEV).view(torch.float8_e4m3fn)
        os_ = torch.zeros((T, H // 128), dtype=torch.float32, device=DEV)
        ops[0].dispatch(out_expert_num_tokens=n, out_expert_x=ox, out_expert_x_scale=os_, dp_x=x.to(DEV),
                        dp_x_scale=None, indices=idx.view(torch.uint32).to(DEV), weights=w.to(DEV))
        torch.cuda.synchronize(DEV)
        assert ops[0].context.status() == 0
        q, s = oracle.quantize_block128(x_codes)
        np.testing.assert_array_equal(ox.view(torch.uint8).cpu().numpy(), q)       # one expert, token order
        np.testing.assert_array_equal(os_.cpu().numpy().view(np.uint32), s.view(np.uint32))
        assert n.cpu().tolist() == [T, 0, 0, 0]
    finally:
        ops[0].destroy()


@pytest.mark.parametrize("split", [False, True], ids=["group", "split"])
@pytest.mark.parametrize("repeat", [1, 110, 450], ids=["one_launch_small", "one_launch_single", "two_launch"])
def test_quantiser_on_nan_infinity_and_the_largest_bf16_value(repeat, split):
    """A NaN poisons its group of 128 (scale NaN, every code the NaN code), an infinity makes the
    scale infinite: bit for bit what the oracle says (which the CPU tests pin against a hand-written
    expectation and torch's operations), in every dispatch kernel that quantises (10, 1100 and 4500
    tokens take the three paths of the group call and of the split send)."""
    from a2a_nonfinite import bad_rows, expected_special_groups

    bits, kinds = bad_rows()
    H = bits.shape[1]
    x_codes = np.tile(bits, (repeat, 1))
    T = x_codes.shape[0]
    case = replace(C0, name="quant_bad", num_tokens=T, hidden_dim=H, topk=2, num_experts=8, world_size=2)
    x = torch.from_numpy(x_codes.view(np.int16).copy()).view(torch.bfloat16)
    gen = torch.Generator().manual_seed(5)
    idx = torch.rand((T, 8), generator=gen).topk(2, dim=-1).indices.to(torch.int32)
    w = torch.full((T, 2), 0.5, dtype=torch.float32)
    empty = dict(x=torch.zeros((0, H), dtype=torch.bfloat16), idx=torch.zeros((0, 2), dtype=torch.int32),
                 w=torch.zeros((0, 2), dtype=torch.float32))
    ins = [dict(x=x, idx=idx, w=w), empty]
    want = oracle.dispatch_world(
        [oracle.RankInput(x=bf16_codes(i["x"]), indices=i["idx"].numpy()) for i in ins],
        num_experts=8, world_size=2, node_size=2, expert_padding=1, out_rows=2 * T, quantize=True)
    _, ops = make_ops(case, DEV, max_num_tokens=T)
    try:
        outs = [dict(n=torch.full((4,), -1, dtype=torch.int32, device=DEV),
                     x=torch.full((2 * T, H), SENTINEL, dtype=torch.uint8, device=DEV).view(torch.float8_e4m3fn),
                     s=torch.full((2 * T, H // 128), -7.0, dtype=torch.float32, device=DEV)) for _ in range(2)]
        phases = [dict(do_send=True, do_recv=False), dict(do_send=False, do_recv=True)] if split else [dict()]
        for kw in phases:
            for r in range(2):
                ops[r].dispatch(out_expert_num_tokens=outs[r]["n"], out_expert_x=outs[r]["x"],
                                out_expert_x_scale=outs[r]["s"], dp_x=ins[r]["x"].to(DEV), dp_x_scale=None,
                                indices=ins[r]["idx"].view(torch.uint32).to(DEV), weights=ins[r]["w"].to(DEV), **kw)
        torch.cuda.synchronize(DEV)
        assert ops[0].context.status() == 0
        for r in range(2):
            wr = want[r].written
            np.testing.assert_array_equal(outs[r]["n"].cpu().numpy(), want[r].num_tokens)
            np.testing.assert_array_equal(outs[r]["x"].view(torch.uint8).cpu().numpy()[wr], want[r].x[wr])
            np.testing.assert_array_equal(outs[r]["s"].cpu().numpy().view(np.uint32)[wr],
                                          want[r].x_scale.view(np.uint32)[wr])
        # and against the hand-written expectation directly, on the copies of the first ten tokens
        slots = want[0].slots[0]
        for row, group, codes, scale_bits in expected_special_groups(bits, kinds):
            for k in range(2):
                r, slot = int(idx[row, k]) // 4, int(slots[row, k])
                got = outs[r]["x"].view(torch.uint8)[slot, group * 128:(group + 1) * 128].cpu().numpy()
                np.testing.assert_array_equal(got, codes)
                assert int(outs[r]["s"][slot, group].view(torch.int32).item()) & 0xFFFFFFFF == scale_bits
    finally:
        for op in ops:
            op.destroy()


@pytest.mark.parametrize("split", [False, True], ids=["group", "split"])
@pytest.mark.parametrize("case", [C0, scaled(C0, 700), scaled(C0, 1200)], ids=["one_launch", "one_launch_mid_size", "two_launch"])
def test_bound_m_limits_the_tokens(case, split):
    world = make_world(case, "all")
    bounds = [case.num_tokens, 0, 17, 1]
    rows = rows_needed(case, world)
    N, Le, H, Hs = case.world_size, case.experts_per_rank, case.hidden_dim, case.hidden_dim_scale
    inputs = [oracle.RankInput(x=bf16_codes(rd.x), indices=rd.indices.numpy(), bound_m=b) for rd, b in zip(world, bounds)]
    want = oracle.dispatch_world(inputs, num_experts=case.num_experts, world_size=N, node_size=N,
                                 expert_padding=1, out_rows=rows, quantize=True)
    _, ops = make_ops(case, DEV)
    try:
        t = []
        for r, rd in enumerate(world):
            t.append(dict(x=rd.x.to(DEV), idx=rd.indices_u32.to(DEV), w=rd.weights.to(DEV),
                          b=torch.tensor([bounds[r]], dtype=torch.int32, device=DEV),
                          n=torch.full((Le,), -1, dtype=torch.int32, device=DEV),
                          ox=torch.full((rows, H), SENTINEL, dtype=torch.uint8, device=DEV).view(torch.float8_e4m3fn),
                          os=torch.full((rows, Hs), -7.0, dtype=torch.float32, device=DEV),
                          o=torch.full((rd.x.shape[0], H), 3.0, dtype=torch.bfloat16, device=DEV)))
        phases = [dict(do_send=True, do_recv=False), dict(do_send=False, do_recv=True)] if split else [dict()]
        for ph in phases:
            for r in range(N):
                ops[r].dispatch(out_expert_num_tokens=t[r]["n"], out_expert_x=t[r]["ox"], out_expert_x_scale=t[r]["os"],
                                dp_x=t[r]["x"], dp_x_scale=None, indices=t[r]["idx"], weights=t[r]["w"],
                                bound_m=t[r]["b"], **ph)
        torch.cuda.synchronize(DEV)
        assert ops[0].context.status() == 0
        ys = []
        for r in range(N):
            np.testing.assert_array_equal(t[r]["n"].cpu().numpy(), want[r].num_tokens)
            wr = want[r].written
            got_x = t[r]["ox"].view(torch.uint8).cpu().numpy()
            np.testing.assert_array_equal(got_x[wr], want[r].x[wr])
            assert (got_x[~wr] == SENTINEL).all()
            y = oracle.f32_to_bf16(np.where(wr[:, None], oracle.dequantize_block128(want[r].x, want[r].x_scale), 0).astype(np.float32))
            ys.append(y)
        yd = [torch.from_numpy(y.view(np.int16)).view(torch.bfloat16).to(DEV) for y in ys]
        for ph in phases:
            for r in range(N):
                ops[r].combine(out_tokens=t[r]["o"], indices=t[r]["idx"], weights=t[r]["w"], expert_y=yd[r],
                               bound_m=t[r]["b"], **ph)
        torch.cuda.synchronize(DEV)
        assert ops[0].context.status() == 0
        comb = oracle.combine_world(ys, [rd.indices.numpy() for rd in world], [rd.weights.numpy() for rd in world],
                                    want[0].slots, num_experts=case.num_experts, world_size=N, bound_m=bounds)
        for g in range(N):
            got = t[g]["o"].view(torch.int16).cpu().numpy().view(np.uint16)
            b = bounds[g]
            np.testing.assert_allclose(oracle.bf16_to_f32(got[:b]), oracle.bf16_to_f32(comb[g][:b]), rtol=1e-2, atol=1e-3)
            assert (oracle.bf16_to_f32(got[b:]) == 3.0).all()          # tokens beyond bound_m are not written
    finally:
        for op in ops:
            op.destroy()


def _check_split_combine_refuses_narrow_rows(in_dtype, out_dtype):
    """combine-send copies staging rows sized for out_dtype and is not told the type of expert_y:
    narrower rows are refused before any launch, by the operator and by the C ABI."""
    cfg = RefConfig("types", 4, 1, 48, 16, 256, None, 4, torch.bfloat16, out_dtype, None)
    world = [make_ref_rank(cfg, r) for r in range(4)]
    rows = rows_for(cfg, world)
    ops = make_transport_ops(cfg, DEV)
    try:
        t = []
        for r, rd in enumerate(world):
            t.append(dict(x=rd.dp_x.to(DEV), idx=rd.indices.view(torch.uint32).to(DEV), w=rd.weights.to(DEV),
                          n=torch.zeros(4, dtype=torch.int32, device=DEV),
                          ox=torch.zeros((rows, cfg.hidden_dim), dtype=torch.bfloat16, device=DEV),
                          y=torch.zeros((rows, cfg.hidden_dim), dtype=in_dtype, device=DEV),
                          o=torch.zeros((cfg.max_num_tokens, cfg.hidden_dim), dtype=out_dtype, device=DEV)))
        for ph in (dict(do_send=True, do_recv=False), dict(do_send=False, do_recv=True)):
            for r in range(4):
                ops[r].dispatch(out_expert_num_tokens=t[r]["n"], out_expert_x=t[r]["ox"], out_expert_x_scale=None,
                                dp_x=t[r]["x"], dp_x_scale=None, indices=t[r]["idx"], weights=t[r]["w"], **ph)
        with pytest.raises(RuntimeError, match="element size of out_dtype"):
            ops[0].combine(out_tokens=t[0]["o"], indices=t[0]["idx"], weights=t[0]["w"], expert_y=t[0]["y"],
                           do_send=True, do_recv=False)
        if in_dtype.itemsize < out_dtype.itemsize:
            with pytest.raises(RuntimeError, match="as wide as out_dtype"):
                ops[0].context.combine_send(0, t[0]["y"].data_ptr(), cfg.hidden_dim * in_dtype.itemsize, rows, 0)
        else:
            # wider rows can be copied (their first bytes), but the recv is told the type and refuses
            # to read staging rows sized for 2-byte elements as 4-byte ones
            for r in range(4):
                ops[r].context.combine_send(r, t[r]["y"].data_ptr(), cfg.hidden_dim * in_dtype.itemsize, rows, 0)
            with pytest.raises(RuntimeError, match="does not have the 2-byte elements"):
                ops[0].context.combine_recv(0, cfg.max_num_tokens, rows, in_dtype, t[0]["o"].data_ptr(),
                                            cfg.hidden_dim, t[0]["idx"].data_ptr(), cfg.num_experts_per_token,
                                            t[0]["w"].data_ptr(), cfg.num_experts_per_token, None, False, 0)
        torch.cuda.synchronize(DEV)
        assert ops[0].context.status() == 0
    finally:
        for op in ops:
            op.destroy()


@pytest.mark.parametrize("split", [False, True], ids=["group", "split"])
@pytest.mark.parametrize("in_dtype,out_dtype", [
    (torch.bfloat16, torch.bfloat16), (torch.float32, torch.float32), (torch.float16, torch.float16),
    (torch.bfloat16, torch.float32), (torch.float16, torch.float32),
    (torch.bfloat16, torch.float16), (torch.float16, torch.bfloat16),
    (torch.float32, torch.bfloat16), (torch.float32, torch.float16),
], ids=lambda d: str(d).split(".")[-1])
def test_combine_types_and_accumulate(in_dtype, out_dtype, split):
    """All nine pairs expert_y in {f16, bf16, f32} x out in {f16, bf16, f32} that the reference
    instantiates (a2a_combine_recv.cu:237-238, launch_utils.cuh:183-194), with and without accumulate
    (a2a_combine_recv.cu:132).  The split calls stage rows sized for the output type, so there
    expert_y has the output's element size (seven pairs through the group call only)."""
    if split and in_dtype.itemsize != out_dtype.itemsize:
        _check_split_combine_refuses_narrow_rows(in_dtype, out_dtype)
        return
    cfg = RefConfig("types", 4, 1, 48, 16, 256, None, 4, torch.bfloat16, out_dtype, None)
    world = [make_ref_rank(cfg, r) for r in range(4)]
    rows = rows_for(cfg, world)
    want = oracle_dispatch(cfg, world, rows)
    gen = torch.Generator().manual_seed(9)
    ys = [torch.randn((rows, cfg.hidden_dim), generator=gen).to(in_dtype) for _ in range(4)]
    prev = [torch.randn((cfg.max_num_tokens, cfg.hidden_dim), generator=gen).to(out_dtype) for _ in range(4)]
    ops = make_transport_ops(cfg, DEV)
    try:
        t = []
        for r, rd in enumerate(world):
            t.append(dict(x=rd.dp_x.to(DEV), idx=rd.indices.view(torch.uint32).to(DEV), w=rd.weights.to(DEV),
                          n=torch.zeros(4, dtype=torch.int32, device=DEV),
                          ox=torch.zeros((rows, cfg.hidden_dim), dtype=torch.bfloat16, device=DEV), y=ys[r].to(DEV)))
        phases = [dict(do_send=True, do_recv=False), dict(do_send=False, do_recv=True)] if split else [dict()]
        for ph in phases:
            for r in range(4):
                ops[r].dispatch(out_expert_num_tokens=t[r]["n"], out_expert_x=t[r]["ox"], out_expert_x_scale=None,
                                dp_x=t[r]["x"], dp_x_scale=None, indices=t[r]["idx"], weights=t[r]["w"], **ph)
        for accumulate in (False, True):
            outs = [p.clone().to(DEV) for p in prev]
            for ph in phases:
                for r in range(4):
                    ops[r].combine(out_tokens=outs[r], indices=t[r]["idx"], weights=t[r]["w"], expert_y=t[r]["y"],
                                   accumulate=accumulate, **ph)
            torch.cuda.synchronize(DEV)
            assert ops[0].context.status() == 0
            prev_np = None
            if accumulate:
                prev_np = [p.numpy() if out_dtype == torch.float32 else p.view(torch.int16).numpy().view(np.uint16) for p in prev]
            comb = oracle_combine(cfg, world, ys, want[0].slots, out_prev=prev_np)
            for g in range(4):
                got = outs[g].cpu().to(torch.float32).numpy()
                ref = comb[g] if out_dtype == torch.float32 else (
                    oracle.bf16_to_f32(comb[g]) if out_dtype == torch.bfloat16 else oracle.f16_to_f32(comb[g]))
                tol = 1e-5 if out_dtype == torch.float32 and in_dtype == torch.float32 else 1e-2
                np.testing.assert_allclose(got, ref, rtol=tol, atol=tol)
    finally:
        for op in ops:
            op.destroy()


def test_errors_are_reported_not_faulted():
    case = C0
    world = make_world(case, "one")
    N, Le, H, Hs = case.world_size, case.experts_per_rank, case.hidden_dim, case.hidden_dim_scale
    _, ops = make_ops(case, DEV)
    try:
        ctx = ops[0].context
        rd = world[0]
        bad = rd.indices.clone()
        bad[3, 1] = case.num_experts + 5                 # an expert id out of range: that copy is dropped
        rows = 4                                           # far too few rows: overflowing copies are dropped
        t = [dict(n=torch.zeros(Le, dtype=torch.int32, device=DEV),
                  ox=torch.full((rows, H), SENTINEL, dtype=torch.uint8, device=DEV).view(torch.float8_e4m3fn),
                  os=torch.zeros((rows, Hs), dtype=torch.float32, device=DEV)) for _ in range(N)]
        x = rd.x.to(DEV)
        w = rd.weights.to(DEV)
        for r in range(N):
            xr = x if r == 0 else x[:0]
            ir = (bad if r == 0 else bad[:0]).view(torch.uint32).to(DEV)
            ops[r].dispatch(out_expert_num_tokens=t[r]["n"], out_expert_x=t[r]["ox"], out_expert_x_scale=t[r]["os"],
                            dp_x=xr, dp_x_scale=None, indices=ir, weights=w if r == 0 else w[:0])
        flags = ctx.status()
        assert flags & native.DEV_BAD_EXPERT_ID and flags & native.DEV_RECV_OVERFLOW
        assert ctx.status() == 0                           # reading clears the word
        # host-side errors: too many tokens (a2a_context.rs:290-292), bad rank, combine before dispatch
        big = torch.zeros((case.num_tokens + 1, H), dtype=torch.bfloat16, device=DEV)
        with pytest.raises(RuntimeError, match="exceeds maximum"):
            ctx.dispatch_send(0, case.num_tokens + 1, big.data_ptr(), 2 * H, None, None, None, bad.data_ptr(),
                              case.topk, 0, case.topk, None, 0, quantize=True)
        with pytest.raises(RuntimeError, match="rank"):
            ctx.dispatch_recv(N, 0, 0, H, 0, None, None, None, 0)
        with pytest.raises(RuntimeError, match="16-byte"):
            ctx.dispatch_send(0, 4, x.data_ptr() + 2, 2 * H, None, None, None, bad.data_ptr(), case.topk, 0,
                              case.topk, None, 0, quantize=True)
        # index rows closer together than K ids, and a stride the kernels' 32-bit fields cannot carry
        with pytest.raises(RuntimeError, match="indices_stride"):
            ctx.dispatch_send(0, 4, x.data_ptr(), 2 * H, None, None, None, bad.data_ptr(), case.topk - 1, 0,
                              case.topk, None, 0, quantize=True)
        with pytest.raises(RuntimeError, match="32 bits"):
            ctx.dispatch_send(0, 4, x.data_ptr(), 2 * H, None, None, None, bad.data_ptr(), 1 << 32, 0,
                              case.topk, None, 0, quantize=True)
        # a combine of more tokens than the step's dispatch routed for that rank would gather stale routes
        out = torch.zeros((case.num_tokens, H), dtype=torch.bfloat16, device=DEV)
        y = torch.zeros((rows, H), dtype=torch.bfloat16, device=DEV)
        with pytest.raises(RuntimeError, match="combines"):
            per_rank = []
            for r in range(N):
                a = native.A2ACombineArgs()
                a.expert_y, a.expert_y_stride, a.expert_y_rows = y.data_ptr(), 2 * H, rows
                if r == 1:                                 # rank 1 sent nothing in the dispatch above
                    a.num_tokens, a.out_tokens, a.out_tokens_stride = 2, out.data_ptr(), H
                    a.indices, a.indices_stride = bad.view(torch.uint32).to(DEV).data_ptr(), case.topk
                    a.weights, a.weights_stride = w.data_ptr(), case.topk
                per_rank.append(a)
            ctx.combine(per_rank, torch.bfloat16, False, 0)
    finally:
        for op in ops:
            op.destroy()
    _, ops = make_ops(case, DEV)
    try:
        ctx = ops[0].context
        with pytest.raises(RuntimeError, match="before"):
            ctx.dispatch_recv(0, 0, 0, H, 0, None, None, None, 0)
        with pytest.raises(RuntimeError, match="a2a_dispatch"):
            ctx.combine([native.A2ACombineArgs() for _ in range(N)], torch.bfloat16, False, 0)
    finally:
        for op in ops:
            op.destroy()


@pytest.mark.parametrize("split", [False, True], ids=["group", "split"])
def test_device_errors_in_the_two_launch_paths(split):
    """The same two device-side errors (an expert id out of range, receive buffers that are too small)
    on a step large enough for the two-launch dispatch and send: flagged, not faulted, and the context
    keeps working afterwards."""
    case = scaled(C0, 1500)
    world = make_world(case, "one")
    N, Le, H, Hs = case.world_size, case.experts_per_rank, case.hidden_dim, case.hidden_dim_scale
    _, ops = make_ops(case, DEV)
    try:
        ctx = ops[0].context
        rd = world[0]
        bad = rd.indices.clone()
        bad[1234, 2] = case.num_experts + 1
        phases = [dict(do_send=True, do_recv=False), dict(do_send=False, do_recv=True)] if split else [dict()]

        def run(indices, rows):
            t = [dict(n=torch.zeros(Le, dtype=torch.int32, device=DEV),
                      ox=torch.full((rows, H), SENTINEL, dtype=torch.uint8, device=DEV).view(torch.float8_e4m3fn),
                      os=torch.zeros((rows, Hs), dtype=torch.float32, device=DEV)) for _ in range(N)]
            x, w = rd.x.to(DEV), rd.weights.to(DEV)
            for ph in phases:
                for r in range(N):
                    ops[r].dispatch(out_expert_num_tokens=t[r]["n"], out_expert_x=t[r]["ox"],
                                    out_expert_x_scale=t[r]["os"], dp_x=x if r == 0 else x[:0], dp_x_scale=None,
                                    indices=(indices if r == 0 else indices[:0]).view(torch.uint32).to(DEV),
                                    weights=w if r == 0 else w[:0], **ph)
            return t

        run(bad, 16)
        flags = ctx.status()
        assert flags & native.DEV_BAD_EXPERT_ID and flags & native.DEV_RECV_OVERFLOW
        assert ctx.status() == 0
        # a clean step on the same context afterwards
        rows = rows_needed(case, world)
        t = run(rd.indices, rows)
        assert ctx.status() == 0
        want = run_oracle(case, world, rows)
        for r in range(N):
            np.testing.assert_array_equal(t[r]["n"].cpu().numpy(), want.num_tokens[r])
            wr = want.written[r]
            np.testing.assert_array_equal(t[r]["ox"].view(torch.uint8).cpu().numpy()[wr], want.x[r][wr])
    finally:
        for op in ops:
            op.destroy()


def test_operator_asserts_like_the_reference():
    case = C0
    _, ops = make_ops(case, DEV)
    try:
        Le, H, Hs, K = case.experts_per_rank, case.hidden_dim, case.hidden_dim_scale, case.topk
        good = dict(out_expert_num_tokens=torch.zeros(Le, dtype=torch.int32, device=DEV),
                    out_expert_x=torch.zeros((8, H), dtype=torch.uint8, device=DEV).view(torch.float8_e4m3fn),
                    out_expert_x_scale=torch.zeros((8, Hs), dtype=torch.float32, device=DEV),
                    dp_x=torch.zeros((2, H), dtype=torch.bfloat16, device=DEV), dp_x_scale=None,
                    indices=torch.zeros((2, K), dtype=torch.int32, device=DEV).view(torch.uint32),
                    weights=torch.zeros((2, K), dtype=torch.float32, device=DEV))
        for key, value in [
            ("out_expert_num_tokens", torch.zeros(Le + 1, dtype=torch.int32, device=DEV)),    # p2p_all_to_all.py:337
            ("out_expert_num_tokens", torch.zeros(Le, dtype=torch.int64, device=DEV)),         # :339
            ("out_expert_x", torch.zeros((8, H), dtype=torch.bfloat16, device=DEV)),           # :346
            ("indices", torch.zeros((2, K), dtype=torch.int32, device=DEV)),                   # :393 uint32 only
            ("weights", torch.zeros((2, K), dtype=torch.float64, device=DEV)),                 # :400
            ("bound_m", torch.zeros(2, dtype=torch.int32, device=DEV)),                        # :407
        ]:
            with pytest.raises(AssertionError):
                ops[0].dispatch(**{**good, key: value})
        with pytest.raises(AssertionError):
            ops[0].dispatch(**good, do_send=False, do_recv=False)                              # :332
    finally:
        for op in ops:
            op.destroy()


@pytest.mark.parametrize("split", [False, True], ids=["group", "split"])
@pytest.mark.parametrize("case,sources", [(C1, "all"), (scaled(C1, 1200), "one"), (scaled(C1, 300), "all"),
                                          (scaled(C1, 40), "ragged"), (scaled(C1, 900), "one")],
                         ids=["one_launch_dispatch", "two_launch_dispatch_one_source", "two_launch_dispatch", "ragged",
                              "one_launch_dispatch_larger_source"])
def test_calls_can_be_captured_in_a_hip_graph(case, sources, split):
    """The calls only enqueue kernels whose arguments travel by value (no allocation, copy or
    synchronisation inside), so a dispatch + combine can be captured once and replayed
    (docs/fabric-lib.md:15 lists graph capture as a feature of the reference): the two group calls
    of every rank, or the four split calls of every rank (all sends, all recvs, all combine-sends,
    all combine-recvs) on a context whose staging was allocated at create.  Every replay, with eager
    work in between, must reproduce what the ORACLE says, bit for bit for the dispatch and within the
    combine's tolerance.  The larger cases take the two-launch dispatch, whose step totals alternate
    between two copies in device memory: the replays land on either copy."""
    world = make_world(case, sources)
    rows = rows_needed(case, world)
    N, Le, H, Hs = case.world_size, case.experts_per_rank, case.hidden_dim, case.hidden_dim_scale
    want = run_oracle(case, world, rows)
    gen = torch.Generator().manual_seed(3)
    ys = [torch.randn((rows, H), generator=gen).to(torch.bfloat16) for _ in range(N)]
    want_out = oracle.combine_world([bf16_codes(y) for y in ys], [rd.indices.numpy() for rd in world],
                                    [rd.weights.numpy() for rd in world], want.slots,
                                    num_experts=case.num_experts, world_size=N)
    _, ops = make_ops(case, DEV, context_flags=native.FLAG_PREALLOC_STAGING if split else 0)
    try:
        t = []
        for r, rd in enumerate(world):
            t.append(dict(x=rd.x.to(DEV), idx=rd.indices_u32.to(DEV), w=rd.weights.to(DEV),
                          n=torch.zeros(Le, dtype=torch.int32, device=DEV),
                          ox=torch.zeros((rows, H), dtype=torch.uint8, device=DEV).view(torch.float8_e4m3fn),
                          os=torch.zeros((rows, Hs), dtype=torch.float32, device=DEV),
                          y=ys[r].to(DEV),
                          o=torch.zeros((rd.x.shape[0], H), dtype=torch.bfloat16, device=DEV)))
        phases = [dict(do_send=True, do_recv=False), dict(do_send=False, do_recv=True)] if split else [dict()]

        def step():
            for ph in phases:
                for r in range(N):
                    ops[r].dispatch(out_expert_num_tokens=t[r]["n"], out_expert_x=t[r]["ox"],
                                    out_expert_x_scale=t[r]["os"], dp_x=t[r]["x"], dp_x_scale=None,
                                    indices=t[r]["idx"], weights=t[r]["w"], **ph)
            for ph in phases:
                for r in range(N):
                    ops[r].combine(out_tokens=t[r]["o"], indices=t[r]["idx"], weights=t[r]["w"],
                                   expert_y=t[r]["y"], **ph)

        def check(label):
            torch.cuda.synchronize(DEV)
            got = WorldResult([a["n"].cpu().numpy() for a in t],
                              [a["ox"].view(torch.uint8).cpu().numpy() for a in t],
                              [a["os"].cpu().numpy() for a in t],
                              [a["o"].view(torch.int16).cpu().numpy().view(np.uint16) for a in t])
            for r in range(N):
                n_local = max(min(Le, case.num_experts - r * Le), 0)
                np.testing.assert_array_equal(got.num_tokens[r][:n_local], want.num_tokens[r][:n_local], err_msg=label)
                w = want.written[r]
                np.testing.assert_array_equal(got.x[r][w], want.x[r][w], err_msg=label)
                np.testing.assert_array_equal(got.x_scale[r][w].view(np.uint32), want.x_scale[r][w].view(np.uint32),
                                              err_msg=label)
                if got.out_tokens[r].size:
                    np.testing.assert_allclose(oracle.bf16_to_f32(got.out_tokens[r]), oracle.bf16_to_f32(want_out[r]),
                                               rtol=1e-2, atol=1e-2, err_msg=label)

        def clear():
            for a in t:
                a["n"].zero_(); a["ox"].view(torch.uint8).zero_(); a["os"].zero_(); a["o"].zero_()

        step()
        check("eager")
        assert ops[0].context.status() == 0
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream(device=DEV)
        side.wait_stream(torch.cuda.current_stream(DEV))
        with torch.cuda.stream(side):
            step()                                       # warm-up on the capture stream
        torch.cuda.current_stream(DEV).wait_stream(side)
        torch.cuda.synchronize(DEV)
        with torch.cuda.graph(graph):
            step()
        for i in range(3):
            clear()
            scratch = torch.randn(1 << 20, device=DEV).sum()       # eager work between replays
            torch.cuda.synchronize(DEV)
            graph.replay()
            check(f"replay {i}")
            del scratch
        assert ops[0].context.status() == 0
    finally:
        for op in ops:
            op.destroy()


def test_a_first_split_send_under_capture_needs_preallocated_staging():
    """The split calls allocate their staging on first use unless the context was created with
    A2A_FLAG_PREALLOC_STAGING; allocating is illegal while a stream is being captured, so that
    first send is refused there instead (and works once the capture is over)."""
    case = scaled(C0, 8)
    world = make_world(case, "all")
    _, ops = make_ops(case, DEV)
    try:
        rd = world[0]
        x, idx, w = rd.x.to(DEV), rd.indices_u32.to(DEV), rd.weights.to(DEV)
        n = torch.zeros(case.experts_per_rank, dtype=torch.int32, device=DEV)
        ox = torch.zeros((64, case.hidden_dim), dtype=torch.uint8, device=DEV).view(torch.float8_e4m3fn)
        os_ = torch.zeros((64, case.hidden_dim_scale), dtype=torch.float32, device=DEV)
        send = lambda: ops[0].dispatch(out_expert_num_tokens=n, out_expert_x=ox, out_expert_x_scale=os_, dp_x=x,
                                       dp_x_scale=None, indices=idx, weights=w, do_send=True, do_recv=False)
        torch.cuda.synchronize(DEV)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            with pytest.raises(RuntimeError, match="A2A_FLAG_PREALLOC_STAGING"):
                send()
        send()
        torch.cuda.synchronize(DEV)
        assert ops[0].context.status() == 0
    finally:
        for op in ops:
            op.destroy()


def test_kernel_own_events():
    """a2a_ctx_time_next_kernel: the pack and the gather of the next group calls record the caller's
    events at their own start and end; the request is one-shot."""
    case = C1
    world = make_world(case, "all")
    rows = rows_needed(case, world)
    N, Le, H, Hs = case.world_size, case.experts_per_rank, case.hidden_dim, case.hidden_dim_scale
    _, ops = make_ops(case, DEV)
    try:
        t = []
        gen = torch.Generator().manual_seed(4)
        for r, rd in enumerate(world):
            t.append(dict(x=rd.x.to(DEV), idx=rd.indices_u32.to(DEV), w=rd.weights.to(DEV),
                          n=torch.zeros(Le, dtype=torch.int32, device=DEV),
                          ox=torch.zeros((rows, H), dtype=torch.uint8, device=DEV).view(torch.float8_e4m3fn),
                          os=torch.zeros((rows, Hs), dtype=torch.float32, device=DEV),
                          y=torch.randn((rows, H), generator=gen).to(torch.bfloat16).to(DEV),
                          o=torch.zeros((rd.x.shape[0], H), dtype=torch.bfloat16, device=DEV)))

        def step():
            for r in range(N):
                ops[r].dispatch(out_expert_num_tokens=t[r]["n"], out_expert_x=t[r]["ox"], out_expert_x_scale=t[r]["os"],
                                dp_x=t[r]["x"], dp_x_scale=None, indices=t[r]["idx"], weights=t[r]["w"])
            for r in range(N):
                ops[r].combine(out_tokens=t[r]["o"], indices=t[r]["idx"], weights=t[r]["w"], expert_y=t[r]["y"])

        step()
        torch.cuda.synchronize(DEV)
        first = [a["o"].clone() for a in t]
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(6)]
        for e in ev:
            e.record()                       # gives the event its handle
        torch.cuda.synchronize(DEV)
        ctx = ops[0].context
        ctx.time_next_kernel(native.KERNEL_PACK, ev[0].cuda_event, ev[1].cuda_event)
        ctx.time_next_kernel(native.KERNEL_GATHER, ev[2].cuda_event, ev[3].cuda_event)
        ev[4].record()
        step()
        ev[5].record()
        torch.cuda.synchronize(DEV)
        pack_ms, gather_ms, both_ms = ev[0].elapsed_time(ev[1]), ev[2].elapsed_time(ev[3]), ev[4].elapsed_time(ev[5])
        assert 0.0 < pack_ms < both_ms and 0.0 < gather_ms < both_ms
        assert ev[1].elapsed_time(ev[2]) >= 0.0          # the pack ends before the gather begins
        for a, want in zip(t, first):
            assert torch.equal(a["o"].view(torch.int16), want.view(torch.int16))
        # one-shot: a further step leaves the events alone
        step()
        torch.cuda.synchronize(DEV)
        assert ev[0].elapsed_time(ev[1]) == pack_ms and ev[2].elapsed_time(ev[3]) == gather_ms
        with pytest.raises(RuntimeError, match="both events or neither"):
            ctx.time_next_kernel(native.KERNEL_PACK, ev[0].cuda_event, None)
        with pytest.raises(RuntimeError, match="unknown kernel"):
            ctx.time_next_kernel(7, None, None)
        assert ctx.status() == 0
    finally:
        for op in ops:
            op.destroy()


def test_routing_kernel_own_events():
    """A large group step has a routing launch of its own before the pack: A2A_KERNEL_ROUTE times it,
    and it ends before the pack begins."""
    case = scaled(C1, 1500)     # 8 x 1500 tokens x 8 entries: far beyond the one-launch step
    world = make_world(case, "all")
    rows = rows_needed(case, world)
    want = run_oracle(case, world, rows)
    _, ops = make_ops(case, DEV)
    try:
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
        for e in ev:
            e.record()
        torch.cuda.synchronize(DEV)
        ctx = ops[0].context
        ctx.time_next_kernel(native.KERNEL_ROUTE, ev[0].cuda_event, ev[1].cuda_event)
        ctx.time_next_kernel(native.KERNEL_PACK, ev[2].cuda_event, ev[3].cuda_event)
        got = run_gpu(case, world, rows, DEV, ops=ops)
        torch.cuda.synchronize(DEV)
        route_ms, pack_ms = ev[0].elapsed_time(ev[1]), ev[2].elapsed_time(ev[3])
        print(f"route {route_ms * 1e3:.1f} us, pack {pack_ms * 1e3:.1f} us", flush=True)
        assert 0.0 < route_ms < 1.0 and 0.0 < pack_ms
        assert ev[1].elapsed_time(ev[2]) >= 0.0          # the routing ends before the pack begins
        assert_dispatch_equal(case, got, want)
        assert_combine_close(case, got, want)
    finally:
        for op in ops:
            op.destroy()
    # a small step counts its routing inside the pack: the request is consumed, nothing is recorded
    case = C0
    world = make_world(case, "all")
    rows = rows_needed(case, world)
    _, ops = make_ops(case, DEV)
    try:
        before = ev[3].elapsed_time(ev[0])
        ops[0].context.time_next_kernel(native.KERNEL_ROUTE, ev[0].cuda_event, ev[1].cuda_event)
        run_gpu(case, world, rows, DEV, ops=ops)
        run_gpu(case, world, rows, DEV, ops=ops)
        torch.cuda.synchronize(DEV)
        assert ev[3].elapsed_time(ev[0]) == before
    finally:
        for op in ops:
            op.destroy()


def test_operator_reports_the_reference_capacities():
    """`P2PAllToAll.max_recv_tokens` / `max_private_tokens` of live operators on the five baseline
    shapes against the oracle's restatement of python/pplx_garden/kernels/p2p_all_to_all.py:92-114,
    and the DeepSeek decode value that those lines give (9216 rows)."""
    from a2a_cases import BASELINE_CASES
    for case in BASELINE_CASES:
        _, ops = make_ops(case, DEV)
        try:
            Le, private, recv = oracle.buffer_capacity(case.num_tokens, case.num_experts, case.topk,
                                                       case.world_size, 1, case.expert_padding)
            for op in ops:
                assert (op.num_local_experts, op.max_private_tokens, op.max_recv_tokens) == (Le, private, recv)
            if case is C2:
                assert ops[0].max_recv_tokens == 9216 and ops[0].max_private_tokens == 128
        finally:
            for op in ops:
                op.destroy()


def _check_single_source(case, sender, bound, strided, repeats=False):
    """Dispatch of a step in which only `sender` has tokens, against the oracle: counts, fp8 bytes, scales,
    untouched rows, and the sender's routing tables.  `repeats`: every third token names its first expert
    twice (the second copy goes to the next row of that expert)."""
    N, Le, H, Hs, K = case.world_size, case.experts_per_rank, case.hidden_dim, case.hidden_dim_scale, case.topk
    world = [make_world(case, "all")[r] if r == sender else make_world(scaled(case, 0), "all")[r] for r in range(N)]
    if repeats:
        world[sender].indices[::3, K - 1] = world[sender].indices[::3, 0]
    rows = rows_needed(case, world)
    inputs = [oracle.RankInput(x=bf16_codes(rd.x), indices=rd.indices.numpy(), bound_m=bound if r == sender else None)
              for r, rd in enumerate(world)]
    want = oracle.dispatch_world(inputs, num_experts=case.num_experts, world_size=N, node_size=N, expert_padding=case.expert_padding,
                                 out_rows=rows, quantize=True)
    _, ops = make_ops(case, DEV)
    try:
        t = []
        for r, rd in enumerate(world):
            idx = rd.indices_u32.to(DEV)
            if strided and rd.indices.shape[0]:
                wide = torch.zeros((rd.indices.shape[0], K + 3), dtype=torch.uint32, device=DEV)
                wide[:, :K] = idx
                idx = wide[:, :K]                  # row stride K + 3
                assert idx.stride(0) == K + 3
            t.append(dict(x=rd.x.to(DEV), idx=idx, w=rd.weights.to(DEV),
                          b=torch.tensor([bound], dtype=torch.int32, device=DEV) if r == sender and bound is not None else None,
                          n=torch.full((Le,), -1, dtype=torch.int32, device=DEV),
                          ox=torch.full((rows, H), SENTINEL, dtype=torch.uint8, device=DEV).view(torch.float8_e4m3fn),
                          os=torch.full((rows, Hs), -7.0, dtype=torch.float32, device=DEV)))
        for r in range(N):
            ops[r].dispatch(out_expert_num_tokens=t[r]["n"], out_expert_x=t[r]["ox"], out_expert_x_scale=t[r]["os"],
                            dp_x=t[r]["x"], dp_x_scale=None, indices=t[r]["idx"], weights=t[r]["w"], bound_m=t[r]["b"])
        torch.cuda.synchronize(DEV)
        ctx = ops[0].context
        assert ctx.status() == 0
        for r in range(N):
            n_local = max(0, min(Le, case.num_experts - r * Le))   # (a2a_dispatch_recv.cu:220-224 writes the experts that exist)
            np.testing.assert_array_equal(t[r]["n"].cpu().numpy()[:n_local], want[r].num_tokens[:n_local])
            assert (t[r]["n"].cpu().numpy()[n_local:] == -1).all()
            wr = want[r].written
            got_x = t[r]["ox"].view(torch.uint8).cpu().numpy()
            np.testing.assert_array_equal(got_x[wr], want[r].x[wr])
            np.testing.assert_array_equal(t[r]["os"].cpu().numpy()[wr].view(np.uint32), want[r].x_scale[wr].view(np.uint32))
            assert (got_x[~wr] == SENTINEL).all()
        n_eff = world[sender].indices.shape[0] if bound is None else bound
        count, toff, eoff = oracle.route(world[sender].indices.numpy()[:n_eff], case.num_experts)
        np.testing.assert_array_equal(ctx.read_table(sender, native.TABLE_NUM_ROUTED, case.num_experts).numpy(), count)
        np.testing.assert_array_equal(ctx.read_table(sender, native.TABLE_EXPERT_OFFSETS, case.num_experts).numpy(), eoff)
        np.testing.assert_array_equal(ctx.read_table(sender, native.TABLE_TOKEN_OFFSET, n_eff * K).numpy(), toff)
        np.testing.assert_array_equal(ctx.read_table(sender, native.TABLE_SLOT, n_eff * K).numpy(),
                                      want[0].slots[sender][:n_eff].reshape(-1))
    finally:
        for op in ops:
            op.destroy()


@pytest.mark.parametrize("sender,bound,strided", [(0, None, False), (2, None, False), (3, 37, False), (1, 0, False),
                                                   (2, None, True), (1, 5, True)],
                         ids=["rank0", "rank2", "rank3_bound37", "rank1_bound0", "rank2_strided", "rank1_bound5_strided"])
def test_one_launch_dispatch_with_a_single_source(sender, bound, strided):
    """A small step in which ONE rank has tokens takes a variant of the one-launch dispatch that reads the
    entries as a flat array, provided the index rows are dense; with a row stride other than K the general
    variant runs.  Either way: any rank may be the sender, `bound_m` may shorten the step on the device, and
    the result is the oracle's, bit for bit."""
    _check_single_source(C1, sender, bound, strided)   # 128 tokens, 128 experts over 8 ranks, top-8


@pytest.mark.parametrize("tokens,sender,bound,topk,pad,experts,hidden,repeats", [
    (1, 0, None, 8, 1, 128, 2048, False), (3, 5, None, 8, 16, 128, 2048, True), (128, 2, 100, 5, 8, 250, 7168, False),
    (200, 7, None, 2, 1, 1024, 2048, True), (17, 1, 16, 8, 128, 64, 384, False), (64, 3, None, 1, 1, 8, 1024, False),
    (100, 4, None, 12, 1, 128, 2048, True)],
    ids=["1_token", "3_tokens_pad16_repeats", "128_top5_pad8_250_experts_bound100", "200_top2_1024_experts_repeats",
         "17_pad128_bound16", "64_top1_one_expert_a_rank", "100_top12_the_general_kernel"])
def test_quick_dispatch_of_a_small_single_source(tokens, sender, bound, topk, pad, experts, hidden, repeats):
    """A small quantising step of one source with at most eight routes per token takes a kernel in which a
    spare wavefront per token resolves the routes while the others quantise, and the first workgroups'
    spare wavefronts write the step's tables.  Fewer workgroups than tables to write, a token that names
    an expert twice, experts that do not divide among the ranks, more experts per rank than a pass of the
    route sums covers, a bound on the device, padded receive slots: the oracle's result, bit for bit.  (More
    than eight routes a token: the general one-launch kernel serves the step.)"""
    case = replace(scaled(C1, tokens), topk=topk, expert_padding=pad, num_experts=experts, hidden_dim=hidden,
                   name=f"quick_{tokens}")
    _check_single_source(case, sender, bound, False, repeats)


@pytest.mark.parametrize("tokens,sender,bound,topk,pad", [(700, 2, None, 8, 1), (1024, 0, None, 8, 16), (702, 5, 333, 8, 1),
                                                          (600, 1, 0, 8, 1), (640, 3, None, 5, 8), (1000, 7, 1, 3, 1), (600, 6, None, 12, 1)],
                         ids=["700", "1024_pad16", "702_bound333", "600_bound0", "640_top5_pad8", "1000_top3_bound1",
                              "600_top12_the_general_kernel"])
def test_one_launch_dispatch_of_a_larger_single_source(tokens, sender, bound, topk, pad):
    """Steps of one source that are too large for the one-launch dispatch of small steps (every token's
    workgroup counting every entry) and have at most 8192 entries take a launch whose workgroups count
    once for four tokens each.  Partial last workgroups, a bound inside a workgroup's four tokens, a bound
    of zero and one, odd top-k, padded receive slots: the oracle's result, bit for bit."""
    case = replace(scaled(C1, tokens), topk=topk, expert_padding=pad, name=f"single_{tokens}")
    _check_single_source(case, sender, bound, False)


@pytest.mark.parametrize("tokens,topk,hidden", [(900, 8, 7168), (500, 3, 2048), (1024, 8, 256)],
                         ids=["900_two_rounds", "500_top3_four_teams", "1024_small_rows"])
def test_larger_single_source_with_experts_named_twice(tokens, topk, hidden):
    """The same steps with tokens that name an expert twice: the second copy takes the next row of that
    expert, also when the two routes belong to different tokens of one workgroup's share."""
    case = replace(scaled(C1, tokens), topk=topk, hidden_dim=hidden, name=f"single_twice_{tokens}")
    _check_single_source(case, 3, None, False, repeats=True)

