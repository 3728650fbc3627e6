"""Run a workload through the HIP library (via the operator) and through the oracle."""

from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence

import numpy as np
import torch

import a2a_oracle as oracle
from a2a_cases import Case, RankData, bf16_codes, rows_needed  # noqa: F401

SENTINEL = 0xA5


@dataclass
class WorldResult:
    num_tokens: List[np.ndarray]      # per rank [Le] int32
    x: List[np.ndarray]               # per rank [rows, H] uint8 (fp8 codes)
    x_scale: List[np.ndarray]         # per rank [rows, Hs] float32
    out_tokens: List[np.ndarray]      # per rank [T, H] bf16 codes (uint16)


def act_numpy(q: np.ndarray, scale: np.ndarray) -> np.ndarray:
    """The 'expert' of the reference's test: 2 * dequantised row, as bf16 codes
    (tests/p2p_all_to_all/test_p2p_all_to_all.py:44-50 with the block layout of
    benchmarks/bench_all_to_all.py:40-50)."""
    deq = oracle.dequantize_block128(q, scale)
    deq = np.nan_to_num(deq, nan=0.0)
    return oracle.f32_to_bf16((deq * np.float32(2.0)).astype(np.float32))


def run_oracle(case: Case, world: Sequence[RankData], rows: int) -> WorldResult:
    inputs = [oracle.RankInput(x=bf16_codes(rd.x), indices=rd.indices.numpy()) for rd in world]
    outs = oracle.dispatch_world(
        inputs, num_experts=case.num_experts, world_size=case.world_size,
        node_size=case.node_size or case.world_size, expert_padding=case.expert_padding,
        out_rows=rows, quantize=True)
    slots = outs[0].slots
    ys = []
    for o in outs:
        y = act_numpy(o.x, o.x_scale)
        y[~o.written] = 0
        ys.append(y)
    comb = oracle.combine_world(
        ys, [rd.indices.numpy() for rd in world], [rd.weights.numpy() for rd in world], slots,
        num_experts=case.num_experts, world_size=case.world_size)
    res = WorldResult([o.num_tokens for o in outs], [o.x for o in outs], [o.x_scale for o in outs], comb)
    res.written = [o.written for o in outs]
    res.slots = slots
    res.expert_y = ys
    return res


def make_ops(case: Case, device: torch.device, max_num_tokens: Optional[int] = None, context_flags: int = 0,
             max_private_tokens: Optional[int] = None):
    from pplx_garden_amd.distributed.loopback import LoopbackWorld
    from pplx_garden_amd.kernels.p2p_all_to_all import P2PAllToAll

    world = LoopbackWorld(case.world_size, node_size=case.node_size, device=device, context_flags=context_flags)
    ops = [
        P2PAllToAll(
            max_num_tokens=max_num_tokens or max(case.num_tokens, 1), num_experts=case.num_experts,
            expert_padding=case.expert_padding, hidden_dim=case.hidden_dim,
            hidden_dim_scale=case.hidden_dim_scale, in_dtype=torch.float8_e4m3fn,
            out_dtype=torch.bfloat16, scale_dtype=torch.float32,
            num_experts_per_token=case.topk, nets_per_gpu=1, max_private_tokens=max_private_tokens, device=device,
            dp_group=None, node_group=None, global_group=world.group(r))
        for r in range(case.world_size)
    ]
    return world, ops


def run_gpu(case: Case, world_data: Sequence[RankData], rows: int, device: torch.device,
            split: bool = False, expert_y_override=None, context_flags: int = 0, ops=None) -> WorldResult:
    """dispatch -> 2*dequant -> combine on the GPU through the operator API.

    split=False: every rank calls dispatch()/combine() with do_send and do_recv
    (the group calls of the library); split=True: all sends, then all recvs (the
    four split calls).  With `ops` the given operators are used (and kept): several
    steps on one context."""
    N, H, Hs, Le = case.world_size, case.hidden_dim, case.hidden_dim_scale, case.experts_per_rank
    own_ops = ops is None
    if own_ops:
        _, ops = make_ops(case, device, context_flags=context_flags)
    try:
        dev = [
            dict(x=rd.x.to(device), idx=rd.indices_u32.to(device), w=rd.weights.to(device))
            for rd in world_data
        ]
        outs = []
        for r in range(N):
            outs.append(dict(
                n=torch.full((Le,), -1, dtype=torch.int32, device=device),
                x=torch.full((rows, H), SENTINEL, dtype=torch.uint8, device=device).view(torch.float8_e4m3fn),
                s=torch.full((rows, Hs), -7.0, dtype=torch.float32, device=device),
                o=torch.zeros((world_data[r].x.shape[0], H), dtype=torch.bfloat16, device=device)))

        def dispatch(r, **kw):
            ops[r].dispatch(out_expert_num_tokens=outs[r]["n"], out_expert_x=outs[r]["x"],
                            out_expert_x_scale=outs[r]["s"], dp_x=dev[r]["x"], dp_x_scale=None,
                            indices=dev[r]["idx"], weights=dev[r]["w"], **kw)

        if split:
            for r in range(N):
                dispatch(r, do_send=True, do_recv=False)
            for r in range(N):
                dispatch(r, do_send=False, do_recv=True)
        else:
            for r in range(N):
                dispatch(r)
        torch.cuda.synchronize(device)
        flags = ops[0].context.status()
        assert flags == 0, f"device error flags {flags}"

        ys = []
        for r in range(N):
            q = outs[r]["x"].view(torch.uint8).cpu().numpy()
            s = outs[r]["s"].cpu().numpy()
            if expert_y_override is not None:
                y = expert_y_override[r]
            else:
                y = act_numpy(q, s)
            ys.append(torch.from_numpy(y.view(np.int16)).view(torch.bfloat16).to(device))

        def combine(r, **kw):
            ops[r].combine(out_tokens=outs[r]["o"], indices=dev[r]["idx"], weights=dev[r]["w"],
                           expert_y=ys[r], **kw)

        if split:
            for r in range(N):
                combine(r, do_send=True, do_recv=False)
            for r in range(N):
                combine(r, do_send=False, do_recv=True)
        else:
            for r in range(N):
                combine(r)
        torch.cuda.synchronize(device)
        flags = ops[0].context.status()
        assert flags == 0, f"device error flags {flags}"

        res = WorldResult(
            [o["n"].cpu().numpy() for o in outs],
            [o["x"].view(torch.uint8).cpu().numpy() for o in outs],
            [o["s"].cpu().numpy() for o in outs],
            [o["o"].view(torch.int16).cpu().numpy().view(np.uint16) for o in outs])
        return res
    finally:
        if own_ops:
            for op in ops:
                op.destroy()


def assert_dispatch_equal(case: Case, got: WorldResult, want: WorldResult) -> None:
    """Bit-exact: counts, fp8 bytes and scales of written rows; untouched rows keep the sentinel."""
    for r in range(case.world_size):
        n_local = max(min(case.experts_per_rank, case.num_experts - r * case.experts_per_rank), 0)
        np.testing.assert_array_equal(got.num_tokens[r][:n_local], want.num_tokens[r][:n_local],
                                      err_msg=f"rank {r} counts")
        w = want.written[r]
        np.testing.assert_array_equal(got.x[r][w], want.x[r][w], err_msg=f"rank {r} fp8 bytes")
        np.testing.assert_array_equal(got.x_scale[r][w].view(np.uint32), want.x_scale[r][w].view(np.uint32),
                                      err_msg=f"rank {r} scales")
        assert (got.x[r][~w] == SENTINEL).all(), f"rank {r}: a padding row was written"
        assert (got.x_scale[r][~w] == -7.0).all(), f"rank {r}: a padding scale row was written"


def assert_combine_close(case: Case, got: WorldResult, want: WorldResult, rtol: float = 1e-2) -> None:
    """Within 1e-2 relative (bf16), the tolerance the baseline states; in practice bit-exact
    up to float64-emulated fused multiply-add corner cases."""
    for r in range(case.world_size):
        g = oracle.bf16_to_f32(got.out_tokens[r])
        w = oracle.bf16_to_f32(want.out_tokens[r])
        assert g.shape == w.shape
        if g.size == 0:
            continue
        np.testing.assert_allclose(g, w, rtol=rtol, atol=1e-2 * max(float(np.abs(w).max()), 1e-6) * 1e-2,
                                   err_msg=f"rank {r} combine")
