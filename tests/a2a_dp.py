"""Harness for groups of ranks that hold the same tokens (dp_size > 1), transport mode."""

from __future__ import annotations

from typing import List

import numpy as np
import torch

import a2a_oracle as oracle
from a2a_transport import SENTINEL, RefConfig, RefRank, _bytes, _NP_OUT, act, out_tokens_numpy, to_f32


def rows_for_dp(cfg: RefConfig, groups: List[RefRank]) -> int:
    Le = -(-cfg.num_experts // cfg.world_size)
    counts = np.zeros(cfg.num_experts, dtype=np.int64)
    for rd in groups:
        counts += np.bincount(rd.indices.numpy().reshape(-1), minlength=cfg.num_experts)
    pad = cfg.expert_padding
    padded = (counts + pad - 1) // pad * pad
    return int(max(max(padded[r * Le:(r + 1) * Le].sum() for r in range(cfg.world_size)), 1))


def run_gpu_dp(cfg: RefConfig, groups: List[RefRank], device: torch.device, split: bool):
    from pplx_garden_amd.distributed.loopback import LoopbackWorld
    from pplx_garden_amd.kernels.p2p_all_to_all import P2PAllToAll

    N, D, H = cfg.world_size, cfg.dp_size, cfg.hidden_dim
    Le = -(-cfg.num_experts // N)
    rows = rows_for_dp(cfg, groups)
    lw = LoopbackWorld(N, node_size=cfg.node_size, device=device)
    ops = [P2PAllToAll(
        max_num_tokens=cfg.max_num_tokens, num_experts=cfg.num_experts, expert_padding=cfg.expert_padding,
        hidden_dim=H, hidden_dim_scale=cfg.hidden_dim_scale, in_dtype=cfg.in_dtype, out_dtype=cfg.out_dtype,
        scale_dtype=cfg.scale_dtype, num_experts_per_token=cfg.num_experts_per_token, nets_per_gpu=1,
        max_private_tokens=cfg.max_private_tokens, device=device, dp_group=lw.dp_group(r, D), node_group=None,
        global_group=lw.group(r)) for r in range(N)]
    try:
        # every rank of a group holds its own copy of the group's tensors
        dev = []
        for r in range(N):
            rd = groups[r // D]
            dev.append(dict(x=rd.dp_x.clone().to(device), idx=rd.indices.clone().view(torch.uint32).to(device),
                            w=rd.weights.clone().to(device),
                            xs=None if rd.dp_x_scale is None else rd.dp_x_scale.clone().to(device)))
        esize = cfg.in_dtype.itemsize
        outs = [dict(n=torch.full((Le,), -1, dtype=torch.int32, device=device),
                     x=torch.full((rows, H * esize), SENTINEL, dtype=torch.uint8, device=device).view(cfg.in_dtype),
                     s=None if cfg.hidden_dim_scale is None else torch.full((rows, cfg.hidden_dim_scale), -7.0, dtype=torch.float32, device=device),
                     o=torch.zeros((groups[r // D].dp_x.shape[0], H), dtype=cfg.out_dtype, device=device))
                for r in range(N)]
        phases = [dict(do_send=True, do_recv=False), dict(do_send=False, do_recv=True)] if split else [dict()]
        for ph in phases:
            for r in range(N):
                ops[r].dispatch(out_expert_num_tokens=outs[r]["n"], out_expert_x=outs[r]["x"],
                                out_expert_x_scale=outs[r]["s"], dp_x=dev[r]["x"], dp_x_scale=dev[r]["xs"],
                                indices=dev[r]["idx"], weights=dev[r]["w"], **ph)
        torch.cuda.synchronize(device)
        assert ops[0].context.status() == 0
        ys = [act(outs[r]["x"], outs[r]["s"]).to(cfg.out_dtype) for r in range(N)]
        for ph in phases:
            for r in range(N):
                ops[r].combine(out_tokens=outs[r]["o"], indices=dev[r]["idx"], weights=dev[r]["w"],
                               expert_y=ys[r], **ph)
        torch.cuda.synchronize(device)
        assert ops[0].context.status() == 0
        got = [dict(n=o["n"].cpu().numpy(), x=_bytes(o["x"].cpu()), s=None if o["s"] is None else o["s"].cpu().numpy(),
                    y=ys[r].cpu(), o=out_tokens_numpy(o["o"])) for r, o in enumerate(outs)]
        return got, rows
    finally:
        for op in ops:
            op.destroy()


def check_dp(cfg: RefConfig, groups: List[RefRank], rows: int, got) -> None:
    N, D = cfg.world_size, cfg.dp_size
    Le = -(-cfg.num_experts // N)
    want, (slot_rank, slot_row) = oracle.world_by_rows(
        [rd.indices.numpy() for rd in groups], [_bytes(rd.dp_x) for rd in groups],
        [None if rd.dp_x_scale is None else rd.dp_x_scale.numpy() for rd in groups],
        num_experts=cfg.num_experts, world_size=N, node_size=cfg.node_size or N, dp_size=D,
        expert_padding=cfg.expert_padding, out_rows=rows)
    for r in range(N):
        n_local = max(min(Le, cfg.num_experts - r * Le), 0)
        np.testing.assert_array_equal(got[r]["n"][:n_local], want[r].num_tokens[:n_local])
        w = want[r].written
        np.testing.assert_array_equal(got[r]["x"][w], want[r].x[w])
        assert (got[r]["x"][~w] == SENTINEL).all()
        if cfg.hidden_dim_scale is not None:
            np.testing.assert_array_equal(got[r]["s"][w], want[r].x_scale[w])
    kind = _NP_OUT[cfg.out_dtype]
    for r in range(N):
        g = r // D
        rd = groups[g]
        T, K = rd.indices.shape
        acc = np.zeros((T, cfg.hidden_dim), dtype=np.float64)
        for k in range(K):
            for t in range(T):
                y = got[int(slot_rank[g][t, k])]["y"][int(slot_row[g][t, k])].to(torch.float32).numpy()
                acc[t] += float(rd.weights[t, k]) * y.astype(np.float64)
        out = to_f32(got[r]["o"], cfg.out_dtype)
        tol = 1e-2 if kind != "f32" else 1e-5
        np.testing.assert_allclose(out, acc, rtol=tol, atol=tol)
        # the reference's round trip: every rank of the group gets act(x) back
        ref = act(rd.dp_x, rd.dp_x_scale).to(cfg.out_dtype).to(torch.float32)
        torch.testing.assert_close(torch.from_numpy(out.copy()), ref, rtol=1.6e-2, atol=1e-2)
