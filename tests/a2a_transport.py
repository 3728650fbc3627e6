"""Harness for the transport mode (rows are copied as bytes, scales are the caller's), used to
replay the reference's own test matrix (tests/p2p_all_to_all/test_p2p_all_to_all.py:243-550)
with every rank on one GPU."""

from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional

import numpy as np
import torch

import a2a_oracle as oracle

SENTINEL = 0xA5
_NP_OUT = {torch.bfloat16: "bf16", torch.float16: "f16", torch.float32: "f32"}


@dataclass(frozen=True)
class RefConfig:
    """One row of the reference's parameter list; transport-only columns dropped."""
    name: str
    world_size: int
    dp_size: int
    max_num_tokens: int
    num_experts: int
    hidden_dim: int
    hidden_dim_scale: Optional[int]
    num_experts_per_token: int
    in_dtype: torch.dtype
    out_dtype: torch.dtype
    scale_dtype: Optional[torch.dtype]
    expert_padding: int = 1
    max_private_tokens: Optional[int] = None
    node_size: Optional[int] = None


@dataclass
class RefRank:
    dp_x: torch.Tensor
    dp_x_scale: Optional[torch.Tensor]
    indices: torch.Tensor      # int32 [T, K]
    weights: torch.Tensor


def make_ref_rank(cfg: RefConfig, rank: int, num_tokens: Optional[int] = None) -> RefRank:
    """Restates RankTestData.create (tests/p2p_all_to_all/data.py:55-108) with a CPU generator
    seeded by the rank (test_p2p_all_to_all.py:53-56)."""
    T = cfg.max_num_tokens if num_tokens is None else num_tokens
    g = torch.Generator(device="cpu")
    g.manual_seed(rank)
    scores = torch.randn((T, cfg.num_experts), generator=g).abs() + 1
    idx = torch.topk(scores, cfg.num_experts_per_token, dim=-1, largest=True, sorted=True).indices.to(torch.int32)
    x = torch.randn((T, cfg.hidden_dim), generator=g).to(cfg.in_dtype)
    xs = None
    if cfg.hidden_dim_scale is not None:
        xs = torch.randn((T, cfg.hidden_dim_scale), generator=g).to(cfg.scale_dtype)
    w = torch.rand((T, cfg.num_experts_per_token), generator=g)
    w = (w / w.sum(dim=-1, keepdim=True)).to(torch.float32)
    return RefRank(x, xs, idx, w)


def act(x: torch.Tensor, x_scale: Optional[torch.Tensor]) -> torch.Tensor:
    """The stand-in for the experts, block layout of the scales
    (benchmarks/bench_all_to_all.py:40-50; test_p2p_all_to_all.py:44-50 for the unscaled case)."""
    if x_scale is None:
        return x * 2
    b, h = x.shape
    hs = x_scale.shape[1]
    r = x.view(b, hs, h // hs).to(torch.float32) * x_scale.view(b, hs, 1) * 2
    return r.view(b, h)


def rows_for(cfg: RefConfig, world: List[RefRank]) -> int:
    Le = -(-cfg.num_experts // cfg.world_size)
    counts = np.zeros(cfg.num_experts, dtype=np.int64)
    for rd in world:
        counts += np.bincount(rd.indices.numpy().reshape(-1), minlength=cfg.num_experts)
    pad = cfg.expert_padding
    padded = (counts + pad - 1) // pad * pad
    return int(max(max(padded[r * Le:(r + 1) * Le].sum() for r in range(cfg.world_size)), 1))


def _bytes(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.uint8).numpy().reshape(t.shape[0], t.shape[1] * t.element_size())


def oracle_dispatch(cfg: RefConfig, world: List[RefRank], rows: int):
    inputs = [oracle.RankInput(x=_bytes(rd.dp_x), indices=rd.indices.numpy(),
                               x_scale=None if rd.dp_x_scale is None else rd.dp_x_scale.numpy())
              for rd in world]
    return oracle.dispatch_world(
        inputs, num_experts=cfg.num_experts, world_size=cfg.world_size,
        node_size=cfg.node_size or cfg.world_size, expert_padding=cfg.expert_padding, out_rows=rows,
        quantize=False, hidden_dim_scale=cfg.hidden_dim_scale or 0)


def oracle_combine(cfg: RefConfig, world: List[RefRank], expert_y: List[torch.Tensor], slots,
                   out_prev=None, bound_m=None):
    kind = _NP_OUT[expert_y[0].dtype]
    ys = [y.contiguous().view(torch.int16).numpy().view(np.uint16) if kind != "f32" else y.numpy() for y in expert_y]
    return oracle.combine_world(
        ys, [rd.indices.numpy() for rd in world], [rd.weights.numpy() for rd in world], slots,
        num_experts=cfg.num_experts, world_size=cfg.world_size, in_dtype=kind,
        out_dtype=_NP_OUT[cfg.out_dtype], out_prev=out_prev, bound_m=bound_m)


def make_ops(cfg: RefConfig, device: torch.device):
    from pplx_garden_amd.distributed.loopback import LoopbackWorld
    from pplx_garden_amd.kernels.p2p_all_to_all import P2PAllToAll

    lw = LoopbackWorld(cfg.world_size, node_size=cfg.node_size, device=device)
    return [
        P2PAllToAll(
            max_num_tokens=cfg.max_num_tokens, num_experts=cfg.num_experts, expert_padding=cfg.expert_padding,
            hidden_dim=cfg.hidden_dim, hidden_dim_scale=cfg.hidden_dim_scale, in_dtype=cfg.in_dtype,
            out_dtype=cfg.out_dtype, scale_dtype=cfg.scale_dtype,
            num_experts_per_token=cfg.num_experts_per_token, nets_per_gpu=1,
            max_private_tokens=cfg.max_private_tokens, device=device, dp_group=None, node_group=None,
            global_group=lw.group(r))
        for r in range(cfg.world_size)
    ]


def out_tokens_numpy(t: torch.Tensor) -> np.ndarray:
    t = t.cpu()
    return t.numpy() if t.dtype == torch.float32 else t.view(torch.int16).numpy().view(np.uint16)


def to_f32(a: np.ndarray, dtype: torch.dtype) -> np.ndarray:
    if dtype == torch.float32:
        return a
    return oracle.bf16_to_f32(a) if dtype == torch.bfloat16 else oracle.f16_to_f32(a)


def run_gpu(cfg: RefConfig, world: List[RefRank], rows: int, device: torch.device, split: bool,
            scale_layout: str = "row"):
    """dispatch -> act -> combine through the operator; returns per-rank dicts of numpy results.
    scale_layout "col": the output scale tensor is the transpose of a [Hs, rows] buffer (strided)."""
    N, H, Hs = cfg.world_size, cfg.hidden_dim, cfg.hidden_dim_scale
    Le = -(-cfg.num_experts // N)
    ops = make_ops(cfg, device)
    try:
        dev = [dict(x=rd.dp_x.to(device), xs=None if rd.dp_x_scale is None else rd.dp_x_scale.to(device),
                    idx=rd.indices.view(torch.uint32).to(device), w=rd.weights.to(device)) for rd in world]
        outs = []
        esize = cfg.in_dtype.itemsize
        for r in range(N):
            x = torch.full((rows, H * esize), SENTINEL, dtype=torch.uint8, device=device).view(cfg.in_dtype)
            s = None
            if Hs is not None:
                if scale_layout == "col":
                    s = torch.full((Hs, rows), -7.0, dtype=torch.float32, device=device).t()
                else:
                    s = torch.full((rows, Hs), -7.0, dtype=torch.float32, device=device)
            outs.append(dict(n=torch.full((Le,), -1, dtype=torch.int32, device=device), x=x, s=s,
                             o=torch.zeros((world[r].dp_x.shape[0], H), dtype=cfg.out_dtype, device=device)))

        def dispatch(r, **kw):
            ops[r].dispatch(out_expert_num_tokens=outs[r]["n"], out_expert_x=outs[r]["x"],
                            out_expert_x_scale=outs[r]["s"], dp_x=dev[r]["x"], dp_x_scale=dev[r]["xs"],
                            indices=dev[r]["idx"], weights=dev[r]["w"], bound_m=None, **kw)

        if split:
            for r in range(N):
                dispatch(r, do_send=True, do_recv=False)
            for r in range(N):
                dispatch(r, do_send=False, do_recv=True)
        else:
            for r in range(N):
                dispatch(r)
        torch.cuda.synchronize(device)
        assert ops[0].context.status() == 0

        ys = [act(outs[r]["x"], outs[r]["s"]).to(cfg.out_dtype) for r in range(N)]

        def combine(r, **kw):
            ops[r].combine(out_tokens=outs[r]["o"], indices=dev[r]["idx"], weights=dev[r]["w"],
                           expert_y=ys[r], bound_m=None, **kw)

        if split:
            for r in range(N):
                combine(r, do_send=True, do_recv=False)
            for r in range(N):
                combine(r, do_send=False, do_recv=True)
        else:
            for r in range(N):
                combine(r)
        torch.cuda.synchronize(device)
        assert ops[0].context.status() == 0
        return [dict(n=o["n"].cpu().numpy(), x=_bytes(o["x"].cpu()),
                     s=None if o["s"] is None else o["s"].cpu().numpy(), y=ys[r].cpu(),
                     o=out_tokens_numpy(o["o"])) for r, o in enumerate(outs)]
    finally:
        for op in ops:
            op.destroy()


def check(cfg: RefConfig, world: List[RefRank], rows: int, got) -> None:
    """The three checks of the reference's test (counts, rows inside the right expert's slot
    range, round trip), the first two strengthened to exact placement."""
    want = oracle_dispatch(cfg, world, rows)
    N = cfg.world_size
    Le = -(-cfg.num_experts // N)
    for r in range(N):
        n_local = max(min(Le, cfg.num_experts - r * Le), 0)
        np.testing.assert_array_equal(got[r]["n"][:n_local], want[r].num_tokens[:n_local])
        w = want[r].written
        np.testing.assert_array_equal(got[r]["x"][w], want[r].x[w])
        assert (got[r]["x"][~w] == SENTINEL).all()
        if cfg.hidden_dim_scale is not None:
            np.testing.assert_array_equal(got[r]["s"][w].view(np.uint32), want[r].x_scale[w].view(np.uint32))
            assert (got[r]["s"][~w] == -7.0).all()
    # combine against the oracle on the same expert outputs (zero the rows nobody wrote)
    ys = []
    for r in range(N):
        y = got[r]["y"].clone()
        y[torch.from_numpy(~want[r].written)] = 0
        ys.append(y)
    comb = oracle_combine(cfg, world, ys, want[0].slots)
    for g in range(N):
        a = to_f32(got[g]["o"], cfg.out_dtype)
        b = to_f32(comb[g], cfg.out_dtype)
        if b.size == 0:   # a rank without tokens gets none back
            assert a.size == 0
            continue
        tol = 1e-2 if cfg.out_dtype != torch.float32 else 1e-5
        np.testing.assert_allclose(a, b, rtol=tol, atol=tol * max(float(np.abs(b).max()), 1e-3) * 1e-2)
        # the reference's own round-trip check: combine(act(dispatch(x))) == act(x)
        ref = act(world[g].dp_x, world[g].dp_x_scale).to(cfg.out_dtype)
        torch.testing.assert_close(torch.from_numpy(a.copy()), ref.to(torch.float32), rtol=1.6e-2, atol=1e-2)
