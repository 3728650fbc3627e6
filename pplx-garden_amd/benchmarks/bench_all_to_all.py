#!/usr/bin/env python3
"""All-to-all benchmark with the command line and the output of the reference's.

Mirrors `benchmarks/bench_all_to_all.py` of the reference: the same flags
(`:569-594`), the same loop (`:355-433`: fresh routing every iteration, a
"back-to-back" dispatch and combine, then the same step with send and recv
split and filler work between the halves), the same statistics and the same
JSON document (`:501-515`): `{"dispatch": {"both", "send", "recv"}, "combine":
{...}}`, every entry a `Statistics` of microseconds.

What differs: all `--world-size` ranks are logical ranks on ONE GPU.  By
default only rank 0 has tokens (`--sources one`): the GPU then does the work of
one rank of the group, which is what a rank of the reference times.
`--sources all` makes every logical rank send, i.e. the work of the whole group
on one GPU.  `--init-method`, `--node-rank`, `--nets-per-gpu` and
`--max-private-tokens` are accepted and have no effect; `--dp-size` must be 1.
`--quantize` feeds bf16 tokens and lets dispatch quantise them to fp8 (the
reference always transports rows quantised by the caller).
"""

from __future__ import annotations

import argparse
import json
import sys
import time
from dataclasses import asdict
from pathlib import Path
from typing import Optional

import torch

PKG_ROOT = Path(__file__).resolve().parent.parent
if str(PKG_ROOT) not in sys.path:
    sys.path.insert(0, str(PKG_ROOT))

from pplx_garden_amd.distributed.loopback import LoopbackWorld  # noqa: E402
from pplx_garden_amd.kernels.p2p_all_to_all import P2PAllToAll  # noqa: E402
from pplx_garden_amd.utils.math import Statistics, round_up  # noqa: E402

_DTYPES = {
    "float8_e4m3fn": torch.float8_e4m3fn, "fp8": torch.float8_e4m3fn, "bfloat16": torch.bfloat16,
    "bf16": torch.bfloat16, "float16": torch.float16, "fp16": torch.float16, "float32": torch.float32,
    "fp32": torch.float32,
}


def str_to_dtype(name: str) -> torch.dtype:
    key = name.replace("torch.", "").lower()
    if key not in _DTYPES:
        raise argparse.ArgumentTypeError(f"unknown dtype {name}")
    return _DTYPES[key]


def rand_topk_idx(num_tokens, num_experts, num_topk, generator, device):
    """K distinct experts per token (benchmarks/bench_all_to_all.py:22-37)."""
    scores = torch.randn((num_tokens, num_experts), dtype=torch.float32, device=device, generator=generator)
    scores = scores.abs() + 1
    return torch.topk(scores, num_topk, dim=-1, largest=True, sorted=True)[1].to(torch.int32).view(torch.uint32)


def act(x: torch.Tensor, x_scale: Optional[torch.Tensor]) -> torch.Tensor:
    """The stand-in for the experts (benchmarks/bench_all_to_all.py:40-50)."""
    if x_scale is None:
        return x * 2
    b, h = x.shape
    hs = x_scale.shape[1]
    return (x.view(b, hs, h // hs).to(torch.float32) * x_scale.view(b, hs, 1) * 2).view(b, h)


class Rank:
    """Buffers of one logical rank."""

    def __init__(self, args, op: P2PAllToAll, rank: int, num_tokens: int, rows: int, device, quantize: bool):
        self.op = op
        self.gen = torch.Generator(device=device)
        self.gen.manual_seed(rank + 123)                           # bench_all_to_all.py:53-56
        T, H, Hs, K = num_tokens, args.hidden_dim, args.hidden_dim_scale, args.num_experts_per_token
        self.T = T
        x = torch.randn((T, H), device=device, generator=self.gen)
        if quantize:
            self.dp_x, self.dp_x_scale = x.to(torch.bfloat16), None
        else:
            self.dp_x = x.to(args.in_dtype)
            self.dp_x_scale = None if Hs is None else torch.randn((T, Hs), device=device, generator=self.gen)
        w = torch.rand((T, K), dtype=torch.float32, device=device, generator=self.gen)
        self.weights = w / torch.sum(w, dim=-1, keepdim=True) if T else w
        self.indices = rand_topk_idx(T, args.num_experts, K, self.gen, device)
        self.expert_num_tokens = torch.empty((op.num_local_experts,), dtype=torch.int32, device=device)
        self.out_expert_x = torch.empty((rows, H), dtype=args.in_dtype, device=device)
        self.out_expert_x_scale = None if Hs is None else torch.empty((rows, Hs), dtype=torch.float32, device=device)
        self.expert_y = torch.zeros((rows, H), dtype=args.out_dtype, device=device)
        self.out_tokens = torch.empty((T, H), dtype=args.out_dtype, device=device)

    def new_routing(self, args, device):
        self.indices = rand_topk_idx(self.T, args.num_experts, args.num_experts_per_token, self.gen, device)

    def dispatch(self, do_send: bool, do_recv: bool):
        self.op.dispatch(out_expert_num_tokens=self.expert_num_tokens, out_expert_x=self.out_expert_x,
                         out_expert_x_scale=self.out_expert_x_scale, dp_x=self.dp_x, dp_x_scale=self.dp_x_scale,
                         indices=self.indices, weights=self.weights, bound_m=None, do_send=do_send, do_recv=do_recv)

    def combine(self, do_send: bool, do_recv: bool):
        self.op.combine(out_tokens=self.out_tokens, indices=self.indices, weights=self.weights,
                        expert_y=self.expert_y, bound_m=None, do_send=do_send, do_recv=do_recv)


def correctness_check(ranks, args, quantize: bool) -> None:
    """Counts, then combine(act(dispatch(x))) == act(x) (bench_all_to_all.py:188-266)."""
    for r in ranks:
        r.dispatch(True, True)
    torch.cuda.synchronize()
    counts = sum(torch.bincount(r.indices.view(torch.int32).flatten().long(), minlength=args.num_experts)
                 for r in ranks if r.T)
    Le = ranks[0].op.num_local_experts
    for i, r in enumerate(ranks):
        torch.testing.assert_close(r.expert_num_tokens.cpu().long(), counts[i * Le:(i + 1) * Le].cpu())
        n = int(r.expert_num_tokens.sum())
        r.expert_y[:n] = act(r.out_expert_x[:n], None if r.out_expert_x_scale is None
                             else r.out_expert_x_scale[:n]).to(args.out_dtype)
    for r in ranks:
        r.combine(True, True)
    torch.cuda.synchronize()
    for r in ranks:
        if not r.T:
            continue
        if quantize:
            ref = (r.dp_x.float() * 2).to(args.out_dtype)
            torch.testing.assert_close(r.out_tokens.float(), ref.float(), rtol=0.14, atol=0.14 * float(ref.abs().max()) / 8)
        else:
            ref = act(r.dp_x, r.dp_x_scale).to(args.out_dtype)
            torch.testing.assert_close(r.out_tokens, ref)


def main() -> None:
    parser = argparse.ArgumentParser(description="All-to-All Benchmark (one GPU, logical ranks)")
    parser.add_argument("--world-size", type=int, required=True)
    parser.add_argument("--init-method", type=str, default=None)
    parser.add_argument("--dp-size", type=int, default=1)
    parser.add_argument("--node-rank", type=int, default=0)
    parser.add_argument("--num-warmup", type=int, default=10000)
    parser.add_argument("--num-repeats", type=int, default=10000)
    parser.add_argument("--nets-per-gpu", type=int, default=2)
    parser.add_argument("--max-num-tokens", type=int, default=128)
    parser.add_argument("--max-private-tokens", type=int, default=256)
    parser.add_argument("--num-experts", type=int, default=256)
    parser.add_argument("--hidden-dim", type=int, default=7168)
    parser.add_argument("--hidden-dim-scale", type=int, default=56)
    parser.add_argument("--num-experts-per-token", type=int, default=8)
    parser.add_argument("--in-dtype", type=str_to_dtype, default=torch.float8_e4m3fn)
    parser.add_argument("--out-dtype", type=str_to_dtype, default=torch.bfloat16)
    parser.add_argument("--scale-dtype", type=str_to_dtype, default=torch.float32)
    parser.add_argument("--nvlink", type=int, default=None)
    parser.add_argument("--output", type=Path, default=Path("/dev/stdout"))
    parser.add_argument("--check", type=bool, default=True, action=argparse.BooleanOptionalAction)
    parser.add_argument("--sources", choices=("one", "all"), default="one")
    parser.add_argument("--quantize", action="store_true")
    args = parser.parse_args()
    if args.dp_size != 1:
        parser.error("--dp-size other than 1 is not supported")
    if args.hidden_dim_scale is not None and args.hidden_dim_scale <= 0:
        args.hidden_dim_scale = None

    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    N, K, T = args.world_size, args.num_experts_per_token, args.max_num_tokens
    world = LoopbackWorld(N, node_size=args.nvlink or N, device=device)
    ops = [P2PAllToAll(max_num_tokens=T, num_experts=args.num_experts, expert_padding=1, hidden_dim=args.hidden_dim,
                       hidden_dim_scale=args.hidden_dim_scale, in_dtype=args.in_dtype, out_dtype=args.out_dtype,
                       scale_dtype=args.scale_dtype if args.hidden_dim_scale else None, num_experts_per_token=K,
                       nets_per_gpu=args.nets_per_gpu, max_private_tokens=args.max_private_tokens, device=device,
                       dp_group=None, node_group=None, global_group=world.group(r)) for r in range(N)]
    senders = N if args.sources == "all" else 1
    Le = ops[0].num_local_experts
    rows = round_up(max(min(senders * T * K, senders * T * Le), Le), 1)     # bench_all_to_all.py:107-118
    ranks = [Rank(args, ops[r], r, T if r < senders else 0, rows, device, args.quantize) for r in range(N)]

    try:
        if args.check:
            correctness_check(ranks, args, args.quantize)
        gemm = torch.empty((2048, 2048) if T <= 128 else (8192, 8192), dtype=torch.float32, device=device)

        def wait() -> None:       # the delay of other layers (bench_all_to_all.py:281-285, without the all-reduce)
            _ = gemm @ gemm

        def every_rank(fn, *a):
            for r in ranks:
                fn(r, *a)

        total = args.num_warmup + args.num_repeats
        events = [[torch.cuda.Event(enable_timing=True) for _ in range(12)] for _ in range(total)]
        last_report = time.time()
        for i in range(total):
            if time.time() - last_report > 1 or i + 1 == total:
                print(f"Iteration {i + 1}/{total}", file=sys.stderr)
                last_report = time.time()
            ev = events[i]
            for r in ranks:
                r.new_routing(args, device)
            wait()
            ev[0].record(); every_rank(Rank.dispatch, True, True); ev[1].record()
            wait()
            ev[2].record(); every_rank(Rank.combine, True, True); ev[3].record()
            wait()
            ev[4].record(); every_rank(Rank.dispatch, True, False); ev[5].record()
            wait()
            ev[6].record(); every_rank(Rank.dispatch, False, True); ev[7].record()
            wait()
            ev[8].record(); every_rank(Rank.combine, True, False); ev[9].record()
            wait()
            ev[10].record(); every_rank(Rank.combine, False, True); ev[11].record()
        torch.cuda.synchronize()
        assert ops[0].context.status() == 0

        def series(a: int) -> Statistics:
            return Statistics.create([e[a].elapsed_time(e[a + 1]) * 1000 for e in events[args.num_warmup:]])

        stats = {"dispatch": {"both": series(0), "send": series(4), "recv": series(6)},
                 "combine": {"both": series(2), "send": series(8), "recv": series(10)}}
        itemsize = torch.float8_e4m3fn.itemsize if args.quantize else args.in_dtype.itemsize
        token_bytes = args.hidden_dim * itemsize + (args.hidden_dim_scale or 0) * 4
        dispatch_bytes = senders * T * K * token_bytes                      # bench_all_to_all.py:73-84
        combine_bytes = senders * T * K * args.hidden_dim * args.out_dtype.itemsize
        print(f"Dispatch both time: {stats['dispatch']['both']}, "
              f"{dispatch_bytes / stats['dispatch']['both'].p50 * 1e-3:.1f} GB/s", file=sys.stderr)
        print(f"Combine both time: {stats['combine']['both']}, "
              f"{combine_bytes / stats['combine']['both'].p50 * 1e-3:.1f} GB/s", file=sys.stderr)
        data = {phase: {k: asdict(v) for k, v in d.items()} for phase, d in stats.items()}
        with args.output.open("w") as f:
            f.write(json.dumps(data))
            f.write("\n")
    finally:
        for op in ops:
            op.destroy()


if __name__ == "__main__":
    main()
