#!/usr/bin/env python3
"""Benchmark of the MoE dispatch + combine path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one dispatch (routing pass + fp8 quantising pack) followed by one
combine (top-k weighted gather) over one batch of synthetic tokens, through the
C ABI of the library (`a2a_dispatch`, `a2a_combine`), with every tensor already
resident in HBM.  The workload is the DeepSeek-V3 prefill chunk of the baseline
(4096 tokens, hidden 7168, 256 experts over 8 logical ranks, top-8 with Zipf(1.2)
expert popularity): the GPU sends its 4096 tokens and holds the receive buffers
of all 8 logical ranks, which is one GPU's share of the group's work.  Routing
changes every step (a few pre-generated routings are cycled), as in the
reference's benchmark (benchmarks/bench_all_to_all.py:382-389).

Prints one JSON line.  `value` is algorithmic bytes per step over the wall time
of the timed region; per-phase times come from events recorded on the stream
the kernels run on, around about 25 steps of the same region (an event between
two launches idles the GPU for about 3 us, so they are kept sparse).  The 128-token decode shape is timed too and reported in
the same line.  The CPU baseline is the oracle's C restatement, single thread,
on the same workload.
"""

from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time
from dataclasses import replace
from pathlib import Path

REPO = Path(__file__).resolve().parent
for _p in (REPO / "pplx-garden_amd", REPO / "oracle", REPO / "tests"):
    if str(_p) not in sys.path:
        sys.path.insert(0, str(_p))

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published

# HBM bytes per launch on the default workload, from hardware counters (FETCH_SIZE and WRITE_SIZE
# passes, scaled by what the same counters read for a 512 MiB copy: x2.000 and x1.000).  The counter
# runs and their commands are summarised in profiles/hbm_traffic_dsv3_prefill_4096_pack_and_combine.md.
MEASURED_TRAFFIC_BYTES = {"combine_gather_kernel": 531_696_000, "dispatch_resolve_kernel": 303_561_000,
                          "dispatch_push_kernel": 303_073_000}


def algorithmic_bytes(T: int, H: int, K: int):
    """One-hop minimum per step: dispatch reads the bf16 row and the indices and
    writes K fp8 rows with their scales; combine reads K bf16 rows, the indices
    and the weights and writes one bf16 row."""
    dispatch = T * (2 * H + 4 * K + K * (H + 4 * (H // 128)))
    combine = T * (K * 2 * H + 8 * K + 2 * H)
    return dispatch, combine


class Workload:
    """Buffers of one case with the GPU as rank 0 of N logical ranks."""

    def __init__(self, case, device, num_routings: int, context_flags: int = 0):
        import torch
        from a2a_cases import make_rank
        from a2a_harness import rows_needed
        from pplx_garden_amd.native.p2p_all_to_all import (A2ACombineArgs, A2ADispatchArgs,
                                                           AllToAllContext)

        self.case = case
        self.device = device
        N, H, Hs, K = case.world_size, case.hidden_dim, case.hidden_dim_scale, case.topk
        Le, T = case.experts_per_rank, case.num_tokens
        self.ctx = AllToAllContext.create(
            hidden_dim=H, hidden_dim_scale=Hs, in_elemsize=1, out_elemsize=2,
            out_dtype=torch.bfloat16, scale_elemsize=4, max_num_tokens=T, max_recv_tokens=T * K,
            max_private_tokens=0, num_experts=case.num_experts, expert_padding=case.expert_padding,
            num_experts_per_token=K, dp_size=1, node_size=case.node_size or N, world_size=N,
            device=device.index or 0, flags=context_flags)
        self.routings = []
        rows = 1
        for i in range(num_routings):
            rd = make_rank(replace(case, seed=case.seed + 100 * i), 0)
            self.routings.append(rd)
            empty = [make_rank(case, r, 0) for r in range(1, N)]
            rows = max(rows, rows_needed(case, [rd] + empty))
        self.rows = rows
        self.cpu_first = self.routings[0]
        self.x = self.routings[0].x.to(device)
        self.idx = [rd.indices.to(device) for rd in self.routings]
        self.w = [rd.weights.to(device) for rd in self.routings]
        self.out_n = [torch.zeros(Le, dtype=torch.int32, device=device) for _ in range(N)]
        self.out_x = [torch.zeros((rows, H), dtype=torch.uint8, device=device) for _ in range(N)]
        self.out_s = [torch.zeros((rows, Hs), dtype=torch.float32, device=device) for _ in range(N)]
        gen = torch.Generator(device="cpu")
        gen.manual_seed(case.seed + 5)
        self.y = [torch.randn((rows, H), generator=gen).to(torch.bfloat16).to(device) for _ in range(N)]
        self.out_tokens = torch.zeros((T, H), dtype=torch.bfloat16, device=device)
        self.dispatch_args = []
        self.combine_args = []
        for i in range(num_routings):
            d, c = [], []
            for r in range(N):
                src = r == 0
                d.append(A2ADispatchArgs(
                    num_tokens=T if src else 0, x_ptr=self.x.data_ptr() if src else None, x_stride=2 * H,
                    x_scale_ptr=None, x_scale_stride_elem=0, x_scale_stride_token=0,
                    indices=self.idx[i].data_ptr() if src else None, indices_stride=K,
                    weights=self.w[i].data_ptr() if src else None, weights_stride=K, bound_m=None,
                    out_num_tokens=self.out_n[r].data_ptr(), out_x=self.out_x[r].data_ptr(),
                    out_x_stride=H, out_x_rows=rows, out_x_scale=self.out_s[r].data_ptr(),
                    out_x_scale_stride_elem=1, out_x_scale_stride_token=Hs))
                c.append(A2ACombineArgs(
                    expert_y=self.y[r].data_ptr(), expert_y_stride=2 * H, expert_y_rows=rows,
                    num_tokens=T if src else 0, out_tokens=self.out_tokens.data_ptr() if src else None,
                    out_tokens_stride=H, indices=self.idx[i].data_ptr() if src else None,
                    indices_stride=K, weights=self.w[i].data_ptr() if src else None, weights_stride=K,
                    bound_m=None))
            self.dispatch_args.append(self.ctx.pack_dispatch_args(d))
            self.combine_args.append(self.ctx.pack_combine_args(c))

    def step(self, i: int, stream: int, events=None, kernel_events=None):
        """One dispatch + combine.  `events` = (start, middle, end) recorded around the two calls;
        `kernel_events` = (pack start, pack stop, gather start, gather stop[, route start, route stop]),
        which the library records at the start and end of those kernels themselves (the last pair only
        in a step whose dispatch has a routing launch of its own)."""
        import torch
        j = i % len(self.routings)
        if kernel_events is not None:
            self.ctx.time_next_kernel(0, kernel_events[0].cuda_event, kernel_events[1].cuda_event)
            self.ctx.time_next_kernel(1, kernel_events[2].cuda_event, kernel_events[3].cuda_event)
            if len(kernel_events) >= 6:
                self.ctx.time_next_kernel(2, kernel_events[4].cuda_event, kernel_events[5].cuda_event)
        if events is not None:
            events[0].record()
        self.ctx.dispatch(self.dispatch_args[j], True, stream)
        if events is not None:
            events[1].record()
        self.ctx.combine(self.combine_args[j], torch.bfloat16, False, stream)
        if events is not None:
            events[2].record()

    def close(self):
        self.ctx.destroy()


def time_workload(wl: Workload, steps: int, warmup: int, kernel_every: int = 32, call_every: int = 0,
                  route_events: bool = False):
    """W untimed steps, then exactly K timed steps between two synchronisations.

    Events cost idle GPU time (measured on the 4096-token step: 146.8 us per step without events,
    152.5 us with one after each call; a launch that records its own start and end costs about 3 us
    more), so the timed region carries them sparsely.  Every `kernel_every`-th step has the library record
    events at the start and end of the pack and the gather kernel themselves: the kernels' own durations
    (with `route_events` also of the routing launch, where the step has one).  Every `call_every`-th
    step (0 = none), never one of those, carries three events around the two calls (before the dispatch,
    between dispatch and combine, after the combine).

    Returns wall seconds and, in microseconds per sampled step: dispatch call, combine call, both,
    pack kernel, gather kernel, routing kernel (empty without `route_events`, or when the dispatch
    counts its routing inside the pack)."""
    import torch
    stream = torch.cuda.current_stream(wl.device).cuda_stream
    kernel_steps = []
    if kernel_every > 0:
        kernel_steps = [i for i in range(steps) if i % kernel_every == kernel_every // 2]
        if not kernel_steps and steps > 0:      # a very short run still gets a sample
            kernel_steps = [steps // 2]
    call_steps = [i for i in range(steps) if call_every > 0 and i % call_every == 0 and i not in kernel_steps]
    call_ev = {i: [torch.cuda.Event(enable_timing=True) for _ in range(3)] for i in call_steps}
    kern_ev = {i: [torch.cuda.Event(enable_timing=True) for _ in range(6 if route_events else 4)]
               for i in kernel_steps}
    for evs in kern_ev.values():         # an event gets its handle when it is first recorded
        for ev in evs:
            ev.record()
    for i in range(warmup):
        wl.step(i, stream)
    torch.cuda.synchronize(wl.device)
    t0 = time.perf_counter()
    for i in range(steps):
        wl.step(warmup + i, stream, call_ev.get(i), kern_ev.get(i))
    torch.cuda.synchronize(wl.device)
    wall_s = time.perf_counter() - t0
    flags = wl.ctx.status(stream)
    if flags:
        raise RuntimeError(f"device error flags {flags}")
    us = lambda a, b: a.elapsed_time(b) * 1e3
    disp = [us(call_ev[i][0], call_ev[i][1]) for i in call_steps]
    comb = [us(call_ev[i][1], call_ev[i][2]) for i in call_steps]
    both = [us(call_ev[i][0], call_ev[i][2]) for i in call_steps]
    pack = [us(kern_ev[i][0], kern_ev[i][1]) for i in kernel_steps]
    gather = [us(kern_ev[i][2], kern_ev[i][3]) for i in kernel_steps]
    route = []
    if route_events:
        # a routing launch that ran in this step started shortly before the pack; events that no launch
        # recorded still hold the time of their first recording, long before
        route = [us(kern_ev[i][4], kern_ev[i][5]) for i in kernel_steps
                 if 0.0 <= us(kern_ev[i][4], kern_ev[i][0]) < 500.0]
    return wall_s, disp, comb, both, pack, gather, route


def cpu_baseline(case, rd, reps: int, threads: int = 1):
    """The oracle's C restatement on the same batch; best of `reps`.  Returns seconds per step and the
    seconds of its routing part (histogram, ranks, receiver layout: what the reference does on one host
    thread, a2a_worker.rs:526-703)."""
    import numpy as np
    from a2a_cases import bf16_codes
    from a2a_harness import rows_needed
    import c_oracle

    N = case.world_size
    from a2a_cases import make_rank
    world = [rd] + [make_rank(case, r, 0) for r in range(1, N)]
    rows = rows_needed(case, world)
    cw = c_oracle.CWorld(case.num_experts, N, case.node_size or N, case.expert_padding,
                         case.hidden_dim, case.topk, rows)
    rng = np.random.default_rng(case.seed)
    for r in range(N):
        cw.y[r][:] = rng.integers(0x3C00, 0x4000, size=cw.y[r].shape, dtype=np.uint16)
    idx = [w.indices.numpy() for w in world]
    xs = [bf16_codes(w.x) for w in world]
    ws = [w.weights.numpy() for w in world]
    best = route_best = None
    c_oracle.set_threads(threads)
    try:
        for _ in range(reps):
            t0 = time.perf_counter()
            cw.route_all(idx)
            t1 = time.perf_counter()
            cw.dispatch(xs)
            cw.combine(ws)
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
            route_best = t1 - t0 if route_best is None else min(route_best, t1 - t0)
    finally:
        c_oracle.set_threads(1)
    return best, route_best


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--routings", type=int, default=4, help="distinct routings cycled over the steps")
    ap.add_argument("--kernel-every", type=int, default=0,
                    help="every how many timed steps have the pack and the gather kernel record their own "
                         "start and end (0 = about 12 such steps, at least 16 apart)")
    ap.add_argument("--cpu-reps", type=int, default=3, help="repetitions of the CPU baseline (0 = skip)")
    ap.add_argument("--no-decode", action="store_true", help="skip the 128-token shape")
    ap.add_argument("--decode-only", action="store_true",
                    help="time only the 128-token shape (for a kernel trace of the decode step alone)")
    ap.add_argument("--separate-routing", action="store_true",
                    help="create the context with A2A_FLAG_SEPARATE_ROUTING (routing kernels, then the pack): "
                         "for comparisons with the default paths")
    ap.add_argument("--context-flags", type=int, default=None,
                    help="create the context with these A2A_FLAG_* bits (for comparisons between paths)")
    ap.add_argument("--probe-copy", action="store_true",
                    help="also run plain device-to-device copies of 512 MiB (torch's copy kernel): the "
                         "known-size kernel that hardware byte counters are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: every logical rank of the expert-parallel group lives in "
              "this GPU's HBM and nothing here uses a second GPU; run with --gpus 1", file=sys.stderr)
        return 2

    import torch
    from a2a_cases import C2, C3
    from pplx_garden_amd.utils.math import Statistics

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (the HIP library has no CPU fallback)", file=sys.stderr)
        return 3
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)

    if args.probe_copy:
        src = torch.empty(512 << 20, dtype=torch.uint8, device=device).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize(device)
        del src, dst

    ctx_flags = 2 if args.separate_routing else 0   # A2A_FLAG_SEPARATE_ROUTING
    if args.context_flags is not None:
        ctx_flags = args.context_flags
    if args.kernel_every <= 0:
        args.kernel_every = max(16, args.steps // 12)
    if args.decode_only:
        wl2 = Workload(C2, device, args.routings, ctx_flags)
        w2, _, _, _, p2, g2, _ = time_workload(wl2, args.steps, args.warmup, args.kernel_every)
        _, d2, c2, b2, _, _, _ = time_workload(wl2, max(args.steps, 200), 0, 0, call_every=1)
        wl2.close()
        print(json.dumps({"decode_128_only": {"step_us_wall": round(w2 / args.steps * 1e6, 2),
                                              "pack_kernel_us_mean": round(Statistics.create(p2).mean, 2),
                                              "gather_kernel_us_mean": round(Statistics.create(g2).mean, 2),
                                              "dispatch_us_p50": round(Statistics.create(d2).p50, 2),
                                              "combine_us_p50": round(Statistics.create(c2).p50, 2),
                                              "total_us_p50": round(Statistics.create(b2).p50, 2)}}))
        return 0

    case = C3
    wl = Workload(case, device, args.routings, ctx_flags)
    wall_s, _, _, _, pack, gather, _ = time_workload(wl, args.steps, args.warmup, args.kernel_every)
    # Phase statistics as the reference's benchmark reports them (events around each phase of EVERY
    # iteration, benchmarks/bench_all_to_all.py:391-433), outside the timed region above; every fourth
    # step times the routing launch by its own events instead.
    _, disp, comb, both, _, _, route = time_workload(wl, max(args.steps, 200), 0, 4, call_every=1,
                                                     route_events=True)
    rows = wl.rows
    cpu_rd = wl.cpu_first
    wl.close()

    d_bytes, c_bytes = algorithmic_bytes(case.num_tokens, case.hidden_dim, case.topk)
    ms_per_step = wall_s / args.steps * 1e3
    value = (d_bytes + c_bytes) / (ms_per_step * 1e-3) / 1e9
    p_stats, g_stats = Statistics.create(pack), Statistics.create(gather)

    def stats_dict(xs):
        return {k: round(v, 2) for k, v in Statistics.create(xs).as_dict().items()}

    def roof(bytes_, mean_us, kernel, note):
        achieved = bytes_ / (mean_us * 1e-6) / 1e9
        return {"kernel": kernel, "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                "traffic": MEASURED_TRAFFIC_BYTES.get(kernel), "bytes_per_launch": bytes_,
                "avg_us": round(mean_us, 2), "timing": note}

    note = ("events recorded by the launch itself at the start and end of this kernel (hipExtLaunchKernelGGL), "
            f"on {len(gather)} of the {args.steps} timed steps")
    combine_roof = roof(c_bytes, g_stats.mean, "combine_gather_kernel", note)
    dispatch_roof = roof(d_bytes, p_stats.mean,
                         "dispatch_push_kernel" if args.separate_routing else "dispatch_resolve_kernel", note)
    dominant, other = ((combine_roof, dispatch_roof) if g_stats.mean >= p_stats.mean
                       else (dispatch_roof, combine_roof))

    decode = None
    if not args.no_decode:
        wl2 = Workload(C2, device, args.routings, ctx_flags)
        steps2 = max(args.steps, 200)
        w2, _, _, _, p2, g2, _ = time_workload(wl2, steps2, args.warmup, args.kernel_every)
        _, d2, c2, b2, _, _, _ = time_workload(wl2, steps2, 0, 0, call_every=1)
        wl2.close()
        decode = {
            "workload": "DeepSeek-V3 decode: 128 tokens, hidden 7168, 256 experts / 8 logical ranks, top-8 uniform, 1% x50 outliers",
            "step_us_wall": round(w2 / steps2 * 1e6, 2),
            "pack_kernel_us_mean": round(Statistics.create(p2).mean, 2),
            "gather_kernel_us_mean": round(Statistics.create(g2).mean, 2),
            "dispatch_us_p50": round(Statistics.create(d2).p50, 2),
            "combine_us_p50": round(Statistics.create(c2).p50, 2),
            "total_us_p50": round(Statistics.create(b2).p50, 2),
            "total_us_mean": round(Statistics.create(b2).mean, 2),
            "note": "working set (26 MB) fits the 256 MB Infinity Cache and is not flushed between steps; "
                    "step_us_wall is wall time over the timed steps, the kernel figures come from events the "
                    "launches record themselves on a few of those steps, the p50 figures from a second pass "
                    "with events around the calls of every step (each event adds about 3 us)",
        }

    cpu = cpu_more = None
    if args.cpu_reps > 0:
        dt, route_dt = cpu_baseline(case, cpu_rd, args.cpu_reps)
        cpu = {
            "value": round((d_bytes + c_bytes) / dt / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "us_per_step": round(dt * 1e6, 1),
            "sample": f"the full {case.num_tokens}-token batch (routing pass, quantising dispatch, combine), "
                      f"best of {args.cpu_reps} runs of the oracle's C restatement, one thread of "
                      f"{os.cpu_count()} host cores",
        }
        cores = min(16, os.cpu_count() or 1)
        dt_all, _ = cpu_baseline(case, cpu_rd, args.cpu_reps, threads=cores)
        cpu_more = {
            "routing_only_us_one_thread": round(route_dt * 1e6, 1),
            "all_cores": {"value": round((d_bytes + c_bytes) / dt_all / 1e9, 3), "unit": "GB/s", "cores": cores,
                          "us_per_step": round(dt_all * 1e6, 1),
                          "note": "same code, tokens split over OpenMP threads; routing stays on one thread"},
        }

    line = {
        "metric": "dispatch+combine µs & HBM GB/s (% peak), DSv3 shape, 128 and 4096 tokens",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "DeepSeek-V3 prefill chunk: 4096 tokens, hidden 7168 bf16, 256 experts over 8 logical "
                        "ranks in one HBM, top-8 Zipf(1.2), fp8 e4m3 dispatch with float scale per 128, bf16 "
                        "combine with float accumulation",
            "tokens": case.num_tokens, "hidden_dim": case.hidden_dim, "num_experts": case.num_experts,
            "logical_ranks": case.world_size, "topk": case.topk, "receive_rows_per_rank": rows,
            "routings_cycled": args.routings,
        },
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
        "prefill_4096": {
            "step_us_wall": round(ms_per_step * 1e3, 2),
            "timed_steps_with_kernel_events": len(gather),
            "pack_kernel_us": {"p50": round(p_stats.p50, 2), "mean": round(p_stats.mean, 2)},
            "gather_kernel_us": {"p50": round(g_stats.p50, 2), "mean": round(g_stats.mean, 2)},
            "algorithmic_bytes": {"dispatch": d_bytes, "combine": c_bytes},
            "with_events_on_every_step": {
                "note": "a second pass outside the timed region, events around each phase of every iteration as "
                        "in the reference's benchmark (each event adds about 3 us); every fourth step has the "
                        "routing launch record its own start and end instead",
                "dispatch_us": stats_dict(disp),
                "combine_us": stats_dict(comb),
                "total_us": stats_dict(both),
                "route_kernel_us": ({"p50": round(Statistics.create(route).p50, 2),
                                     "mean": round(Statistics.create(route).mean, 2)} if route else None),
            },
        },
        "decode_128": decode,
        "roofline": dominant,
        "roofline_other": other,
        "cpu_baseline": cpu,
        "cpu_baseline_more": cpu_more,
    }
    print(json.dumps(line, ensure_ascii=False))
    return 0


if __name__ == "__main__":
    sys.exit(main())
