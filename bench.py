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

Prints one JSON line.  Order of the run:
 1. a pass of at least 200 steps that carries events, as the reference's benchmark does
    (around each phase of every step); every fourth step instead has the pack, the gather and
    the routing launch record events at their own start and end: those are the kernels' own
    durations, the samples behind `roofline`;
 2. the timed region: W warm-up steps, then exactly K steps between two synchronisations with
    no event in between; `value` is algorithmic bytes per step over that wall time;
 3. the same K steps as replays of a captured HIP graph (reported beside it);
 4. the other shapes of the baseline (128-token decode at both hidden sizes, the 1024-token
    mixed batch) and the CPU baselines.
"""

from __future__ import annotations

import argparse
import hashlib
import json
import os
import re
import sys
import time
from dataclasses import replace
from pathlib import Path

REPO = Path(__file__).resolve().parent
for _p in (REPO / "pplx-garden_amd", REPO / "pplx-garden_amd" / "benchmarks"):
    if str(_p) not in sys.path:
        sys.path.insert(0, str(_p))

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
TRAFFIC_PROFILE = REPO / "profiles" / "hbm_traffic_pack_and_combine_dsv3_prefill_4096_and_kimi_1024.md"


def algorithmic_bytes(T: int, H: int, K: int):
    """One-hop minimum per step: dispatch reads the bf16 row and the indices and
    writes K fp8 rows with their scales; combine reads K bf16 rows, the indices
    and the weights and writes one bf16 row."""
    dispatch = T * (2 * H + 4 * K + K * (H + 4 * (H // 128)))
    combine = T * (K * 2 * H + 8 * K + 2 * H)
    return dispatch, combine


def code_only(text: str) -> str:
    """C++ source without its comments and blank lines, lines stripped: what the compiler sees, more or
    less, so that rewording a comment does not make a counter summary look stale.  (No string literal
    in these sources holds a comment marker.)"""
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    return "\n".join(line.strip() for line in text.splitlines() if line.strip())


def kernel_sources_sha256() -> str:
    """Fingerprint of the kernel sources this run uses: sha256 over the names and the code (comments
    and blank lines left out) of pplx-garden_amd/csrc/*, sorted by name."""
    h = hashlib.sha256()
    for path in sorted((REPO / "pplx-garden_amd" / "csrc").iterdir()):
        if path.is_file():
            h.update(path.name.encode() + b"\0" + code_only(path.read_text()).encode() + b"\0")
    return h.hexdigest()


def measured_traffic():
    """HBM bytes per launch from the hardware-counter summary under profiles/, or {} when that
    summary was taken on other kernel sources than the ones this run uses (then it says nothing
    about this build)."""
    try:
        text = TRAFFIC_PROFILE.read_text()
    except OSError:
        return {}, "no counter summary under profiles/"
    sha = re.search(r"^csrc_sha256:\s*([0-9a-f]{64})\s*$", text, flags=re.M)
    if sha is None or sha.group(1) != kernel_sources_sha256():
        return {}, "the counter summary under profiles/ was taken on other kernel sources"
    out = {m.group(1): int(m.group(2)) for m in re.finditer(r"^traffic_bytes:\s*(\w+)\s*=\s*(\d+)\s*$", text, flags=re.M)}
    # the other shapes of the baseline: lines "traffic_bytes_<shape>: <kernel>=<bytes>"
    for m in re.finditer(r"^traffic_bytes_(\w+):\s*(\w+)\s*=\s*(\d+)\s*$", text, flags=re.M):
        out.setdefault(m.group(1), {})[m.group(2)] = int(m.group(3))
    return out, f"FETCH_SIZE and WRITE_SIZE passes of this build, profiles/{TRAFFIC_PROFILE.name}"


class Workload:
    """Buffers of one case with the GPU as rank 0 of N logical ranks (`senders` "one": one GPU's share
    of the group's work), or with every logical rank sending its own batch (`senders` "all": the work
    of the whole group on this GPU)."""

    def __init__(self, case, device, num_routings: int, context_flags: int = 0, senders: str = "one"):
        import torch
        from workloads import make_rank, rows_needed
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
        self.senders = list(range(N)) if senders == "all" else [0]
        self.routings = []                 # [routing][sender]
        rows = 1
        for i in range(num_routings):
            sent = [make_rank(replace(case, seed=case.seed + 100 * i), r, T if r in self.senders else 0)
                    for r in range(N)]
            self.routings.append([sent[r] for r in self.senders])
            rows = max(rows, rows_needed(case, sent))
        self.rows = rows
        self.cpu_first = self.routings[0][0]
        self.x = [rd.x.to(device) for rd in self.routings[0]]                       # [sender]
        self.idx = [[rd.indices.to(device) for rd in routing] for routing in self.routings]
        self.w = [[rd.weights.to(device) for rd in routing] for routing in self.routings]
        self.out_n = [torch.zeros(Le, dtype=torch.int32, device=device) for _ in range(N)]
        self.out_x = [torch.zeros((rows, H), dtype=torch.uint8, device=device) for _ in range(N)]
        self.out_s = [torch.zeros((rows, Hs), dtype=torch.float32, device=device) for _ in range(N)]
        if senders == "all":               # N times the rows: drawn on the device
            gen = torch.Generator(device=device)
            gen.manual_seed(case.seed + 5)
            self.y = [torch.randn((rows, H), generator=gen, device=device, dtype=torch.float32).to(torch.bfloat16)
                      for _ in range(N)]
        else:
            gen = torch.Generator(device="cpu")
            gen.manual_seed(case.seed + 5)
            self.y = [torch.randn((rows, H), generator=gen).to(torch.bfloat16).to(device) for _ in range(N)]
        self.out_tokens = [torch.zeros((T, H), dtype=torch.bfloat16, device=device) for _ in self.senders]
        self.dispatch_args = []
        self.combine_args = []
        for i in range(num_routings):
            d, c = [], []
            for r in range(N):
                src = r in self.senders
                j = self.senders.index(r) if src else 0
                d.append(A2ADispatchArgs(
                    num_tokens=T if src else 0, x_ptr=self.x[j].data_ptr() if src else None, x_stride=2 * H,
                    x_scale_ptr=None, x_scale_stride_elem=0, x_scale_stride_token=0,
                    indices=self.idx[i][j].data_ptr() if src else None, indices_stride=K,
                    weights=self.w[i][j].data_ptr() if src else None, weights_stride=K, bound_m=None,
                    out_num_tokens=self.out_n[r].data_ptr(), out_x=self.out_x[r].data_ptr(),
                    out_x_stride=H, out_x_rows=rows, out_x_scale=self.out_s[r].data_ptr(),
                    out_x_scale_stride_elem=1, out_x_scale_stride_token=Hs))
                c.append(A2ACombineArgs(
                    expert_y=self.y[r].data_ptr(), expert_y_stride=2 * H, expert_y_rows=rows,
                    num_tokens=T if src else 0, out_tokens=self.out_tokens[j].data_ptr() if src else None,
                    out_tokens_stride=H, indices=self.idx[i][j].data_ptr() if src else None,
                    indices_stride=K, weights=self.w[i][j].data_ptr() if src else None, weights_stride=K,
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


def time_workload(wl: Workload, steps: int, warmup: int, kernel_every: int = 0, call_every: int = 0,
                  route_events: bool = False):
    """W untimed steps, then exactly K timed steps between two synchronisations.

    Events cost idle GPU time (measured on the 4096-token step: 146.8 us per step without events,
    152.5 us with one after each call; a launch that records its own start and end costs about 3 us
    more), so the timed region of the headline carries none (`kernel_every` = `call_every` = 0).
    With `kernel_every` > 0 every such step has the library record events at the start and end of
    the pack and the gather kernel themselves: the kernels' own durations (with `route_events` also
    of the routing launch, where the step has one).  Every `call_every`-th step (0 = none), never
    one of those, carries three events around the two calls (before the dispatch, between dispatch
    and combine, after the combine).

    Returns wall seconds and, in microseconds per sampled step: dispatch call, combine call, both,
    pack kernel, gather kernel, routing kernel (empty without `route_events`, or when the dispatch
    counts its routing inside the pack)."""
    import torch
    stream = torch.cuda.current_stream(wl.device).cuda_stream
    kernel_steps = []
    if kernel_every > 0:
        kernel_steps = [i for i in range(steps) if i % kernel_every == kernel_every // 2]
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


def time_graph_replay(wl: Workload, steps: int, warmup: int):
    """The same steps as replays of ONE captured HIP graph that holds a step per routing (the calls
    only enqueue kernels whose arguments travel by value, so they can be recorded; graph capture
    is a stated feature of the reference, docs/fabric-lib.md:15).  Returns wall seconds per step."""
    import torch
    n = len(wl.routings)
    side = torch.cuda.Stream(device=wl.device)
    side.wait_stream(torch.cuda.current_stream(wl.device))
    with torch.cuda.stream(side):
        for i in range(n):
            wl.step(i, side.cuda_stream)
    torch.cuda.current_stream(wl.device).wait_stream(side)
    torch.cuda.synchronize(wl.device)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        stream = torch.cuda.current_stream(wl.device).cuda_stream
        for i in range(n):
            wl.step(i, stream)
    replays = max(1, -(-steps // n))
    for _ in range(max(1, -(-warmup // n))):
        graph.replay()
    torch.cuda.synchronize(wl.device)
    t0 = time.perf_counter()
    for _ in range(replays):
        graph.replay()
    torch.cuda.synchronize(wl.device)
    wall_s = time.perf_counter() - t0
    flags = wl.ctx.status(torch.cuda.current_stream(wl.device).cuda_stream)
    if flags:
        raise RuntimeError(f"device error flags {flags}")
    del graph
    return wall_s / (replays * n), replays * n


def time_gpu_pace(wl: Workload, batches: int = 5, steps_each: int = 100, step_fn=None):
    """The GPU's own pace per step: `steps_each` steps are enqueued behind a kernel that holds the queue
    for a few milliseconds, so the host is ahead of the GPU for all of them, and two events around them
    give the time the GPU took.  For steps of about 10 us the host's share of a step (two calls through
    ctypes and the launches behind them, 7 to 10 us on this pool's hosts) is of the same size as the
    GPU's, and the wall time of a loop then says which host the box has.  Returns the median over
    `batches` in microseconds, or None where torch has no such kernel."""
    import torch
    hold = getattr(torch.cuda, "_sleep", None)
    if hold is None:
        return None
    stream = torch.cuda.current_stream(wl.device).cuda_stream
    paces = []
    for _ in range(batches):
        first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        hold(20_000_000)
        first.record()
        for i in range(steps_each):
            if step_fn is None:
                wl.step(i, stream)
            else:
                step_fn(i)
        last.record()
        torch.cuda.synchronize(wl.device)
        paces.append(first.elapsed_time(last) * 1e3 / steps_each)
    flags = wl.ctx.status(stream)
    if flags:
        raise RuntimeError(f"device error flags {flags}")
    paces.sort()
    return paces[len(paces) // 2]


def cpu_baseline(case, rd, reps: int, threads: int = 1):
    """The oracle's C restatement on the same batch; best of `reps`.  Returns seconds per step and the
    seconds of its routing part (histogram, ranks, receiver layout: what the reference does on one host
    thread, a2a_worker.rs:526-703).  The only part of this file that touches oracle/."""
    import numpy as np
    from workloads import bf16_codes, make_rank, rows_needed
    sys.path.insert(0, str(REPO / "oracle"))
    import c_oracle

    N = case.world_size
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


def cpu_baseline_numpy(case, tokens: int):
    """The numpy oracle (array code, whatever threads numpy's kernels use: its element-wise loops run
    on one) on a sample of `tokens` tokens of the same workload.  Returns seconds for the sample."""
    import numpy as np
    from workloads import bf16_codes, make_rank, rows_needed
    sys.path.insert(0, str(REPO / "oracle"))
    import a2a_oracle as oracle

    N = case.world_size
    world = [make_rank(case, 0, tokens)] + [make_rank(case, r, 0) for r in range(1, N)]
    rows = rows_needed(case, world)
    rng = np.random.default_rng(case.seed)
    ys = [rng.integers(0x3C00, 0x4000, size=(rows, case.hidden_dim), dtype=np.uint16) for _ in range(N)]
    t0 = time.perf_counter()
    inputs = [oracle.RankInput(x=bf16_codes(w.x), indices=w.indices.numpy()) for w in world]
    outs = oracle.dispatch_world(inputs, num_experts=case.num_experts, world_size=N,
                                 node_size=case.node_size or N, expert_padding=case.expert_padding,
                                 out_rows=rows, quantize=True)
    oracle.combine_world(ys, [w.indices.numpy() for w in world], [w.weights.numpy() for w in world],
                         outs[0].slots, num_experts=case.num_experts, world_size=N)
    return time.perf_counter() - t0


def cpu_baseline_torch(case, tokens: int):
    """The torch restatement of the path (tensor ops on the CPU, torch's intra-op threads) on a sample of
    `tokens` tokens of the same workload.  Returns (seconds for the sample, threads used)."""
    import torch
    from workloads import make_rank, rows_needed
    sys.path.insert(0, str(REPO / "oracle"))
    import a2a_oracle_torch as torch_oracle

    N = case.world_size
    world = [make_rank(case, 0, tokens)] + [make_rank(case, r, 0) for r in range(1, N)]
    rows = rows_needed(case, world)
    gen = torch.Generator().manual_seed(case.seed)
    ys = [torch.rand((rows, case.hidden_dim), generator=gen).to(torch.bfloat16) for _ in range(N)]
    t0 = time.perf_counter()
    _, _, _, slots = torch_oracle.dispatch_world(
        [w.x for w in world], [w.indices for w in world], num_experts=case.num_experts, world_size=N,
        node_size=case.node_size or N, expert_padding=case.expert_padding, out_rows=rows)
    torch_oracle.combine_world(ys, [w.indices for w in world], [w.weights for w in world], slots,
                               num_experts=case.num_experts, world_size=N)
    return time.perf_counter() - t0, torch.get_num_threads()


def other_shape(case, device, routings: int, steps: int, warmup: int, ctx_flags: int, label: str, bar_us=None,
                senders: str = "one"):
    """Wall time per step without events, the kernels' own durations from a pass with events, and the
    calls' p50 from a pass with events around every call."""
    from pplx_garden_amd.utils.math import Statistics
    wl = Workload(case, device, routings, ctx_flags, senders=senders)
    num_senders = len(wl.senders)
    _, d, c, b, p, g, _ = time_workload(wl, steps, warmup, kernel_every=4, call_every=1)
    w, _, _, _, _, _, _ = time_workload(wl, steps, warmup)
    graph_s, _ = time_graph_replay(wl, steps, warmup)
    pace_us = time_gpu_pace(wl) if w / steps < 100e-6 else None
    wl.close()
    d_bytes, c_bytes = algorithmic_bytes(case.num_tokens * num_senders, case.hidden_dim, case.topk)
    step_us = w / steps * 1e6
    out = {
        "workload": label,
        "step_us_wall": round(step_us, 2),
        "step_us_graph_replay": round(graph_s * 1e6, 2),
        "step_us_gpu_pace": None if pace_us is None else round(pace_us, 2),
        "pack_kernel_us_mean": round(Statistics.create(p).mean, 2),
        "gather_kernel_us_mean": round(Statistics.create(g).mean, 2),
        "kernel_samples": len(g),
        "dispatch_us_p50": round(Statistics.create(d).p50, 2),
        "combine_us_p50": round(Statistics.create(c).p50, 2),
        "total_us_p50": round(Statistics.create(b).p50, 2),
        "total_us_mean": round(Statistics.create(b).mean, 2),
        "algorithmic_bytes": d_bytes + c_bytes,
        "pct_of_hbm_peak": round(100.0 * (d_bytes + c_bytes) / (step_us * 1e-6) / 1e9 / HBM_PEAK_GBS, 2),
    }
    if bar_us is not None:
        out["bar_us_for_70pct"] = bar_us
    return out


def split_calls(case, device, routings: int, steps: int, warmup: int, label: str):
    """The four split calls (`a2a_dispatch_send / _recv`, `a2a_combine_send / _recv`: the calls the
    reference's FFI binds, a2a_context.rs:275-487) at the headline's shape, rank 0 holding the tokens.
    Rows move twice here (sender -> staging -> receiver, and back), so the bytes are two-hop bytes.

    Three passes: (1) whole steps (the send, every rank's recv, every rank's combine-send, rank 0's
    combine-recv) in which every kernel records events at its own start and end: the kernels' own
    durations, per kernel; (2) the same steps between two synchronisations, no events: wall time of the
    work of the whole group on this GPU; (3) only rank 0's four calls per step, no events: what a rank
    on a GPU of its own runs (its combine-recv reads the rows the other ranks' combine-sends of the
    passes before left in the staging buffer)."""
    import numpy as np
    import torch
    from pplx_garden_amd.native import p2p_all_to_all as native
    from pplx_garden_amd.utils.math import Statistics

    wl = Workload(case, device, routings, native.FLAG_PREALLOC_STAGING)
    ctx = wl.ctx
    N, H, Hs, K, T = case.world_size, case.hidden_dim, case.hidden_dim_scale, case.topk, case.num_tokens
    Le = case.experts_per_rank
    stream = torch.cuda.current_stream(device).cuda_stream
    rows_of = []                           # [routing][rank]: rows a rank receives
    for routing in wl.routings:
        owner = routing[0].indices.numpy().reshape(-1) // Le
        rows_of.append(np.bincount(owner, minlength=N)[:N])

    def send(j):
        ctx.dispatch_send(0, T, wl.x[0].data_ptr(), 2 * H, None, 0, 0, wl.idx[j][0].data_ptr(), K,
                          wl.w[j][0].data_ptr(), K, None, stream, quantize=True)

    def empty_send(r):
        ctx.dispatch_send(r, 0, None, 2 * H, None, 0, 0, None, K, None, K, None, stream, quantize=True)

    def recv(r):
        ctx.dispatch_recv(r, wl.out_n[r].data_ptr(), wl.out_x[r].data_ptr(), H, wl.rows, wl.out_s[r].data_ptr(), 1, Hs,
                          stream)

    def combine_send(r):
        ctx.combine_send(r, wl.y[r].data_ptr(), 2 * H, wl.rows, stream)

    def combine_recv(j):
        ctx.combine_recv(0, T, wl.rows, torch.bfloat16, wl.out_tokens[0].data_ptr(), H, wl.idx[j][0].data_ptr(), K,
                         wl.w[j][0].data_ptr(), K, None, False, stream)

    def whole_step(i, timed=None):
        j = i % len(wl.routings)

        def own(which, key):
            if timed is not None:
                pair = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
                for ev in pair:
                    ev.record()             # an event gets its handle when it is first recorded
                ctx.time_next_kernel(which, pair[0].cuda_event, pair[1].cuda_event)
                timed.append((key, j, pair))

        own(native.KERNEL_ROUTE, "route")
        own(native.KERNEL_STAGE_SEND, "send")
        send(j)
        for r in range(1, N):
            empty_send(r)
        for r in range(N):
            own(native.KERNEL_STAGE_RECV, ("recv", r))
            recv(r)
        for r in range(N):
            own(native.KERNEL_COMBINE_SEND, ("combine_send", r))
            combine_send(r)
        own(native.KERNEL_GATHER, "combine_recv")
        combine_recv(j)

    def one_rank_step(i):
        j = i % len(wl.routings)
        send(j)
        recv(0)
        combine_send(0)
        combine_recv(j)

    def wall(step_fn, n):
        for i in range(warmup):
            step_fn(i)
        torch.cuda.synchronize(device)
        t0 = time.perf_counter()
        for i in range(n):
            step_fn(warmup + i)
        torch.cuda.synchronize(device)
        dt = time.perf_counter() - t0
        flags = ctx.status(stream)
        if flags:
            raise RuntimeError(f"device error flags {flags}")
        return dt / n * 1e6

    # (1) the kernels' own durations
    timed = []
    sample_steps = min(steps, 100)
    for i in range(min(warmup, 20)):
        whole_step(i)
    torch.cuda.synchronize(device)
    for i in range(sample_steps):
        whole_step(i, timed)
    torch.cuda.synchronize(device)
    if ctx.status(stream):
        raise RuntimeError("device error flags in the split calls")
    us = {}
    for key, j, (a, b) in timed:
        us.setdefault(key, []).append((a.elapsed_time(b) * 1e3, j))
    # (2), (3) wall time without events
    whole_us = wall(whole_step, steps)
    one_rank_us = wall(one_rank_step, steps)
    wl.close()

    row_d = H + 4 * Hs                     # a dispatched row: fp8 payload and its float scales
    row_c = 2 * H                          # a combined row: bf16

    def kernel(name, samples, bytes_of):
        if not samples:
            return None
        t = [x for x, _ in samples]
        total_bytes = sum(bytes_of(j) for _, j in samples)
        st = Statistics.create(t)
        out = {"kernel": name, "avg_us": round(st.mean, 2), "p50_us": round(st.p50, 2), "samples": len(t)}
        if total_bytes:
            rate = total_bytes / (sum(t) * 1e-6) / 1e9
            out.update({"bytes_per_launch": int(total_bytes / len(t)), "achieved_gbs": round(rate, 1),
                        "frac_of_hbm_peak": round(rate / HBM_PEAK_GBS, 4)})
        return out

    d_bytes, c_bytes = algorithmic_bytes(T, H, K)
    later = [x for r in range(1, N) for x in us.get(("recv", r), [])]
    # bytes of the later recvs: per sample, in the order the samples were taken
    later_seq = [2 * int(rows_of[j][r]) * row_d for r in range(1, N) for _, j in us.get(("recv", r), [])]
    csend = [x for r in range(N) for x in us.get(("combine_send", r), [])]
    csend_seq = [2 * int(rows_of[j][r]) * row_c for r in range(N) for _, j in us.get(("combine_send", r), [])]

    def seq_kernel(name, samples, byte_seq):
        if not samples:
            return None
        t = [x for x, _ in samples]
        st = Statistics.create(t)
        rate = sum(byte_seq) / (sum(t) * 1e-6) / 1e9
        return {"kernel": name, "avg_us": round(st.mean, 2), "p50_us": round(st.p50, 2), "samples": len(t),
                "bytes_per_launch": int(sum(byte_seq) / len(t)), "achieved_gbs": round(rate, 1),
                "frac_of_hbm_peak": round(rate / HBM_PEAK_GBS, 4)}

    kernels = {
        "dispatch_send": [
            kernel("route_hist_kernel", us.get("route", []), lambda j: 0),
            kernel("stage_send_resolve_kernel", us.get("send", []), lambda j: T * (2 * H + 4 * K) + T * row_d),
        ],
        "dispatch_recv": [
            kernel("stage_recv_first_kernel", us.get(("recv", 0), []), lambda j: 2 * int(rows_of[j][0]) * row_d),
            seq_kernel("stage_recv_kernel", later, later_seq),
        ],
        "combine_send": [seq_kernel("combine_send_kernel", csend, csend_seq)],
        "combine_recv": [kernel("combine_gather_kernel", us.get("combine_recv", []), lambda j: c_bytes)],
    }
    one_rank_kernels = sum(k["avg_us"] for k in (kernels["dispatch_send"] + kernels["dispatch_recv"][:1]
                                                 + kernels["combine_send"] + kernels["combine_recv"]) if k)
    return {
        "workload": label,
        "one_rank_step_us_wall": round(one_rank_us, 2),
        "one_rank_step_us_kernels": round(one_rank_kernels, 2),
        "all_ranks_step_us_wall": round(whole_us, 2),
        "kernels": kernels,
        "rows_received_per_rank_first_routing": [int(v) for v in rows_of[0]],
        "note": "two-hop bytes: a send reads 4096 bf16 rows and their index rows and stages one fp8 row with its "
                "scales per token; a recv reads and writes the rows its rank receives; a combine-send reads and "
                "writes the bf16 rows of its rank; the combine-recv is the gather of the group call over the "
                "staging buffer.  one_rank_step = rank 0's four calls (what a rank on a GPU of its own runs; "
                "its recv is the step's first and also lays out the other receivers); all_ranks_step = the "
                "send, every rank's recv, every rank's combine-send and rank 0's combine-recv (the work of "
                "the whole group for one sender's tokens, on this GPU).  Kernel durations come from events "
                f"the launches record themselves, over {sample_steps} steps; wall times from {steps} steps "
                "without events.",
    }


def split_calls_small(case, device, routings: int, steps: int, warmup: int, label: str):
    """The four split calls at a step of a few tens of microseconds at most (a decode shape, the
    1024-token mixed batch), rank 0 holding the tokens:
    wall time of a loop of steps and the GPU's own pace (the steps enqueued behind a kernel that holds the
    queue), for rank 0's four calls (what a rank on a GPU of its own runs) and for the calls of the whole
    group, and the pace of the sequences send / send + recv / send + recv + combine-send, whose
    differences are what each call adds."""
    import torch
    from pplx_garden_amd.native import p2p_all_to_all as native

    wl = Workload(case, device, routings, native.FLAG_PREALLOC_STAGING)
    ctx = wl.ctx
    N, H, Hs, K, T = case.world_size, case.hidden_dim, case.hidden_dim_scale, case.topk, case.num_tokens
    stream = torch.cuda.current_stream(device).cuda_stream
    R = len(wl.routings)

    def send(i):
        j = i % R
        ctx.dispatch_send(0, T, wl.x[0].data_ptr(), 2 * H, None, 0, 0, wl.idx[j][0].data_ptr(), K,
                          wl.w[j][0].data_ptr(), K, None, stream, quantize=True)

    def empty_send(r):
        ctx.dispatch_send(r, 0, None, 2 * H, None, 0, 0, None, K, None, K, None, stream, quantize=True)

    def recv(r):
        ctx.dispatch_recv(r, wl.out_n[r].data_ptr(), wl.out_x[r].data_ptr(), H, wl.rows, wl.out_s[r].data_ptr(), 1, Hs,
                          stream)

    def combine_send(r):
        ctx.combine_send(r, wl.y[r].data_ptr(), 2 * H, wl.rows, stream)

    def combine_recv(i):
        j = i % R
        ctx.combine_recv(0, T, wl.rows, torch.bfloat16, wl.out_tokens[0].data_ptr(), H, wl.idx[j][0].data_ptr(), K,
                         wl.w[j][0].data_ptr(), K, None, False, stream)

    def one_rank_step(i):
        send(i)
        recv(0)
        combine_send(0)
        combine_recv(i)

    def whole_step(i):
        send(i)
        for r in range(1, N):
            empty_send(r)
        for r in range(N):
            recv(r)
        for r in range(N):
            combine_send(r)
        combine_recv(i)

    def wall(step_fn, n):
        for i in range(warmup):
            step_fn(i)
        torch.cuda.synchronize(device)
        t0 = time.perf_counter()
        for i in range(n):
            step_fn(warmup + i)
        torch.cuda.synchronize(device)
        dt = time.perf_counter() - t0
        flags = ctx.status(stream)
        if flags:
            raise RuntimeError(f"device error flags {flags}")
        return dt / n * 1e6

    def pace(step_fn):
        p = time_gpu_pace(wl, step_fn=step_fn)
        return None if p is None else round(p, 2)

    for i in range(min(warmup, 20)):
        whole_step(i)               # every rank's tables exist before rank 0's calls are timed alone
    one_wall = wall(one_rank_step, steps)
    whole_wall = wall(whole_step, steps)
    out = {
        "workload": label,
        "one_rank_step_us_wall": round(one_wall, 2),
        "one_rank_step_us_gpu_pace": pace(one_rank_step),
        "all_ranks_step_us_wall": round(whole_wall, 2),
        "gpu_pace_us_of_call_sequences": {
            "send": pace(send),
            "send_recv": pace(lambda i: (send(i), recv(0))),
            "send_recv_combine_send": pace(lambda i: (send(i), recv(0), combine_send(0))),
        },
        "note": "rank 0 holds the tokens.  one_rank_step = rank 0's send, recv, combine-send and combine-recv: "
                "four launches; the recv is the step's first and also lays out the other receivers.  "
                "all_ranks_step = those plus the other ranks' (empty) sends, recvs and combine-sends: 3 N + 1 "
                "calls for N ranks, whose wall time is mostly the host's.  gpu_pace: the calls enqueued behind a kernel that "
                "holds the queue, two events around 100 steps, median of 5.",
    }
    wl.close()
    return out


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--routings", type=int, default=4, help="distinct routings cycled over the steps")
    ap.add_argument("--regions", type=int, default=5,
                    help="repetitions of the timed region (warm-up, then K steps without events); the line's "
                         "value is the median region")
    ap.add_argument("--cpu-reps", type=int, default=3, help="repetitions of the CPU baseline (0 = skip)")
    ap.add_argument("--no-decode", action="store_true", help="skip the shapes other than the 4096-token one")
    ap.add_argument("--no-split", action="store_true", help="skip the pass through the four split calls")
    ap.add_argument("--split-small-only", action="store_true",
                    help="time only the four split calls at the two decode shapes (for a kernel trace of them alone)")
    ap.add_argument("--split-only", action="store_true",
                    help="time only the four split calls at the headline's shape (for a kernel trace of them alone)")
    ap.add_argument("--decode-only", action="store_true",
                    help="time only the 128-token shape (for a kernel trace of the decode step alone)")
    ap.add_argument("--only-shape", choices=("decode_128", "qwen3_decode_128", "kimi_1024"), default=None,
                    help="time only this one of the other shapes of the baseline (for a kernel trace of it alone)")
    ap.add_argument("--separate-routing", action="store_true",
                    help="create the context with A2A_FLAG_SEPARATE_ROUTING (routing kernels, then the pack): "
                         "for comparisons with the default paths")
    ap.add_argument("--context-flags", type=int, default=None,
                    help="create the context with these A2A_FLAG_* bits (for comparisons between paths)")
    ap.add_argument("--probe-copy", action="store_true",
                    help="also run plain device-to-device copies of 512 MiB (torch's copy kernel): the "
                         "known-size kernel that hardware byte counters are scaled by")
    ap.add_argument("--print-source-hash", action="store_true",
                    help="print the fingerprint of the kernel sources (what a counter summary under "
                         "profiles/ records as csrc_sha256) and exit")
    args = ap.parse_args()
    if args.print_source_hash:
        print(kernel_sources_sha256())
        return 0
    if args.gpus != 1:
        print("bench.py measures one GPU: every logical rank of the expert-parallel group lives in "
              "this GPU's HBM and nothing here uses a second GPU; run with --gpus 1", file=sys.stderr)
        return 2

    import torch
    from workloads import C1, C2, C3, C4
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
    side_steps = max(args.steps, 200)
    decode_label = ("DeepSeek-V3 decode: 128 tokens, hidden 7168, 256 experts / 8 logical ranks, top-8 uniform, "
                    "1% x50 outliers")
    qwen_label = "Qwen3-30B-A3B decode: 128 tokens, hidden 2048, 128 experts / 8 logical ranks, top-8 uniform"
    kimi_label = ("Kimi-K2 mixed batch: 1024 tokens, hidden 7168, 384 experts / 16 logical ranks, top-8 Zipf(1.0), "
                  "receive slots padded to 128 per expert")
    others = {"decode_128": (C2, decode_label, None), "qwen3_decode_128": (C1, qwen_label, None),
              "kimi_1024": (C4, kimi_label, 37.0)}
    if args.split_small_only:
        print(json.dumps({
            "split_calls_128_only": split_calls_small(C2, device, args.routings, side_steps, args.warmup,
                                                      decode_label + ", through the four split calls"),
            "split_calls_qwen3_128_only": split_calls_small(C1, device, args.routings, side_steps, args.warmup,
                                                            qwen_label + ", through the four split calls"),
            "split_calls_kimi_1024_only": split_calls_small(C4, device, args.routings, side_steps, args.warmup,
                                                            kimi_label + ", through the four split calls")}))
        return 0
    if args.split_only:
        print(json.dumps({"split_calls_4096_only": split_calls(
            C3, device, args.routings, side_steps, args.warmup,
            "DeepSeek-V3 prefill through the four split calls, rank 0 holds the 4096 tokens")}))
        return 0
    if args.decode_only:
        args.only_shape = "decode_128"
    if args.only_shape is not None:
        shape, label, bar = others[args.only_shape]
        print(json.dumps({args.only_shape + "_only": other_shape(shape, device, args.routings, side_steps, args.warmup,
                                                                 ctx_flags, label, bar_us=bar)}))
        return 0

    case = C3
    wl = Workload(case, device, args.routings, ctx_flags)
    # 1. Phase statistics as the reference's benchmark reports them (events around each phase of every
    #    iteration, benchmarks/bench_all_to_all.py:391-433); every fourth step has the three kernels
    #    record their own start and end instead: the samples of the roofline figures.
    _, disp, comb, both, pack, gather, route = time_workload(wl, side_steps, args.warmup, kernel_every=4,
                                                             call_every=1, route_events=True)
    # 2. The timed region: W warm-up steps, then exactly K steps between two synchronisations, no events.
    #    Run `regions` times over; the line's value is the MEDIAN region, the spread is reported.
    region_s = sorted(time_workload(wl, args.steps, args.warmup)[0] for _ in range(args.regions))
    wall_s = region_s[len(region_s) // 2]
    # 3. The same as graph replays.
    graph_step_s, graph_steps = time_graph_replay(wl, args.steps, args.warmup)
    rows = wl.rows
    cpu_rd = wl.cpu_first
    wl.close()

    d_bytes, c_bytes = algorithmic_bytes(case.num_tokens, case.hidden_dim, case.topk)
    ms_per_step = wall_s / args.steps * 1e3
    value = (d_bytes + c_bytes) / (ms_per_step * 1e-3) / 1e9
    p_stats, g_stats = Statistics.create(pack), Statistics.create(gather)
    traffic, traffic_note = measured_traffic()

    def stats_dict(xs):
        return {k: round(v, 2) for k, v in Statistics.create(xs).as_dict().items()}

    def roof(bytes_, stats, samples, kernel):
        achieved = bytes_ / (stats.mean * 1e-6) / 1e9
        return {"kernel": kernel, "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                "traffic": traffic.get(kernel), "traffic_source": traffic_note,
                "bytes_per_launch": bytes_, "avg_us": round(stats.mean, 2), "p50_us": round(stats.p50, 2),
                "samples": samples,
                "timing": "events recorded by the launch itself at the start and end of this kernel "
                          f"(hipExtLaunchKernelGGL), on every fourth of the {side_steps} steps of the pass "
                          "that precedes the timed region"}

    combine_roof = roof(c_bytes, g_stats, len(gather), "combine_gather_kernel")
    dispatch_roof = roof(d_bytes, p_stats, len(pack),
                         "dispatch_push_kernel" if args.separate_routing else "dispatch_resolve_kernel")
    dominant, other = ((combine_roof, dispatch_roof) if g_stats.mean >= p_stats.mean
                       else (dispatch_roof, combine_roof))

    decode = qwen = kimi = whole_group = split = None
    if not args.no_split:
        split = split_calls(C3, device, args.routings, side_steps, args.warmup,
                            "DeepSeek-V3 prefill through the four split calls (send, recv, combine-send, "
                            "combine-recv), rank 0 holds the 4096 tokens")
    split_decode = split_qwen = split_kimi = None
    if not args.no_decode and not args.no_split:
        split_decode = split_calls_small(C2, device, args.routings, side_steps, args.warmup,
                                         decode_label + ", through the four split calls")
        split_qwen = split_calls_small(C1, device, args.routings, side_steps, args.warmup,
                                       qwen_label + ", through the four split calls")
        split_kimi = split_calls_small(C4, device, args.routings, side_steps, args.warmup,
                                       kimi_label + ", through the four split calls")
    if not args.no_decode:
        decode = other_shape(C2, device, args.routings, side_steps, args.warmup, ctx_flags, decode_label)
        decode["note"] = ("working set (26 MB) fits the 256 MB Infinity Cache and is not flushed between steps; "
                          "step_us_wall is wall time over steps without events, the kernel figures come from "
                          "events the launches record themselves, the p50 figures from events around the calls "
                          "of every step (each event adds about 3 us); step_us_gpu_pace is the time per step "
                          "between two events when the steps are enqueued behind a kernel that holds the queue, "
                          "i.e. with the host ahead of the GPU (the host's share of such a step, two calls "
                          "through ctypes and their launches, is 7-10 us on this pool's hosts)")
        qwen = other_shape(C1, device, args.routings, side_steps, args.warmup, ctx_flags, qwen_label)
        kimi = other_shape(C4, device, args.routings, side_steps, args.warmup, ctx_flags, kimi_label, bar_us=37.0)
        kimi_d, kimi_c = algorithmic_bytes(C4.num_tokens, C4.hidden_dim, C4.topk)
        kimi["traffic"] = traffic.get("kimi_1024")      # HBM bytes per launch by kernel, same rule as roofline.traffic
        kimi["traffic_source"] = traffic_note
        kimi["algorithmic_bytes_by_kernel"] = {"dispatch_teams_kernel": kimi_d, "combine_gather_kernel": kimi_c}
        # The work of the WHOLE group on this GPU: every logical rank sends its 4096 tokens (8 times the
        # bytes of the headline's step, which is one GPU's share).  Not the baseline's configuration;
        # reported beside it as the same kernels' sustained rate over a longer step.
        whole_group = other_shape(C3, device, 2, 100, 20, ctx_flags,
                                  "DeepSeek-V3 prefill, all 8 logical ranks send 4096 tokens each (32 768 tokens per "
                                  "step on one GPU: 8 times one GPU's share)", senders="all")

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
        sample_tokens = case.num_tokens
        dt_np = cpu_baseline_numpy(case, sample_tokens)
        dt_torch, torch_threads = cpu_baseline_torch(case, sample_tokens)
        s_d, s_c = algorithmic_bytes(sample_tokens, case.hidden_dim, case.topk)
        cpu_more = {
            "routing_only_us_one_thread": round(route_dt * 1e6, 1),
            "all_cores": {"value": round((d_bytes + c_bytes) / dt_all / 1e9, 3), "unit": "GB/s", "cores": cores,
                          "us_per_step": round(dt_all * 1e6, 1),
                          "note": "same code, tokens split over OpenMP threads; routing stays on one thread"},
            "torch_oracle_all_cores": {"value": round((s_d + s_c) / dt_torch / 1e9, 3), "unit": "GB/s",
                                       "cores": torch_threads, "seconds": round(dt_torch, 2),
                                       "sample": "the same 4096-token batch, once, through the torch restatement "
                                                 "of the path (tensor ops on the CPU, torch's intra-op threads)"},
            "numpy_oracle": {"value": round((s_d + s_c) / dt_np / 1e9, 3), "unit": "GB/s",
                             "cores": 1, "seconds": round(dt_np, 2),
                             "sample": f"the same {sample_tokens}-token batch, once, through the numpy oracle "
                                       "(array code; numpy's element-wise loops use one thread whatever the "
                                       f"host has: {os.cpu_count()} cores here)"},
        }

    graph_value = (d_bytes + c_bytes) / graph_step_s / 1e9
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
        "pct_of_hbm_peak_p50_with_events": round(
            100.0 * (d_bytes + c_bytes) / (Statistics.create(both).p50 * 1e-6) / 1e9 / HBM_PEAK_GBS, 2),
        "timed_regions": {
            "regions": len(region_s), "steps_each": args.steps, "warmup_each": args.warmup,
            "us_per_step": {"min": round(region_s[0] / args.steps * 1e6, 2),
                            "median": round(wall_s / args.steps * 1e6, 2),
                            "max": round(region_s[-1] / args.steps * 1e6, 2)},
            "note": "each region: W warm-up steps, then exactly K steps between two synchronisations, no event in "
                    "between; `value`, `ms_per_step` and `pct_of_hbm_peak` are the median region; "
                    "`pct_of_hbm_peak_p50_with_events` is the same bytes over the p50 of the per-step time of the "
                    "pass that records events around each phase of every step (the reference benchmark's method: "
                    "every event idles the queue for about 3 us)",
        },
        "prefill_4096": {
            "step_us_wall": round(ms_per_step * 1e3, 2),
            "graph_replay": {"step_us_wall": round(graph_step_s * 1e6, 2), "steps": graph_steps,
                             "value": round(graph_value, 1),
                             "pct_of_hbm_peak": round(100.0 * graph_value / HBM_PEAK_GBS, 2),
                             "note": f"one captured HIP graph of {args.routings} steps (one per routing), replayed"},
            "pack_kernel_us": {"p50": round(p_stats.p50, 2), "mean": round(p_stats.mean, 2), "samples": len(pack)},
            "gather_kernel_us": {"p50": round(g_stats.p50, 2), "mean": round(g_stats.mean, 2), "samples": len(gather)},
            "route_kernel_us": ({"p50": round(Statistics.create(route).p50, 2),
                                 "mean": round(Statistics.create(route).mean, 2), "samples": len(route)}
                                if route else None),
            "algorithmic_bytes": {"dispatch": d_bytes, "combine": c_bytes},
            "with_events_on_every_step": {
                "note": f"the pass of {side_steps} steps before the timed region, events around each phase of every "
                        "iteration as in the reference's benchmark (each event adds about 3 us); every fourth step "
                        "has the three kernels record their own start and end instead",
                "dispatch_us": stats_dict(disp),
                "combine_us": stats_dict(comb),
                "total_us": stats_dict(both),
            },
        },
        "split_calls_4096": split,
        "split_calls_128": split_decode,
        "split_calls_qwen3_128": split_qwen,
        "split_calls_kimi_1024": split_kimi,
        "decode_128": decode,
        "qwen3_decode_128": qwen,
        "kimi_1024": kimi,
        "prefill_4096_all_ranks_send": whole_group,
        "roofline": dominant,
        "roofline_other": other,
        "cpu_baseline": cpu,
        "cpu_baseline_more": cpu_more,
    }
    print(json.dumps(line, ensure_ascii=False))
    return 0


if __name__ == "__main__":
    sys.exit(main())
