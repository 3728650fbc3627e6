"""The dispatch / combine path restated with torch tensor ops on the CPU.

TEST INFRASTRUCTURE ONLY: imported by `tests/` (where it is pinned against the
numpy oracle, which in turn is pinned against library routines and brute
force) and by the `cpu_baseline` leg of `bench.py`, where it is the
many-threaded CPU figure (torch's intra-op thread pool).  Nothing the library
ships imports it.

Dispatch mode: bf16 rows are quantised to fp8 e4m3 with one float32 scale per
128 elements; ranks without dp groups (every rank a source and a receiver).

What it follows, as the numpy oracle does:
  route        a2a_dispatch_send.cu:176-242 (histogram, rank of every copy in its
               expert in ascending (token, k) order, inclusive offset scan)
  slot rule    a2a_worker.rs:577-606,621-634,669-671,681-694
  payload      a2a_dispatch_send.cu:341-367, a2a_dispatch_recv.cu:139-155,220-224
  combine      a2a_combine_recv.cu:94-148, combine_utils.cuh:14-23,108-114
"""

from __future__ import annotations

from typing import List, Sequence

import torch

QUANT_GROUP = 128
FP8_MAX = 448.0


def route(indices: torch.Tensor, num_experts: int):
    """`indices` [T, K] int64 -> (count [E], token_offset [T, K], inclusive offsets [E])."""
    flat = indices.reshape(-1)
    count = torch.bincount(flat, minlength=num_experts)
    incl = torch.cumsum(count, 0)
    order = torch.argsort(flat, stable=True)          # entries sorted by expert, ascending (token, k) inside
    first = (incl - count)[flat[order]]               # position of the expert's first entry
    token_offset = torch.empty_like(flat)
    token_offset[order] = torch.arange(flat.numel(), dtype=flat.dtype) - first
    return count, token_offset.reshape(indices.shape), incl


def source_order(rank: int, world_size: int, node_size: int) -> List[int]:
    """Sources in the order receiver `rank` lays them out (a2a_worker.rs:681-694): the ranks of the
    other nodes from the next node on, the rest of the own node after `rank`, then `rank`."""
    nodes = world_size // node_size
    node = rank // node_size
    out = []
    for i in range(1, nodes):
        other = (node + i) % nodes
        out.extend(range(other * node_size, (other + 1) * node_size))
    for i in range(1, node_size):
        out.append(node * node_size + (rank % node_size + i) % node_size)
    out.append(rank)
    return out


def quantize_block128(x: torch.Tensor):
    """bf16 [T, H] -> (fp8 e4m3 codes uint8 [T, H], float32 scales [T, H / 128]).

    A NaN or an infinity in a group goes through the same operations (torch's maxima propagate
    NaN); on output NaN has one spelling: code 0x7F, scale bits 0x7FC00000."""
    T, H = x.shape
    f = x.to(torch.float32).reshape(T, H // QUANT_GROUP, QUANT_GROUP)
    amax = f.abs().amax(dim=-1, keepdim=True).clamp_min(1e-4)
    inv = torch.tensor(FP8_MAX, dtype=torch.float32) / amax
    q = (f * inv).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)
    scale = (amax / torch.tensor(FP8_MAX, dtype=torch.float32)).reshape(T, H // QUANT_GROUP)
    codes = q.reshape(T, H).view(torch.uint8)
    codes = torch.where((codes & 0x7F) == 0x7F, torch.full_like(codes, 0x7F), codes)
    scale = torch.where(scale.isnan(), torch.full_like(scale, float("nan")), scale)
    return codes, scale


def dispatch_world(xs: Sequence[torch.Tensor], indices: Sequence[torch.Tensor], *, num_experts: int,
                   world_size: int, node_size: int, expert_padding: int, out_rows: int):
    """dispatch() of every rank.  Returns (num_tokens [N][Le], out_x [N][rows, H] uint8, out_scale
    [N][rows, Hs], slots [N][T, K]): per receiver the per-expert counts and its rows, per source the
    receiver row of every copy."""
    N, E, pad = world_size, num_experts, expert_padding
    Le = -(-E // N)
    H = xs[0].shape[1]
    routed = [route(idx.to(torch.int64), E) for idx in indices]
    num_routed = torch.stack([c for c, _, _ in routed])                    # [N, E]
    padded_E = Le * N
    per = torch.zeros((N, padded_E), dtype=torch.int64)
    per[:, :E] = num_routed
    per = per.reshape(N, N, Le)                                            # [source, receiver, local expert]
    tpe = per.sum(0)                                                       # [receiver, local expert]
    padded = (tpe + pad - 1) // pad * pad
    padded_offset = torch.cumsum(padded, 1) - padded
    base = torch.zeros((N, N, Le), dtype=torch.int64)                      # first row of (source, receiver, le)
    for r in range(N):
        running = padded_offset[r].clone()
        for g in source_order(r, N, node_size):
            base[g, r] = running
            running = running + per[g, r]
    out_x = [torch.zeros((out_rows, H), dtype=torch.uint8) for _ in range(N)]
    out_s = [torch.zeros((out_rows, H // QUANT_GROUP), dtype=torch.float32) for _ in range(N)]
    slots = []
    for g in range(N):
        idx = indices[g].to(torch.int64)
        T, K = idx.shape
        owner = idx // Le
        slot = base[g].reshape(-1)[idx] + routed[g][1] if T else idx       # base[g][owner, le] flattened = [e]
        slots.append(slot)
        if T == 0:
            continue
        q, s = quantize_block128(xs[g])
        token = torch.arange(T).unsqueeze(1).expand(T, K)
        for r in range(N):
            sel = owner == r
            if not bool(sel.any()):
                continue
            rows, toks = slot[sel], token[sel]
            if int(rows.max()) >= out_rows:
                raise ValueError("receive buffer too small")
            out_x[r][rows] = q[toks]
            out_s[r][rows] = s[toks]
    num_tokens = [tpe[r].to(torch.int32) for r in range(N)]
    return num_tokens, out_x, out_s, slots


def combine_world(ys: Sequence[torch.Tensor], indices: Sequence[torch.Tensor], weights: Sequence[torch.Tensor],
                  slots: Sequence[torch.Tensor], *, num_experts: int, world_size: int):
    """combine() of every rank: out[t] = sum over k ascending of w[t, k] * y(t, k), accumulated in
    float32 (one multiply and one add per term, each rounded: torch has no fused form here), one
    rounding to bf16.  `ys` [N][rows, H] bf16."""
    Le = -(-num_experts // world_size)
    H = ys[0].shape[1]
    outs = []
    for g in range(world_size):
        idx = indices[g].to(torch.int64)
        T, K = idx.shape
        acc = torch.zeros((T, H), dtype=torch.float32)
        owner = idx // Le
        for k in range(K):
            rows = torch.zeros((T, H), dtype=torch.float32)
            for r in range(world_size):
                sel = owner[:, k] == r
                if bool(sel.any()):
                    rows[sel] = ys[r][slots[g][sel, k]].to(torch.float32)
            acc += weights[g][:, k : k + 1] * rows
        outs.append(acc.to(torch.bfloat16))
    return outs
