"""CPU oracle for the MoE dispatch / combine path.  TEST INFRASTRUCTURE ONLY.

This module restates, in numpy, the algorithm of the reference's p2p-all-to-all
path so that the HIP kernels can be checked against it.  Nothing in the product
package may import it: only tests, the smoke check and the benchmark's
CPU-baseline leg do, and only as the checker.

Every function cites the reference file:line it follows (paths relative to the
reference checkout).  Where the reference leaves something open the choice made
here is stated:

* token order inside an expert: the reference hands out `token_offset` with
  `atomicAdd` in arrival order (a2a_dispatch_send.cu:183-190), which is not
  deterministic.  Here the order is the stable one, ascending `(token, k)`.
* the bf16 -> fp8 e4m3 quantiser is not part of the reference at all (it only
  transports caller-quantised bytes and caller-supplied scales,
  a2a_dispatch_send.cu:341-367).  Its rule is defined in `quantize_block128`.

How each function is pinned (tests/test_oracle_*.py):
  route / expert offsets   numpy.bincount and numpy.cumsum, a brute-force loop
  process_routing_info     invariants of the reference's test (counts, slot
                           ranges, injectivity) and the closed form `slot_base`
  e4m3fn_encode            torch's float8_e4m3fn cast on every bf16 value and a
                           brute-force nearest-value search over the 256 codes
  quantize_block128        torch ops (amax, division, cast) and the dequant bound
  combine                  float64 weighted sum; the round-trip identity of the
                           reference's test (test_p2p_all_to_all.py:44-50,233)
  strides / capacity       hand-computed values quoted in the reference
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Sequence

import numpy as np

# ---------------------------------------------------------------------------
# small integer helpers (python/pplx_garden/utils/math.py:5-10)
# ---------------------------------------------------------------------------


def ceil_div(n: int, m: int) -> int:
    return (n + m - 1) // m


def round_up(n: int, m: int) -> int:
    return (n + m - 1) // m * m


# ScalarType tags that cross the FFI (rust/torch-lib/src/lib.rs:31-49).
SCALAR_TYPES = (
    "BOOL", "I8", "U8", "I16", "U16", "I32", "U32", "I64", "U64",
    "F8_E4M3", "F8_E5M2", "F16", "BF16", "F32", "F64",
)
SCALAR_TYPE = {name: i for i, name in enumerate(SCALAR_TYPES)}


# ---------------------------------------------------------------------------
# geometry: row strides and buffer capacities
# ---------------------------------------------------------------------------


def dispatch_token_stride(hidden_dim: int, in_elemsize: int,
                          hidden_dim_scale: int, scale_elemsize: int) -> int:
    """Bytes per staged dispatch row: payload, scales, 16 spare bytes.

    a2a_worker.rs:317-321, a2a_dispatch_send.cu:586-588.
    """
    token_dim = round_up(hidden_dim * in_elemsize, 16)
    scale_dim = round_up(hidden_dim_scale * scale_elemsize, 16)
    return token_dim + scale_dim + 16


def combine_token_stride(hidden_dim: int, out_elemsize: int) -> int:
    """Bytes per staged combine row (a2a_worker.rs:323-325)."""
    return round_up(hidden_dim * out_elemsize, 16)


def buffer_capacity(max_num_tokens: int, num_experts: int,
                    num_experts_per_token: int, world_size: int, dp_size: int,
                    expert_padding: int,
                    max_private_tokens: Optional[int] = None):
    """(num_local_experts, max_private_tokens, max_recv_tokens).

    python/pplx_garden/kernels/p2p_all_to_all.py:91-114.
    """
    num_dp_groups = world_size // dp_size
    num_local_experts = ceil_div(num_experts, world_size)
    avg_tokens_per_expert = int(
        ceil_div(max_num_tokens * num_experts_per_token, num_experts) * 1.2)
    if max_private_tokens is None:
        max_private_tokens = avg_tokens_per_expert * num_local_experts
    num_tokens = max_num_tokens * num_dp_groups
    max_recv_tokens = max_private_tokens * num_dp_groups + round_up(
        max(
            min(num_tokens * num_experts_per_token
                + num_local_experts * (expert_padding - 1),
                num_tokens * num_local_experts),
            num_local_experts * expert_padding),
        expert_padding)
    return num_local_experts, max_private_tokens, max_recv_tokens


# ---------------------------------------------------------------------------
# sender-side routing: histogram, per-entry rank, offset scan
# ---------------------------------------------------------------------------


def route(indices: np.ndarray, num_experts: int):
    """Histogram of expert ids, stable rank of every entry, inclusive scan.

    a2a_dispatch_send.cu:176-243.  `indices` is [T, K]; entries are visited in
    row-major order, so `token_offset[t*K+k]` is the number of earlier entries
    with the same expert id.  Returns (count[E], token_offset[T*K],
    expert_offsets[E]) as uint32, `expert_offsets` being the INCLUSIVE sum the
    reference stores (a2a_dispatch_send.cu:236-242).
    """
    flat = np.asarray(indices).reshape(-1).astype(np.int64)
    if flat.size and (flat.min() < 0 or flat.max() >= num_experts):
        raise ValueError("expert id out of range")
    count = np.zeros(num_experts, dtype=np.uint32)
    token_offset = np.zeros(flat.size, dtype=np.uint32)
    if flat.size:
        order = np.argsort(flat, kind="stable")
        sorted_e = flat[order]
        starts = np.flatnonzero(np.r_[True, sorted_e[1:] != sorted_e[:-1]])
        run_len = np.diff(np.r_[starts, sorted_e.size])
        within = np.arange(sorted_e.size) - np.repeat(starts, run_len)
        token_offset[order] = within.astype(np.uint32)
        count[sorted_e[starts]] = run_len.astype(np.uint32)
    expert_offsets = np.cumsum(count, dtype=np.uint64).astype(np.uint32)
    return count, token_offset, expert_offsets


def positions(indices: np.ndarray, token_offset: np.ndarray,
              expert_offsets: np.ndarray, experts_per_rank: int):
    """Row of every (token, k) in the sender's expert-sorted order.

    ExpertIterator, a2a_dispatch_send.cu:50-58: position = exclusive offset of
    the expert + token_offset; offset = position - exclusive offset of the
    destination rank's first expert.  Returns (position[T,K], offset[T,K]).
    """
    idx = np.asarray(indices).astype(np.int64)
    excl = np.r_[0, expert_offsets[:-1].astype(np.int64)]
    pos = excl[idx] + token_offset.reshape(idx.shape).astype(np.int64)
    dst_rank = idx // experts_per_rank
    rank_off = excl[np.minimum(dst_rank * experts_per_rank, len(excl) - 1)]
    return pos.astype(np.uint32), (pos - rank_off).astype(np.uint32)


# ---------------------------------------------------------------------------
# receiver-side layout
# ---------------------------------------------------------------------------


def source_order(rank: int, world_size: int, node_size: int,
                 dp_size: int = 1) -> list:
    """dp groups in the order receiver `rank` lays their rows out.

    a2a_worker.rs:681-694: groups on other nodes starting at the next node,
    then the other groups of the own node starting after the own group, then
    the own group.
    """
    num_nodes = world_size // node_size
    groups_per_node = node_size // dp_size
    rank_node = rank // node_size
    dp_group = rank // dp_size
    order = []
    for i in range(1, num_nodes):
        for j in range(groups_per_node):
            order.append((rank_node + i) % num_nodes * groups_per_node + j)
    for local_group in range(1, groups_per_node):
        order.append(rank_node * groups_per_node
                     + (dp_group + local_group) % groups_per_node)
    order.append(dp_group)
    return order


@dataclass
class RecvLayout:
    tokens_per_expert: np.ndarray      # [Le] uint32
    padded_offset: np.ndarray          # [n_local] uint32
    num_recv_tokens: int
    num_efa_tokens: int
    padded_index: np.ndarray           # [num_recv_tokens] uint32
    source_rank: np.ndarray
    source_dispatch_offset: np.ndarray
    combine_send_offset: np.ndarray
    source_position: np.ndarray        # row in the sender's expert-sorted order


def process_routing_info(num_routed: np.ndarray, rank: int, world_size: int,
                         node_size: int, dp_size: int, expert_padding: int,
                         max_private_tokens: int) -> RecvLayout:
    """Receiver-side metadata, a loop-for-loop restatement of the host worker.

    a2a_worker.rs:526-703.  `num_routed` is [num_dp_groups, E]: row g is what
    dp group g counted for every expert.  `source_position` is extra: the row
    of the copy in the sender's expert-sorted send order
    (`dst_group_offset + running index`, a2a_worker.rs:571-575,641-651), which
    is what every variant of `source_dispatch_offset` ultimately refers to.
    """
    num_routed = np.asarray(num_routed, dtype=np.int64)
    num_dp_groups, num_experts = num_routed.shape
    assert num_dp_groups == world_size // dp_size
    experts_per_rank = ceil_div(num_experts, world_size)
    first_local = rank * experts_per_rank
    last_local = min(first_local + experts_per_rank, num_experts)
    num_local = max(last_local - first_local, 0)
    rank_node = rank // node_size
    own_group = rank // dp_size
    dp_rank = rank % dp_size

    src_group_offset = [0] * num_dp_groups
    dst_group_offset = [0] * num_dp_groups
    tokens_per_expert = [0] * experts_per_rank
    source_expert_offset = [0] * num_experts
    num_recv_tokens = 0
    rank_offset = 0
    for g in range(num_dp_groups):
        for i in range(dp_size):
            r = g * dp_size + i
            fe = r * experts_per_rank
            le = min(fe + experts_per_rank, num_experts)
            for e in range(fe, le):
                n = int(num_routed[own_group, e])
                source_expert_offset[e] = rank_offset
                rank_offset += n
        dst_group_offset[g] = int(num_routed[g, :first_local].sum())
        n_tok = 0
        for e in range(first_local, last_local):
            n = int(num_routed[g, e])
            n_tok += n
            tokens_per_expert[e - first_local] += n
        src_group_offset[g] = num_recv_tokens
        num_recv_tokens += n_tok

    padded_offset = []
    base = 0
    for c in tokens_per_expert[:num_local]:
        padded_offset.append(base)
        base += ceil_div(c, expert_padding) * expert_padding

    sdo = np.zeros(num_recv_tokens, dtype=np.uint32)
    cso = np.zeros(num_recv_tokens, dtype=np.uint32)
    srk = np.zeros(num_recv_tokens, dtype=np.uint32)
    pidx = np.zeros(num_recv_tokens, dtype=np.uint32)
    spos = np.zeros(num_recv_tokens, dtype=np.uint32)
    base_offset = max_private_tokens * num_dp_groups
    state = {"last": 0}
    src_dispatch_count = [0] * num_dp_groups
    src_combine_count = [0] * num_dp_groups
    expert_count = [0] * num_local

    def route_group(peer_group: int) -> int:
        routed_total = 0
        for e in range(first_local, last_local):
            private_offset = max_private_tokens * peer_group
            routed = int(num_routed[peer_group, e])
            routed_total += routed
            le = e - first_local
            src_offset = src_group_offset[peer_group]
            dst_offset = dst_group_offset[peer_group]
            peer_rank = peer_group * dp_size + dp_rank
            for _ in range(routed):
                last = state["last"]
                if peer_rank == rank:
                    local_offset = source_expert_offset[e]
                    source_expert_offset[e] += 1
                    sdo[last] = local_offset
                    cso[last] = local_offset
                    spos[last] = local_offset
                else:
                    index_on_rank = src_dispatch_count[peer_group]
                    src_dispatch_count[peer_group] += 1
                    spos[last] = dst_offset + index_on_rank
                    if index_on_rank < max_private_tokens:
                        sdo[last] = private_offset + index_on_rank
                    elif peer_rank // node_size == rank_node:
                        sdo[last] = (dst_offset + index_on_rank) | (1 << 31)
                    else:
                        sdo[last] = (src_offset + index_on_rank
                                     + base_offset - max_private_tokens)
                if peer_rank != rank or dp_size > 1:
                    combine_index = src_combine_count[peer_group]
                    src_combine_count[peer_group] += 1
                    if peer_rank // node_size == rank_node:
                        cso[last] = dst_offset + combine_index
                    else:
                        cso[last] = src_offset + combine_index
                srk[last] = peer_rank
                pidx[last] = padded_offset[le] + expert_count[le]
                expert_count[le] += 1
                state["last"] = last + 1
        return routed_total

    num_efa = 0
    order = source_order(rank, world_size, node_size, dp_size)
    num_nodes = world_size // node_size
    groups_per_node = node_size // dp_size
    n_remote = (num_nodes - 1) * groups_per_node
    for i, g in enumerate(order):
        n = route_group(g)
        if i < n_remote:
            num_efa += n

    return RecvLayout(
        tokens_per_expert=np.asarray(tokens_per_expert, dtype=np.uint32),
        padded_offset=np.asarray(padded_offset, dtype=np.uint32),
        num_recv_tokens=num_recv_tokens,
        num_efa_tokens=num_efa,
        padded_index=pidx, source_rank=srk, source_dispatch_offset=sdo,
        combine_send_offset=cso, source_position=spos)


def slot_base(num_routed: np.ndarray, world_size: int, node_size: int,
              expert_padding: int) -> np.ndarray:
    """Closed form of the receiver layout for dp_size = 1: base[g, e].

    The copy `(g, t, k)` with expert `e` lands in row
    `base[g, e] + token_offset_g[t, k]` of the receiver `e // Le`:
    padded offset of the local expert plus the counts of the sources that come
    earlier in `source_order` (a2a_worker.rs:598-606,621-634,669-671).
    """
    num_routed = np.asarray(num_routed, dtype=np.int64)
    G, E = num_routed.shape
    assert G == world_size
    Le = ceil_div(E, world_size)
    base = np.zeros((G, E), dtype=np.int64)
    for r in range(world_size):
        fe, le_end = r * Le, min((r + 1) * Le, E)
        if fe >= le_end:
            continue
        tpe = num_routed[:, fe:le_end].sum(axis=0)
        padded = (tpe + expert_padding - 1) // expert_padding * expert_padding
        poff = np.r_[0, np.cumsum(padded)[:-1]]
        running = poff.copy()
        for g in source_order(r, world_size, node_size):
            base[g, fe:le_end] = running
            running = running + num_routed[g, fe:le_end]
    return base.astype(np.uint32)


# ---------------------------------------------------------------------------
# number formats
# ---------------------------------------------------------------------------


def bf16_to_f32(u16: np.ndarray) -> np.ndarray:
    """bf16 bit patterns (uint16) -> float32 (exact)."""
    return (np.asarray(u16, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16(f: np.ndarray) -> np.ndarray:
    """float32 -> bf16 bit patterns, round to nearest even.

    The rounding of `cvt.rn.bf16x2.f32` (combine_utils.cuh:14-23).  NaN stays
    NaN (quiet bit forced).
    """
    bits = np.asarray(f, dtype=np.float32).view(np.uint32).astype(np.uint64)
    lsb = (bits >> 16) & 1
    rounded = ((bits + 0x7FFF + lsb) >> 16).astype(np.uint32)
    is_nan = (bits & 0x7FFFFFFF) > 0x7F800000
    rounded = np.where(is_nan, (bits >> 16) | 0x40, rounded)
    return rounded.astype(np.uint16)


def f16_to_f32(u16: np.ndarray) -> np.ndarray:
    return np.asarray(u16, dtype=np.uint16).view(np.float16).astype(np.float32)


def f32_to_f16(f: np.ndarray) -> np.ndarray:
    return np.asarray(f, dtype=np.float32).astype(np.float16).view(np.uint16)


def e4m3fn_encode(f: np.ndarray) -> np.ndarray:
    """float32 -> OCP fp8 e4m3 ("fn": no infinities, one NaN) codes, RNE.

    Arithmetic formulation: the grid spacing is 2^-9 below 2^-6 (subnormals)
    and 2^(e-3) in the binade of 2^e.  No saturation: a magnitude that rounds
    beyond 448 becomes the NaN code 0x7F, like torch's cast.
    """
    f = np.ascontiguousarray(f, dtype=np.float32)
    sign = (f.view(np.uint32) >> 24).astype(np.uint8) & 0x80
    with np.errstate(invalid="ignore"):
        a = np.abs(f).astype(np.float64)
    nan = np.isnan(a)
    a = np.where(nan, 0.0, a)
    inf = np.isinf(a)
    a = np.where(inf, 1024.0, a)
    sub = a < 2.0 ** -6
    code_sub = np.rint(a * 2.0 ** 9)                     # 0..8, ties to even
    mant, expo = np.frexp(np.where(sub, 1.0, a))         # a = mant * 2^expo, mant in [.5,1)
    e = expo - 1
    m = np.rint((mant * 2.0 - 1.0) * 8.0)                # 0..8, ties to even
    carry = m == 8
    e = np.where(carry, e + 1, e)
    m = np.where(carry, 0, m)
    code_norm = (e + 7) * 8 + m
    code = np.where(sub, code_sub, code_norm)
    code = np.where(code > 0x7E, 0x7F, code)
    code = np.where(nan | inf, 0x7F, code)
    return (code.astype(np.uint8) | sign).astype(np.uint8)


def e4m3fn_decode(code: np.ndarray) -> np.ndarray:
    """fp8 e4m3fn codes -> float32 (exact)."""
    c = np.asarray(code, dtype=np.uint8).astype(np.int64)
    s = np.where(c & 0x80, -1.0, 1.0)
    e = (c >> 3) & 0xF
    m = c & 7
    val = np.where(e == 0, m * 2.0 ** -9, (1.0 + m / 8.0) * 2.0 ** (e - 7.0))
    val = np.where((c & 0x7F) == 0x7F, np.nan, val)
    return (s * val).astype(np.float32)


FP8_MAX = np.float32(448.0)
AMAX_FLOOR = np.float32(1e-4)
QUANT_GROUP = 128


NAN_CODE = np.uint8(0x7F)
QUIET_NAN_BITS = np.uint32(0x7FC00000)


def quantize_block128(x_bf16: np.ndarray):
    """bf16 rows -> (fp8 e4m3fn codes [T,H], float32 scales [T,H/128]).

    Not in the reference (it transports caller-quantised data).  Rule, all in
    float32, per token and per group of 128 consecutive elements:
        amax  = max(max_i |x_i|, 1e-4)
        scale = amax / 448
        q_i   = e4m3fn_rne(clamp(x_i * (448 / amax), -448, 448))
    The multiply and the two divisions are separate correctly rounded float32
    operations (no fused multiply-add, no reciprocal approximation).

    Non-finite values follow from the same arithmetic with NaN-propagating
    maxima (numpy's, torch's), and NaN has ONE spelling on output (code 0x7F,
    scale bits 0x7FC00000; which NaN an operation returns differs between
    machines):
      * a NaN in the group: amax, scale and every product are NaN, so the
        scale is NaN and all 128 codes are 0x7F;
      * an infinity and no NaN: amax = scale = +inf, 448 / amax = 0, so a
        finite value becomes a zero with its sign (0x00 / 0x80) and an infinite
        one (inf * 0 = NaN) the code 0x7F.
    Either way the group dequantises to NaN throughout: a bad activation stays
    visible, as it does in the reference, which moves the caller's bytes
    untouched (a2a_dispatch_send.cu:341-367).
    """
    x = bf16_to_f32(x_bf16)
    T, H = x.shape
    assert H % QUANT_GROUP == 0
    g = x.reshape(T, H // QUANT_GROUP, QUANT_GROUP)
    with np.errstate(invalid="ignore", over="ignore"):
        amax = np.maximum(np.abs(g).max(axis=2), AMAX_FLOOR).astype(np.float32)
        inv = (FP8_MAX / amax).astype(np.float32)
        scale = (amax / FP8_MAX).astype(np.float32)
        y = (g * inv[:, :, None]).astype(np.float32)
        y = np.clip(y, -FP8_MAX, FP8_MAX)
    codes = e4m3fn_encode(y).reshape(T, H)
    codes = np.where((codes & 0x7F) == 0x7F, NAN_CODE, codes).astype(np.uint8)
    scale_bits = scale.view(np.uint32)
    scale = np.where(np.isnan(scale), QUIET_NAN_BITS, scale_bits).astype(np.uint32).view(np.float32)
    return codes, scale


def dequantize_block128(q: np.ndarray, scale: np.ndarray) -> np.ndarray:
    T, H = q.shape
    v = e4m3fn_decode(q).reshape(T, H // QUANT_GROUP, QUANT_GROUP)
    with np.errstate(invalid="ignore"):
        return (v * scale[:, :, None]).astype(np.float32).reshape(T, H)


# ---------------------------------------------------------------------------
# whole-group dispatch and combine (dp_size = 1)
# ---------------------------------------------------------------------------


@dataclass
class RankInput:
    """What one rank passes to dispatch(): rows, optional scales, routing."""
    x: np.ndarray                       # [T, row_bytes] uint8 (payload bytes) or bf16 codes [T,H] uint16 in quantise mode
    indices: np.ndarray                 # [T, K]
    x_scale: Optional[np.ndarray] = None  # [T, Hs] float32 (transport mode)
    bound_m: Optional[int] = None


@dataclass
class RankOutput:
    num_tokens: np.ndarray              # [Le] int32
    x: np.ndarray                       # [rows, row_bytes] uint8
    x_scale: Optional[np.ndarray]       # [rows, Hs] float32
    written: np.ndarray                 # [rows] bool: rows the dispatch writes
    slots: list = field(default_factory=list)


def world_routing(indices_per_rank: Sequence[np.ndarray], num_experts: int,
                  world_size: int, node_size: int, expert_padding: int,
                  bound_m: Optional[Sequence[Optional[int]]] = None):
    """Routing of the whole group: per-source route() and slot of every copy.

    Returns (num_routed[G,E], token_offsets, expert_offsets, slots) where
    `slots[g]` is int64 [T,K], the receiver row of copy (g,t,k); rows of tokens
    beyond `bound_m[g]` are -1 (a2a_dispatch_send.cu:172).
    """
    Le = ceil_div(num_experts, world_size)
    num_routed = np.zeros((world_size, num_experts), dtype=np.uint32)
    toffs, eoffs = [], []
    for g, idx in enumerate(indices_per_rank):
        n = idx.shape[0] if bound_m is None or bound_m[g] is None else int(bound_m[g])
        c, to, eo = route(idx[:n], num_experts)
        num_routed[g] = c
        toffs.append(to)
        eoffs.append(eo)
    base = slot_base(num_routed, world_size, node_size, expert_padding).astype(np.int64)
    slots = []
    for g, idx in enumerate(indices_per_rank):
        n = idx.shape[0] if bound_m is None or bound_m[g] is None else int(bound_m[g])
        s = np.full(idx.shape, -1, dtype=np.int64)
        if n:
            e = idx[:n].astype(np.int64)
            s[:n] = base[g][e] + toffs[g].reshape(n, -1).astype(np.int64)
        slots.append(s)
    del Le
    return num_routed, toffs, eoffs, slots


def dispatch_world(inputs: Sequence[RankInput], *, num_experts: int,
                   world_size: int, node_size: int, expert_padding: int,
                   out_rows: int, quantize: bool, hidden_dim_scale: int = 0):
    """dispatch() of every rank at once; returns one RankOutput per rank.

    Payload movement: a2a_dispatch_send.cu:341-367 (row + scales to each of the
    K destinations) and a2a_dispatch_recv.cu:139-155 (into
    `out_x[padded_index]`, scales with it); `out_num_tokens`:
    a2a_dispatch_recv.cu:220-224.  Rows in padding gaps are never written.
    In quantise mode `x` holds bf16 codes and the payload is
    `quantize_block128(x)`; otherwise `x` is raw row bytes, copied verbatim.
    """
    Le = ceil_div(num_experts, world_size)
    idxs = [np.asarray(i.indices) for i in inputs]
    bms = [i.bound_m for i in inputs]
    num_routed, _, _, slots = world_routing(
        idxs, num_experts, world_size, node_size, expert_padding, bms)
    payloads, scales = [], []
    for inp in inputs:
        if quantize:
            q, s = quantize_block128(inp.x) if inp.x.shape[0] else (
                np.zeros(inp.x.shape, np.uint8), np.zeros((0, inp.x.shape[1] // QUANT_GROUP), np.float32))
            payloads.append(q)
            scales.append(s)
        else:
            payloads.append(np.asarray(inp.x, dtype=np.uint8))
            scales.append(inp.x_scale)
    row_bytes = payloads[0].shape[1]
    Hs = scales[0].shape[1] if scales[0] is not None else 0
    if not quantize and hidden_dim_scale:
        assert Hs == hidden_dim_scale
    outs = []
    for r in range(world_size):
        fe, le_end = r * Le, min((r + 1) * Le, num_experts)
        tpe = np.zeros(Le, dtype=np.int32)
        if fe < le_end:
            tpe[: le_end - fe] = num_routed[:, fe:le_end].sum(axis=0)
        outs.append(RankOutput(
            num_tokens=tpe,
            x=np.zeros((out_rows, row_bytes), dtype=np.uint8),
            x_scale=np.zeros((out_rows, Hs), dtype=np.float32) if Hs else None,
            written=np.zeros(out_rows, dtype=bool)))
    for g, inp in enumerate(inputs):
        idx = idxs[g].astype(np.int64)
        s = slots[g]
        T, K = idx.shape
        for k in range(K):
            valid = s[:, k] >= 0
            if not valid.any():
                continue
            dst_rank = idx[valid, k] // Le
            rows = s[valid, k]
            tok = np.flatnonzero(valid)
            for r in np.unique(dst_rank):
                sel = dst_rank == r
                if rows[sel].max() >= out_rows:
                    raise ValueError("receive buffer too small")
                outs[r].x[rows[sel]] = payloads[g][tok[sel]]
                if Hs:
                    outs[r].x_scale[rows[sel]] = scales[g][tok[sel]]
                if outs[r].written[rows[sel]].any():
                    raise AssertionError("slot written twice")
                outs[r].written[rows[sel]] = True
    for r in range(world_size):
        outs[r].slots = slots
    return outs


def world_by_rows(indices_per_group: Sequence[np.ndarray], payload_per_group: Sequence[np.ndarray],
                  scales_per_group: Sequence[Optional[np.ndarray]], *, num_experts: int,
                  world_size: int, node_size: int, dp_size: int, expert_padding: int, out_rows: int):
    """dispatch() of the whole group, written as the reference's receive loop.

    For every receiver, `process_routing_info` lists the received rows with
    their source rank, their position in the source's expert-sorted order and
    their destination row; the row behind a position is found by sorting the
    source's entries by (expert, token, k).  Handles dp groups (ranks of a group
    hold the same tokens: a2a_dispatch_send.cu:304,508, a2a_worker.rs:633).
    Returns (outs, slots): one RankOutput per RANK and, per GROUP, the pair
    (receiver, row) of every copy as two [T,K] arrays.
    """
    G = world_size // dp_size
    Le = ceil_div(num_experts, world_size)
    num_routed = np.zeros((G, num_experts), dtype=np.uint32)
    entry_at = []                          # per group: entry index behind each position
    for g in range(G):
        idx = np.asarray(indices_per_group[g]).astype(np.int64)
        count, _, _ = route(idx, num_experts)
        num_routed[g] = count
        entry_at.append(np.argsort(idx.reshape(-1), kind="stable"))
    row_bytes = payload_per_group[0].shape[1]
    Hs = scales_per_group[0].shape[1] if scales_per_group[0] is not None else 0
    outs, slot_rank, slot_row = [], [], []
    for g in range(G):
        shape = np.asarray(indices_per_group[g]).shape
        slot_rank.append(np.full(shape, -1, dtype=np.int64))
        slot_row.append(np.full(shape, -1, dtype=np.int64))
    for r in range(world_size):
        lay = process_routing_info(num_routed, r, world_size, node_size, dp_size, expert_padding, 0)
        tpe = np.zeros(Le, dtype=np.int32)
        tpe[: len(lay.tokens_per_expert)] = lay.tokens_per_expert
        out = RankOutput(num_tokens=tpe, x=np.zeros((out_rows, row_bytes), dtype=np.uint8),
                         x_scale=np.zeros((out_rows, Hs), dtype=np.float32) if Hs else None,
                         written=np.zeros(out_rows, dtype=bool))
        for i in range(lay.num_recv_tokens):
            g = int(lay.source_rank[i]) // dp_size
            entry = int(entry_at[g][int(lay.source_position[i])])
            K = np.asarray(indices_per_group[g]).shape[1]
            token, k = divmod(entry, K)
            row = int(lay.padded_index[i])
            assert not out.written[row]
            out.x[row] = payload_per_group[g][token]
            if Hs:
                out.x_scale[row] = scales_per_group[g][token]
            out.written[row] = True
            slot_rank[g][token, k] = r
            slot_row[g][token, k] = row
        outs.append(out)
    return outs, (slot_rank, slot_row)


def _load_rows(y: np.ndarray, dtype: str) -> np.ndarray:
    if dtype == "bf16":
        return bf16_to_f32(y)
    if dtype == "f16":
        return f16_to_f32(y)
    if dtype == "f32":
        return np.asarray(y, dtype=np.float32)
    raise ValueError(dtype)


def _store_rows(acc: np.ndarray, dtype: str) -> np.ndarray:
    if dtype == "bf16":
        return f32_to_bf16(acc)
    if dtype == "f16":
        return f32_to_f16(acc)
    if dtype == "f32":
        return np.asarray(acc, dtype=np.float32)
    raise ValueError(dtype)


def combine_world(expert_y: Sequence[np.ndarray], indices_per_rank,
                  weights_per_rank, slots, *, num_experts: int, world_size: int,
                  in_dtype: str = "bf16", out_dtype: str = "bf16",
                  out_prev: Optional[Sequence[Optional[np.ndarray]]] = None,
                  bound_m: Optional[Sequence[Optional[int]]] = None):
    """combine() of every rank at once; returns out_tokens per rank.

    a2a_combine_send.cu:124-136,196-205 moves `expert_y[padded_index]` back to
    the sender's row `position`; a2a_combine_recv.cu:94-148 then computes, per
    element, acc = accumulate ? out : 0; for k ascending acc += w[k]*y[k] in
    float32, and rounds once to the output type (combine_utils.cuh:108-114,
    14-23).  The multiply-add is fused (one rounding per k), emulated here in
    float64, which differs from a true fused multiply-add only in
    double-rounding corner cases.  `expert_y[r]` holds bf16/f16 codes (uint16)
    or float32; tokens beyond bound_m keep their previous contents (zeros when
    no previous output is given).
    """
    Le = ceil_div(num_experts, world_size)
    outs = []
    for g, idx in enumerate(indices_per_rank):
        idx = np.asarray(idx).astype(np.int64)
        T, K = idx.shape
        H = expert_y[0].shape[1]
        n = T if bound_m is None or bound_m[g] is None else int(bound_m[g])
        prev = None if out_prev is None else out_prev[g]
        if prev is not None:
            acc = _load_rows(prev, out_dtype).astype(np.float32).copy()
        else:
            acc = np.zeros((T, H), dtype=np.float32)
        w = np.asarray(weights_per_rank[g], dtype=np.float32)
        for k in range(K):
            if n == 0:
                break
            rows = np.zeros((n, H), dtype=np.float32)
            dst_rank = idx[:n, k] // Le
            for r in np.unique(dst_rank):
                sel = np.flatnonzero(dst_rank == r)
                rows[sel] = _load_rows(expert_y[r][slots[g][sel, k]], in_dtype)
            fused = acc[:n].astype(np.float64) + w[:n, k, None].astype(np.float64) * rows.astype(np.float64)
            acc[:n] = fused.astype(np.float32)
        out = _store_rows(acc, out_dtype)
        if prev is not None and n < T:
            out[n:] = prev[n:]
        elif n < T:
            out[n:] = 0
        outs.append(out)
    return outs
