// Device helpers shared by the routing kernels and the one-launch dispatch of
// small steps: wavefront and workgroup scans, and the layout of a receiver's
// rows from per-source totals.
#pragma once

#include "a2a_device.h"
#include "a2a_internal.h"

namespace a2a {

constexpr int kRouteWaves = kRouteBlock / kWave;

// Inclusive scan over the 64 lanes of a wavefront, on the DPP path of the
// vector unit (no LDS traffic): shifts by 1, 2, 4, 8 inside each row of 16
// lanes, then the last lane of row 0 and 2 is added to rows 1 and 3, then lane
// 31 to the upper half.
template <int CTRL, int ROW_MASK, bool ZERO_INVALID>
__device__ __forceinline__ uint32_t dpp_take(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, ROW_MASK, 0xF, ZERO_INVALID);
}

__device__ __forceinline__ uint32_t wave_inclusive_scan(uint32_t v, uint32_t lane) {
    (void)lane;
    v += dpp_take<0x111, 0xF, true>(v);    // row_shr:1
    v += dpp_take<0x112, 0xF, true>(v);    // row_shr:2
    v += dpp_take<0x114, 0xF, true>(v);    // row_shr:4
    v += dpp_take<0x118, 0xF, true>(v);    // row_shr:8
    v += dpp_take<0x142, 0xA, false>(v);   // row_bcast:15 into rows 1 and 3
    v += dpp_take<0x143, 0xC, false>(v);   // row_bcast:31 into rows 2 and 3
    return v;
}

// Inclusive scan over the first blockDim.x values (one per thread); `scratch`
// holds one word per wavefront.  Every thread of the workgroup must call.
// LDS_ONLY: with barriers that leave loads from memory in flight (lds_barrier).
template <bool LDS_ONLY = false>
__device__ __forceinline__ uint32_t block_inclusive_scan(uint32_t v, uint32_t *scratch) {
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = threadIdx.x / kWave;
    const uint32_t incl = wave_inclusive_scan(v, lane);
    if constexpr (LDS_ONLY) lds_barrier(); else __syncthreads();
    if (lane == kWave - 1) scratch[wave] = incl;
    if constexpr (LDS_ONLY) lds_barrier(); else __syncthreads();
    uint32_t before = 0;
    for (uint32_t w = 0; w < wave; ++w) before += scratch[w];
    return before + incl;
}

// The order in which receiver `r` lays out the sources (kMaxWorld bytes, four to
// a word), asked for in one go: eight independent loads, so that whoever needs the
// order later does not walk it source by source, one dependent trip each.
struct OrderWords {
    uint32_t w[kMaxWorld / 4];
};

__device__ __forceinline__ OrderWords load_order_words(const Workspace &ws, uint32_t r) {
    OrderWords o;
#pragma unroll
    for (uint32_t i = 0; i < (uint32_t)kMaxWorld / 4; ++i) o.w[i] = ws.order[r * (kMaxWorld / 4) + i];
    return o;
}

// Rows of receiver `r` from `tot[g * Le + le]`, the number of copies source g
// sends to local expert le.  `order` = load_order_words(ws, r), asked for by the
// caller as early as it can.  Whole workgroup.
__device__ inline void layout_from_totals(const FinalizeArgs &args, const Workspace &ws, uint32_t r,
                                          const uint32_t *tot, uint32_t *scratch, const OrderWords &order) {
    const uint32_t N = ws.num_groups, E = ws.num_experts, Le = ws.experts_per_rank;
    const uint32_t tid = threadIdx.x;
    const uint32_t pad = ws.expert_padding;
    const uint32_t e = r * Le + tid;
    const bool mine = tid < Le && e < E;
    uint32_t tpe = 0;
    if (mine) {
        for (uint32_t g = 0; g < N; ++g) tpe += tot[g * Le + tid];
    }
    const uint32_t padded = (tpe + pad - 1) / pad * pad;
    const uint32_t poff = block_inclusive_scan(mine ? padded : 0, scratch) - padded;
    if (mine) {
        ws.tokens_per_expert[e] = tpe;
        ws.padded_offset[e] = poff;
        if (args.out_num_tokens[r] != nullptr) args.out_num_tokens[r][tid] = (int32_t)tpe;
        if (poff + tpe > args.out_rows[r]) atomicOr(ws.err, A2A_DEV_RECV_OVERFLOW);
        // Sources in the order the reference's host worker visits them
        // (a2a_worker.rs:681-694); each gets a contiguous run of rows.
        uint32_t running = poff;
#pragma unroll
        for (uint32_t i = 0; i < (uint32_t)kMaxWorld; ++i) {
            if (i < N) {
                const uint32_t g = order.w[i / 4] >> (8 * (i % 4)) & 0xFFu;
                ws.slot_base[g * E + e] = running;
                running += tot[g * Le + tid];
            }
        }
    }
}

__device__ inline void layout_from_totals(const FinalizeArgs &args, const Workspace &ws, uint32_t r,
                                          const uint32_t *tot, uint32_t *scratch) {
    layout_from_totals(args, ws, r, tot, scratch, load_order_words(ws, r));
}

}  // namespace a2a
