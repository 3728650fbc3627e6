// Dispatch pack: read every token row once, optionally quantise it to fp8 e4m3
// with one float scale per 128 elements, and write one copy per route straight
// into the receiver's rows.
//
// What it replaces: phase 2 of the reference's dispatch-send kernel (row ->
// staging buffer per route, a2a_dispatch_send.cu:266-523) fused with the
// dispatch-recv kernel (staging -> out_x[padded_index], a2a_dispatch_recv.cu:
// 122-156).  The reference moves every copy twice; here it moves once.
//
// Design for CDNA4: one workgroup per token, one 16-byte fp8 store per lane per
// route.  In quantise mode a lane owns 16 consecutive bf16 (two 16-byte loads),
// so a 128-element scale group is exactly 8 lanes, i.e. half a DPP row: the
// group maximum takes two quad permutes and one half-row mirror, no LDS.  The
// eight scales a wavefront produces are spread over the lanes so that a single
// store instruction writes them for eight routes at once.  Row pointers are
// computed once per token by the first K lanes and read back as wave-uniform
// scalars.  Token rows are loaded non-temporally (each is read once).  The
// copies are written with cached stores at device scope: measured on this part,
// non-temporal stores to this many rows at once sustain about two thirds of
// that rate (see store_copy).
#include "a2a_device.h"
#include "a2a_scan.h"

namespace a2a {

namespace {

constexpr int kMaxLdsScales = 1024;

// Arguments travel by value; a launch can carry 4 KB of them.
static_assert(sizeof(PushArgs) + sizeof(FinalizeArgs) + sizeof(Workspace) <= 4096, "kernel arguments too large");

// The 16-byte store of a dispatched copy, at device scope (`sc1`): the line is written through
// instead of staying dirty in the L2 of the storing die.  Measured on the 4096-token pack against
// the other policies of the store: non-temporal 62 us, ordinary 50.3 us, device scope 49.7 us
// (plain kernels of the same shape: 63 / 48.5 / 47.4 us).
__device__ __forceinline__ void store_copy(u32x4 v, u32x4 *p) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
}

// Moves the row of `token` to its copies.  Lanes 0..K-1 of EVERY wavefront hold
// the row pointer, scale pointer and scale stride of route k (0 = no copy).
// The row is loaded here, AFTER the routes are known, unless the caller passes
// its first piece (PRE): in the bandwidth-bound pack of a large step asking for
// it earlier was 4 us slower; the latency-bound one-launch kernels ask for it at
// their head.
// The work is done by a TEAM of `team_threads` threads (a multiple of 64), in
// which the caller is thread `team_tid`; a workgroup is one team or several of
// the same size, each with a token and LDS arrays of its own.  Every thread of
// the workgroup must call (there is a barrier inside); a team without a token
// passes `live` false.
// PRE: the thread's first piece of the row was asked for earlier (first_piece) and is passed in.
template <bool QUANT, bool PRE = false>
__device__ __forceinline__ void push_rows(const PushArgs &args, const PushSrc &src, uint32_t token, uint32_t K,
                                          uint64_t row_ptr, uint64_t scale_ptr, uint32_t scale_stride,
                                          float *s_scale, uint64_t *s_scale_ptr, uint32_t *s_scale_stride,
                                          uint32_t team_tid, uint32_t team_threads, bool live,
                                          u32x4 pre_a = u32x4{0, 0, 0, 0}, u32x4 pre_b = u32x4{0, 0, 0, 0}) {
    const uint32_t tid = team_tid;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = tid / kWave;
    const uint8_t *x_row = src.x + (size_t)token * src.x_stride;

    if constexpr (QUANT) {
        const uint32_t num_chunks = live ? args.hidden_dim / 16 : 0;  // 16 bf16 in, 16 fp8 out per lane
        const uint32_t Hs = args.hidden_dim_scale;
        for (uint32_t base = wave * kWave; base < num_chunks; base += team_threads) {
            const uint32_t c = base + lane;
            const bool active = c < num_chunks;
            u32x4 a = {0, 0, 0, 0}, b = {0, 0, 0, 0};
            if (PRE && base == wave * kWave) {
                a = pre_a;
                b = pre_b;
            } else if (active) {
                const u32x4 *p = reinterpret_cast<const u32x4 *>(x_row + (size_t)c * 32);
                a = __builtin_nontemporal_load(p);
                b = __builtin_nontemporal_load(p + 1);
            }
            float scale;
            const u32x4 q = quantize16(a, b, &scale);
            for (uint32_t k = 0; k < K; ++k) {
                const uint64_t row = read_lane64(row_ptr, k);
                if (row != 0 && active) {
                    store_copy(q, reinterpret_cast<u32x4 *>(row + (size_t)c * 16));
                }
            }
            if (active && (lane & 7) == 0 && c / 8 < kMaxLdsScales) s_scale[c / 8] = scale;
        }
        // The token's scales meet in LDS so that each copy's scale row goes out
        // as one contiguous run instead of one 32-byte piece per wavefront.
        if (wave == 0 && lane < K) {
            s_scale_ptr[lane] = live ? scale_ptr : 0;
            s_scale_stride[lane] = scale_stride;
        }
        lds_barrier();   // (the row's stores and whatever the caller has asked for stay in flight)
        const uint32_t Hl = Hs < (uint32_t)kMaxLdsScales ? Hs : (uint32_t)kMaxLdsScales;
        for (uint32_t i = tid; i < K * Hl; i += team_threads) {
            const uint32_t k = i / Hl;
            const uint32_t j = i - k * Hl;
            const uint64_t sp = s_scale_ptr[k];
            if (sp != 0) reinterpret_cast<float *>(sp)[(size_t)j * s_scale_stride[k]] = s_scale[j];
        }
    } else {
        const uint32_t num_chunks = live ? args.row_bytes / 16 : 0;
        for (uint32_t c = tid; c < num_chunks; c += team_threads) {
            const u32x4 v = PRE && c == tid ? pre_a : __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(x_row) + c);
            for (uint32_t k = 0; k < K; ++k) {
                const uint64_t row = read_lane64(row_ptr, k);
                if (row != 0) {
                    reinterpret_cast<u32x4 *>(row)[c] = v;
                }
            }
        }
        if (src.x_scale != nullptr && live) {
            const float *xs = src.x_scale + (size_t)token * src.xs_stride_token;
            for (uint32_t j = tid; j < args.hidden_dim_scale; j += team_threads) {
                const float s = xs[(size_t)j * src.xs_stride_elem];
                for (uint32_t k = 0; k < K; ++k) {
                    const uint64_t sp = read_lane64(scale_ptr, k);
                    const uint32_t ss = __builtin_amdgcn_readlane((int)scale_stride, (int)k);
                    if (sp != 0) reinterpret_cast<float *>(sp)[(size_t)j * ss] = s;
                }
            }
        }
    }
}

// The piece of `token`'s row that thread `team_tid` of a team handles first in push_rows, asked for
// ahead of time (zeros where push_rows would not load).
template <bool QUANT>
__device__ __forceinline__ void first_piece(const PushArgs &args, const PushSrc &src, uint32_t token,
                                            uint32_t team_tid, bool live, u32x4 *a, u32x4 *b) {
    const uint8_t *x_row = src.x + (size_t)token * src.x_stride;
    *a = u32x4{0, 0, 0, 0};
    *b = u32x4{0, 0, 0, 0};
    if constexpr (QUANT) {
        if (live && team_tid < args.hidden_dim / 16) {
            const u32x4 *p = reinterpret_cast<const u32x4 *>(x_row + (size_t)team_tid * 32);
            *a = __builtin_nontemporal_load(p);
            *b = __builtin_nontemporal_load(p + 1);
        }
    } else {
        if (live && team_tid < args.row_bytes / 16) {
            *a = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(x_row) + team_tid);
        }
    }
}

// Where the copy of one route goes: row `slot` of the receiver described by `dst`.
// Returns the slot that is recorded for the combine (kInvalidSlot if the row
// does not fit the receiver's buffer).  Written without branches on purpose:
// the descriptor is read in one go and everything else is a select, so a lane
// that resolves a route makes ONE trip to memory here, not one per condition
// (under a saturated memory system every dependent trip costs microseconds).
__device__ __forceinline__ uint32_t resolve_copy(const PushDst &dst, const Workspace &ws, uint32_t slot,
                                                 bool flag_overflow, uint64_t *row_ptr, uint64_t *scale_ptr,
                                                 uint32_t *scale_stride) {
    const uint64_t out_x = (uint64_t)dst.out_x;
    const uint64_t out_scale = (uint64_t)dst.out_scale;
    const uint64_t out_stride = dst.out_stride;
    const uint32_t os_elem = dst.os_stride_elem;
    const uint32_t os_token = dst.os_stride_token;
    const uint32_t out_rows = dst.out_rows;
    const bool wanted = out_x != 0;
    const bool fits = slot < out_rows;
    const bool copy = wanted && fits;
    const bool scales = copy && out_scale != 0;
    *row_ptr = copy ? out_x + (uint64_t)slot * out_stride : 0;
    *scale_ptr = scales ? out_scale + (uint64_t)slot * os_token * sizeof(float) : 0;
    *scale_stride = scales ? os_elem : 0;
    if (wanted && !fits && flag_overflow) atomicOr(ws.err, A2A_DEV_RECV_OVERFLOW);
    return wanted && !fits ? kInvalidSlot : slot;
}

uint32_t push_threads(const PushArgs &args, bool quantize) {
    const uint32_t chunks = quantize ? args.hidden_dim / 16 : args.row_bytes / 16;
    uint32_t threads = (chunks + kWave - 1) / kWave * kWave;
    if (threads < (uint32_t)kWave) threads = kWave;
    if (threads > 1024) threads = 1024;
    return threads;
}

}  // namespace

template <bool QUANT>
__global__ __launch_bounds__(1024) void dispatch_push_kernel(const PushArgs args,
                                                             const Workspace ws) {
    // Scales of one token (one per 128 elements) and where each copy's go.
    __shared__ float s_scale[QUANT ? kMaxLdsScales : 1];
    __shared__ uint64_t s_scale_ptr[A2A_MAX_EXPERTS_PER_TOKEN];
    __shared__ uint32_t s_scale_stride[A2A_MAX_EXPERTS_PER_TOKEN];
    __shared__ uint64_t s_row_ptr[A2A_MAX_EXPERTS_PER_TOKEN];
    __shared__ uint64_t s_route_scale_ptr[A2A_MAX_EXPERTS_PER_TOKEN];
    __shared__ uint32_t s_route_scale_stride[A2A_MAX_EXPERTS_PER_TOKEN];

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = tid / kWave;
    const uint32_t E = ws.num_experts;
    const uint32_t K = ws.topk;

    uint32_t g = 0;
    while (g + 1 < ws.num_groups && blockIdx.x >= args.token_start[g + 1]) ++g;
    const uint32_t token = blockIdx.x - args.token_start[g];
    const PushSrc &src = args.src[g];
    if (token >= effective_tokens(src.bound_m, src.num_tokens)) return;

    // Lanes 0..K-1 of wavefront 0 resolve one route each and hand the result to
    // the other wavefronts through LDS.
    if (wave == 0 && lane < K) {
        uint64_t row_ptr = 0, scale_ptr = 0;
        uint32_t scale_stride = 0;
        const uint32_t entry = token * K + lane;
        const uint32_t expert =
            (uint32_t)src.indices[(size_t)token * src.indices_stride + lane];
        uint32_t slot = kInvalidSlot, toff = 0;
        if (expert < E) {
            const uint32_t chunk = entry / kRouteBlock;
            toff = ws.block_prefix[((size_t)g * ws.nb_max + chunk) * E + expert] +
                   ws.local_rank[(size_t)g * ws.max_tk + entry];
            slot = ws.slot_base[g * E + expert] + toff;
            slot = resolve_copy(args.dst[owner_of_expert(ws, expert)], ws, slot, true, &row_ptr, &scale_ptr,
                                &scale_stride);
        }
        ws.route_slot[(size_t)g * ws.max_tk + entry] = slot;
        ws.token_offset[(size_t)g * ws.max_tk + entry] = toff;
        s_row_ptr[lane] = row_ptr;
        s_route_scale_ptr[lane] = scale_ptr;
        s_route_scale_stride[lane] = scale_stride;
    }
    __syncthreads();
    uint64_t row_ptr = 0, scale_ptr = 0;
    uint32_t scale_stride = 0;
    if (lane < K) {
        row_ptr = s_row_ptr[lane];
        scale_ptr = s_route_scale_ptr[lane];
        scale_stride = s_route_scale_stride[lane];
    }
    push_rows<QUANT>(args, src, token, K, row_ptr, scale_ptr, scale_stride, s_scale, s_scale_ptr, s_scale_stride,
                     threadIdx.x, blockDim.x, true);
}

// Routing pass and dispatch pack in ONE launch, for small steps (decode).  The
// grid holds one workgroup per token, then one per receiver; none depends on
// another, because every workgroup counts, by itself, what it needs to know
// about the whole step:
//  - a token workgroup counts the entries of every
//    source per (source, expert) and the entries of its own source before its
//    token per expert (LDS atomics: counts do not depend on arrival order), and
//    from those derives the receiver rows of its K copies exactly as the
//    two-launch pass does: first row of the expert in its receiver + copies of
//    the sources the receiver lays out earlier + copies of its own source
//    before it, in (token, k) order.  The workgroup of a source's first token
//    also publishes the source's per-expert totals and their scan.
//  - a receiver workgroup counts the copies bound for its experts and lays out
//    its rows (expert counts for the caller, first row per expert and source).
// The counting is redundant: its cost grows with tokens x entries, so the host
// takes this path only below a bound on the entries of a step.
//
//
// SINGLE: the common shape of a decode step on one GPU's share: exactly one
// source has tokens and its index rows are dense (stride K).  Then the entries
// of the step are one flat array, read directly: no table of where every
// token's ids are (building it costs a trip to memory before the counting can
// start), no division of entry numbers, and no copies of other sources to
// place before mine, so the order in which receivers lay out their sources
// drops out too.  (With at most eight routes a token and a row that one
// workgroup covers with a wavefront to spare, such a step takes
// dispatch_quick_kernel instead; this variant serves the rest.)
//
// Dynamic LDS: (G + 3) * E words and 8 bytes per token of the step; SINGLE:
// 4 * E words (or G * Le, if that is more: the receiver workgroups' table).
template <bool QUANT, bool SINGLE>
__global__ __launch_bounds__(1024) void dispatch_small_kernel(const PushArgs args, const FinalizeArgs fin,
                                                              const Workspace ws) {
    if constexpr (SINGLE) {
        // everything the head of a workgroup needs from the argument block, asked for in one go; the
        // same in the kernel of a larger single source gained nothing and is left out there
        A2A_PIN(args.token_start[kMaxWorld]);
        A2A_PIN(args.single_source);
        A2A_PIN(args.hidden_dim);
        A2A_PIN(args.hidden_dim_scale);
        A2A_PIN(args.row_bytes);
        A2A_PIN(args.single.x);
        A2A_PIN(args.single.indices);
        A2A_PIN(args.single.bound_m);
        A2A_PIN(args.single.x_stride);
        A2A_PIN(args.single.indices_stride);
        A2A_PIN(args.single.num_tokens);
        A2A_PIN(fin.recv_mask);
        A2A_PIN(ws.world);
        A2A_PIN(ws.num_groups);
        A2A_PIN(ws.num_experts);
        A2A_PIN(ws.topk);
        A2A_PIN(ws.experts_per_rank);
        A2A_PIN(ws.le_magic);
        A2A_PIN(ws.expert_padding);
        A2A_PIN(ws.max_tk);
        A2A_PIN(ws.order);
        A2A_PIN(ws.num_routed);
        A2A_PIN(ws.expert_offsets);
        A2A_PIN(ws.route_slot);
        A2A_PIN(ws.token_offset);
        A2A_PIN(ws.err);
    }
    extern __shared__ uint64_t s_dyn64[];
    uint32_t *s_dyn = reinterpret_cast<uint32_t *>(s_dyn64);
    __shared__ float s_scale[QUANT ? kMaxLdsScales : 1];
    __shared__ uint64_t s_scale_ptr[A2A_MAX_EXPERTS_PER_TOKEN];
    __shared__ uint32_t s_scale_stride[A2A_MAX_EXPERTS_PER_TOKEN];
    __shared__ PushDst s_dst[kMaxWorld];                      // per receiver: its buffers
    __shared__ uint32_t s_order[kMaxWorld * kMaxWorld / 4];   // [receiver] bytes: i -> source
    __shared__ uint32_t scratch[kRouteWaves];
    __shared__ uint32_t s_carry;

    const uint32_t tid = threadIdx.x;
    // read once: used after LDS atomics and barriers, the compiler would fetch it again from the
    // launch's implicit arguments each time, a trip to memory in the middle of the chain
    const uint32_t nthreads = blockDim.x;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = tid / kWave;
    const uint32_t G = ws.num_groups, E = ws.num_experts, K = ws.topk, Le = ws.experts_per_rank;
    const uint32_t total_tokens = args.token_start[kMaxWorld];   // the total, at a fixed place
    const uint32_t total_entries = total_tokens * K;
    const bool receiver = blockIdx.x >= total_tokens;

    // SINGLE: the entries are asked for first of all: they travel while the tables are cleared and
    // the receivers' descriptors copied, instead of after them (one trip to memory less in a chain
    // of five).
    constexpr uint32_t kBatch = 8;
    uint32_t early[kBatch];
    uint32_t early_mine = 0xFFFFFFFFu;
    if constexpr (SINGLE) {
        // Without a branch around any of them (an address inside the array for every lane; which of the
        // values count is decided where they are used), so that all of them are in flight together and
        // each is waited for by itself.
        const PushSrc &one = args.single;
        const uint32_t entries = one.num_tokens * K;   // > 0: the one source has tokens
#pragma unroll
        for (uint32_t j = 0; j < kBatch; ++j) {
            const uint32_t f = j * nthreads + tid;
            early[j] = (uint32_t)one.indices[f < entries ? f : entries - 1];
        }
        early_mine = (uint32_t)one.indices[(size_t)(receiver ? 0 : blockIdx.x) * one.indices_stride + (lane < K ? lane : 0)];
    }
    // A receiver workgroup also asks for the order in which it lays out the sources, a token
    // workgroup, further down, for its row (what the chain waits for first goes first).  A step
    // this small leaves the memory system idle, so the row is there when the routes are known; in
    // the larger steps of the other dispatch kernels the same early request delays the entries.
    OrderWords my_order = {};
    if (receiver) my_order = load_order_words(ws, blockIdx.x - total_tokens);

    // Per token of the step (all sources, in grid order): where its K expert ids
    // are, with the source in the top byte; 0 for tokens past their source's
    // bound.  This is what the counting pass below looks up per entry.
    const uint32_t table_words = ((G + 3) * E + 1) & ~1u;
    uint64_t *tok_ids = reinterpret_cast<uint64_t *>(s_dyn + table_words);
    for (uint32_t ft = tid; !SINGLE && ft < total_tokens; ft += nthreads) {
        // token_start is non-decreasing and equals the total from G on, so the
        // fixed trip count is safe and lets the loads go out together
        uint32_t g = 0, start = 0;
#pragma unroll
        for (uint32_t gg = 1; gg < (uint32_t)kMaxWorld; ++gg) {
            const uint32_t first = args.token_start[gg];
            if (ft >= first) {
                g = gg;
                start = first;
            }
        }
        const PushSrc &from = args.src[g];
        const uint32_t t = ft - start;
        const uint64_t ids = (uint64_t)(from.indices + (size_t)t * from.indices_stride) | (uint64_t)g << 56;
        tok_ids[ft] = t < effective_tokens(from.bound_m, from.num_tokens) ? ids : 0;
    }
    // SINGLE: a token workgroup keeps only the row of the one source, at the front
    // [G][E] (SINGLE: [E]): low half of a word the entries of (source, expert), high half (own source only)
    // those of the tokens before mine; receivers: [G][Le] plain counts.  A step of this kernel has at most
    // kSmallMaxEntries < 2^16 entries.
    uint32_t *cnt = s_dyn;
    uint32_t *rows_before = s_dyn + (SINGLE ? (size_t)E : (size_t)G * E);   // [E] padded rows of all experts before e
    uint32_t *copies_before = rows_before + E;              // [E] copies of the sources laid out before mine
    const uint32_t table = receiver ? G * Le : G * E;
    if (SINGLE && !receiver) {
        for (uint32_t i = tid; i < E; i += nthreads) s_dyn[i] = 0;
    } else {
        for (uint32_t i = tid; i < table; i += nthreads) s_dyn[i] = 0;
    }
    uint32_t my_g = 0, token = 0;
    if constexpr (SINGLE) {
        my_g = args.single_source - 1;      // receivers too: the one source they count
        token = receiver ? 0 : blockIdx.x;
    } else if (!receiver) {
        while (my_g + 1 < G && blockIdx.x >= args.token_start[my_g + 1]) ++my_g;
        token = blockIdx.x - args.token_start[my_g];
    }
    // The receivers' descriptors are asked for here and written to LDS after the counting: written
    // here, the wait for them would also wait for the entries and the row asked for above.
    // (field by field and without a branch, so that they stay in registers and nothing waits for them
    // before their use)
    const PushDst &dst_of_tid = args.dst[tid < ws.world ? tid : 0];
    uint8_t *const my_out_x = dst_of_tid.out_x;
    float *const my_out_scale = dst_of_tid.out_scale;
    const uint64_t my_out_stride = dst_of_tid.out_stride;
    const uint32_t my_os_elem = dst_of_tid.os_stride_elem, my_os_token = dst_of_tid.os_stride_token;
    const uint32_t my_out_rows = dst_of_tid.out_rows;
    // The row comes last: the chain needs it last, and what is asked for later is waited for later.
    u32x4 pre_a = {0, 0, 0, 0}, pre_b = {0, 0, 0, 0};
    bool pre_live = false;
    if constexpr (SINGLE) {
        const PushSrc &one = args.single;
        pre_live = !receiver && blockIdx.x < effective_tokens(one.bound_m, one.num_tokens);
        first_piece<QUANT>(args, one, blockIdx.x, tid, pre_live, &pre_a, &pre_b);
    }
    // Sources without tokens have no workgroup of their own: the first receiver
    // workgroup (the first workgroup, if nobody receives) clears their tables.
    if (blockIdx.x == (fin.recv_mask != 0 ? total_tokens : 0)) {
        for (uint32_t g = 0; g < G; ++g) {
            if (args.src[g].num_tokens != 0) continue;
            for (uint32_t e = tid; e < E; e += nthreads) {
                ws.num_routed[g * E + e] = 0;
                ws.expert_offsets[g * E + e] = 0;
            }
        }
    }
    __syncthreads();

    // One pass over the entries of all sources, kBatch loads in flight per lane.
    const PushSrc &src = SINGLE ? args.single : args.src[my_g];
    const uint32_t rank = blockIdx.x - total_tokens;        // receivers only
    // flat index of my first entry (the one source of SINGLE is the first with tokens: it starts at 0)
    const uint32_t my_first = ((SINGLE ? 0 : args.token_start[my_g]) + token) * K;
    uint32_t my_expert = 0xFFFFFFFFu;
    // The order in which every receiver lays out the sources comes from device
    // memory: asked for here, stored to LDS after the counting.
    const uint32_t order_words = receiver || SINGLE ? 0 : ws.world * (kMaxWorld / 4);
    const uint32_t order_word = tid < order_words ? ws.order[tid] : 0;
    const uint32_t flat_entries = SINGLE ? effective_tokens(src.bound_m, src.num_tokens) * K : 0;
    // counts one batch of entries: entry j of the batch is f0 + j * nthreads + tid
    auto count_batch = [&](const uint32_t (&expert)[kBatch], const uint32_t (&src_of)[kBatch], uint32_t f0) {
#pragma unroll
        for (uint32_t j = 0; j < kBatch; ++j) {
            const uint32_t x = expert[j];
            if (x >= E) continue;
            if (receiver) {
                const uint32_t le = x - rank * Le;   // wraps for experts of lower ranks
                if (le < Le) atomicAdd(&cnt[src_of[j] * Le + le], 1u);
            } else {
                const uint32_t f = f0 + j * nthreads + tid;
                atomicAdd(&cnt[(SINGLE ? 0 : src_of[j]) * E + x], src_of[j] == my_g && f < my_first ? 0x10001u : 1u);
            }
        }
    };
    uint32_t f_begin = 0;
    if constexpr (SINGLE) {
        // The first batch was asked for at the head.  It is counted here in straight-line code, outside
        // the loop: each of its values is then waited for by itself, and the row and the descriptors
        // asked for after them stay in flight meanwhile.
        uint32_t expert[kBatch], src_of[kBatch];
#pragma unroll
        for (uint32_t j = 0; j < kBatch; ++j) {
            const uint32_t f = j * nthreads + tid;
            expert[j] = f < flat_entries ? early[j] : 0xFFFFFFFFu;
            src_of[j] = my_g;
        }
        if (!receiver && lane < K) my_expert = early_mine;
        count_batch(expert, src_of, 0);
        f_begin = kBatch * nthreads;
    }
    for (uint32_t f0 = f_begin; f0 < total_entries || (!SINGLE && f0 == 0); f0 += kBatch * nthreads) {
        uint32_t expert[kBatch], src_of[kBatch];
#pragma unroll
        for (uint32_t j = 0; j < kBatch; ++j) {
            const uint32_t f = f0 + j * nthreads + tid;
            expert[j] = 0xFFFFFFFFu;
            src_of[j] = SINGLE ? my_g : 0;
            if constexpr (SINGLE) {
                if (f < flat_entries) expert[j] = (uint32_t)src.indices[f];
            } else if (f < total_entries) {
                const uint32_t flat_token = K > 1 ? __umulhi(f, args.topk_magic) : f;
                const uint64_t ids = tok_ids[flat_token];
                src_of[j] = (uint32_t)(ids >> 56);
                if (ids != 0) {
                    expert[j] = (uint32_t) reinterpret_cast<const int32_t *>(ids & 0x00FFFFFFFFFFFFFFull)[f - flat_token * K];
                }
            }
        }
        if (!SINGLE && f0 == 0 && !receiver && lane < K) {
            my_expert = (uint32_t)src.indices[(size_t)token * src.indices_stride + lane];
        }
        count_batch(expert, src_of, f0);
    }
    if (!receiver && tid < ws.world) {
        s_dst[tid] = PushDst{my_out_x, my_out_scale, my_out_stride, my_os_elem, my_os_token, my_out_rows, 0};
    }
    if (tid < order_words) s_order[tid] = order_word;
    for (uint32_t i = tid + nthreads; i < order_words; i += nthreads) s_order[i] = ws.order[i];
    __syncthreads();

    if (receiver) {
        if (fin.recv_mask >> rank & 1) layout_from_totals(fin, ws, rank, cnt, scratch, my_order);
        return;
    }

    const uint32_t pad = ws.expert_padding;
    // Per expert: padded rows of the experts before it (a scan; the difference to
    // the scan at the first expert of a receiver is the expert's first row there)
    // and the copies of the sources its receiver lays out before mine.
    uint32_t carry = 0;
    for (uint32_t e0 = 0; e0 < E; e0 += nthreads) {
        const uint32_t e = e0 + tid;
        uint32_t total = 0, before = 0;
        if (SINGLE) {
            total = e < E ? cnt[e] & 0xFFFFu : 0;   // nobody else sends: nothing is laid out before mine
        } else if (e < E) {
            const uint32_t r = owner_of_expert(ws, e);
            bool seen = false;
            // eight sources at a time, their LDS reads in flight together
            for (uint32_t i0 = 0; i0 < G; i0 += 8) {
                const uint32_t w0 = s_order[r * (kMaxWorld / 4) + i0 / 4];
                const uint32_t w1 = s_order[r * (kMaxWorld / 4) + i0 / 4 + 1];
                uint32_t g[8], c[8];
#pragma unroll
                for (uint32_t j = 0; j < 8; ++j) {
                    g[j] = (j < 4 ? w0 >> (8 * j) : w1 >> (8 * (j - 4))) & 0xFFu;
                    c[j] = i0 + j < G ? cnt[g[j] * E + e] & 0xFFFFu : 0;
                }
#pragma unroll
                for (uint32_t j = 0; j < 8; ++j) {
                    seen = seen || (i0 + j < G && g[j] == my_g);
                    if (!seen) before += c[j];
                    total += c[j];
                }
            }
        }
        const uint32_t padded = e < E ? (total + pad - 1) / pad * pad : 0;
        const uint32_t incl = carry + block_inclusive_scan(padded, scratch);
        if (e < E) {
            rows_before[e] = incl - padded;
            copies_before[e] = before;
        }
        if (e0 + nthreads < E) {   // uniform: another round follows
            if (tid == nthreads - 1) s_carry = incl;
            __syncthreads();
            carry = s_carry;
        }
    }
    __syncthreads();

    // The first token's workgroup publishes its source's totals (last wavefront).
    if (token == 0 && wave == nthreads / kWave - 1) {
        uint32_t run = 0;
        for (uint32_t e0 = 0; e0 < E; e0 += kWave) {
            const uint32_t e = e0 + lane;
            const uint32_t v = e < E ? cnt[(SINGLE ? 0 : my_g) * E + e] & 0xFFFFu : 0;
            const uint32_t incl = run + wave_inclusive_scan(v, lane);
            if (e < E) {
                ws.num_routed[my_g * E + e] = v;
                ws.expert_offsets[my_g * E + e] = incl;
            }
            run = __shfl(incl, kWave - 1);
        }
    }
    if (token >= effective_tokens(src.bound_m, src.num_tokens)) return;   // nothing to send (uniform)

    // Lanes 0..K-1 of every wavefront resolve one route each, from LDS alone.
    uint32_t repeats = 0;   // copies of this token to the same expert at an earlier k
    for (uint32_t k = 0; k + 1 < K; ++k) {
        const uint32_t other = (uint32_t)__builtin_amdgcn_readlane((int)my_expert, (int)k);
        if (k < lane && other == my_expert) ++repeats;
    }
    uint64_t row_ptr = 0, scale_ptr = 0;
    uint32_t scale_stride = 0;
    if (lane < K) {
        const uint32_t entry = token * K + lane;
        uint32_t slot = kInvalidSlot, toff = 0;
        if (my_expert < E) {
            // copies of my source before this one: earlier tokens, then earlier k of this token
            toff = (cnt[(SINGLE ? 0 : my_g) * E + my_expert] >> 16) + repeats;
            const uint32_t r = owner_of_expert(ws, my_expert);
            const uint32_t row = rows_before[my_expert] - rows_before[r * Le] + copies_before[my_expert];
            slot = resolve_copy(s_dst[r], ws, row + toff, wave == 0, &row_ptr, &scale_ptr, &scale_stride);
        } else if (wave == 0) {
            atomicOr(ws.err, A2A_DEV_BAD_EXPERT_ID);
        }
        if (wave == 0) {
            ws.route_slot[(size_t)my_g * ws.max_tk + entry] = slot;
            ws.token_offset[(size_t)my_g * ws.max_tk + entry] = toff;
        }
    }
    if constexpr (SINGLE) {
        push_rows<QUANT, true>(args, src, token, K, row_ptr, scale_ptr, scale_stride, s_scale, s_scale_ptr,
                               s_scale_stride, threadIdx.x, nthreads, true, pre_a, pre_b);
    } else {
        push_rows<QUANT>(args, src, token, K, row_ptr, scale_ptr, scale_stride, s_scale, s_scale_ptr, s_scale_stride,
                         threadIdx.x, nthreads, true);
    }
}

// The quick form of the one-launch dispatch of a small step: ONE source has tokens, its index rows
// are dense, a token has at most eight routes, and the row is one piece per thread (16 elements to
// quantise, or 16 bytes to move as they are) with a wavefront to spare (the host launches one more
// than the row has pieces for).
// One workgroup per token, no receiver workgroups.
//
// In dispatch_small_kernel every wavefront walks the same chain once its data is there: count, a
// scan of all experts' rows, its routes, quantise, K stores behind a loop's branches, scales; at
// 128 tokens that chain was 2.9 us of a 4.1 us kernel with everything it reads already arrived,
// and the receivers' workgroups, which start last and walk a chain of their own, ended 1.5 us
// after the last row was out.  Here
//  - the spare wavefront (the RESOLVER) does not count: from the token's ids it prepares what the
//    routes need that no count decides (receiver, descriptor, copies of the token to the same
//    expert at an earlier k), waits until every counting wavefront has said that its entries are
//    counted (a word in LDS, not a barrier: the counting wavefronts do not wait for each other or
//    for the resolver here), and then needs five words of the table per lane: a route's first row
//    is the padded rows of the experts of ITS receiver before it, at most Le - 1 terms, summed by
//    eight lanes, not a scan over all experts;
//  - the other wavefronts count their entries, say so, and quantise their piece of the row while
//    the resolver works; the routes and the scales meet in LDS at the one barrier that follows;
//  - the K stores of a piece are straight-line code for K = 8;
//  - with one source a workgroup's own table holds everything a receiver's layout needs: the
//    resolvers of the first world + G + 1 workgroups write the step's tables, one job each, while
//    the others store rows (done by all workgroups, a share of the experts each, the same stores
//    were 0.3 us slower than with receiver workgroups: many wavefronts writing parts of the
//    same lines).
// 128 tokens, hidden 7168: 5.95 -> 4.5 us per dispatch at the GPU's own pace; hidden 2048: 5.8 -> 4.2.
// (Two workgroups per token, half a row each, so that all compute units have one: 4.65 and 5.3 us.)
//
// Dynamic LDS: E words.
constexpr uint32_t kQuickSpinLimit = 1u << 22;   // (a resolver that gives up flags A2A_DEV_INTERNAL; never seen)

//
// NB: entries a counting thread asks for at the head (the host picks the smallest of 1, 2, 3, 4, 8
// that covers the step; entries beyond NB per thread are counted by a loop).  Every one of them
// costs each wavefront a dozen instructions whether it exists or not, and two wavefronts share a
// SIMD here.
//
// QUANT false: the rows travel as they are (the caller's fp8 bytes, or any other element type), one
// 16-byte piece per thread, and the caller's scales, if it passed any, are copied beside them.
template <uint32_t NB, bool QUANT>
__global__ __launch_bounds__(1024) void dispatch_quick_kernel(const PushArgs args, const FinalizeArgs fin,
                                                              const Workspace ws) {
    // everything the head of a workgroup needs from the argument block, asked for in one go
    A2A_PIN(args.single_source);
    A2A_PIN(args.hidden_dim);
    A2A_PIN(args.hidden_dim_scale);
    A2A_PIN(args.single.x);
    A2A_PIN(args.single.indices);
    A2A_PIN(args.single.bound_m);
    A2A_PIN(args.single.x_stride);
    A2A_PIN(args.single.num_tokens);
    if constexpr (!QUANT) {
        A2A_PIN(args.row_bytes);
        A2A_PIN(args.single.x_scale);
        A2A_PIN(args.single.xs_stride_elem);
        A2A_PIN(args.single.xs_stride_token);
    }
    A2A_PIN(fin.recv_mask);
    A2A_PIN(ws.world);
    A2A_PIN(ws.num_groups);
    A2A_PIN(ws.num_experts);
    A2A_PIN(ws.topk);
    A2A_PIN(ws.experts_per_rank);
    A2A_PIN(ws.le_magic);
    A2A_PIN(ws.expert_padding);
    A2A_PIN(ws.max_tk);
    A2A_PIN(ws.laid_before);
    A2A_PIN(ws.route_slot);
    A2A_PIN(ws.token_offset);
    A2A_PIN(ws.err);
    // the buffer for the counts and the rows of the receiver this workgroup's resolver may lay out at
    // its end (receiver blockIdx.x; the index is kept inside the array, whether it is a receiver is
    // decided at the use)
    int32_t *const duty_out_tokens = fin.out_num_tokens[blockIdx.x & (kMaxWorld - 1)];
    const uint32_t duty_out_rows = fin.out_rows[blockIdx.x & (kMaxWorld - 1)];
    A2A_PIN(duty_out_tokens);
    A2A_PIN(duty_out_rows);

    extern __shared__ uint32_t s_cnt[];   // [E]: low half of a word the entries of the expert, high half those of
                                          // the tokens before mine (a step of this kernel has < 2^16 entries)
    __shared__ float s_scale[kMaxLdsScales];
    __shared__ uint64_t s_row_ptr[8];
    __shared__ uint64_t s_scale_ptr[8];
    __shared__ uint32_t s_scale_stride[8];
    __shared__ uint32_t s_counted;        // counting wavefronts whose entries are in the table

    const uint32_t tid = threadIdx.x;
    const uint32_t nthreads = blockDim.x;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = tid / kWave;
    const uint32_t waves = nthreads / kWave;
    const bool resolver = wave == waves - 1;
    const uint32_t counters = nthreads - kWave;   // threads that count entries and move the row
    const uint32_t G = ws.num_groups, E = ws.num_experts, K = ws.topk, Le = ws.experts_per_rank;
    const uint32_t pad = ws.expert_padding;
    const PushSrc &one = args.single;
    const uint32_t my_g = args.single_source - 1;
    const uint32_t token = blockIdx.x;
    const uint32_t tokens = one.num_tokens;        // the grid: one workgroup per token
    const uint32_t entries = tokens * K;           // > 0
    const uint32_t my_first = token * K;
    const uint32_t num_chunks = QUANT ? args.hidden_dim / 16 : args.row_bytes / 16;   // pieces of a row, one per thread
    const uint32_t Hs = args.hidden_dim_scale;

    // What each kind of wavefront takes from memory, asked for before anything else is done: the
    // entries, then the thread's piece of the row; the resolver its token's ids (laid out as it uses
    // them: eight lanes per route), the receivers' descriptors (lane r: receiver r) and which sources
    // the receiver it may lay out visits before mine.
    constexpr uint32_t kBatch = NB;
    uint32_t early[kBatch] = {};
    u32x4 pre_a = {0, 0, 0, 0}, pre_b = {0, 0, 0, 0};
    uint32_t id_route = 0xFFFFFFFFu, id_part = 0xFFFFFFFFu, duty_before = 0;
    uint64_t my_out_x = 0, my_out_scale = 0, my_out_stride = 0;
    uint32_t my_os_elem = 0, my_os_token = 0, my_out_rows = 0;
    const uint32_t part = lane & 7, route = lane >> 3;
    if (!resolver) {
#pragma unroll
        for (uint32_t j = 0; j < kBatch; ++j) {
            const uint32_t f = j * counters + tid;
            early[j] = (uint32_t)one.indices[f < entries ? f : entries - 1];
        }
        if (tid < num_chunks) {
            if constexpr (QUANT) {
                const u32x4 *p = reinterpret_cast<const u32x4 *>(one.x + (size_t)token * one.x_stride + (size_t)tid * 32);
                pre_a = __builtin_nontemporal_load(p);
                pre_b = __builtin_nontemporal_load(p + 1);
            } else {
                pre_a = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(one.x + (size_t)token * one.x_stride) + tid);
            }
        }
        if constexpr (!QUANT) {
            // the caller's scales of this token (one per thread; kept in pre_b's first word)
            if (one.x_scale != nullptr && tid < Hs && tid < (uint32_t)kMaxLdsScales) {
                pre_b.x = __float_as_uint(one.x_scale[(size_t)token * one.xs_stride_token + (size_t)tid * one.xs_stride_elem]);
            }
        }
    } else {
        // (the resolver shares its SIMD with a wavefront that quantises while the routes are resolved,
        // and the routes are what every wavefront of the workgroup waits for)
        __builtin_amdgcn_s_setprio(3);
        id_route = (uint32_t)one.indices[my_first + (route < K ? route : 0)];
        id_part = (uint32_t)one.indices[my_first + (part < K ? part : 0)];
        const PushDst &dst_of_lane = args.dst[lane < ws.world ? lane : 0];
        my_out_x = (uint64_t)dst_of_lane.out_x;
        my_out_scale = (uint64_t)dst_of_lane.out_scale;
        my_out_stride = dst_of_lane.out_stride;
        my_os_elem = dst_of_lane.os_stride_elem;
        my_os_token = dst_of_lane.os_stride_token;
        my_out_rows = dst_of_lane.out_rows;
        duty_before = ws.laid_before[(blockIdx.x < ws.world ? blockIdx.x : 0) * G + my_g];
    }
    const uint32_t live_tokens = effective_tokens(one.bound_m, tokens);
    const uint32_t flat_entries = live_tokens * K;
    const bool live = token < live_tokens;   // uniform

    for (uint32_t i = tid; i < E; i += nthreads) s_cnt[i] = 0;
    if (tid == 0) s_counted = 0;
    lds_barrier();

    if (!resolver) {
        // The first batch in straight-line code: each of its values is waited for by itself, and the
        // row asked for after them stays in flight meanwhile.
#pragma unroll
        for (uint32_t j = 0; j < kBatch; ++j) {
            const uint32_t f = j * counters + tid;
            const uint32_t x = f < flat_entries ? early[j] : 0xFFFFFFFFu;
            if (x < E) atomicAdd(&s_cnt[x], f < my_first ? 0x10001u : 1u);
        }
        for (uint32_t f0 = kBatch * counters; f0 < flat_entries; f0 += kBatch * counters) {
            uint32_t x[kBatch];
#pragma unroll
            for (uint32_t j = 0; j < kBatch; ++j) {
                const uint32_t f = f0 + j * counters + tid;
                x[j] = f < flat_entries ? (uint32_t)one.indices[f] : 0xFFFFFFFFu;
            }
#pragma unroll
            for (uint32_t j = 0; j < kBatch; ++j) {
                const uint32_t f = f0 + j * counters + tid;
                if (x[j] < E) atomicAdd(&s_cnt[x[j]], f < my_first ? 0x10001u : 1u);
            }
        }
        // this wavefront's entries are in the table before its arrival is counted
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (lane == 0) atomicAdd(&s_counted, 1u);
        if (!live) return;   // nothing to send (uniform; the resolver does not wait at the barrier either)

        const bool has_piece = tid < num_chunks;
        u32x4 q;
        if constexpr (QUANT) {
            float scale;
            q = quantize16(pre_a, pre_b, &scale);
            if (has_piece && (lane & 7) == 0) s_scale[tid / 8] = scale;
        } else {
            q = pre_a;
            if (tid < Hs && tid < (uint32_t)kMaxLdsScales) s_scale[tid] = __uint_as_float(pre_b.x);
        }
        lds_barrier();
        const uint64_t row_ptr = lane < K ? s_row_ptr[lane] : 0;
        if (K == 8) {
#pragma unroll
            for (uint32_t k = 0; k < 8; ++k) {
                const uint64_t row = read_lane64(row_ptr, k);
                if (row != 0 && has_piece) store_copy(q, reinterpret_cast<u32x4 *>(row + (size_t)tid * 16));
            }
        } else {
            for (uint32_t k = 0; k < K; ++k) {
                const uint64_t row = read_lane64(row_ptr, k);
                if (row != 0 && has_piece) store_copy(q, reinterpret_cast<u32x4 *>(row + (size_t)tid * 16));
            }
        }
        // each copy's scale row goes out as one contiguous run: wavefront w takes routes w, w + waves - 1, ...
        if (!QUANT && one.x_scale == nullptr) return;   // rows without scales
        for (uint32_t k = wave; k < K; k += waves - 1) {
            const uint64_t sp = s_scale_ptr[k];
            const uint32_t ss = s_scale_stride[k];
            if (sp == 0) continue;
            for (uint32_t j = lane; j < Hs; j += kWave) reinterpret_cast<float *>(sp)[(size_t)j * ss] = s_scale[j];
        }
        return;
    }

    // ---- the resolver ----
    // what no count decides: the route's expert and receiver, the receiver's descriptor (from the lane
    // that holds it), the copies of this token to the same expert at an earlier k
    const bool in = route < K;
    const bool route_live = in && id_route < E;
    const uint32_t e = route_live ? id_route : 0;
    const uint32_t r = owner_of_expert(ws, e);
    const uint32_t le = e - r * Le;
    const uint32_t repeats = group8_sum(part < route && id_part == id_route ? 1u : 0u);
    PushDst dst;
    dst.out_x = reinterpret_cast<uint8_t *>(__shfl(my_out_x, (int)r));
    dst.out_scale = reinterpret_cast<float *>(__shfl(my_out_scale, (int)r));
    dst.out_stride = __shfl(my_out_stride, (int)r);
    dst.os_stride_elem = __shfl(my_os_elem, (int)r);
    dst.os_stride_token = __shfl(my_os_token, (int)r);
    dst.out_rows = __shfl(my_out_rows, (int)r);
    dst.pad_ = 0;

    // until the counting wavefronts have all said that their entries are in the table (at the lowest
    // priority: the wavefront that shares this SIMD is one of those waited for)
    __builtin_amdgcn_s_setprio(0);
    for (uint32_t spins = 0; __hip_atomic_load(&s_counted, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) != waves - 1;) {
        if (++spins == kQuickSpinLimit) {
            if (lane == 0) atomicOr(ws.err, A2A_DEV_INTERNAL);
            break;
        }
    }
    __builtin_amdgcn_s_setprio(3);
    asm volatile("" ::: "memory");

    // The source's per-expert totals and their scan, for the caller and the combine.
    auto publish_totals = [&]() {
        uint32_t run = 0;
        for (uint32_t e0 = 0; e0 < E; e0 += kWave) {
            const uint32_t x = e0 + lane;
            const uint32_t v = x < E ? s_cnt[x] & 0xFFFFu : 0;
            const uint32_t incl = run + wave_inclusive_scan(v, lane);
            if (x < E) {
                ws.num_routed[my_g * E + x] = v;
                ws.expert_offsets[my_g * E + x] = incl;
            }
            run = __shfl(incl, kWave - 1);
        }
    };
    // What the resolver does once the routes are out, while the others store rows: one of the step's
    // world + G + 1 jobs (with fewer workgroups than jobs, several).  Every store of a job is a run of
    // neighbouring words from neighbouring lanes.
    auto duties = [&]() {
        const uint32_t jobs = ws.world + G + 1;
        for (uint32_t job = blockIdx.x; job < jobs; job += tokens) {
            if (job < ws.world) {
                // a receiver's layout
                const uint32_t rr = job;
                if (!(fin.recv_mask >> rr & 1)) continue;
                const uint32_t before_mine = rr == blockIdx.x ? duty_before : ws.laid_before[rr * G + my_g];
                int32_t *const out_tokens = rr == blockIdx.x ? duty_out_tokens : fin.out_num_tokens[rr];
                const uint32_t out_rows = rr == blockIdx.x ? duty_out_rows : fin.out_rows[rr];
                uint32_t run = 0;
                for (uint32_t l0 = 0; l0 < Le; l0 += kWave) {
                    const uint32_t l = l0 + lane;
                    const uint32_t x = rr * Le + l;
                    const bool valid = l < Le && x < E;
                    const uint32_t tpe = valid ? s_cnt[x] & 0xFFFFu : 0;
                    const uint32_t padded = pad > 1 ? (tpe + pad - 1) / pad * pad : tpe;
                    const uint32_t incl = run + wave_inclusive_scan(padded, lane);
                    const uint32_t poff = incl - padded;
                    if (valid) {
                        ws.tokens_per_expert[x] = tpe;
                        ws.padded_offset[x] = poff;
                        if (out_tokens != nullptr) out_tokens[l] = (int32_t)tpe;
                        if (poff + tpe > out_rows) atomicOr(ws.err, A2A_DEV_RECV_OVERFLOW);
                        for (uint32_t g = 0; g < G; ++g) {
                            ws.slot_base[g * E + x] = g == my_g || (before_mine >> g & 1) ? poff : poff + tpe;
                        }
                    }
                    run = __shfl(incl, kWave - 1);
                }
            } else if (job < ws.world + G) {
                // a source without tokens has no workgroup of its own: its tables read as zeros
                const uint32_t g = job - ws.world;
                if (g == my_g) continue;
                for (uint32_t x = lane; x < E; x += kWave) {
                    ws.num_routed[g * E + x] = 0;
                    ws.expert_offsets[g * E + x] = 0;
                }
            } else {
                publish_totals();
            }
        }
    };
    if (!live) {   // nothing to send (uniform)
        duties();
        return;
    }

    // padded rows of the receiver's experts before mine: four terms per lane without a branch
    // (clamped index, masked value), the rest in a loop
    const uint32_t mine = s_cnt[e];
    uint32_t v_rows[4];
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) {
        const uint32_t n = part + 8 * i;
        v_rows[i] = s_cnt[r * Le + (n < le ? n : 0)] & 0xFFFFu;
    }
    uint32_t base = 0;
    if (pad > 1) {   // uniform
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) base += part + 8 * i < le ? (v_rows[i] + pad - 1) / pad * pad : 0;
        for (uint32_t n = 32 + part; n < le; n += 8) base += ((s_cnt[r * Le + n] & 0xFFFFu) + pad - 1) / pad * pad;
    } else {
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) base += part + 8 * i < le ? v_rows[i] : 0;
        for (uint32_t n = 32 + part; n < le; n += 8) base += s_cnt[r * Le + n] & 0xFFFFu;
    }
    base = group8_sum(base);
    // copies of my source before this one: earlier tokens, then earlier k of this token
    const uint32_t toff = route_live ? (mine >> 16) + repeats : 0;
    uint64_t to_row, to_scale;
    uint32_t to_stride;
    uint32_t slot = resolve_copy(dst, ws, base + toff, part == 0 && route_live, &to_row, &to_scale, &to_stride);
    if (!route_live) {
        slot = kInvalidSlot;
        to_row = 0;
        to_scale = 0;
        to_stride = 0;
    }
    if (part == 0 && in) {
        s_row_ptr[route] = to_row;
        s_scale_ptr[route] = to_scale;
        s_scale_stride[route] = to_stride;
    }
    lds_barrier();
    // (after the barrier: nothing of the resolver's that goes to memory stands between the others and their rows)
    if (part == 0 && in) {
        if (!route_live) atomicOr(ws.err, A2A_DEV_BAD_EXPERT_ID);
        ws.route_slot[(size_t)my_g * ws.max_tk + my_first + route] = slot;
        ws.token_offset[(size_t)my_g * ws.max_tk + my_first + route] = toff;
    }
    duties();
}

// Routing pass and dispatch pack in ONE launch for steps of ONE source with
// dense index rows that are too large for dispatch_small_kernel (a mixed batch
// of about a thousand tokens on one GPU's share).  What makes the one-launch
// dispatch of small steps expensive as steps grow is that every token's
// workgroup counts every entry of the step; here a workgroup counts once for
// `per_group` tokens (at most kTokensPerGroup; the host picks it so that the
// token workgroups are about as many as the compute units): it is made of
// teams of wavefronts, each as wide as a token row needs, that move one token
// each per round.  As in dispatch_small_kernel no workgroup depends on another,
// and the rows are the same: first row of the expert in its receiver + copies of
// earlier tokens to the expert + copies of this token at an earlier k.  There are
// no receiver workgroups: with one source a token workgroup's own tables hold
// everything a receiver's layout needs, and the first workgroups write it.
//
// Dynamic LDS: 2 * E words.
//
// Two of these workgroups should fit a compute unit at once: where the grid has more workgroups than
// the GPU has compute units, a workgroup that has to wait for another to end starts its whole chain
// a step late (4 us on the 1024-token step when its grid still had the receivers' workgroups on top
// of one token workgroup per compute unit).  With 14 wavefronts each that means at most 72 vector
// registers a lane, which the kernel is held to (amdgpu_waves_per_eu): left to itself the compiler
// moved between 62 and 75 with unrelated changes to the code.
constexpr uint32_t kTokensPerGroup = 4;
constexpr uint32_t kMaxGroupRoutes = kTokensPerGroup * A2A_MAX_EXPERTS_PER_TOKEN;

template <bool QUANT>
__global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(7))) void dispatch_single_kernel(const PushArgs args, const FinalizeArgs fin,
                                                               const Workspace ws, const uint32_t team_threads,
                                                               const uint32_t per_group) {
    extern __shared__ uint32_t s_tab[];
    __shared__ float s_scale[kTokensPerGroup][QUANT ? kMaxLdsScales : 1];   // [team]: at most kTokensPerGroup teams
    __shared__ uint64_t s_scale_ptr[kTokensPerGroup][A2A_MAX_EXPERTS_PER_TOKEN];
    __shared__ uint32_t s_scale_stride[kTokensPerGroup][A2A_MAX_EXPERTS_PER_TOKEN];
    __shared__ uint64_t s_row_ptr[kMaxGroupRoutes];            // per route of the workgroup's tokens
    __shared__ uint64_t s_route_scale_ptr[kMaxGroupRoutes];
    __shared__ uint32_t s_route_scale_stride[kMaxGroupRoutes];
    __shared__ uint32_t s_route_expert[kMaxGroupRoutes];
    __shared__ PushDst s_dst[kMaxWorld];                       // per receiver: its buffers
    __shared__ uint32_t scratch[kRouteWaves];
    __shared__ uint32_t s_carry;

    const uint32_t tid = threadIdx.x;
    const uint32_t nthreads = blockDim.x;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t G = ws.num_groups, E = ws.num_experts, K = ws.topk, Le = ws.experts_per_rank;
    const uint32_t my_g = args.single_source - 1;
    const PushSrc &src = args.single;
    const uint32_t token_groups = gridDim.x;                            // every workgroup has tokens
    const uint32_t tokens = effective_tokens(src.bound_m, src.num_tokens);
    const uint32_t flat_entries = tokens * K;
    const uint32_t first_token = blockIdx.x * per_group;
    const uint32_t my_first = first_token * K;                          // flat index of my first entry
    // Every token of mine is past the bound: nothing to send.  The first workgroups stay: they publish the
    // totals, lay out the receivers and clear the tables of the sources without tokens (workgroup b:
    // receivers and sources b, b + grid, ...).
    const bool has_duty = blockIdx.x < ws.world;   // (there are at most as many sources as receivers)
    if (!has_duty && first_token >= tokens) return;

    // The first entries and the ids of my tokens' routes are asked for first of all, then the rows of the
    // first round: they travel while the entries are counted and the routes resolved.
    constexpr uint32_t kBatch = 10;   // 8192 entries over 896 threads in one batch: one trip to memory, not two
    uint32_t early[kBatch];
#pragma unroll
    for (uint32_t j = 0; j < kBatch; ++j) {
        const uint32_t f = j * nthreads + tid;
        early[j] = f < flat_entries ? (uint32_t)src.indices[f] : 0xFFFFFFFFu;
    }
    const uint32_t my_routes = per_group * K;    // one thread each
    uint32_t my_expert = 0xFFFFFFFFu;
    if (tid < my_routes && my_first + tid < flat_entries) {
        my_expert = (uint32_t)src.indices[my_first + tid];
    }
    // The descriptor of receiver `tid` is asked for here too and written to LDS after the counting (written
    // here, the wait for it would cover the entries; asked for later, it would cover the rows).
    const PushDst &dst_of_tid = args.dst[tid < ws.world ? tid : 0];
    uint8_t *const my_out_x = dst_of_tid.out_x;
    float *const my_out_scale = dst_of_tid.out_scale;
    const uint64_t my_out_stride = dst_of_tid.out_stride;
    const uint32_t my_os_elem = dst_of_tid.os_stride_elem, my_os_token = dst_of_tid.os_stride_token;
    const uint32_t my_out_rows = dst_of_tid.out_rows;
    // (The rows without a condition: a thread that has no piece asks for one it ignores later, from a row
    // that exists; a value picked by a condition would be waited for right here.  Every barrier between
    // here and the rows' use is an lds_barrier, and nothing is stored to memory in front of them: the
    // compiler's own barrier after such stores waits for every outstanding load.)
    const uint32_t teams = nthreads / team_threads;
    const uint32_t team = tid / team_threads;
    const uint32_t team_tid = tid - team * team_threads;
    // The same for the team's token of the SECOND round, asked for ahead of the first round's (it is
    // needed later): a workgroup of two rounds then has all its rows on their way from the start and its
    // rounds only store (1024 tokens: 41.3 -> 39.8 us per step).
    u32x4 pre_a, pre_b = {0, 0, 0, 0};
    u32x4 next_a = {0, 0, 0, 0}, next_b = {0, 0, 0, 0};
    {
        const uint32_t last_token = src.num_tokens - 1;
        const uint32_t any_token = first_token + team < src.num_tokens ? first_token + team : last_token;
        const uint32_t second = first_token + teams + team;
        const uint32_t next_token = second < src.num_tokens ? second : last_token;
        const uint8_t *x_row = src.x + (size_t)any_token * src.x_stride;
        const uint8_t *x_next = src.x + (size_t)next_token * src.x_stride;
        const bool two_rounds = per_group > teams;   // uniform: a branch, not a select (nothing waits at its end)
        if constexpr (QUANT) {
            const uint32_t pieces = args.hidden_dim / 16;
            const size_t at = (size_t)(team_tid < pieces ? team_tid : 0) * 32;
            if (two_rounds) {
                next_a = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(x_next + at));
                next_b = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(x_next + at) + 1);
            }
            pre_a = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(x_row + at));
            pre_b = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(x_row + at) + 1);
        } else {
            const uint32_t pieces = args.row_bytes / 16;
            const uint32_t at = team_tid < pieces ? team_tid : 0;
            if (two_rounds) next_a = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(x_next) + at);
            pre_a = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(x_row) + at);
        }
    }

    uint32_t *cnt = s_tab;                 // [E] low half: entries per expert, high half: those before my first token
    uint32_t *rows_before = cnt + E;       // [E] padded rows of all experts before e
    for (uint32_t i = tid; i < E; i += nthreads) s_tab[i] = 0;
    lds_barrier();

    // One pass over the entries of the step, kBatch loads in flight per lane.
    // (the first batch in straight-line code: inside the loop the compiler waits for every outstanding
    // load, the rows included, before it uses the first entry)
    auto count_batch = [&](const uint32_t (&expert)[kBatch], uint32_t f0) {
#pragma unroll
        for (uint32_t j = 0; j < kBatch; ++j) {
            const uint32_t x = expert[j];
            if (x >= E) continue;
            // one word per expert: low half all its entries, high half those before my first token
            // (a step of this kernel has at most kSingleMaxEntries < 2^16 entries)
            atomicAdd(&cnt[x], f0 + j * nthreads + tid < my_first ? 0x10001u : 1u);
        }
    };
    count_batch(early, 0);
    for (uint32_t f0 = kBatch * nthreads; f0 < flat_entries; f0 += kBatch * nthreads) {
        uint32_t expert[kBatch];
#pragma unroll
        for (uint32_t j = 0; j < kBatch; ++j) {
            const uint32_t f = f0 + j * nthreads + tid;
            expert[j] = f < flat_entries ? (uint32_t)src.indices[f] : 0xFFFFFFFFu;
        }
        count_batch(expert, f0);
    }
    if (tid < my_routes) s_route_expert[tid] = my_expert;
    if (tid < ws.world) {
        s_dst[tid] = PushDst{my_out_x, my_out_scale, my_out_stride, my_os_elem, my_os_token, my_out_rows, 0};
    }
    lds_barrier();

    // Per expert: padded rows of the experts before it (the difference to the scan
    // at the first expert of a receiver is the expert's first row there).
    const uint32_t pad = ws.expert_padding;
    uint32_t carry = 0;
    for (uint32_t e0 = 0; e0 < E; e0 += nthreads) {
        const uint32_t e = e0 + tid;
        const uint32_t total = e < E ? cnt[e] & 0xFFFFu : 0;
        const uint32_t padded = e < E ? (total + pad - 1) / pad * pad : 0;
        const uint32_t incl = carry + block_inclusive_scan<true>(padded, scratch);
        if (e < E) rows_before[e] = incl - padded;
        if (e0 + nthreads < E) {   // uniform: another round follows
            if (tid == nthreads - 1) s_carry = incl;
            lds_barrier();
            carry = s_carry;
        }
    }
    lds_barrier();

    // The receivers' layouts, by the last wavefront of the first workgroups (workgroup b: receivers b,
    // b + grid, ...), beside the other wavefronts' work.  With one source everything a receiver needs
    // is in this workgroup's tables: an expert's rows are its count, its first row the difference of two
    // values of the scan, and of the other sources (all empty) those the receiver lays out after mine
    // begin behind my rows (a2a_worker.rs:598-606,669-671,681-694).
    if (has_duty && tid / kWave == nthreads / kWave - 1) {
        // Sources without tokens have no workgroup of their own: their tables read as zeros.  (Early in
        // the kernel's life and spread over workgroups: stores issued at the very end of a kernel delay
        // the start of the next one.)
        for (uint32_t g = blockIdx.x; g < G; g += token_groups) {
            if (args.src[g].num_tokens != 0) continue;
            for (uint32_t e = lane; e < E; e += kWave) {
                ws.num_routed[g * E + e] = 0;
                ws.expert_offsets[g * E + e] = 0;
            }
        }
        for (uint32_t r = blockIdx.x; r < ws.world; r += token_groups) {
            if (!(fin.recv_mask >> r & 1)) continue;
            const uint32_t before_mine = ws.laid_before[r * G + my_g];   // sources receiver r lays out before mine
            const uint32_t base = r * Le < E ? rows_before[r * Le] : 0;
            for (uint32_t l0 = 0; l0 < Le; l0 += kWave) {
                const uint32_t le = l0 + lane;
                const uint32_t e = r * Le + le;
                if (le >= Le || e >= E) continue;
                const uint32_t tpe = cnt[e] & 0xFFFFu;
                const uint32_t poff = rows_before[e] - base;
                ws.tokens_per_expert[e] = tpe;
                ws.padded_offset[e] = poff;
                if (fin.out_num_tokens[r] != nullptr) fin.out_num_tokens[r][le] = (int32_t)tpe;
                if (poff + tpe > fin.out_rows[r]) atomicOr(ws.err, A2A_DEV_RECV_OVERFLOW);
                for (uint32_t g = 0; g < G; ++g) {
                    ws.slot_base[g * E + e] = g == my_g || (before_mine >> g & 1) ? poff : poff + tpe;
                }
            }
        }
    }

    // The first workgroup publishes the source's totals (last wavefront).
    if (blockIdx.x == 0 && tid / kWave == nthreads / kWave - 1) {
        uint32_t run = 0;
        for (uint32_t e0 = 0; e0 < E; e0 += kWave) {
            const uint32_t e = e0 + lane;
            const uint32_t v = e < E ? cnt[e] & 0xFFFFu : 0;
            const uint32_t incl = run + wave_inclusive_scan(v, lane);
            if (e < E) {
                ws.num_routed[my_g * E + e] = v;
                ws.expert_offsets[my_g * E + e] = incl;
            }
            run = __shfl(incl, kWave - 1);
        }
    }

    // One thread per route of my tokens resolves it from LDS alone.
    if (tid < my_routes && my_first + tid < flat_entries) {
        uint64_t row_ptr = 0, scale_ptr = 0;
        uint32_t scale_stride = 0;
        uint32_t slot = kInvalidSlot, toff = 0;
        if (my_expert < E) {
            // copies of the source before this one: those of earlier workgroups' tokens, then mine
            uint32_t earlier = 0;
            for (uint32_t q = 0; q < tid; ++q) earlier += s_route_expert[q] == my_expert ? 1u : 0u;
            toff = (cnt[my_expert] >> 16) + earlier;
            const uint32_t r = owner_of_expert(ws, my_expert);
            const uint32_t row = rows_before[my_expert] - rows_before[r * Le];
            slot = resolve_copy(s_dst[r], ws, row + toff, true, &row_ptr, &scale_ptr, &scale_stride);
        } else {
            atomicOr(ws.err, A2A_DEV_BAD_EXPERT_ID);
        }
        ws.route_slot[(size_t)my_g * ws.max_tk + my_first + tid] = slot;
        ws.token_offset[(size_t)my_g * ws.max_tk + my_first + tid] = toff;
        s_row_ptr[tid] = row_ptr;
        s_route_scale_ptr[tid] = scale_ptr;
        s_route_scale_stride[tid] = scale_stride;
    }
    lds_barrier();

    // The teams move one token each per round; the rows of the first two rounds are on their way since the head.
    for (uint32_t first = 0; first < per_group; first += teams) {
        const uint32_t mine = first + team;                  // which of the workgroup's tokens
        const uint32_t token = first_token + mine;
        const bool live = mine < per_group && token < tokens;
        uint64_t row_ptr = 0, scale_ptr = 0;
        uint32_t scale_stride = 0;
        if (live && lane < K) {
            row_ptr = s_row_ptr[mine * K + lane];
            scale_ptr = s_route_scale_ptr[mine * K + lane];
            scale_stride = s_route_scale_stride[mine * K + lane];
        }
        if (first == 0) {
            push_rows<QUANT, true>(args, src, token, K, row_ptr, scale_ptr, scale_stride, s_scale[team],
                                   s_scale_ptr[team], s_scale_stride[team], team_tid, team_threads, live, pre_a,
                                   pre_b);
        } else if (first == teams) {
            push_rows<QUANT, true>(args, src, token, K, row_ptr, scale_ptr, scale_stride, s_scale[team],
                                   s_scale_ptr[team], s_scale_stride[team], team_tid, team_threads, live, next_a,
                                   next_b);
        } else {
            push_rows<QUANT>(args, src, token, K, row_ptr, scale_ptr, scale_stride, s_scale[team],
                             s_scale_ptr[team], s_scale_stride[team], team_tid, team_threads, live);
        }
        __syncthreads();   // the team's LDS arrays are reused by the next round
    }
}

// The same division of labour for the larger steps of one source that dispatch_single_kernel serves
// (448 to 1024 tokens at top-8): a workgroup counts the step's entries once for `per_group` tokens,
// its teams of wavefronts (one token each per round, at most two rounds) quantise both rounds' pieces
// while the spare wavefront resolves the per_group * K <= 32 routes, eight, four or two lanes per
// route, and after the one barrier the teams only store.  The resolvers of the first workgroups
// write the step's tables.  1024 tokens, hidden 7168, 384 experts over 16 ranks: the head of the
// kernel (everything in front of the first store) shrinks by about a microsecond.
//
// QUANT false: the rows travel as they are, with the caller's scales if it passed any.
//
// Dynamic LDS: E words.
constexpr uint32_t kTeamsMaxRoutes = 32;
constexpr uint32_t kTeamsMaxScales = 128;   // scale groups of a row of at most (1024 - 64) pieces

template <uint32_t NB, uint32_t ROUNDS, bool QUANT>
__global__ __launch_bounds__(1024) void dispatch_teams_kernel(const PushArgs args, const FinalizeArgs fin,
                                                              const Workspace ws, const uint32_t team_threads,
                                                              const uint32_t per_group) {
    A2A_PIN(args.single_source);
    A2A_PIN(args.hidden_dim);
    A2A_PIN(args.hidden_dim_scale);
    A2A_PIN(args.single.x);
    A2A_PIN(args.single.indices);
    A2A_PIN(args.single.bound_m);
    A2A_PIN(args.single.x_stride);
    A2A_PIN(args.single.num_tokens);
    if constexpr (!QUANT) {
        A2A_PIN(args.row_bytes);
        A2A_PIN(args.single.x_scale);
        A2A_PIN(args.single.xs_stride_elem);
        A2A_PIN(args.single.xs_stride_token);
    }
    A2A_PIN(fin.recv_mask);
    A2A_PIN(ws.world);
    A2A_PIN(ws.num_groups);
    A2A_PIN(ws.num_experts);
    A2A_PIN(ws.topk);
    A2A_PIN(ws.experts_per_rank);
    A2A_PIN(ws.le_magic);
    A2A_PIN(ws.expert_padding);
    A2A_PIN(ws.max_tk);
    A2A_PIN(ws.laid_before);
    A2A_PIN(ws.route_slot);
    A2A_PIN(ws.token_offset);
    A2A_PIN(ws.err);
    int32_t *const duty_out_tokens = fin.out_num_tokens[blockIdx.x & (kMaxWorld - 1)];
    const uint32_t duty_out_rows = fin.out_rows[blockIdx.x & (kMaxWorld - 1)];
    A2A_PIN(duty_out_tokens);
    A2A_PIN(duty_out_rows);

    extern __shared__ uint32_t s_cnt[];   // [E]: low half the entries of the expert, high half those before my first token
    __shared__ float s_scale[ROUNDS][kTokensPerGroup][kTeamsMaxScales];   // [round][team]
    __shared__ uint64_t s_row_ptr[kTeamsMaxRoutes];
    __shared__ uint64_t s_scale_ptr[kTeamsMaxRoutes];
    __shared__ uint32_t s_scale_stride[kTeamsMaxRoutes];
    __shared__ uint32_t s_route_expert[kTeamsMaxRoutes];
    __shared__ uint32_t s_counted;

    const uint32_t tid = threadIdx.x;
    const uint32_t nthreads = blockDim.x;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = tid / kWave;
    const uint32_t waves = nthreads / kWave;
    const bool resolver = wave == waves - 1;
    const uint32_t counters = nthreads - kWave;          // threads that count entries and move rows
    const uint32_t teams = counters / team_threads;
    const uint32_t team = tid / team_threads;            // (row wavefronts)
    const uint32_t team_tid = tid - team * team_threads;
    const uint32_t G = ws.num_groups, E = ws.num_experts, K = ws.topk, Le = ws.experts_per_rank;
    const uint32_t pad = ws.expert_padding;
    const PushSrc &one = args.single;
    const uint32_t my_g = args.single_source - 1;
    const uint32_t tokens = one.num_tokens;
    const uint32_t entries = tokens * K;                 // > 0
    const uint32_t first_token = blockIdx.x * per_group;
    const uint32_t my_first = first_token * K;           // flat index of my first entry
    const uint32_t routes = per_group * K;               // <= kTeamsMaxRoutes
    const uint32_t num_chunks = QUANT ? args.hidden_dim / 16 : args.row_bytes / 16;   // pieces of a row
    const uint32_t Hs = args.hidden_dim_scale;
    const uint32_t token_groups = gridDim.x;

    // lanes of the resolver per route: 8, 4 or 2
    const uint32_t lpr_log = routes <= 8 ? 3 : routes <= 16 ? 2 : 1;
    const uint32_t part = lane & ((1u << lpr_log) - 1), route = lane >> lpr_log;
    const uint32_t lpr = 1u << lpr_log;

    uint32_t early[NB] = {};
    u32x4 pre_a[ROUNDS], pre_b[ROUNDS];
#pragma unroll
    for (uint32_t rd = 0; rd < ROUNDS; ++rd) {
        pre_a[rd] = u32x4{0, 0, 0, 0};
        pre_b[rd] = u32x4{0, 0, 0, 0};
    }
    uint32_t id_route = 0xFFFFFFFFu, duty_before = 0;
    uint64_t my_out_x = 0, my_out_scale = 0, my_out_stride = 0;
    uint32_t my_os_elem = 0, my_os_token = 0, my_out_rows = 0;
    if (!resolver) {
#pragma unroll
        for (uint32_t j = 0; j < NB; ++j) {
            const uint32_t f = j * counters + tid;
            early[j] = (uint32_t)one.indices[f < entries ? f : entries - 1];
        }
        // the pieces of both rounds' rows, the later round first (it is needed later); a team without a
        // token asks for a row that exists and ignores it
#pragma unroll
        for (uint32_t i = 0; i < ROUNDS; ++i) {
            const uint32_t rd = ROUNDS - 1 - i;
            const uint32_t t = first_token + rd * teams + team;
            const uint32_t row_t = t < tokens ? t : tokens - 1;
            if constexpr (QUANT) {
                const u32x4 *p = reinterpret_cast<const u32x4 *>(one.x + (size_t)row_t * one.x_stride +
                                                                 (size_t)(team_tid < num_chunks ? team_tid : 0) * 32);
                pre_a[rd] = __builtin_nontemporal_load(p);
                pre_b[rd] = __builtin_nontemporal_load(p + 1);
            } else {
                pre_a[rd] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(one.x + (size_t)row_t * one.x_stride) +
                                                       (team_tid < num_chunks ? team_tid : 0));
                // the caller's scales of the token (one per thread of the team; kept in pre_b's first word)
                if (one.x_scale != nullptr && team_tid < Hs) {
                    pre_b[rd].x = __float_as_uint(
                        one.x_scale[(size_t)row_t * one.xs_stride_token + (size_t)team_tid * one.xs_stride_elem]);
                }
            }
        }
    } else {
        __builtin_amdgcn_s_setprio(3);
        const uint32_t f = my_first + route;
        id_route = (uint32_t)one.indices[f < entries ? f : entries - 1];
        const PushDst &dst_of_lane = args.dst[lane < ws.world ? lane : 0];
        my_out_x = (uint64_t)dst_of_lane.out_x;
        my_out_scale = (uint64_t)dst_of_lane.out_scale;
        my_out_stride = dst_of_lane.out_stride;
        my_os_elem = dst_of_lane.os_stride_elem;
        my_os_token = dst_of_lane.os_stride_token;
        my_out_rows = dst_of_lane.out_rows;
        duty_before = ws.laid_before[(blockIdx.x < ws.world ? blockIdx.x : 0) * G + my_g];
    }
    const uint32_t live_tokens = effective_tokens(one.bound_m, tokens);
    const uint32_t flat_entries = live_tokens * K;
    const bool group_live = first_token < live_tokens;   // uniform

    for (uint32_t i = tid; i < E; i += nthreads) s_cnt[i] = 0;
    if (tid == 0) s_counted = 0;
    lds_barrier();

    if (!resolver) {
#pragma unroll
        for (uint32_t j = 0; j < NB; ++j) {
            const uint32_t f = j * counters + tid;
            const uint32_t x = f < flat_entries ? early[j] : 0xFFFFFFFFu;
            if (x < E) atomicAdd(&s_cnt[x], f < my_first ? 0x10001u : 1u);
        }
        for (uint32_t f0 = NB * counters; f0 < flat_entries; f0 += counters) {
            const uint32_t f = f0 + tid;
            const uint32_t x = f < flat_entries ? (uint32_t)one.indices[f] : 0xFFFFFFFFu;
            if (x < E) atomicAdd(&s_cnt[x], f < my_first ? 0x10001u : 1u);
        }
        // this wavefront's entries are in the table before its arrival is counted
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (lane == 0) atomicAdd(&s_counted, 1u);
        if (!group_live) return;   // nothing to send (uniform; the resolver does not wait at the barrier either)

        const bool has_piece = team_tid < num_chunks;
        u32x4 q[ROUNDS];
#pragma unroll
        for (uint32_t rd = 0; rd < ROUNDS; ++rd) {
            if constexpr (QUANT) {
                float scale;
                q[rd] = quantize16(pre_a[rd], pre_b[rd], &scale);
                if (has_piece && (lane & 7) == 0) s_scale[rd][team][team_tid / 8] = scale;
            } else {
                q[rd] = pre_a[rd];
                if (team_tid < Hs) s_scale[rd][team][team_tid] = __uint_as_float(pre_b[rd].x);
            }
        }
        lds_barrier();
        const uint32_t team_waves = team_threads / kWave, team_wave = team_tid / kWave;
#pragma unroll
        for (uint32_t rd = 0; rd < ROUNDS; ++rd) {
            const uint32_t mine = rd * teams + team;   // which of the workgroup's tokens
            if (mine >= per_group || first_token + mine >= live_tokens) continue;   // uniform in a team
            const uint64_t row_ptr = lane < K ? s_row_ptr[mine * K + lane] : 0;
            if (K == 8) {
#pragma unroll
                for (uint32_t k = 0; k < 8; ++k) {
                    const uint64_t row = read_lane64(row_ptr, k);
                    if (row != 0 && has_piece) store_copy(q[rd], reinterpret_cast<u32x4 *>(row + (size_t)team_tid * 16));
                }
            } else {
                for (uint32_t k = 0; k < K; ++k) {
                    const uint64_t row = read_lane64(row_ptr, k);
                    if (row != 0 && has_piece) store_copy(q[rd], reinterpret_cast<u32x4 *>(row + (size_t)team_tid * 16));
                }
            }
            // each copy's scale row goes out as one contiguous run: wavefront w of the team takes routes w, w + team_waves, ...
            if (!QUANT && one.x_scale == nullptr) continue;   // rows without scales
            for (uint32_t k = team_wave; k < K; k += team_waves) {
                const uint64_t sp = s_scale_ptr[mine * K + k];
                const uint32_t ss = s_scale_stride[mine * K + k];
                if (sp == 0) continue;
                for (uint32_t j = lane; j < Hs; j += kWave) {
                    reinterpret_cast<float *>(sp)[(size_t)j * ss] = s_scale[rd][team][j];
                }
            }
        }
        return;
    }

    // ---- the resolver ----
    auto group_sum = [&](uint32_t v) {
        v += dpp_move_u32<0xB1>(v);                      // quad_perm [1,0,3,2]
        if (lpr_log >= 2) v += dpp_move_u32<0x4E>(v);    // quad_perm [2,3,0,1]
        if (lpr_log >= 3) v += dpp_move_u32<0x141>(v);   // row_half_mirror
        return v;
    };
    const bool in = route < routes && my_first + route < flat_entries;
    const bool route_live = in && id_route < E;
    const uint32_t e = route_live ? id_route : 0;
    const uint32_t r = owner_of_expert(ws, e);
    const uint32_t le = e - r * Le;
    // copies of my tokens to the same expert at an earlier route of the workgroup
    if (part == 0 && route < kTeamsMaxRoutes) s_route_expert[route] = in ? id_route : 0xFFFFFFFFu;
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    uint32_t earlier = 0;
    for (uint32_t qd = part; qd < route && qd < kTeamsMaxRoutes; qd += lpr) earlier += s_route_expert[qd] == id_route ? 1u : 0u;
    earlier = group_sum(earlier);
    PushDst dst;
    dst.out_x = reinterpret_cast<uint8_t *>(__shfl(my_out_x, (int)r));
    dst.out_scale = reinterpret_cast<float *>(__shfl(my_out_scale, (int)r));
    dst.out_stride = __shfl(my_out_stride, (int)r);
    dst.os_stride_elem = __shfl(my_os_elem, (int)r);
    dst.os_stride_token = __shfl(my_os_token, (int)r);
    dst.out_rows = __shfl(my_out_rows, (int)r);
    dst.pad_ = 0;

    __builtin_amdgcn_s_setprio(0);
    for (uint32_t spins = 0; __hip_atomic_load(&s_counted, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) != waves - 1;) {
        if (++spins == kQuickSpinLimit) {
            if (lane == 0) atomicOr(ws.err, A2A_DEV_INTERNAL);
            break;
        }
    }
    __builtin_amdgcn_s_setprio(3);
    asm volatile("" ::: "memory");

    auto publish_totals = [&]() {
        uint32_t run = 0;
        for (uint32_t e0 = 0; e0 < E; e0 += kWave) {
            const uint32_t x = e0 + lane;
            const uint32_t v = x < E ? s_cnt[x] & 0xFFFFu : 0;
            const uint32_t incl = run + wave_inclusive_scan(v, lane);
            if (x < E) {
                ws.num_routed[my_g * E + x] = v;
                ws.expert_offsets[my_g * E + x] = incl;
            }
            run = __shfl(incl, kWave - 1);
        }
    };
    auto duties = [&]() {
        const uint32_t jobs = ws.world + G + 1;
        for (uint32_t job = blockIdx.x; job < jobs; job += token_groups) {
            if (job < ws.world) {
                const uint32_t rr = job;
                if (!(fin.recv_mask >> rr & 1)) continue;
                const uint32_t before_mine = rr == blockIdx.x ? duty_before : ws.laid_before[rr * G + my_g];
                int32_t *const out_tokens = rr == blockIdx.x ? duty_out_tokens : fin.out_num_tokens[rr];
                const uint32_t out_rows = rr == blockIdx.x ? duty_out_rows : fin.out_rows[rr];
                uint32_t run = 0;
                for (uint32_t l0 = 0; l0 < Le; l0 += kWave) {
                    const uint32_t l = l0 + lane;
                    const uint32_t x = rr * Le + l;
                    const bool valid = l < Le && x < E;
                    const uint32_t tpe = valid ? s_cnt[x] & 0xFFFFu : 0;
                    const uint32_t padded = pad > 1 ? (tpe + pad - 1) / pad * pad : tpe;
                    const uint32_t incl = run + wave_inclusive_scan(padded, lane);
                    const uint32_t poff = incl - padded;
                    if (valid) {
                        ws.tokens_per_expert[x] = tpe;
                        ws.padded_offset[x] = poff;
                        if (out_tokens != nullptr) out_tokens[l] = (int32_t)tpe;
                        if (poff + tpe > out_rows) atomicOr(ws.err, A2A_DEV_RECV_OVERFLOW);
                        for (uint32_t g = 0; g < G; ++g) {
                            ws.slot_base[g * E + x] = g == my_g || (before_mine >> g & 1) ? poff : poff + tpe;
                        }
                    }
                    run = __shfl(incl, kWave - 1);
                }
            } else if (job < ws.world + G) {
                const uint32_t g = job - ws.world;
                if (g == my_g) continue;
                for (uint32_t x = lane; x < E; x += kWave) {
                    ws.num_routed[g * E + x] = 0;
                    ws.expert_offsets[g * E + x] = 0;
                }
            } else {
                publish_totals();
            }
        }
    };
    if (!group_live) {   // nothing to send (uniform)
        duties();
        return;
    }

    const uint32_t mine = s_cnt[e];
    uint32_t v_rows[4];
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) {
        const uint32_t n = part + lpr * i;
        v_rows[i] = s_cnt[r * Le + (n < le ? n : 0)] & 0xFFFFu;
    }
    uint32_t base = 0;
    if (pad > 1) {   // uniform
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) base += part + lpr * i < le ? (v_rows[i] + pad - 1) / pad * pad : 0;
        for (uint32_t n = 4 * lpr + part; n < le; n += lpr) base += ((s_cnt[r * Le + n] & 0xFFFFu) + pad - 1) / pad * pad;
    } else {
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) base += part + lpr * i < le ? v_rows[i] : 0;
        for (uint32_t n = 4 * lpr + part; n < le; n += lpr) base += s_cnt[r * Le + n] & 0xFFFFu;
    }
    base = group_sum(base);
    const uint32_t toff = route_live ? (mine >> 16) + earlier : 0;
    uint64_t to_row, to_scale;
    uint32_t to_stride;
    uint32_t slot = resolve_copy(dst, ws, base + toff, part == 0 && route_live, &to_row, &to_scale, &to_stride);
    if (!route_live) {
        slot = kInvalidSlot;
        to_row = 0;
        to_scale = 0;
        to_stride = 0;
    }
    if (part == 0 && route < routes) {
        s_row_ptr[route] = to_row;
        s_scale_ptr[route] = to_scale;
        s_scale_stride[route] = to_stride;
    }
    lds_barrier();
    if (part == 0 && in) {
        if (!route_live) atomicOr(ws.err, A2A_DEV_BAD_EXPERT_ID);
        ws.route_slot[(size_t)my_g * ws.max_tk + my_first + route] = slot;
        ws.token_offset[(size_t)my_g * ws.max_tk + my_first + route] = toff;
    }
    duties();
}

// Pack of a large group step, after a routing launch that left, per chunk, the
// histogram and the rank of every entry inside its chunk, and, for the whole
// step, the totals per (source, expert) and per expert.  No launch in between
// lays anything out: wavefront 0 of a token workgroup resolves the K rows
// itself, eight lanes per route, each route with three short sums whose terms
// are spread over the lanes and added on the DPP path:
//   copies of the same source and expert in earlier chunks      (chunk histograms)
//   copies of the sources the receiver lays out before mine     (totals per source)
//   padded rows of the receiver's experts before mine           (totals per expert)
// The terms come from tables of a few KB that stay in cache, and they travel
// while the token's row is on its way from memory.  Before the token workgroups
// the grid holds one workgroup per receiver (expert counts for the caller,
// layout tables) and one per source (its totals and their scan); the last of
// them hands the totals over to the next step.
template <bool QUANT>
__global__ __launch_bounds__(1024) void dispatch_resolve_kernel(const PushArgs args, const FinalizeArgs fin,
                                                                const Workspace ws) {
    __shared__ float s_scale[QUANT ? kMaxLdsScales : 1];
    __shared__ uint64_t s_scale_ptr[A2A_MAX_EXPERTS_PER_TOKEN];
    __shared__ uint32_t s_scale_stride[A2A_MAX_EXPERTS_PER_TOKEN];
    __shared__ uint64_t s_row_ptr[A2A_MAX_EXPERTS_PER_TOKEN];
    __shared__ uint64_t s_route_scale_ptr[A2A_MAX_EXPERTS_PER_TOKEN];
    __shared__ uint32_t s_route_scale_stride[A2A_MAX_EXPERTS_PER_TOKEN];
    __shared__ uint32_t tot[A2A_MAX_EXPERTS + kMaxWorld];
    __shared__ uint32_t scratch[kRouteWaves];
    __shared__ uint32_t s_carry;

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = tid / kWave;
    const uint32_t G = ws.num_groups, E = ws.num_experts, K = ws.topk, Le = ws.experts_per_rank;
    // (read at index G, not at its fixed place at the end of the array: with the fixed index the
    // compiler's schedule of this kernel's head came out 0.7 us slower on the 4096-token step)
    const uint32_t total_tokens = args.token_start[G];
    const uint32_t use = ws.turn[1] & 1u;
    const uint32_t *per_source = ws.totals + (size_t)use * (G + 1) * E;   // [E][G]
    const uint32_t *per_expert = per_source + (size_t)G * E;              // [E]

    // The receiver and source workgroups come first in the grid, so that they run
    // beside the token workgroups instead of after them.
    const uint32_t extras = ws.world + G;
    if (blockIdx.x < extras) {
        const uint32_t extra = blockIdx.x;
        if (extra < ws.world) {
            // receiver: rows per expert, padded offsets, first row of every (source, expert) run
            const uint32_t r = extra;
            if (!(fin.recv_mask >> r & 1)) return;
            for (uint32_t w = tid; w < G * Le; w += blockDim.x) {
                const uint32_t g = Le > 1 ? __umulhi(w, ws.le_magic) : w;
                const uint32_t e = r * Le + (w - g * Le);
                tot[w] = e < E ? per_source[e * G + g] : 0;
            }
            __syncthreads();
            layout_from_totals(fin, ws, r, tot, scratch);
            return;
        }
        // source: its totals and their inclusive scan over the experts
        const uint32_t g = extra - ws.world;
        uint32_t carry = 0;
        for (uint32_t e0 = 0; e0 < E; e0 += blockDim.x) {
            const uint32_t e = e0 + tid;
            const uint32_t c = e < E ? per_source[e * G + g] : 0;
            const uint32_t incl = carry + block_inclusive_scan(c, scratch);
            if (e < E) {
                ws.num_routed[g * E + e] = c;
                ws.expert_offsets[g * E + e] = incl;
            }
            if (e0 + blockDim.x < E) {   // uniform: another round follows
                if (tid == blockDim.x - 1) s_carry = incl;
                __syncthreads();
                carry = s_carry;
            }
        }
        // the next routing launch fills the other copy of the totals
        if (g + 1 == G && tid == 0) ws.turn[0] = use ^ 1u;
        return;
    }

    const uint32_t work = blockIdx.x - extras;
    if (work >= total_tokens) return;
    uint32_t g = 0;
    while (g + 1 < G && work >= args.token_start[g + 1]) ++g;
    const uint32_t token = work - args.token_start[g];
    const PushSrc &src = args.src[g];
    if (token >= effective_tokens(src.bound_m, src.num_tokens)) return;

    // Wavefront 0 resolves the K routes, eight at a time with eight lanes per
    // route, and hands them to the others through LDS.  Two dependent trips to
    // memory: the expert ids and in-chunk ranks, then every term of the sums and
    // the receivers' descriptors in one go.  Measured on the prefill shape: done
    // by all seven wavefronts the lookups were three times the cache requests of
    // the rows themselves and cost 7 us; asking for the token's row BEFORE the
    // lookups (to hide its latency) cost another 4 us, because under a saturated
    // memory system what counts is to store a row as soon as it has arrived.
    const uint32_t *counts = ws.chunk_counts + (size_t)g * E * ws.nb_max;   // [E][nb_max]
    const uint32_t pad = ws.expert_padding;
    const uint32_t part = lane & 7, route = lane >> 3;
    const uint32_t passes = wave == 0 ? (K + 7) / 8 : 0;
    for (uint32_t pass = 0; pass < passes; ++pass) {
        const uint32_t k = pass * 8 + route;
        const bool in = k < K;
        const uint32_t kk = in ? k : 0;   // a lane without a route reads route 0 and is dropped below
        const uint32_t id = (uint32_t)src.indices[(size_t)token * src.indices_stride + kk];
        const uint32_t local = ws.local_rank[(size_t)g * ws.max_tk + token * K + kk];
        const bool live = in && id < E;
        const uint32_t e = live ? id : 0;
        const uint32_t upto = live ? (token * K + k) / kRouteBlock : 0;   // chunk of this entry
        const uint32_t r = owner_of_expert(ws, e);
        const uint32_t le = live ? e - r * Le : 0;
        // four terms of each sum per lane without a branch (clamped index, masked value)
        // When no other source has tokens nothing is laid out before mine: the second sum and its
        // loads drop out (five of sixteen lookups per lane; 0.75 us of the 4096-token step).
        const bool alone = args.single_source != 0;
        const uint32_t before = alone ? 0 : ws.laid_before[r * G + g];
        const PushDst dst = args.dst[r];
        uint32_t v_chunk[4], v_source[4], v_rows[4];
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) {
            const uint32_t n = part + 8 * i;
            v_chunk[i] = counts[(size_t)e * ws.nb_max + (n < upto ? n : 0)];
            v_source[i] = alone ? 0 : per_source[e * G + (n < G ? n : 0)];
            v_rows[i] = per_expert[r * Le + (n < le ? n : 0)];
        }
        uint32_t earlier = 0, base = 0;
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) {
            const uint32_t n = part + 8 * i;
            earlier += n < upto ? v_chunk[i] : 0;
            base += n < G && (before >> n & 1) ? v_source[i] : 0;
            const uint32_t padded = pad > 1 ? (v_rows[i] + pad - 1) / pad * pad : v_rows[i];
            base += n < le ? padded : 0;
        }
        // longer sums (more than 32 chunks in a source, more than 32 experts in a rank)
        for (uint32_t c = 32 + part; c < upto; c += 8) earlier += counts[(size_t)e * ws.nb_max + c];
        for (uint32_t q = 32 + part; q < le; q += 8) {
            const uint32_t rows = per_expert[r * Le + q];
            base += pad > 1 ? (rows + pad - 1) / pad * pad : rows;
        }
        earlier = group8_sum(earlier);
        base = group8_sum(base);
        const uint32_t toff = live ? earlier + local : 0;
        uint64_t to_row, to_scale;
        uint32_t to_stride;
        uint32_t slot = resolve_copy(dst, ws, base + toff, part == 0 && live, &to_row, &to_scale, &to_stride);
        if (!live) {
            slot = kInvalidSlot;
            to_row = 0;
            to_scale = 0;
            to_stride = 0;
        }
        if (part == 0 && in) {
            const uint32_t entry = token * K + k;
            ws.route_slot[(size_t)g * ws.max_tk + entry] = slot;
            ws.token_offset[(size_t)g * ws.max_tk + entry] = toff;
            s_row_ptr[k] = to_row;
            s_route_scale_ptr[k] = to_scale;
            s_route_scale_stride[k] = to_stride;
        }
    }
    __syncthreads();
    uint64_t row_ptr = 0, scale_ptr = 0;   // lane k: where the copy of route k goes
    uint32_t scale_stride = 0;
    if (lane < K) {
        row_ptr = s_row_ptr[lane];
        scale_ptr = s_route_scale_ptr[lane];
        scale_stride = s_route_scale_stride[lane];
    }
    push_rows<QUANT>(args, src, token, K, row_ptr, scale_ptr, scale_stride, s_scale, s_scale_ptr, s_scale_stride,
                     threadIdx.x, blockDim.x, true);
}

hipError_t launch_dispatch_push(const PushArgs &args, const Workspace &ws, bool quantize,
                                uint32_t total_tokens, hipStream_t stream, KernelTiming timing) {
    if (total_tokens == 0) return hipSuccess;
    const uint32_t threads = push_threads(args, quantize);
    if (quantize) {
        hipExtLaunchKernelGGL(dispatch_push_kernel<true>, dim3(total_tokens), dim3(threads), 0, stream,
                              timing.start, timing.stop, 0, args, ws);
    } else {
        hipExtLaunchKernelGGL(dispatch_push_kernel<false>, dim3(total_tokens), dim3(threads), 0, stream,
                              timing.start, timing.stop, 0, args, ws);
    }
    return hipGetLastError();
}

bool dispatch_small_fits(const PushArgs &args, const Workspace &ws, bool quantize, uint32_t total_tokens) {
    const uint64_t entries = (uint64_t)total_tokens * ws.topk;
    const uint64_t table = ((uint64_t)ws.num_groups + 3) * ws.num_experts;
    // The counting is redundant: every token workgroup visits every entry.  Measured with 8
    // sources and 8 entries per token against the two-launch dispatch: 13.0 against 15.4 us at
    // 256 tokens x 2048 entries, 17.0 against 16.3 us at 512 x 4096, 32.8 against 25.8 us at
    // 1024 x 8192.
    return entries <= kSmallMaxEntries && entries * total_tokens <= kSmallMaxVisits &&
           total_tokens <= 1024 && table <= 8192 + 3072 &&
           ws.experts_per_rank <= push_threads(args, quantize);
}

hipError_t launch_dispatch_small(const PushArgs &args, const FinalizeArgs &fin, const Workspace &ws,
                                 bool quantize, uint32_t total_tokens, hipStream_t stream, KernelTiming timing) {
    const uint32_t threads = push_threads(args, quantize);
    const uint32_t blocks = total_tokens + (fin.recv_mask != 0 ? ws.world : 0);
    if (blocks == 0) return hipSuccess;
    const size_t table_words = (((size_t)ws.num_groups + 3) * ws.num_experts + 1) & ~(size_t)1;
    size_t lds = table_words * sizeof(uint32_t) + (size_t)total_tokens * sizeof(uint64_t);
    // One source with tokens whose index rows are dense: the flat-array variant.
    PushArgs a = args;
    a.single_source = 0;
    uint32_t senders = 0;
    for (uint32_t g = 0; g < ws.num_groups; ++g) {
        if (args.src[g].num_tokens == 0) continue;
        ++senders;
        a.single_source = g + 1;
    }
    if (senders != 1 || args.src[a.single_source - 1].indices_stride != ws.topk) a.single_source = 0;
    if (a.single_source != 0) {
        a.single = args.src[a.single_source - 1];
        const size_t tokens_words = 4 * (size_t)ws.num_experts;
        const size_t receiver_words = (size_t)ws.num_groups * ws.experts_per_rank;
        lds = (tokens_words > receiver_words ? tokens_words : receiver_words) * sizeof(uint32_t);
        // The quick form: a wavefront beside those that move the row, and no receiver workgroups.
        const uint32_t pieces = quantize ? args.hidden_dim / 16 : args.row_bytes / 16;
        if (ws.topk <= 8 && pieces + kWave <= 1024 && (quantize || args.hidden_dim_scale <= pieces)) {
            const uint32_t quick_threads = (pieces + kWave - 1) / kWave * kWave + kWave;
            const uint32_t counters = quick_threads - kWave;
            const uint32_t per_thread = (total_tokens * ws.topk + counters - 1) / counters;
#define A2A_LAUNCH_QUICK(NB)                                                                                         \
    do {                                                                                                             \
        if (quantize)                                                                                                \
            hipExtLaunchKernelGGL((dispatch_quick_kernel<NB, true>), dim3(total_tokens), dim3(quick_threads),        \
                                  (size_t)ws.num_experts * sizeof(uint32_t), stream, timing.start, timing.stop, 0,   \
                                  a, fin, ws);                                                                       \
        else                                                                                                         \
            hipExtLaunchKernelGGL((dispatch_quick_kernel<NB, false>), dim3(total_tokens), dim3(quick_threads),       \
                                  (size_t)ws.num_experts * sizeof(uint32_t), stream, timing.start, timing.stop, 0,   \
                                  a, fin, ws);                                                                       \
    } while (0)
            if (per_thread <= 1) A2A_LAUNCH_QUICK(1);
            else if (per_thread == 2) A2A_LAUNCH_QUICK(2);
            else if (per_thread == 3) A2A_LAUNCH_QUICK(3);
            else if (per_thread == 4) A2A_LAUNCH_QUICK(4);
            else A2A_LAUNCH_QUICK(8);
#undef A2A_LAUNCH_QUICK
            return hipGetLastError();
        }
    }
#define A2A_LAUNCH_SMALL(Q, S)                                                                                       \
    hipExtLaunchKernelGGL((dispatch_small_kernel<Q, S>), dim3(blocks), dim3(threads), lds, stream, timing.start,  \
                          timing.stop, 0, a, fin, ws)
    if (quantize) {
        if (a.single_source != 0) A2A_LAUNCH_SMALL(true, true); else A2A_LAUNCH_SMALL(true, false);
    } else {
        if (a.single_source != 0) A2A_LAUNCH_SMALL(false, true); else A2A_LAUNCH_SMALL(false, false);
    }
#undef A2A_LAUNCH_SMALL
    return hipGetLastError();
}

// Tokens per workgroup of dispatch_single_kernel: as many as it takes to have about one token
// workgroup per compute unit (every workgroup counts all entries, so fewer workgroups count
// less; but a compute unit without a workgroup moves no rows).  Measured on the 1024-token
// step with 2 / 4 / 8 tokens a workgroup: 47.4 / 44.9 / 51.1 us.
uint32_t single_tokens_per_group(uint32_t total_tokens) {
    constexpr uint32_t kComputeUnits = 256;
    const uint32_t per_group = (total_tokens + kComputeUnits - 1) / kComputeUnits;
    return per_group < 1 ? 1 : per_group > kTokensPerGroup ? kTokensPerGroup : per_group;
}

// Threads of a dispatch_single_kernel workgroup: as many teams of `team` threads as fit, at most
// one per token of the workgroup.
uint32_t single_threads(uint32_t team, uint32_t per_group) {
    uint32_t teams = 1024 / team;
    if (teams > per_group) teams = per_group;
    return teams * team;
}

// Whether a step takes dispatch_single_kernel: one source has tokens, its index rows are dense,
// and the step is of the size where counting its entries once per kTokensPerGroup tokens is
// cheaper than a routing launch in front of the pack.
bool dispatch_single_fits(const PushArgs &args, const Workspace &ws, bool quantize, uint32_t total_tokens) {
    uint32_t senders = 0, g_single = 0;
    for (uint32_t g = 0; g < ws.num_groups; ++g) {
        if (args.src[g].num_tokens == 0) continue;
        ++senders;
        g_single = g;
    }
    if (senders != 1 || args.src[g_single].indices_stride != ws.topk) return false;
    const uint64_t entries = (uint64_t)total_tokens * ws.topk;
    const uint32_t per_group = single_tokens_per_group(total_tokens);
    const uint32_t threads = single_threads(push_threads(args, quantize), per_group);
    // one thread per route of the workgroup's tokens and per local expert; the receivers' table in LDS
    return entries <= kSingleMaxEntries && per_group * ws.topk <= threads && ws.experts_per_rank <= threads &&
           (size_t)ws.num_groups * ws.experts_per_rank <= 8192;
}

hipError_t launch_dispatch_single(const PushArgs &args, const FinalizeArgs &fin, const Workspace &ws,
                                  bool quantize, uint32_t total_tokens, hipStream_t stream, KernelTiming timing) {
    if (total_tokens == 0) return hipSuccess;
    const uint32_t team = push_threads(args, quantize);
    const uint32_t per_group = single_tokens_per_group(total_tokens);
    const uint32_t threads = single_threads(team, per_group);
    const uint32_t blocks = (total_tokens + per_group - 1) / per_group;   // the receivers are laid out by the first of them
    const size_t lds = 2 * (size_t)ws.num_experts * sizeof(uint32_t);
    PushArgs a = args;
    a.single_source = 0;
    for (uint32_t g = 0; g < ws.num_groups; ++g) {
        if (args.src[g].num_tokens != 0) a.single_source = g + 1;
    }
    a.single = args.src[a.single_source - 1];
    // The form with a spare wavefront per workgroup that resolves the routes while the teams quantise:
    // at most eight routes a token, 32 a workgroup, and two rounds.
    if (ws.topk <= 8 && per_group * ws.topk <= kTeamsMaxRoutes && team + kWave <= 1024 &&
        (quantize || args.hidden_dim_scale <= (team < kTeamsMaxScales ? team : kTeamsMaxScales))) {
        uint32_t teams = (1024 - kWave) / team;
        if (teams > per_group) teams = per_group;
        const uint32_t rounds = (per_group + teams - 1) / teams;
        const uint32_t counters = teams * team;
        const uint32_t per_thread = (total_tokens * ws.topk + counters - 1) / counters;
        if (rounds <= 2 && (!quantize || args.hidden_dim / 128 <= kTeamsMaxScales)) {
            const size_t cnt_bytes = (size_t)ws.num_experts * sizeof(uint32_t);
#define A2A_LAUNCH_TEAMS(NB, R)                                                                                   \
    do {                                                                                                          \
        if (quantize)                                                                                             \
            hipExtLaunchKernelGGL((dispatch_teams_kernel<NB, R, true>), dim3(blocks), dim3(counters + kWave),     \
                                  cnt_bytes, stream, timing.start, timing.stop, 0, a, fin, ws, team, per_group);  \
        else                                                                                                      \
            hipExtLaunchKernelGGL((dispatch_teams_kernel<NB, R, false>), dim3(blocks), dim3(counters + kWave),    \
                                  cnt_bytes, stream, timing.start, timing.stop, 0, a, fin, ws, team, per_group);  \
    } while (0)
            if (rounds == 1) {
                if (per_thread <= 5) A2A_LAUNCH_TEAMS(5, 1);
                else if (per_thread <= 10) A2A_LAUNCH_TEAMS(10, 1);
                else A2A_LAUNCH_TEAMS(16, 1);
            } else {
                if (per_thread <= 5) A2A_LAUNCH_TEAMS(5, 2);
                else if (per_thread <= 10) A2A_LAUNCH_TEAMS(10, 2);
                else A2A_LAUNCH_TEAMS(16, 2);
            }
#undef A2A_LAUNCH_TEAMS
            return hipGetLastError();
        }
    }
    if (quantize) {
        hipExtLaunchKernelGGL(dispatch_single_kernel<true>, dim3(blocks), dim3(threads), lds, stream, timing.start,
                              timing.stop, 0, a, fin, ws, team, per_group);
    } else {
        hipExtLaunchKernelGGL(dispatch_single_kernel<false>, dim3(blocks), dim3(threads), lds, stream, timing.start,
                              timing.stop, 0, a, fin, ws, team, per_group);
    }
    return hipGetLastError();
}

hipError_t launch_dispatch_resolve(const PushArgs &args, const FinalizeArgs &fin, const Workspace &ws,
                                   bool quantize, uint32_t total_tokens, hipStream_t stream, KernelTiming timing) {
    uint32_t threads = push_threads(args, quantize);
    if (threads < ws.experts_per_rank) {   // a receiver workgroup has one thread per local expert
        threads = (ws.experts_per_rank + kWave - 1) / kWave * kWave;
    }
    const uint32_t blocks = total_tokens + ws.world + ws.num_groups;
    PushArgs a = args;
    uint32_t senders = 0;
    a.single_source = 0;
    for (uint32_t g = 0; g < ws.num_groups; ++g) {
        if (args.src[g].num_tokens == 0) continue;
        ++senders;
        a.single_source = g + 1;
    }
    if (senders != 1) a.single_source = 0;    // here only "one source has tokens": the rows may be strided
    if (a.single_source != 0) a.single = args.src[a.single_source - 1];
    if (quantize) {
        hipExtLaunchKernelGGL(dispatch_resolve_kernel<true>, dim3(blocks), dim3(threads), 0, stream, timing.start,
                              timing.stop, 0, a, fin, ws);
    } else {
        hipExtLaunchKernelGGL(dispatch_resolve_kernel<false>, dim3(blocks), dim3(threads), 0, stream, timing.start,
                              timing.stop, 0, a, fin, ws);
    }
    return hipGetLastError();
}

}  // namespace a2a
