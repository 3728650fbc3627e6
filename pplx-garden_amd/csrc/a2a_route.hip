// Routing pass: per-expert histogram of the top-k expert ids, a deterministic
// rank for every (token, k) entry inside its expert, the offset scan, and the
// receiver-side layout.
//
// What it replaces: phase 1 of the reference's dispatch-send kernel, which runs
// on ONE block and hands out ranks with shared-memory atomicAdd in arrival
// order (a2a_dispatch_send.cu:176-243), and the per-receiver layout the
// reference computes on a CPU thread (a2a_worker.rs:577-606,621-694).
//
// Design for CDNA4, two launches and no device-wide fence or atomic:
//
// route_hist_kernel: the entries are cut into chunks of 1024, one workgroup of
// 16 wavefronts per chunk.  Inside a wavefront, equal expert ids are matched
// with one 64-bit ballot per id bit (no LDS atomics, so the result does not
// depend on scheduling); the lane's rank among its matches is a popcount of
// the match mask below it.  Wavefront totals meet in a [16][E] LDS table whose
// columns are scanned by E threads.  The rank of an entry is then
// `block_prefix[chunk][e] + local_rank[entry]`, ascending in (token, k):
// stable, reproducible, and never materialised in a second pass over the
// entries.
//
// route_finalize_kernel: two workgroups per logical rank.  Workgroup i turns
// the chunk histograms of SOURCE i into prefixes over chunks and scans its
// expert offsets; workgroup N + i lays out RECEIVER i from the chunk histograms
// of every source.  Each workgroup reads what it needs straight from the
// histograms (one round trip to memory, all loads in flight together), so no
// workgroup depends on another.
#include "a2a_scan.h"

namespace a2a {

namespace {

// Sum of `n` words spaced `stride` apart, loads batched eight at a time so
// that they are in flight together.
__device__ __forceinline__ uint32_t strided_sum(const uint32_t *p, uint32_t n, size_t stride) {
    uint32_t sum = 0;
    for (uint32_t b = 0; b < n; b += 8) {
        uint32_t v[8];
#pragma unroll
        for (uint32_t j = 0; j < 8; ++j) v[j] = b + j < n ? p[(size_t)(b + j) * stride] : 0;
#pragma unroll
        for (uint32_t j = 0; j < 8; ++j) sum += v[j];
    }
    return sum;
}

// Source part of the finalize: chunk histograms of source `g` -> exclusive
// prefixes over chunks, per-expert totals, their inclusive scan over experts
// (a2a_dispatch_send.cu:199-204,209-242).  Whole workgroup.
__device__ void fold_source(const FinalizeArgs &args, const Workspace &ws, uint32_t g, uint32_t *part_sum,
                            uint32_t *scratch) {
    const uint32_t E = ws.num_experts;
    const uint32_t tid = threadIdx.x;
    const uint32_t num_blocks = args.num_blocks[g];
    if (num_blocks == 0) {
        if (tid < E) {
            ws.num_routed[g * E + tid] = 0;
            ws.expert_offsets[g * E + tid] = 0;
        }
        return;
    }
    const uint32_t parts = blockDim.x / E;   // >= 1: threads that share a column
    const uint32_t part = tid / E;
    const uint32_t e0 = tid - part * E;
    const uint32_t per = (num_blocks + parts - 1) / parts;
    const bool has_column = part < parts;
    uint32_t b0 = 0, nb = 0;
    uint32_t first[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) first[j] = 0;
    if (has_column) {
        b0 = part * per < num_blocks ? part * per : num_blocks;
        const uint32_t b1 = b0 + per < num_blocks ? b0 + per : num_blocks;
        nb = b1 - b0;
        const uint32_t *col = ws.block_hist + ((size_t)g * ws.nb_max + b0) * E + e0;
#pragma unroll
        for (uint32_t j = 0; j < 8; ++j) first[j] = j < nb ? col[(size_t)j * E] : 0;
        uint32_t sum = 0;
#pragma unroll
        for (uint32_t j = 0; j < 8; ++j) sum += first[j];
        if (nb > 8) sum += strided_sum(col + (size_t)8 * E, nb - 8, E);
        part_sum[part * E + e0] = sum;
    }
    __syncthreads();
    uint32_t total = 0;
    if (has_column) {
        uint32_t run = 0;
        for (uint32_t p = 0; p < parts; ++p) {
            const uint32_t s = part_sum[p * E + e0];
            if (p < part) run += s;
            total += s;
        }
        const uint32_t *col = ws.block_hist + ((size_t)g * ws.nb_max + b0) * E + e0;
        uint32_t *out = ws.block_prefix + ((size_t)g * ws.nb_max + b0) * E + e0;
#pragma unroll
        for (uint32_t j = 0; j < 8; ++j) {
            if (j < nb) out[(size_t)j * E] = run;
            run += first[j];
        }
        for (uint32_t j = 8; j < nb; ++j) {
            out[(size_t)j * E] = run;
            run += col[(size_t)j * E];
        }
    }
    const bool owner = has_column && part == 0;
    if (owner) ws.num_routed[g * E + e0] = total;
    const uint32_t incl = block_inclusive_scan(owner ? total : 0, scratch);
    if (owner) ws.expert_offsets[g * E + e0] = incl;
}

// Receiver part of the finalize: rows of receiver `r`, from the chunk
// histograms of the sources folded by this launch and the published counts of
// the sources that sent earlier in the step.  Whole workgroup; `tot` holds
// N * Le words.
__device__ void layout_receiver(const FinalizeArgs &args, const Workspace &ws, uint32_t r, uint32_t *tot,
                                uint32_t *scratch) {
    const uint32_t N = ws.num_groups, E = ws.num_experts, Le = ws.experts_per_rank;
    const uint32_t tid = threadIdx.x;
    const uint32_t items = N * Le;              // (source, local expert) pairs
    for (uint32_t i = tid; i < items; i += blockDim.x) tot[i] = 0;
    __syncthreads();
    uint32_t parts = blockDim.x / items;
    if (parts == 0) parts = 1;
    for (uint32_t w = tid; w < parts * items; w += blockDim.x) {
        const uint32_t part = w / items;
        const uint32_t item = w - part * items;
        const uint32_t g = item / Le;
        const uint32_t e = r * Le + (item - g * Le);
        if (e >= E || !(args.valid_mask >> g & 1)) continue;
        uint32_t sum = 0;
        if (args.fold_mask >> g & 1) {
            const uint32_t num_blocks = args.num_blocks[g];
            const uint32_t per = (num_blocks + parts - 1) / parts;
            const uint32_t b0 = part * per < num_blocks ? part * per : num_blocks;
            const uint32_t b1 = b0 + per < num_blocks ? b0 + per : num_blocks;
            sum = strided_sum(ws.block_hist + ((size_t)g * ws.nb_max + b0) * E + e, b1 - b0, E);
        } else if (part == 0) {
            sum = ws.num_routed[g * E + e];
        }
        if (sum != 0) atomicAdd(&tot[item], sum);
    }
    __syncthreads();
    layout_from_totals(args, ws, r, tot, scratch);
}

// Ranks the entries of chunk `chunk` of source `g` inside their experts and
// returns, to thread e < E, the number of entries of the chunk with expert e.
// Whole workgroup (kRouteBlock threads).
__device__ uint32_t rank_chunk(const RouteSrc &src, const Workspace &ws, uint32_t g, uint32_t chunk,
                               uint16_t (*wave_hist)[A2A_MAX_EXPERTS]) {
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = tid / kWave;
    const uint32_t E = ws.num_experts;
    const uint32_t K = ws.topk;
    const uint32_t num_entries = effective_tokens(src.bound_m, src.num_tokens) * K;

    // The entry's expert id is asked for first: it travels while the table is cleared.
    const uint32_t entry = chunk * kRouteBlock + tid;
    bool valid = entry < num_entries;
    uint32_t expert = 0;
    if (valid) {
        const uint32_t token = entry / K;
        const uint32_t k = entry - token * K;
        expert = (uint32_t)src.indices[(size_t)token * src.indices_stride + k];
    }
    if (tid < E) {
#pragma unroll
        for (int w = 0; w < kRouteWaves; ++w) wave_hist[w][tid] = 0;
    }
    __syncthreads();
    if (valid && expert >= E) {
        valid = false;
        atomicOr(ws.err, A2A_DEV_BAD_EXPERT_ID);
    }

    // Lanes of this wavefront that hold the same expert id.
    uint64_t peers = __ballot(valid);
    const uint32_t nbits = 32 - __clz((int)(E - 1) | 1);
    for (uint32_t b = 0; b < nbits; ++b) {
        const bool bit = (expert >> b) & 1;
        const uint64_t set = __ballot(valid && bit);
        peers &= bit ? set : ~set;
    }
    const uint32_t rank_in_wave = __popcll(peers & ((1ull << lane) - 1));
    if (valid && rank_in_wave == 0) wave_hist[wave][expert] = (uint16_t)__popcll(peers);
    __syncthreads();

    // Exclusive scan of each expert's column over the 16 wavefronts.
    uint32_t run = 0;
    if (tid < E) {
#pragma unroll
        for (int w = 0; w < kRouteWaves; ++w) {
            const uint32_t c = wave_hist[w][tid];
            wave_hist[w][tid] = (uint16_t)run;
            run += c;
        }
    }
    __syncthreads();

    if (entry < num_entries) {
        ws.local_rank[(size_t)g * ws.max_tk + entry] =
            valid ? (uint16_t)(wave_hist[wave][expert] + rank_in_wave) : (uint16_t)0;
    }
    return run;
}

}  // namespace

// MODE 1 (group steps): the launch also adds every chunk's counts to the step's
// totals (per source and expert, and per expert), which the pack of a large
// group step resolves its rows from.  MODE 2 (the send of a split call, one
// source per launch): to that source's totals per expert and per owning rank,
// which the staging launch resolves its positions from.  The totals exist twice
// and are used in turn, so that this launch can clear the copy of the NEXT step
// while it fills its own: turn[0] says which copy to fill (flipped by the launch
// that follows and consumes them), turn[1] tells that launch which copy this
// one filled.  All of it lives on the device, so a recorded sequence of launches
// can be replayed.
template <int MODE>
__global__ __launch_bounds__(kRouteBlock) void route_hist_kernel(const RouteArgs args,
                                                                 const Workspace ws) {
    __shared__ uint16_t wave_hist[kRouteWaves][A2A_MAX_EXPERTS];
    if constexpr (MODE == 1) {
        // what the head of a workgroup takes from the argument block, asked for in one go
        A2A_PIN(args.block_start[0]);
        A2A_PIN(args.block_start[1]);
        A2A_PIN(ws.num_groups);
        A2A_PIN(ws.num_experts);
        A2A_PIN(ws.topk);
        A2A_PIN(ws.nb_max);
        A2A_PIN(ws.max_tk);
        A2A_PIN(ws.turn);
        A2A_PIN(ws.totals);
        A2A_PIN(ws.chunk_counts);
        A2A_PIN(ws.local_rank);
        A2A_PIN(ws.err);
    }
    const uint32_t G = ws.num_groups, E = ws.num_experts;
    const uint32_t words = MODE == 2 ? E + ws.world : (G + 1) * E;
    uint32_t *totals = MODE == 2 ? ws.send_totals : ws.totals;
    uint32_t *turn = MODE == 2 ? ws.send_turn : ws.turn;
    uint32_t fill = 0;
    if constexpr (MODE != 0) {
        fill = turn[0] & 1u;
        // The hand-over between steps is the job of one workgroup of its own, the last of the grid:
        // it has to wait for `turn` before it can do anything, which a chunk workgroup has not (its
        // entries travel meanwhile, and it needs `fill` only for its final atomics).
        if (blockIdx.x + 1 == gridDim.x) {
            uint32_t *next = totals + (size_t)(fill ^ 1u) * words;
            for (uint32_t i = threadIdx.x; i < words; i += kRouteBlock) next[i] = 0;
            if (threadIdx.x == 0) turn[1] = fill;
            return;
        }
    }
    // Which source and which chunk of it this workgroup handles (uniform).
    uint32_t g = 0;
    while (g + 1 < G && blockIdx.x >= args.block_start[g + 1]) ++g;
    const uint32_t chunk = blockIdx.x - args.block_start[g];
    const uint32_t count = rank_chunk(args.src[g], ws, g, chunk, wave_hist);
    uint32_t *mine = totals + (size_t)fill * words;
    if (threadIdx.x < E) {
        if constexpr (MODE == 0) {
            ws.block_hist[((size_t)g * ws.nb_max + chunk) * E + threadIdx.x] = count;
        } else {
            // the consumer reads all chunks of ONE expert, and all sources of one expert: keep those together
            ws.chunk_counts[((size_t)g * E + threadIdx.x) * ws.nb_max + chunk] = count;
            if (count != 0) {
                if constexpr (MODE == 1) {
                    atomicAdd(&mine[threadIdx.x * G + g], count);
                    atomicAdd(&mine[G * E + threadIdx.x], count);
                } else {
                    atomicAdd(&mine[threadIdx.x], count);
                }
            }
        }
    }
    if constexpr (MODE == 2) {
        // Per owning rank: the experts of a rank are added up in LDS first, so that one atomic per
        // rank and chunk reaches memory (one per expert would pile hundreds onto a few addresses).
        __shared__ uint32_t rank_sum[kMaxWorld];
        if (threadIdx.x < ws.world) rank_sum[threadIdx.x] = 0;
        __syncthreads();
        if (threadIdx.x < E && count != 0) atomicAdd(&rank_sum[owner_of_expert(ws, threadIdx.x)], count);
        __syncthreads();
        if (threadIdx.x < ws.world && rank_sum[threadIdx.x] != 0) {
            atomicAdd(&mine[E + threadIdx.x], rank_sum[threadIdx.x]);
        }
    }
}

// Tables of sources that were routed with no tokens: no chunk workgroup exists
// for them, so somebody else clears them.
__device__ void clear_empty_sources(const FinalizeArgs &fin, const Workspace &ws) {
    const uint32_t E = ws.num_experts;
    for (uint32_t g = 0; g < ws.num_groups; ++g) {
        if ((fin.fold_mask >> g & 1) && fin.num_blocks[g] == 0 && threadIdx.x < E) {
            ws.num_routed[g * E + threadIdx.x] = 0;
            ws.expert_offsets[g * E + threadIdx.x] = 0;
        }
    }
}

// Per-expert number of entries of source `g` in the chunks before `chunk`,
// returned to thread e < E.  Counts do not depend on the order of arrival, so
// plain LDS atomics do (eight loads in flight per lane, one atomic per entry).
// `counts` holds E words.  Whole workgroup.
__device__ uint32_t count_prior_chunks(const RouteSrc &src, const Workspace &ws, uint32_t chunk,
                                       uint32_t *counts) {
    const uint32_t tid = threadIdx.x;
    const uint32_t E = ws.num_experts;
    const uint32_t K = ws.topk;
    if (chunk == 0) return 0;
    uint32_t num_entries = effective_tokens(src.bound_m, src.num_tokens) * K;
    if (num_entries > chunk * kRouteBlock) num_entries = chunk * kRouteBlock;
    if (tid < E) counts[tid] = 0;
    __syncthreads();
    for (uint32_t e0 = 0; e0 < num_entries; e0 += 8 * kRouteBlock) {
        uint32_t expert[8];
#pragma unroll
        for (uint32_t j = 0; j < 8; ++j) {
            const uint32_t entry = e0 + j * kRouteBlock + tid;
            expert[j] = 0xFFFFFFFFu;
            if (entry < num_entries) {
                const uint32_t token = entry / K;
                expert[j] = (uint32_t)src.indices[(size_t)token * src.indices_stride + (entry - token * K)];
            }
        }
#pragma unroll
        for (uint32_t j = 0; j < 8; ++j) {
            if (expert[j] < E) atomicAdd(&counts[expert[j]], 1u);
        }
    }
    __syncthreads();
    const uint32_t sum = tid < E ? counts[tid] : 0;
    __syncthreads();
    return sum;
}

// The whole routing pass in ONE launch, for steps of moderate size.  The grid
// holds one workgroup per chunk of every source, then one per receiver; none
// depends on another:
//  - a chunk workgroup counts the entries of the chunks before its own (that is
//    its prefix), ranks its own entries, and, if it is the last chunk of its
//    source, publishes the source's totals and their scan over experts;
//  - a receiver workgroup counts, over the entries of EVERY source, the copies
//    bound for its experts and lays out its rows.
// The redundant counting is quadratic in the number of chunks of a source, so
// long inputs take the two-launch path (route_hist + route_finalize) instead.
__global__ __launch_bounds__(kRouteBlock) void route_fused_kernel(const RouteArgs args,
                                                                  const FinalizeArgs fin,
                                                                  const Workspace ws) {
    __shared__ uint16_t wave_hist[kRouteWaves][A2A_MAX_EXPERTS];
    __shared__ uint32_t tot[A2A_MAX_EXPERTS + kMaxWorld];
    __shared__ uint32_t scratch[kRouteWaves];
    const uint32_t N = ws.num_groups, E = ws.num_experts, K = ws.topk, Le = ws.experts_per_rank;
    const uint32_t tid = threadIdx.x;
    const uint32_t chunk_blocks = args.block_start[N];

    if (blockIdx.x == 0) clear_empty_sources(fin, ws);
    if (blockIdx.x >= chunk_blocks) {
        // receiver workgroup
        const uint32_t rank = blockIdx.x - chunk_blocks;
        if (!(fin.recv_mask >> rank & 1)) return;
        for (uint32_t i = tid; i < N * Le; i += kRouteBlock) tot[i] = 0;
        __syncthreads();
        for (uint32_t g = 0; g < N; ++g) {
            if (!(fin.valid_mask >> g & 1)) continue;
            if (!(fin.fold_mask >> g & 1)) {
                // a source that sent earlier in this step: its counts are published
                if (tid < Le && rank * Le + tid < E) tot[g * Le + tid] = ws.num_routed[g * E + rank * Le + tid];
                continue;
            }
            const RouteSrc &src = args.src[g];
            const uint32_t entries = effective_tokens(src.bound_m, src.num_tokens) * K;
            for (uint32_t e0 = 0; e0 < entries; e0 += 8 * kRouteBlock) {
                uint32_t expert[8];
#pragma unroll
                for (uint32_t j = 0; j < 8; ++j) {
                    const uint32_t entry = e0 + j * kRouteBlock + tid;
                    expert[j] = 0xFFFFFFFFu;
                    if (entry < entries) {
                        const uint32_t token = entry / K;
                        expert[j] = (uint32_t)src.indices[(size_t)token * src.indices_stride + (entry - token * K)];
                    }
                }
#pragma unroll
                for (uint32_t j = 0; j < 8; ++j) {
                    if (expert[j] < E && expert[j] / Le == rank) atomicAdd(&tot[g * Le + expert[j] - rank * Le], 1u);
                }
            }
        }
        __syncthreads();
        layout_from_totals(fin, ws, rank, tot, scratch);
        return;
    }

    // chunk workgroup
    uint32_t g = 0;
    while (g + 1 < N && blockIdx.x >= args.block_start[g + 1]) ++g;
    const uint32_t chunk = blockIdx.x - args.block_start[g];
    const RouteSrc &src = args.src[g];
    const uint32_t prior = count_prior_chunks(src, ws, chunk, tot);
    const uint32_t own = rank_chunk(src, ws, g, chunk, wave_hist);
    if (tid < E) {
        ws.block_hist[((size_t)g * ws.nb_max + chunk) * E + tid] = own;
        ws.block_prefix[((size_t)g * ws.nb_max + chunk) * E + tid] = prior;
    }
    if (chunk + 1 == fin.num_blocks[g]) {
        const uint32_t total = prior + own;
        if (tid < E) ws.num_routed[g * E + tid] = total;
        const uint32_t incl = block_inclusive_scan(tid < E ? total : 0, scratch);
        if (tid < E) ws.expert_offsets[g * E + tid] = incl;
    }
}

// Two workgroups per logical rank, independent of each other: workgroup i folds
// source i, workgroup N + i lays out receiver i.
__global__ __launch_bounds__(kRouteBlock) void route_finalize_kernel(const FinalizeArgs args,
                                                                     const Workspace ws) {
    __shared__ uint32_t part_sum[kRouteBlock];
    __shared__ uint32_t tot[A2A_MAX_EXPERTS + kMaxWorld];
    __shared__ uint32_t scratch[kRouteWaves];
    if (blockIdx.x < ws.world) {
        const uint32_t group = blockIdx.x;
        if (group < ws.num_groups && (args.fold_mask >> group & 1)) fold_source(args, ws, group, part_sum, scratch);
    } else {
        const uint32_t rank = blockIdx.x - ws.world;
        if (args.recv_mask >> rank & 1) layout_receiver(args, ws, rank, tot, scratch);
    }
}

hipError_t launch_route(const RouteArgs &args, const Workspace &ws, uint32_t total_blocks,
                        hipStream_t stream) {
    if (total_blocks == 0) return hipSuccess;
    hipLaunchKernelGGL(route_hist_kernel<0>, dim3(total_blocks), dim3(kRouteBlock), 0, stream, args, ws);
    return hipGetLastError();
}

hipError_t launch_route_accumulate(const RouteArgs &args, const Workspace &ws, uint32_t total_blocks,
                                   hipStream_t stream, bool for_send, KernelTiming timing) {
    // one workgroup per chunk and one more that hands over the totals between steps
    const dim3 grid(total_blocks + 1);
    if (for_send) {
        hipLaunchKernelGGL(route_hist_kernel<2>, grid, dim3(kRouteBlock), 0, stream, args, ws);
    } else {
        hipExtLaunchKernelGGL(route_hist_kernel<1>, grid, dim3(kRouteBlock), 0, stream, timing.start, timing.stop,
                              0, args, ws);
    }
    return hipGetLastError();
}

hipError_t launch_route_fused(const RouteArgs &args, const FinalizeArgs &fin, const Workspace &ws,
                              hipStream_t stream) {
    const uint32_t blocks = args.block_start[ws.num_groups] + (fin.recv_mask != 0 ? ws.world : 0);
    if (blocks == 0) return hipSuccess;   // nothing routed, nobody laid out
    hipLaunchKernelGGL(route_fused_kernel, dim3(blocks), dim3(kRouteBlock), 0, stream, args, fin, ws);
    return hipGetLastError();
}

hipError_t launch_finalize(const FinalizeArgs &args, const Workspace &ws, hipStream_t stream) {
    hipLaunchKernelGGL(route_finalize_kernel, dim3(2 * ws.world), dim3(kRouteBlock), 0, stream, args, ws);
    return hipGetLastError();
}

}  // namespace a2a
