// Routing pass: per-expert histogram of the top-k expert ids, a deterministic
// rank for every (token, k) entry inside its expert, the offset scan, and the
// receiver-side layout.
//
// What it replaces: phase 1 of the reference's dispatch-send kernel, which runs
// on ONE block and hands out ranks with shared-memory atomicAdd in arrival
// order (a2a_dispatch_send.cu:176-243), and the per-receiver layout the
// reference computes on a CPU thread (a2a_worker.rs:577-606,621-694).
//
// Design for CDNA4: the entries are cut into chunks of 1024, one workgroup of
// 16 wavefronts per chunk.  Inside a wavefront, equal expert ids are matched
// with one 64-bit ballot per id bit (no LDS atomics, so the result does not
// depend on scheduling); the lane's rank among its matches is a popcount of
// the match mask below it.  Wavefront totals meet in a [16][E] LDS table whose
// columns are scanned by E threads.  A second, single-workgroup kernel folds
// the per-chunk histograms into prefixes and computes all scans.  The rank of
// an entry is therefore `block_prefix[chunk][e] + local_rank[entry]`, ascending
// in (token, k): stable, reproducible, and never materialised in a second pass
// over the entries.
#include "a2a_internal.h"

namespace a2a {

__global__ __launch_bounds__(kRouteBlock) void route_hist_kernel(const RouteArgs args,
                                                                 const Workspace ws) {
    __shared__ uint16_t wave_hist[kRouteBlock / kWave][A2A_MAX_EXPERTS];

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = tid / kWave;
    const uint32_t E = ws.num_experts;
    const uint32_t K = ws.topk;

    // Which source and which chunk of it this workgroup handles (uniform).
    uint32_t g = 0;
    while (g + 1 < ws.world && blockIdx.x >= args.block_start[g + 1]) ++g;
    const uint32_t chunk = blockIdx.x - args.block_start[g];
    const RouteSrc src = args.src[g];
    const uint32_t num_entries = effective_tokens(src.bound_m, src.num_tokens) * K;

    for (uint32_t i = tid; i < (kRouteBlock / kWave) * E; i += kRouteBlock) {
        wave_hist[i / E][i % E] = 0;
    }
    __syncthreads();

    const uint32_t entry = chunk * kRouteBlock + tid;
    bool valid = entry < num_entries;
    uint32_t expert = 0;
    if (valid) {
        const uint32_t token = entry / K;
        const uint32_t k = entry - token * K;
        expert = (uint32_t)__builtin_nontemporal_load(
            &src.indices[(size_t)token * src.indices_stride + k]);
        if (expert >= E) {
            valid = false;
            atomicOr(ws.err, A2A_DEV_BAD_EXPERT_ID);
        }
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
    if (valid && rank_in_wave == 0) {
        wave_hist[wave][expert] = (uint16_t)__popcll(peers);
    }
    __syncthreads();

    // Exclusive scan of each expert's column over the 16 wavefronts.
    uint32_t *block_hist = ws.block_prefix + ((size_t)g * ws.nb_max + chunk) * E;
    for (uint32_t e = tid; e < E; e += kRouteBlock) {
        uint32_t run = 0;
#pragma unroll
        for (int w = 0; w < kRouteBlock / kWave; ++w) {
            const uint32_t c = wave_hist[w][e];
            wave_hist[w][e] = (uint16_t)run;
            run += c;
        }
        block_hist[e] = run;
    }
    __syncthreads();

    if (entry < num_entries) {
        ws.local_rank[(size_t)g * ws.max_tk + entry] =
            valid ? (uint16_t)(wave_hist[wave][expert] + rank_in_wave) : (uint16_t)0;
    }
}

// Inclusive scan over the 64 lanes of a wavefront.
__device__ __forceinline__ uint32_t wave_inclusive_scan(uint32_t v, uint32_t lane) {
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        const uint32_t up = __shfl_up(v, d);
        if (lane >= (uint32_t)d) v += up;
    }
    return v;
}

// One workgroup.  Dynamic LDS: counts[N*E] then scratch[E + 32].
__global__ __launch_bounds__(1024) void route_finalize_kernel(const FinalizeArgs args,
                                                              const Workspace ws) {
    extern __shared__ uint32_t lds[];
    const uint32_t N = ws.world;
    const uint32_t E = ws.num_experts;
    const uint32_t Le = ws.experts_per_rank;
    uint32_t *cnt = lds;               // [N][E]
    uint32_t *excl = lds + N * E;      // [E] exclusive scan of padded counts
    uint32_t *wave_tot = excl + E;     // [16]

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = tid / kWave;
    const uint32_t nwaves = blockDim.x / kWave;

    // 1. Per (source, expert): exclusive prefix of the chunk histograms, total.
    for (uint32_t p = tid; p < N * E; p += blockDim.x) {
        const uint32_t g = p / E;
        const uint32_t e = p - g * E;
        uint32_t run = 0;
        if (args.fold_mask >> g & 1) {
            uint32_t *col = ws.block_prefix + (size_t)g * ws.nb_max * E + e;
            for (uint32_t b = 0; b < args.num_blocks[g]; ++b) {
                const uint32_t c = col[(size_t)b * E];
                col[(size_t)b * E] = run;
                run += c;
            }
            ws.num_routed[p] = run;
        } else if (args.valid_mask >> g & 1) {
            run = ws.num_routed[p];
        }
        cnt[p] = run;
    }
    __syncthreads();

    // 2. Inclusive scan over experts for every folded source (a2a_dispatch_send.cu:209-242).
    for (uint32_t g = wave; g < N; g += nwaves) {
        if (!(args.fold_mask >> g & 1)) continue;
        uint32_t carry = 0;
        for (uint32_t base = 0; base < E; base += kWave) {
            const uint32_t e = base + lane;
            const uint32_t v = e < E ? cnt[g * E + e] : 0;
            const uint32_t incl = wave_inclusive_scan(v, lane) + carry;
            if (e < E) ws.expert_offsets[g * E + e] = incl;
            carry = __shfl(incl, kWave - 1);
        }
    }

    if (args.recv_mask == 0) return;

    // 3. Receiver layout.  Thread e owns expert e (E <= blockDim.x).
    const uint32_t pad = ws.expert_padding;
    uint32_t tpe = 0, padded = 0;
    if (tid < E) {
        for (uint32_t g = 0; g < N; ++g) tpe += cnt[g * E + tid];
        padded = (tpe + pad - 1) / pad * pad;
    }
    const uint32_t incl = wave_inclusive_scan(padded, lane);
    if (lane == kWave - 1) wave_tot[wave] = incl;
    __syncthreads();
    uint32_t before = 0;
    for (uint32_t w = 0; w < wave; ++w) before += wave_tot[w];
    if (tid < E) excl[tid] = before + incl - padded;
    __syncthreads();

    if (tid < E) {
        const uint32_t e = tid;
        const uint32_t r = e / Le;
        if (args.recv_mask >> r & 1) {
            const uint32_t le = e - r * Le;
            const uint32_t poff = excl[e] - excl[r * Le];
            ws.tokens_per_expert[e] = tpe;
            ws.padded_offset[e] = poff;
            if (args.out_num_tokens[r] != nullptr) args.out_num_tokens[r][le] = (int32_t)tpe;
            if (poff + tpe > args.out_rows[r]) atomicOr(ws.err, A2A_DEV_RECV_OVERFLOW);
            // Sources in the order the reference's host worker visits them
            // (a2a_worker.rs:681-694); each gets a contiguous run of rows.
            uint32_t running = poff;
            for (uint32_t i = 0; i < N; ++i) {
                const uint32_t g = source_order(r, i, N, ws.node_size);
                ws.slot_base[g * E + e] = running;
                running += cnt[g * E + e];
            }
        }
    }
}

hipError_t launch_route(const RouteArgs &args, const Workspace &ws, uint32_t total_blocks,
                        hipStream_t stream) {
    if (total_blocks == 0) return hipSuccess;
    hipLaunchKernelGGL(route_hist_kernel, dim3(total_blocks), dim3(kRouteBlock), 0, stream, args, ws);
    return hipGetLastError();
}

hipError_t launch_finalize(const FinalizeArgs &args, const Workspace &ws, hipStream_t stream) {
    const size_t lds = ((size_t)ws.world * ws.num_experts + ws.num_experts + 32) * sizeof(uint32_t);
    uint32_t threads = (ws.num_experts + kWave - 1) / kWave * kWave;
    if (threads < 256) threads = 256;
    hipLaunchKernelGGL(route_finalize_kernel, dim3(1), dim3(threads), lds, stream, args, ws);
    return hipGetLastError();
}

}  // namespace a2a
