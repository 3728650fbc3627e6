// Kernels of the split calls; see a2a_staged.h for what they mirror.
#include "a2a_staged.h"

#include <cstring>

#include "a2a_device.h"
#include "a2a_scan.h"

namespace a2a {

namespace {

size_t align_up_sz(size_t n, size_t a) { return (n + a - 1) / a * a; }

// ---------------------------------------------------------------------------
// dispatch send: stage one (quantised) row per token, record which token sits
// behind every row of the sender's expert-sorted order.
// ---------------------------------------------------------------------------

// Stages the row of `token` (payload, then scales).  Whole workgroup.
// PRE: the thread's first piece of the row was asked for earlier and is passed in.
template <bool QUANT, bool PRE = false>
__device__ __forceinline__ void stage_row(const StageSendArgs &args, const Staging &st, uint32_t g, uint32_t token,
                                          uint32_t staging_threads, u32x4 pre_a = u32x4{0, 0, 0, 0},
                                          u32x4 pre_b = u32x4{0, 0, 0, 0}, uint32_t first_thread = 0) {
    // the row is the work of threads first_thread .. first_thread + staging_threads - 1 of the workgroup
    const uint32_t tid = threadIdx.x - first_thread;
    if (tid >= staging_threads) return;   // (threads below first_thread wrap around to large numbers)
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = tid / kWave;
    const PushSrc &src = args.src;
    const uint8_t *x_row = src.x + (size_t)token * src.x_stride;
    uint8_t *row = st.send_buf + ((size_t)g * st.max_tokens + token) * st.disp_stride;
    float *row_scale = reinterpret_cast<float *>(row + st.payload_bytes);

    if constexpr (QUANT) {
        const uint32_t num_chunks = args.hidden_dim / 16;
        for (uint32_t base = wave * kWave; base < num_chunks; base += staging_threads) {
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
            if (active) {
                reinterpret_cast<u32x4 *>(row)[c] = q;
                if ((lane & 7) == 0) row_scale[c / 8] = scale;
            }
        }
    } else {
        const uint32_t num_chunks = args.row_bytes / 16;
        for (uint32_t c = tid; c < num_chunks; c += staging_threads) {
            reinterpret_cast<u32x4 *>(row)[c] =
                PRE && c == tid ? pre_a : __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(x_row) + c);
        }
        if (src.x_scale != nullptr) {
            const float *xs = src.x_scale + (size_t)token * src.xs_stride_token;
            for (uint32_t j = tid; j < args.hidden_dim_scale; j += staging_threads) {
                row_scale[j] = xs[(size_t)j * src.xs_stride_elem];
            }
        }
    }
}

template <bool QUANT>
__global__ __launch_bounds__(1024) void stage_send_kernel(const StageSendArgs args, const Workspace ws,
                                                          const Staging st) {
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = tid / kWave;
    const uint32_t E = ws.num_experts;
    const uint32_t K = ws.topk;
    const uint32_t g = args.rank / ws.dp_size;   // ranks of a dp group hold the same tokens
    const uint32_t token = blockIdx.x;
    const PushSrc &src = args.src;
    if (token >= effective_tokens(src.bound_m, src.num_tokens)) return;

    if (wave == 0 && lane < K) {
        const uint32_t entry = token * K + lane;
        const uint32_t expert = (uint32_t)src.indices[(size_t)token * src.indices_stride + lane];
        uint32_t toff = 0, at = kInvalidSlot;
        if (expert < E) {
            toff = ws.block_prefix[((size_t)g * ws.nb_max + entry / kRouteBlock) * E + expert] +
                   ws.local_rank[(size_t)g * ws.max_tk + entry];
            // position of the copy (a2a_dispatch_send.cu:54)
            const uint32_t excl = expert > 0 ? ws.expert_offsets[g * E + expert - 1] : 0;
            at = excl + toff;
            st.pos_token[(size_t)g * ws.max_tk + at] = token;
        }
        ws.token_offset[(size_t)g * ws.max_tk + entry] = toff;
        ws.route_slot[(size_t)g * ws.max_tk + entry] = at;   // (the combine-recv of the step reads the position here)
    }
    stage_row<QUANT>(args, st, g, token, blockDim.x);
}

// The send of a small step in ONE launch (the reference's dispatch-send kernel
// is one launch too, a2a_dispatch_send.cu:158-523): every token workgroup
// counts the entries of the sender per expert and those before its
// own token (LDS atomics; counts do not depend on arrival order), scans the
// counts over the experts, and has the position of each of its K copies in the
// sender's expert-sorted order.  The workgroup of token 0 publishes the counts
// and their scan.  Cost grows with tokens x entries, so the host uses it for
// small steps only.  Dynamic LDS: 3 * E words.
template <bool QUANT>
__global__ __launch_bounds__(1024) void stage_send_small_kernel(const StageSendArgs args, const Workspace ws,
                                                                const Staging st) {
    extern __shared__ uint32_t s_send[];
    __shared__ uint32_t scratch[kRouteWaves];
    __shared__ uint32_t s_carry;
    // everything the head of a workgroup takes from the argument block, asked for in one go
    A2A_PIN(args.src.x);
    A2A_PIN(args.src.indices);
    A2A_PIN(args.src.bound_m);
    A2A_PIN(args.src.x_stride);
    A2A_PIN(args.src.indices_stride);
    A2A_PIN(args.src.num_tokens);
    A2A_PIN(args.rank);
    A2A_PIN(args.hidden_dim);
    A2A_PIN(args.row_bytes);
    A2A_PIN(args.topk_magic);
    A2A_PIN(ws.num_experts);
    A2A_PIN(ws.topk);
    A2A_PIN(ws.dp_size);
    A2A_PIN(ws.max_tk);
    A2A_PIN(ws.num_routed);
    A2A_PIN(ws.expert_offsets);
    A2A_PIN(ws.token_offset);
    A2A_PIN(ws.err);
    A2A_PIN(st.send_buf);
    A2A_PIN(st.pos_token);
    A2A_PIN(st.disp_stride);
    A2A_PIN(st.payload_bytes);
    A2A_PIN(st.max_tokens);
    const uint32_t tid = threadIdx.x;
    const uint32_t nthreads = blockDim.x;   // read once: used after LDS atomics it is fetched again every time
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = tid / kWave;
    const uint32_t E = ws.num_experts;
    const uint32_t K = ws.topk;
    const uint32_t g = args.rank / ws.dp_size;
    const uint32_t token = blockIdx.x;
    const PushSrc &src = args.src;
    const uint32_t eff = effective_tokens(src.bound_m, src.num_tokens);
    const uint32_t entries = eff * K;
    const uint32_t my_first = token * K;
    uint32_t *cnt = s_send;          // [E] entries of the sender per expert
    uint32_t *prior = cnt + E;       // [E] those of the tokens before mine
    uint32_t *excl = prior + E;      // [E] exclusive scan of cnt

    // The first batch of entries is asked for before the tables are cleared and counted in
    // straight-line code, each entry waited for by itself.
    auto load_batch = [&](uint32_t f0, uint32_t (&expert)[8]) {
#pragma unroll
        for (uint32_t j = 0; j < 8; ++j) {
            const uint32_t f = f0 + j * nthreads + tid;
            expert[j] = 0xFFFFFFFFu;
            if (f < entries) {
                const uint32_t t = K > 1 ? __umulhi(f, args.topk_magic) : f;
                expert[j] = (uint32_t)src.indices[(size_t)t * src.indices_stride + (f - t * K)];
            }
        }
    };
    auto count_batch = [&](uint32_t f0, const uint32_t (&expert)[8]) {
#pragma unroll
        for (uint32_t j = 0; j < 8; ++j) {
            const uint32_t x = expert[j];
            if (x >= E) continue;
            atomicAdd(&cnt[x], 1u);
            if (f0 + j * nthreads + tid < my_first) atomicAdd(&prior[x], 1u);
        }
    };
    uint32_t first_batch[8];
    load_batch(0, first_batch);
    uint32_t my_expert = 0xFFFFFFFFu;
    if (lane < K) my_expert = (uint32_t)src.indices[(size_t)token * src.indices_stride + lane];
    // The row is asked for here, after the entries, and travels while they are counted.  Without a
    // condition (a thread without a piece asks for one it ignores), and every barrier up to its use
    // waits for LDS only: otherwise something on the way would wait for it by accident.
    u32x4 pre_a, pre_b = {0, 0, 0, 0};
    {
        const uint8_t *x_row = src.x + (size_t)token * src.x_stride;
        if constexpr (QUANT) {
            const uint32_t pieces = args.hidden_dim / 16;
            const u32x4 *piece = reinterpret_cast<const u32x4 *>(x_row + (size_t)(tid < pieces ? tid : 0) * 32);
            pre_a = __builtin_nontemporal_load(piece);
            pre_b = __builtin_nontemporal_load(piece + 1);
        } else {
            const uint32_t pieces = args.row_bytes / 16;
            pre_a = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(x_row) + (tid < pieces ? tid : 0));
        }
    }

    for (uint32_t i = tid; i < 2 * E; i += nthreads) s_send[i] = 0;
    lds_barrier();
    count_batch(0, first_batch);
    for (uint32_t f0 = 8 * nthreads; f0 < entries; f0 += 8 * nthreads) {
        uint32_t expert[8];
        load_batch(f0, expert);
        count_batch(f0, expert);
    }
    lds_barrier();

    // Scan over the experts (a2a_dispatch_send.cu:236-242); token 0 publishes.
    uint32_t carry = 0;
    for (uint32_t e0 = 0; e0 < E; e0 += nthreads) {
        const uint32_t e = e0 + tid;
        const uint32_t c = e < E ? cnt[e] : 0;
        const uint32_t incl = carry + block_inclusive_scan<true>(c, scratch);
        if (e < E) {
            excl[e] = incl - c;
            if (token == 0) {
                ws.num_routed[g * E + e] = c;
                ws.expert_offsets[g * E + e] = incl;
            }
        }
        if (e0 + nthreads < E) {   // uniform: another round follows
            if (tid == nthreads - 1) s_carry = incl;
            lds_barrier();
            carry = s_carry;
        }
    }
    lds_barrier();
    if (token >= eff) return;   // past bound_m: nothing to stage (uniform)

    if (wave == 0) {
        uint32_t repeats = 0;   // copies of this token to the same expert at an earlier k
        for (uint32_t k = 0; k + 1 < K; ++k) {
            const uint32_t other = (uint32_t)__builtin_amdgcn_readlane((int)my_expert, (int)k);
            if (k < lane && other == my_expert) ++repeats;
        }
        if (lane < K) {
            const uint32_t entry = token * K + lane;
            uint32_t toff = 0, at = kInvalidSlot;
            if (my_expert < E) {
                toff = prior[my_expert] + repeats;
                // position of the copy (a2a_dispatch_send.cu:54)
                at = excl[my_expert] + toff;
                st.pos_token[(size_t)g * ws.max_tk + at] = token;
            } else {
                atomicOr(ws.err, A2A_DEV_BAD_EXPERT_ID);
            }
            ws.token_offset[(size_t)g * ws.max_tk + entry] = toff;
            ws.route_slot[(size_t)g * ws.max_tk + entry] = at;
        }
    }
    stage_row<QUANT, true>(args, st, g, token, nthreads, pre_a, pre_b);
}

// The scan over a sender's per-expert counts (a2a_dispatch_send.cu:236-242) by ONE wavefront, for the
// sends in which a spare wavefront resolves positions.  `s_cnt[e]`: low half of a word the entries of
// expert e.  W passes of 64 experts at a time: their reads, scans and lane exchanges do not depend on
// each other, only the running total `run` does.  A lane whose route's expert `my_id` lies in a pass
// takes the expert's word and the entries of the experts before it from the lane that holds them; with
// `publish` the counts and their inclusive scan go to memory.  Whole wavefront.
template <uint32_t W>
__device__ __forceinline__ void scan_counts_passes(const uint32_t *s_cnt, uint32_t E, uint32_t e0, uint32_t lane,
                                                   uint32_t my_id, bool publish, uint32_t *num_routed,
                                                   uint32_t *expert_offsets, uint32_t &run, uint32_t &my_word,
                                                   uint32_t &my_excl) {
    uint32_t word[W], incl[W];
#pragma unroll
    for (uint32_t u = 0; u < W; ++u) {
        const uint32_t x = e0 + u * kWave + lane;
        word[u] = s_cnt[x < E ? x : 0];
        if (x >= E) word[u] = 0;
    }
#pragma unroll
    for (uint32_t u = 0; u < W; ++u) incl[u] = wave_inclusive_scan(word[u] & 0xFFFFu, lane);
#pragma unroll
    for (uint32_t u = 0; u < W; ++u) {
        const uint32_t x = e0 + u * kWave + lane;
        const uint32_t c = word[u] & 0xFFFFu;
        const uint32_t rel = my_id - (e0 + u * kWave);   // (an id below the pass wraps around to a large number)
        const uint32_t their_word = (uint32_t)__shfl((int)word[u], (int)(rel & (kWave - 1)));   // every lane takes part
        const uint32_t their_excl = (uint32_t)__shfl((int)(incl[u] - c), (int)(rel & (kWave - 1)));
        if (rel < (uint32_t)kWave) {
            my_word = their_word;
            my_excl = run + their_excl;
        }
        if (publish && x < E) {
            num_routed[x] = c;
            expert_offsets[x] = run + incl[u];
        }
        run += (uint32_t)__builtin_amdgcn_readlane((int)incl[u], kWave - 1);
    }
}

// The whole scan: four passes at a time while more than two are left, then two (256 experts: 3.6 ->
// 3.4 us per send of 128 tokens against one pass at a time; a step with 128 experts takes two at a
// time, with four it was 0.1 us slower).
__device__ __forceinline__ void scan_counts_for_routes(const uint32_t *s_cnt, uint32_t E, uint32_t lane, uint32_t my_id,
                                                       bool publish, uint32_t *num_routed, uint32_t *expert_offsets,
                                                       uint32_t &my_word, uint32_t &my_excl) {
    uint32_t run = 0, e0 = 0;
    my_word = my_excl = 0;
    for (; e0 + 2 * kWave < E; e0 += 4 * kWave) {
        scan_counts_passes<4>(s_cnt, E, e0, lane, my_id, publish, num_routed, expert_offsets, run, my_word, my_excl);
    }
    if (e0 < E) scan_counts_passes<2>(s_cnt, E, e0, lane, my_id, publish, num_routed, expert_offsets, run, my_word, my_excl);
}

// The quick form of the one-launch send of a small step: dense index rows and a row that is one piece
// per thread (16 elements to quantise, or 16 bytes to move as they are) with a wavefront to spare (the
// host launches one more than the row has pieces for).  Where a row is staged does not depend on the
// routing (one row per token, at the token's own place), so the wavefronts that move the row count
// their entries, say so (a word in LDS, not a barrier) and then quantise and store without waiting for
// anybody; the spare wavefront (the RESOLVER) does not count: it holds the token's ids, waits until
// every counting wavefront has said that its entries are in the table, scans the table by itself (64
// experts an instruction, no workgroup scan with its barriers), and writes the token's positions; the
// resolver of token 0 publishes the counts and their scan on the way.  In stage_send_small_kernel every
// wavefront walks count, workgroup scan, routes and row one after the other: 128 tokens of 7168,
// 4.1 -> 3.6 us per send at the GPU's own pace; hidden 2048: 3.9 -> 3.2.
// NB: entries a counting thread asks for at the head (the host picks the smallest of 1, 2, 3, 4, 8 that
// covers the step; entries beyond are counted by a loop).  Dynamic LDS: E words (low half of a word:
// the entries of the expert, high half: those of the tokens before this one; a step of this kernel
// has fewer than 2^16 entries).
constexpr uint32_t kSendQuickSpinLimit = 1u << 22;   // (a resolver that gives up flags A2A_DEV_INTERNAL; never seen)

template <uint32_t NB, bool QUANT>
__global__ __launch_bounds__(1024) void stage_send_quick_kernel(const StageSendArgs args, const Workspace ws,
                                                                const Staging st) {
    extern __shared__ uint32_t s_cnt[];
    __shared__ uint32_t s_counted;   // counting wavefronts whose entries are in the table
    // everything the head of a workgroup takes from the argument block, asked for in one go
    A2A_PIN(args.src.x);
    A2A_PIN(args.src.x_scale);
    A2A_PIN(args.src.indices);
    A2A_PIN(args.src.bound_m);
    A2A_PIN(args.src.x_stride);
    A2A_PIN(args.src.num_tokens);
    A2A_PIN(args.rank);
    A2A_PIN(args.hidden_dim);
    A2A_PIN(args.row_bytes);
    A2A_PIN(ws.num_experts);
    A2A_PIN(ws.topk);
    A2A_PIN(ws.dp_size);
    A2A_PIN(ws.max_tk);
    A2A_PIN(ws.num_routed);
    A2A_PIN(ws.expert_offsets);
    A2A_PIN(ws.token_offset);
    A2A_PIN(ws.err);
    A2A_PIN(st.send_buf);
    A2A_PIN(st.pos_token);
    A2A_PIN(st.disp_stride);
    A2A_PIN(st.payload_bytes);
    A2A_PIN(st.max_tokens);
    const uint32_t tid = threadIdx.x;
    const uint32_t nthreads = blockDim.x;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = tid / kWave;
    const uint32_t waves = nthreads / kWave;
    const bool resolver = wave == waves - 1;
    const uint32_t counters = nthreads - kWave;   // threads that count entries and move the row
    const uint32_t E = ws.num_experts;
    const uint32_t K = ws.topk;
    const uint32_t g = args.rank / ws.dp_size;
    const uint32_t token = blockIdx.x;
    const PushSrc &src = args.src;
    const uint32_t tokens = src.num_tokens;   // the grid: one workgroup per token
    const uint32_t entries = tokens * K;      // > 0
    const uint32_t my_first = token * K;
    const uint32_t num_chunks = QUANT ? args.hidden_dim / 16 : args.row_bytes / 16;   // pieces of a row, one per thread
    const bool has_piece = tid < num_chunks;

    // What each kind of wavefront takes from memory, asked for before anything else is done: the
    // entries, then the thread's piece of the row (and the first of the caller's scales it copies);
    // the resolver its token's ids (lane k: route k).
    uint32_t early[NB] = {};
    u32x4 pre_a = {0, 0, 0, 0}, pre_b = {0, 0, 0, 0};
    float first_scale = 0.0f;
    uint32_t my_id = 0xFFFFFFFFu;
    if (!resolver) {
#pragma unroll
        for (uint32_t j = 0; j < NB; ++j) {
            const uint32_t f = j * counters + tid;
            early[j] = (uint32_t)src.indices[f < entries ? f : entries - 1];
        }
        const uint8_t *x_row = src.x + (size_t)token * src.x_stride;
        if (has_piece) {
            if constexpr (QUANT) {
                const u32x4 *piece = reinterpret_cast<const u32x4 *>(x_row + (size_t)tid * 32);
                pre_a = __builtin_nontemporal_load(piece);
                pre_b = __builtin_nontemporal_load(piece + 1);
            } else {
                pre_a = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(x_row) + tid);
            }
        }
        if constexpr (!QUANT) {
            if (src.x_scale != nullptr && tid < args.hidden_dim_scale) {
                first_scale = src.x_scale[(size_t)token * src.xs_stride_token + (size_t)tid * src.xs_stride_elem];
            }
        }
    } else {
        // (the resolver shares its SIMD with wavefronts that quantise while the positions are resolved)
        __builtin_amdgcn_s_setprio(3);
        my_id = (uint32_t)src.indices[my_first + (lane < K ? lane : 0)];
    }
    const uint32_t eff = effective_tokens(src.bound_m, tokens);
    const uint32_t flat_entries = eff * K;
    const bool live = token < eff;   // uniform

    for (uint32_t i = tid; i < E; i += nthreads) s_cnt[i] = 0;
    if (tid == 0) s_counted = 0;
    lds_barrier();

    if (!resolver) {
        // The first batch in straight-line code: each of its values is waited for by itself, and the
        // row asked for after them stays in flight meanwhile.
#pragma unroll
        for (uint32_t j = 0; j < NB; ++j) {
            const uint32_t f = j * counters + tid;
            const uint32_t x = f < flat_entries ? early[j] : 0xFFFFFFFFu;
            if (x < E) atomicAdd(&s_cnt[x], f < my_first ? 0x10001u : 1u);
        }
        for (uint32_t f0 = NB * counters; f0 < flat_entries; f0 += NB * counters) {
            uint32_t x[NB];
#pragma unroll
            for (uint32_t j = 0; j < NB; ++j) {
                const uint32_t f = f0 + j * counters + tid;
                x[j] = f < flat_entries ? (uint32_t)src.indices[f] : 0xFFFFFFFFu;
            }
#pragma unroll
            for (uint32_t j = 0; j < NB; ++j) {
                const uint32_t f = f0 + j * counters + tid;
                if (x[j] < E) atomicAdd(&s_cnt[x[j]], f < my_first ? 0x10001u : 1u);
            }
        }
        // this wavefront's entries are in the table before its arrival is counted
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (lane == 0) atomicAdd(&s_counted, 1u);
        if (!live) return;   // past bound_m: nothing to stage (uniform)

        uint8_t *row = st.send_buf + ((size_t)g * st.max_tokens + token) * st.disp_stride;
        float *row_scale = reinterpret_cast<float *>(row + st.payload_bytes);
        if constexpr (QUANT) {
            float scale;
            const u32x4 q = quantize16(pre_a, pre_b, &scale);
            if (has_piece) {
                reinterpret_cast<u32x4 *>(row)[tid] = q;
                if ((lane & 7) == 0) row_scale[tid / 8] = scale;
            }
        } else {
            if (has_piece) reinterpret_cast<u32x4 *>(row)[tid] = pre_a;
            if (src.x_scale != nullptr) {
                if (tid < args.hidden_dim_scale) row_scale[tid] = first_scale;
                const float *xs = src.x_scale + (size_t)token * src.xs_stride_token;
                for (uint32_t j = tid + counters; j < args.hidden_dim_scale; j += counters) {
                    row_scale[j] = xs[(size_t)j * src.xs_stride_elem];
                }
            }
        }
        return;
    }

    // ---- the resolver ----
    // copies of this token to the same expert at an earlier k: what no count decides
    uint32_t repeats = 0;
    for (uint32_t k = 0; k + 1 < K; ++k) {
        const uint32_t other = (uint32_t)__builtin_amdgcn_readlane((int)my_id, (int)k);
        if (k < lane && other == my_id) ++repeats;
    }
    // until the counting wavefronts have all said that their entries are in the table (at the lowest
    // priority: the wavefronts that share this SIMD are among those waited for)
    __builtin_amdgcn_s_setprio(0);
    for (uint32_t spins = 0; __hip_atomic_load(&s_counted, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) != waves - 1;) {
        if (++spins == kSendQuickSpinLimit) {
            if (lane == 0) atomicOr(ws.err, A2A_DEV_INTERNAL);
            break;
        }
    }
    __builtin_amdgcn_s_setprio(3);
    asm volatile("" ::: "memory");

    // Scan over the experts; a route takes its expert's word and the entries of the experts before it.
    // Token 0 publishes.
    uint32_t my_word, my_excl;
    scan_counts_for_routes(s_cnt, E, lane, my_id, token == 0, ws.num_routed + g * E, ws.expert_offsets + g * E, my_word,
                           my_excl);
    if (!live) return;   // past bound_m: no positions to write (uniform)
    if (lane < K) {
        uint32_t toff = 0, at = kInvalidSlot;
        if (my_id < E) {
            toff = (my_word >> 16) + repeats;
            // position of the copy (a2a_dispatch_send.cu:54)
            at = my_excl + toff;
            st.pos_token[(size_t)g * ws.max_tk + at] = token;
        } else {
            atomicOr(ws.err, A2A_DEV_BAD_EXPERT_ID);
        }
        ws.token_offset[(size_t)g * ws.max_tk + my_first + lane] = toff;
        ws.route_slot[(size_t)g * ws.max_tk + my_first + lane] = at;
    }
}

// The send of a step too large for stage_send_small_kernel and of at most kSendSingleMaxEntries
// entries (448 to 1024 tokens at top-8), in ONE launch: what makes the small kernel expensive as steps
// grow is that every token's workgroup counts every entry of the sender; here a workgroup counts once
// for `per_group` tokens (the host picks it so that the workgroups are about as many as the compute
// units) and stages them with teams of wavefronts, one token per team and round.  One LDS word per
// expert holds its entries (low half) and those of the tokens before the workgroup's first (high half).
// The rows of the first two rounds are asked for at the head and travel while the entries are counted
// (every barrier up to their use waits for LDS only).  Dynamic LDS: 2 * E words.
constexpr uint32_t kSendSingleMaxEntries = 8192;
constexpr uint32_t kSendTokensPerGroup = 4;

template <bool QUANT>
__global__ __launch_bounds__(1024) void stage_send_single_kernel(const StageSendArgs args, const Workspace ws,
                                                                 const Staging st, const uint32_t team_threads,
                                                                 const uint32_t per_group) {
    extern __shared__ uint32_t s_single[];
    __shared__ uint32_t s_route_expert[kSendTokensPerGroup * A2A_MAX_EXPERTS_PER_TOKEN];
    __shared__ uint32_t scratch[kRouteWaves];
    __shared__ uint32_t s_carry;
    const uint32_t tid = threadIdx.x;
    const uint32_t nthreads = blockDim.x;
    const uint32_t E = ws.num_experts, K = ws.topk;
    const uint32_t g = args.rank / ws.dp_size;
    const PushSrc &src = args.src;                     // index rows are dense (the host checks)
    const uint32_t tokens = effective_tokens(src.bound_m, src.num_tokens);
    const uint32_t flat_entries = tokens * K;
    const uint32_t first_token = blockIdx.x * per_group;
    const uint32_t my_first = first_token * K;         // flat index of my first entry
    if (blockIdx.x != 0 && first_token >= tokens) return;   // nothing to stage; the first workgroup publishes

    constexpr uint32_t kBatch = 10;   // 8192 entries over 896 threads in one batch
    uint32_t early[kBatch];
#pragma unroll
    for (uint32_t j = 0; j < kBatch; ++j) {
        const uint32_t f = j * nthreads + tid;
        early[j] = f < flat_entries ? (uint32_t)src.indices[f] : 0xFFFFFFFFu;
    }
    const uint32_t my_routes = per_group * K;          // one thread each
    uint32_t my_expert = 0xFFFFFFFFu;
    if (tid < my_routes && my_first + tid < flat_entries) my_expert = (uint32_t)src.indices[my_first + tid];
    const uint32_t teams = nthreads / team_threads;
    const uint32_t team = tid / team_threads;
    const uint32_t team_tid = tid - team * team_threads;
    u32x4 pre_a, pre_b = {0, 0, 0, 0};
    u32x4 next_a = {0, 0, 0, 0}, next_b = {0, 0, 0, 0};
    {
        const uint32_t last_token = src.num_tokens - 1;
        const uint32_t any_token = first_token + team < src.num_tokens ? first_token + team : last_token;
        const uint32_t second = first_token + teams + team;
        const uint8_t *x_row = src.x + (size_t)any_token * src.x_stride;
        const uint8_t *x_next = src.x + (size_t)(second < src.num_tokens ? second : last_token) * src.x_stride;
        const bool two_rounds = per_group > teams;     // uniform: a branch, not a select
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

    uint32_t *cnt = s_single;      // [E] low half: entries per expert, high half: those before my first token
    uint32_t *excl = cnt + E;      // [E] exclusive scan of the entries per expert
    for (uint32_t i = tid; i < E; i += nthreads) cnt[i] = 0;
    lds_barrier();
    auto count_batch = [&](const uint32_t (&expert)[kBatch], uint32_t f0) {
#pragma unroll
        for (uint32_t j = 0; j < kBatch; ++j) {
            const uint32_t x = expert[j];
            if (x >= E) continue;
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
    lds_barrier();

    // Scan over the experts (a2a_dispatch_send.cu:236-242); the first workgroup publishes.
    uint32_t carry = 0;
    for (uint32_t e0 = 0; e0 < E; e0 += nthreads) {
        const uint32_t e = e0 + tid;
        const uint32_t c = e < E ? cnt[e] & 0xFFFFu : 0;
        const uint32_t incl = carry + block_inclusive_scan<true>(c, scratch);
        if (e < E) {
            excl[e] = incl - c;
            if (blockIdx.x == 0) {
                ws.num_routed[g * E + e] = c;
                ws.expert_offsets[g * E + e] = incl;
            }
        }
        if (e0 + nthreads < E) {   // uniform: another round follows
            if (tid == nthreads - 1) s_carry = incl;
            lds_barrier();
            carry = s_carry;
        }
    }
    lds_barrier();

    // One thread per route of my tokens: its rank inside its expert and the row of the sender's
    // expert-sorted order it stands for (a2a_dispatch_send.cu:54).
    if (tid < my_routes && my_first + tid < flat_entries) {
        uint32_t toff = 0, at = kInvalidSlot;
        if (my_expert < E) {
            uint32_t earlier = 0;
            for (uint32_t q = 0; q < tid; ++q) earlier += s_route_expert[q] == my_expert ? 1u : 0u;
            toff = (cnt[my_expert] >> 16) + earlier;
            at = excl[my_expert] + toff;
            st.pos_token[(size_t)g * ws.max_tk + at] = first_token + tid / K;
        } else {
            atomicOr(ws.err, A2A_DEV_BAD_EXPERT_ID);
        }
        ws.token_offset[(size_t)g * ws.max_tk + my_first + tid] = toff;
        ws.route_slot[(size_t)g * ws.max_tk + my_first + tid] = at;
    }

    // The teams stage one token each per round.
    for (uint32_t first = 0; first < per_group; first += teams) {
        const uint32_t token = first_token + first + team;
        if (first + team >= per_group || token >= tokens) continue;   // (no barrier below: teams work alone)
        if (first == 0) {
            stage_row<QUANT, true>(args, st, g, token, team_threads, pre_a, pre_b, team * team_threads);
        } else if (first == teams) {
            stage_row<QUANT, true>(args, st, g, token, team_threads, next_a, next_b, team * team_threads);
        } else {
            stage_row<QUANT>(args, st, g, token, team_threads, u32x4{0, 0, 0, 0}, u32x4{0, 0, 0, 0}, team * team_threads);
        }
    }
}

// stage_send_single_kernel with the division of labour of stage_send_quick_kernel, for steps whose
// rows are one piece per thread of a team and leave room for a spare wavefront: the teams count the
// step's entries, say so, and quantise and stage their tokens' rows (at most two rounds, both rounds'
// pieces asked for at the head) without waiting for anybody; the spare wavefront holds the routes of
// the workgroup's tokens (a lane each, at most 64), counts for each the earlier routes of the workgroup
// to the same expert, waits for the counting wavefronts, scans the counts by itself and writes the
// positions.  1024 tokens of 7168: 8.5 -> 7.0 us per send at the GPU's own pace.
// NB: entries a counting thread asks for at the head.  Dynamic LDS: E words.
template <uint32_t NB, uint32_t ROUNDS, bool QUANT>
__global__ __launch_bounds__(1024) void stage_send_teams_kernel(const StageSendArgs args, const Workspace ws,
                                                                const Staging st, const uint32_t team_threads,
                                                                const uint32_t per_group) {
    extern __shared__ uint32_t s_cnt[];
    __shared__ uint32_t s_counted;   // counting wavefronts whose entries are in the table
    // everything the head of a workgroup takes from the argument block, asked for in one go
    A2A_PIN(args.src.x);
    A2A_PIN(args.src.x_scale);
    A2A_PIN(args.src.indices);
    A2A_PIN(args.src.bound_m);
    A2A_PIN(args.src.x_stride);
    A2A_PIN(args.src.num_tokens);
    A2A_PIN(args.rank);
    A2A_PIN(args.hidden_dim);
    A2A_PIN(args.row_bytes);
    A2A_PIN(args.topk_magic);
    A2A_PIN(ws.num_experts);
    A2A_PIN(ws.topk);
    A2A_PIN(ws.dp_size);
    A2A_PIN(ws.max_tk);
    A2A_PIN(ws.num_routed);
    A2A_PIN(ws.expert_offsets);
    A2A_PIN(ws.token_offset);
    A2A_PIN(ws.err);
    A2A_PIN(st.send_buf);
    A2A_PIN(st.pos_token);
    A2A_PIN(st.disp_stride);
    A2A_PIN(st.payload_bytes);
    A2A_PIN(st.max_tokens);
    const uint32_t tid = threadIdx.x;
    const uint32_t nthreads = blockDim.x;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = tid / kWave;
    const uint32_t waves = nthreads / kWave;
    const bool resolver = wave == waves - 1;
    const uint32_t counters = nthreads - kWave;   // threads that count entries and move rows
    const uint32_t E = ws.num_experts;
    const uint32_t K = ws.topk;
    const uint32_t g = args.rank / ws.dp_size;
    const PushSrc &src = args.src;              // index rows are dense (the host checks)
    const uint32_t tokens = src.num_tokens;     // the grid: a workgroup per `per_group` tokens
    const uint32_t entries = tokens * K;        // > 0
    const uint32_t first_token = blockIdx.x * per_group;
    const uint32_t my_first = first_token * K;  // flat index of the workgroup's first entry
    const uint32_t routes = per_group * K;      // <= 64 (the host checks)
    const uint32_t num_chunks = QUANT ? args.hidden_dim / 16 : args.row_bytes / 16;   // pieces of a row, one per thread of a team
    const uint32_t teams = counters / team_threads;
    const uint32_t team = tid / team_threads;
    const uint32_t member = tid - team * team_threads;
    const bool has_piece = member < num_chunks;

    uint32_t early[NB] = {};
    u32x4 pre_a[ROUNDS], pre_b[ROUNDS];
    float first_scale[ROUNDS];
    uint32_t my_id = 0xFFFFFFFFu;
    if (!resolver) {
#pragma unroll
        for (uint32_t j = 0; j < NB; ++j) {
            const uint32_t f = j * counters + tid;
            early[j] = (uint32_t)src.indices[f < entries ? f : entries - 1];
        }
#pragma unroll
        for (uint32_t round = 0; round < ROUNDS; ++round) {
            const uint32_t token = first_token + round * teams + team;
            const uint8_t *x_row = src.x + (size_t)(token < tokens ? token : tokens - 1) * src.x_stride;
            pre_a[round] = pre_b[round] = u32x4{0, 0, 0, 0};
            first_scale[round] = 0.0f;
            if (has_piece) {
                if constexpr (QUANT) {
                    const u32x4 *piece = reinterpret_cast<const u32x4 *>(x_row + (size_t)member * 32);
                    pre_a[round] = __builtin_nontemporal_load(piece);
                    pre_b[round] = __builtin_nontemporal_load(piece + 1);
                } else {
                    pre_a[round] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(x_row) + member);
                }
            }
            if constexpr (!QUANT) {
                if (src.x_scale != nullptr && member < args.hidden_dim_scale) {
                    first_scale[round] = src.x_scale[(size_t)(token < tokens ? token : tokens - 1) * src.xs_stride_token +
                                                     (size_t)member * src.xs_stride_elem];
                }
            }
        }
    } else {
        // (the resolver shares its SIMD with wavefronts that quantise while the positions are resolved)
        __builtin_amdgcn_s_setprio(3);
        const uint32_t f = my_first + lane;
        my_id = (uint32_t)src.indices[f < entries ? f : entries - 1];
    }
    const uint32_t eff = effective_tokens(src.bound_m, tokens);
    const uint32_t flat_entries = eff * K;
    if (blockIdx.x != 0 && first_token >= eff) return;   // nothing to stage (uniform); the first workgroup publishes

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
        for (uint32_t f0 = NB * counters; f0 < flat_entries; f0 += NB * counters) {
            uint32_t x[NB];
#pragma unroll
            for (uint32_t j = 0; j < NB; ++j) {
                const uint32_t f = f0 + j * counters + tid;
                x[j] = f < flat_entries ? (uint32_t)src.indices[f] : 0xFFFFFFFFu;
            }
#pragma unroll
            for (uint32_t j = 0; j < NB; ++j) {
                const uint32_t f = f0 + j * counters + tid;
                if (x[j] < E) atomicAdd(&s_cnt[x[j]], f < my_first ? 0x10001u : 1u);
            }
        }
        // this wavefront's entries are in the table before its arrival is counted
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (lane == 0) atomicAdd(&s_counted, 1u);

#pragma unroll
        for (uint32_t round = 0; round < ROUNDS; ++round) {
            const uint32_t token = first_token + round * teams + team;
            if (round * teams + team >= per_group || token >= eff) continue;   // (no barrier below: teams work alone)
            uint8_t *row = st.send_buf + ((size_t)g * st.max_tokens + token) * st.disp_stride;
            float *row_scale = reinterpret_cast<float *>(row + st.payload_bytes);
            if constexpr (QUANT) {
                float scale;
                const u32x4 q = quantize16(pre_a[round], pre_b[round], &scale);
                if (has_piece) {
                    reinterpret_cast<u32x4 *>(row)[member] = q;
                    if ((lane & 7) == 0) row_scale[member / 8] = scale;
                }
            } else {
                if (has_piece) reinterpret_cast<u32x4 *>(row)[member] = pre_a[round];
                if (src.x_scale != nullptr) {
                    if (member < args.hidden_dim_scale) row_scale[member] = first_scale[round];
                    const float *xs = src.x_scale + (size_t)token * src.xs_stride_token;
                    for (uint32_t j = member + team_threads; j < args.hidden_dim_scale; j += team_threads) {
                        row_scale[j] = xs[(size_t)j * src.xs_stride_elem];
                    }
                }
            }
        }
        return;
    }

    // ---- the resolver: lane l holds route l of the workgroup's tokens ----
    const bool route_live = lane < routes && my_first + lane < flat_entries;
    if (!route_live) my_id = 0xFFFFFFFFu;
    // routes of the workgroup before this one (earlier tokens, earlier k) to the same expert: what no count decides
    uint32_t earlier = 0;
    for (uint32_t l = 0; l + 1 < routes; ++l) {
        const uint32_t other = (uint32_t)__builtin_amdgcn_readlane((int)my_id, (int)l);
        if (l < lane && other == my_id) ++earlier;
    }
    // until the counting wavefronts have all said that their entries are in the table (at the lowest
    // priority: the wavefronts that share this SIMD are among those waited for)
    __builtin_amdgcn_s_setprio(0);
    for (uint32_t spins = 0; __hip_atomic_load(&s_counted, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) != waves - 1;) {
        if (++spins == kSendQuickSpinLimit) {
            if (lane == 0) atomicOr(ws.err, A2A_DEV_INTERNAL);
            break;
        }
    }
    __builtin_amdgcn_s_setprio(3);
    asm volatile("" ::: "memory");

    // Scan over the experts; a route takes its expert's word and the entries of the experts before it.
    // The first workgroup publishes.
    uint32_t my_word, my_excl;
    scan_counts_for_routes(s_cnt, E, lane, my_id, blockIdx.x == 0, ws.num_routed + g * E, ws.expert_offsets + g * E,
                           my_word, my_excl);

    if (route_live) {
        uint32_t toff = 0, at = kInvalidSlot;
        if (my_id < E) {
            toff = (my_word >> 16) + earlier;
            // position of the copy (a2a_dispatch_send.cu:54)
            const uint32_t token = first_token + (K > 1 ? __umulhi(lane, args.topk_magic) : lane);
            at = my_excl + toff;
            st.pos_token[(size_t)g * ws.max_tk + at] = token;
        } else {
            atomicOr(ws.err, A2A_DEV_BAD_EXPERT_ID);
        }
        ws.token_offset[(size_t)g * ws.max_tk + my_first + lane] = toff;
        ws.route_slot[(size_t)g * ws.max_tk + my_first + lane] = at;
    }
}

// The send of a large step, after a routing launch that left the chunk counts,
// the in-chunk rank of every entry and the sender's totals per expert and per
// owning rank.  No launch in between scans anything: wavefront 0 of a token
// workgroup finds the position of each of its K copies in the sender's
// expert-sorted order itself, eight lanes per route, from three short sums
// (copies of the same expert in earlier chunks; copies for the ranks before
// the expert's owner; copies for the owner's experts before it), while the
// other wavefronts stage the row.  Workgroup 0 is not a token: it publishes the
// sender's counts and their scan (a2a_dispatch_send.cu:199-204,236-242) and
// hands the totals over to the next send.
template <bool QUANT>
__global__ __launch_bounds__(1024) void stage_send_resolve_kernel(const StageSendArgs args, const Workspace ws,
                                                                  const Staging st) {
    __shared__ uint32_t scratch[kRouteWaves];
    __shared__ uint32_t s_carry;
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = tid / kWave;
    const uint32_t E = ws.num_experts, K = ws.topk, Le = ws.experts_per_rank;
    const uint32_t g = args.rank / ws.dp_size;
    const uint32_t use = ws.send_turn[1] & 1u;
    const uint32_t *per_expert = ws.send_totals + (size_t)use * (E + ws.world);   // [E]
    const uint32_t *per_rank = per_expert + E;                                     // [N]

    if (blockIdx.x == 0) {
        uint32_t carry = 0;
        for (uint32_t e0 = 0; e0 < E; e0 += blockDim.x) {
            const uint32_t e = e0 + tid;
            const uint32_t c = e < E ? per_expert[e] : 0;
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
        if (tid == 0) ws.send_turn[0] = use ^ 1u;
        return;
    }

    const uint32_t token = blockIdx.x - 1;
    const PushSrc &src = args.src;
    if (token >= effective_tokens(src.bound_m, src.num_tokens)) return;

    // With a wavefront to spare the last one resolves and stages nothing, so that no wavefront
    // has both chains of memory trips to walk; otherwise wavefront 0 does both.
    const uint32_t staging_threads = args.resolver_wave != 0 ? args.resolver_wave * kWave : blockDim.x;
    if (wave == args.resolver_wave) {
        const uint32_t *counts = ws.chunk_counts + (size_t)g * E * ws.nb_max;   // [E][nb_max]
        const uint32_t part = lane & 7, route = lane >> 3;
        for (uint32_t k0 = 0; k0 < K; k0 += 8) {
            const uint32_t k = k0 + route;
            const bool in = k < K;
            const uint32_t kk = in ? k : 0;   // a lane without a route reads route 0 and is dropped below
            const uint32_t id = (uint32_t)src.indices[(size_t)token * src.indices_stride + kk];
            const uint32_t local = ws.local_rank[(size_t)g * ws.max_tk + token * K + kk];
            const bool live = in && id < E;
            const uint32_t e = live ? id : 0;
            const uint32_t upto = live ? (token * K + k) / kRouteBlock : 0;   // chunk of this entry
            const uint32_t r = owner_of_expert(ws, e);
            const uint32_t le = live ? e - r * Le : 0;
            const uint32_t ranks_before = live ? r : 0;
            // four terms of each sum per lane without a branch (clamped index, masked value)
            uint32_t v_chunk[4], v_rank[4], v_expert[4];
#pragma unroll
            for (uint32_t i = 0; i < 4; ++i) {
                const uint32_t n = part + 8 * i;
                v_chunk[i] = counts[(size_t)e * ws.nb_max + (n < upto ? n : 0)];
                v_rank[i] = per_rank[n < ranks_before ? n : 0];
                v_expert[i] = per_expert[r * Le + (n < le ? n : 0)];
            }
            uint32_t earlier = 0, excl = 0;
#pragma unroll
            for (uint32_t i = 0; i < 4; ++i) {
                const uint32_t n = part + 8 * i;
                earlier += n < upto ? v_chunk[i] : 0;
                excl += n < ranks_before ? v_rank[i] : 0;
                excl += n < le ? v_expert[i] : 0;
            }
            // longer sums (more than 32 chunks, more than 32 experts in a rank)
            for (uint32_t c = 32 + part; c < upto; c += 8) earlier += counts[(size_t)e * ws.nb_max + c];
            for (uint32_t q = 32 + part; q < le; q += 8) excl += per_expert[r * Le + q];
            earlier = group8_sum(earlier);
            excl = group8_sum(excl);
            if (part == 0 && in) {
                uint32_t toff = 0, at = kInvalidSlot;
                if (live) {
                    toff = earlier + local;
                    // position of the copy (a2a_dispatch_send.cu:54)
                    at = excl + toff;
                    st.pos_token[(size_t)g * ws.max_tk + at] = token;
                }
                ws.token_offset[(size_t)g * ws.max_tk + token * K + k] = toff;
                ws.route_slot[(size_t)g * ws.max_tk + token * K + k] = at;
            }
        }
    }
    stage_row<QUANT>(args, st, g, token, staging_threads);
}

// A team of `team` threads (one or more whole wavefronts) copies a row of
// `num_chunks` 16-byte pieces: eight loads per thread in flight, non-temporal
// both ways (rows are read once and written once).
__device__ __forceinline__ void copy_row_by_team(const u32x4 *src, u32x4 *dst, uint32_t num_chunks, uint32_t member,
                                                 uint32_t team) {
    for (uint32_t c0 = 0; c0 < num_chunks; c0 += 8 * team) {
        u32x4 v[8];
#pragma unroll
        for (uint32_t u = 0; u < 8; ++u) {
            const uint32_t c = c0 + u * team + member;
            if (c < num_chunks) v[u] = __builtin_nontemporal_load(src + c);
        }
#pragma unroll
        for (uint32_t u = 0; u < 8; ++u) {
            const uint32_t c = c0 + u * team + member;
            if (c < num_chunks) dst[c] = v[u];
        }
    }
}

// Payload and scales of one received row, by a team.  The scales are asked for before the payload
// moves: behind the payload's stores their trip would begin only when those have been acknowledged
// (memory operations of a wavefront complete in order).
__device__ __forceinline__ void copy_received_row(const uint8_t *src, uint32_t payload_bytes, uint32_t num_chunks,
                                                  uint32_t num_scales, const PushDst &dst, uint32_t dst_row,
                                                  uint32_t member, uint32_t team) {
    const float *ss = reinterpret_cast<const float *>(src + payload_bytes);
    float first_scale = 0.0f;
    const bool scales = dst.out_scale != nullptr;
    if (scales && member < num_scales) first_scale = ss[member];
    copy_row_by_team(reinterpret_cast<const u32x4 *>(src),
                     reinterpret_cast<u32x4 *>(dst.out_x + (size_t)dst_row * dst.out_stride), num_chunks, member, team);
    if (scales) {
        float *os = dst.out_scale + (size_t)dst_row * dst.os_stride_token;
        if (member < num_scales) os[(size_t)member * dst.os_stride_elem] = first_scale;
        for (uint32_t q = member + team; q < num_scales; q += team) os[(size_t)q * dst.os_stride_elem] = ss[q];
    }
}

// ---------------------------------------------------------------------------
// dispatch recv.  The receivers of a step are laid out ONCE per step, by the
// launch of the step's first recv (the reference's host worker runs
// process_routing_info once per rank and step, a2a_worker.rs:526-703).
//
// stage_recv_first_kernel is that launch.  Its first workgroups serve the rank
// that called: each lays the receiver out in LDS from the published per-source
// counts of its experts (a2a_worker.rs:577-606,621-694: rows per expert, padded
// first row of every expert, first row of every (source, expert) run inside it,
// and the order in which the runs ARRIVE: sources in the worker's order,
// experts inside a source), then teams of wavefronts share the received rows:
// the row's metadata is written (padded_index, source_rank, source position and
// the two offset tables: a2a_worker.rs:636-671) and payload and scales are
// copied from the sender's staged token (a2a_dispatch_recv.cu:139-155).  A rank
// on a GPU of its own would launch only these.  The workgroups behind them lay
// out the OTHER receivers, in the shadow of that copy: the same layout in LDS,
// then one thread per received row writes the row's metadata and the staged row
// it comes from (the token behind its position in the sender's order).
//
// stage_recv_kernel is the launch of every later recv of the step.  It only
// copies: a team of wavefronts per received row reads where the row comes from
// and where it goes (one trip for both) and moves payload and scales; its first
// workgroup hands the receiver's counts to the caller.
//
// Dynamic LDS of a layout: 4 * G * Le + 1 + 3 * G words.
// ---------------------------------------------------------------------------
struct ReceiverTables {   // in LDS, see lay_out_receiver
    uint32_t *tot;       // [g][le]  copies source g sends to local expert le
    uint32_t *excl;      // [g][le]  position of the run in the sender's expert-sorted order
    uint32_t *run_row;   // [i][le]  first row of the run in the receiver's buffer (i = order index)
    uint32_t *seg;       // [i][le]  first ARRIVAL index of the run; seg[items] = rows received
    uint32_t *grp_dst;   // [g]      position of source g's first row for this receiver in g's send order
    uint32_t *grp_src;   // [g]      rows this receiver gets from the sources numbered below g
    uint32_t *grp_cnt;   // [g]      rows this receiver gets from source g
    const uint8_t *order;  // [i]    the i-th source this receiver lays out
    uint32_t rows;       // rows received
    // only with lay_out_receiver_spread (w = i * Le + le is the run of the i-th source visited and local expert le):
    uint32_t *pos;       // [w]      position of the run in the sender's expert-sorted order (excl, by run)
    uint32_t own_g, own_pos, own_seg, own_end, own_row;   // run w = threadIdx.x of this thread (if there is one), in registers
};

// Lays out receiver `r` in LDS.  Whole workgroup.  `publish`: this workgroup also writes the
// receiver's tables to memory and (if given) its counts to the caller.  Returns false, before the
// expensive part, when the workgroup's first row `first_row` lies beyond the rows received and it
// does not publish: the host sizes grids for an upper bound, a receiver typically gets 1/N of it.
__device__ __forceinline__ bool lay_out_receiver(uint32_t valid_mask, const Workspace &ws, const Staging &st, uint32_t r,
                                                 bool publish, uint32_t first_row, int32_t *out_num_tokens,
                                                 uint32_t out_rows, uint32_t *s_recv, uint8_t *s_order,
                                                 ReceiverTables &t) {
    const uint32_t G = ws.num_groups, E = ws.num_experts, Le = ws.experts_per_rank;
    const uint32_t first = r * Le;
    const uint32_t n_local = first >= E ? 0 : (E - first < Le ? E - first : Le);
    const uint32_t items = G * Le;
    const uint32_t tid = threadIdx.x;
    const uint32_t nthreads = blockDim.x;
    const uint32_t lane = tid & (kWave - 1);
    uint32_t *tot = t.tot = s_recv;
    uint32_t *excl = t.excl = tot + items;
    uint32_t *run_row = t.run_row = excl + items;
    uint32_t *seg = t.seg = run_row + items;
    uint32_t *grp_dst = t.grp_dst = seg + items + 1;
    uint32_t *grp_src = t.grp_src = grp_dst + G;
    uint32_t *grp_cnt = t.grp_cnt = grp_src + G;
    t.order = s_order;

    // The order in which this receiver lays out its sources (one byte per source, from the table the
    // context computed once) travels with the counts and is read from LDS from then on: looked up in
    // memory where it is used, it put a dependent trip into the layout and one in front of every row.
    // All loads of a thread are asked for before the first is used (none under a condition of its own:
    // a word that does not count is read from a valid place and dropped), or each would be waited for
    // by itself, one trip to memory after the other.
    const uint32_t order_word = ws.order[r * (kMaxWorld / 4) + (tid < G ? tid >> 2 : 0)];
    for (uint32_t w = tid; w < items; w += nthreads) {
        const uint32_t g = Le > 1 ? __umulhi(w, ws.le_magic) : w;
        const uint32_t le = w - g * Le;
        const uint32_t e = first + le;
        const bool live = le < n_local && (valid_mask >> g & 1);
        const uint32_t at = live ? g * E + e : 0;
        const uint32_t count = ws.num_routed[at];
        const uint32_t upto = ws.expert_offsets[at > 0 ? at - 1 : 0];
        tot[w] = live ? count : 0;
        excl[w] = live && e > 0 ? upto : 0;
    }
    if (tid < G) s_order[tid] = (uint8_t)(order_word >> (8 * (tid & 3)));
    __syncthreads();

    // Rows this receiver gets from source g (lane g; there are at most kMaxWorld <= 64 sources): the
    // sender's scan over its experts gives them without a sum.  Every wavefront adds them up by itself.
    uint32_t from_source = 0;
    if (lane < G && n_local != 0) {
        const uint32_t last = lane * Le + n_local - 1;
        from_source = excl[last] + tot[last] - excl[lane * Le];
    }
    const uint32_t from_lower = wave_inclusive_scan(from_source, lane);   // inclusive over the sources
    const uint32_t rows = t.rows = (uint32_t)__builtin_amdgcn_readlane((int)from_lower, kWave - 1);
    if (!publish && first_row >= rows) return false;   // uniform

    // The layout is the work of two wavefronts, each by itself (scans on the DPP path, no barrier
    // inside); the others wait for them.  Done by every wavefront of every workgroup, with workgroup
    // scans, it was most of the kernel's instructions.
    const uint32_t wave = tid / kWave;
    if (wave == 0) {
        // Per source: where its rows for this receiver begin in its own send order (dst_group_offset,
        // a2a_worker.rs:571-575) and how many rows the lower-numbered sources send here
        // (src_group_offset, a2a_worker.rs:582-590: numeric order, not the order of arrival).
        if (lane < G) {
            grp_dst[lane] = excl[lane * Le];
            grp_cnt[lane] = from_source;
            grp_src[lane] = from_lower - from_source;
        }

        // Rows per expert, padded offsets, first row of every run.
        const uint32_t visited = lane < G ? s_order[lane] : 0;   // lane i: the i-th source in the order of the layout
        const uint32_t pad = ws.expert_padding;
        uint32_t carry = 0;
        for (uint32_t l0 = 0; l0 < Le; l0 += kWave) {
            const uint32_t le = l0 + lane;
            const bool mine = le < n_local;
            uint32_t tpe = 0;
            if (mine) {
                for (uint32_t g = 0; g < G; ++g) tpe += tot[g * Le + le];
            }
            const uint32_t padded = (tpe + pad - 1) / pad * pad;
            const uint32_t scan = wave_inclusive_scan(mine ? padded : 0, lane);
            if (mine) {
                const uint32_t poff = carry + scan - padded;
                const uint32_t e = first + le;
                uint32_t running = poff;
                uint32_t g = (uint32_t)__builtin_amdgcn_readlane((int)visited, 0);
                uint32_t next = tot[g * Le + le];
                for (uint32_t i = 0; i < G; ++i) {
                    // the count of the source after this one is asked for before this one's is used
                    const uint32_t count = next;
                    const uint32_t g_next = (uint32_t)__builtin_amdgcn_readlane((int)visited, (int)(i + 1 < G ? i + 1 : i));
                    next = tot[g_next * Le + le];
                    run_row[i * Le + le] = running;
                    if (publish) ws.slot_base[g * E + e] = running;
                    running += count;
                    g = g_next;
                }
                if (publish) {
                    ws.tokens_per_expert[e] = tpe;
                    ws.padded_offset[e] = poff;
                    if (out_num_tokens != nullptr) out_num_tokens[le] = (int32_t)tpe;
                    if (poff + tpe > out_rows) atomicOr(ws.err, A2A_DEV_RECV_OVERFLOW);
                }
            }
            carry += (uint32_t)__builtin_amdgcn_readlane((int)scan, kWave - 1);
        }
    }
    if (wave == (nthreads > kWave ? 1u : 0u)) {
        // Arrival order: sources as the worker visits them, local experts inside a source.  Lane i has
        // the rows that arrive before those of the i-th source visited; inside a source the sender's
        // scan over its experts says how many rows precede those of a local expert.  No sum, no scan
        // over the runs.
        const uint32_t visited = lane < G ? s_order[lane] : 0;
        const uint32_t theirs = (uint32_t)__shfl((int)from_source, (int)visited);   // every lane takes part
        const uint32_t arrive = lane < G ? theirs : 0;
        const uint32_t before = wave_inclusive_scan(arrive, lane) - arrive;
        for (uint32_t b = 0; b < items; b += kWave) {
            const uint32_t s = b + lane;
            const uint32_t i = s < items ? (Le > 1 ? __umulhi(s, ws.le_magic) : s) : 0;
            const uint32_t base = (uint32_t)__shfl((int)before, (int)i);
            const uint32_t count = (uint32_t)__shfl((int)arrive, (int)i);
            if (s < items) {
                const uint32_t le = s - i * Le;
                const uint32_t g = s_order[i];
                seg[s] = base + (le < n_local ? excl[g * Le + le] - excl[g * Le] : count);
            }
        }
        if (lane == 0) {
            seg[items] = rows;
            if (publish) {
                if (rows > st.max_recv) atomicOr(ws.err, A2A_DEV_RECV_OVERFLOW);
                st.num_recv[2 * r] = rows;
            }
        }
    }
    __syncthreads();
    if (publish && tid == 0) {
        // rows that come from other nodes (num_efa_tokens, a2a_worker.rs:681-687)
        const uint32_t remote_segs = (ws.world / ws.node_size - 1) * (ws.node_size / ws.dp_size) * Le;
        st.num_recv[2 * r + 1] = remote_segs < items ? seg[remote_segs] : rows;
    }
    return true;
}

// What the receiver's tables say of arrival `row` of run `s` (seg[s] <= row < seg[s + 1]).
struct RowMeta {
    uint32_t g;        // source (dp group)
    uint32_t pos;      // position in the source's expert-sorted order
    uint32_t dst_row;  // row in the receiver's buffer
};

__device__ __forceinline__ RowMeta row_of_run(const ReceiverTables &t, const Workspace &ws, uint32_t s, uint32_t row) {
    const uint32_t Le = ws.experts_per_rank;
    const uint32_t i = Le > 1 ? __umulhi(s, ws.le_magic) : s;
    const uint32_t le = s - i * Le;
    RowMeta m;
    m.g = t.order[i];
    const uint32_t j = row - t.seg[s];
    m.pos = t.excl[m.g * Le + le] + j;
    m.dst_row = t.run_row[s] + j;
    return m;
}

// Writes the five per-row tables of the reference's host worker for arrival `row` of receiver `r`
// (a2a_worker.rs:633-671).  One thread.
__device__ __forceinline__ void write_row_tables(const ReceiverTables &t, const Workspace &ws, const Staging &st,
                                                 uint32_t r, uint32_t row, const RowMeta &m, uint32_t max_private) {
    const uint32_t G = ws.num_groups;
    const size_t at = (size_t)r * st.max_recv + row;
    st.padded_index[at] = m.dst_row;
    // the member of the group that sends to this rank (a2a_worker.rs:633)
    const uint32_t peer = m.g * ws.dp_size + r % ws.dp_size;
    st.source_rank[at] = peer;
    st.source_position[at] = m.pos;
    // How the reference addresses the row on its way in and on its way back (a2a_worker.rs:636-667).
    // Nothing here reads these two: they are what a rank on a GPU of its own would consume.
    const uint32_t index_on_rank = m.pos - t.grp_dst[m.g];     // rows of this source before this one
    const bool same_node = peer / ws.node_size == r / ws.node_size;
    uint32_t sdo = m.pos, cso = m.pos;                         // own rows: the sender's position
    if (peer != r) {
        if (index_on_rank < max_private) {
            sdo = max_private * m.g + index_on_rank;                               // private region
        } else if (same_node) {
            sdo = m.pos | 0x80000000u;                                             // read from the peer's send buffer
        } else {
            sdo = t.grp_src[m.g] + index_on_rank + max_private * (G - 1);          // overflow region
        }
    }
    if ((peer != r || ws.dp_size > 1) && !same_node) cso = t.grp_src[m.g] + index_on_rank;
    st.source_dispatch_offset[at] = sdo;
    st.combine_send_offset[at] = cso;
}

__global__ __launch_bounds__(1024) void stage_recv_first_kernel(const StageRecvArgs args, const Workspace ws,
                                                                const Staging st) {
    extern __shared__ uint32_t s_recv[];
    __shared__ uint8_t s_order[kMaxWorld];
    const uint32_t tid = threadIdx.x;
    const uint32_t nthreads = blockDim.x;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t items = ws.num_groups * ws.experts_per_rank;
    ReceiverTables t;

    if (blockIdx.x >= args.copy_blocks) {
        // ---- one of the other receivers: layout, then one thread per received row ----
        const uint32_t w = blockIdx.x - args.copy_blocks;
        uint32_t r = w / args.slices;
        const uint32_t slice = w - r * args.slices;
        if (r >= args.rank) ++r;   // the caller's rank is served by the first workgroups
        if (!lay_out_receiver(args.valid_mask, ws, st, r, slice == 0, slice * nthreads, nullptr, 0xFFFFFFFFu, s_recv,
                              s_order, t))
            return;
        const uint32_t total = t.rows < st.max_recv ? t.rows : st.max_recv;   // beyond: flagged and dropped
        for (uint32_t row = slice * nthreads + tid; row < total; row += args.slices * nthreads) {
            // the run this arrival belongs to: the last one with seg[s] <= row (runs without rows share
            // their first arrival with the run after them, so the last such run is the one with rows)
            uint32_t lo = 0, hi = items;   // seg[lo] <= row < seg[hi]
            while (hi - lo > 1) {
                const uint32_t mid = (lo + hi) / 2;
                if (t.seg[mid] <= row) lo = mid; else hi = mid;
            }
            const RowMeta m = row_of_run(t, ws, lo, row);
            // the token behind the position: asked for first, used last
            const uint32_t token = m.pos < ws.max_tk ? st.pos_token[(size_t)m.g * ws.max_tk + m.pos] : 0;
            write_row_tables(t, ws, st, r, row, m, args.max_private);
            st.source_row[(size_t)r * st.max_recv + row] = m.g * st.max_tokens + token;
        }
        return;
    }

    // ---- the caller's rank: layout, then a team of wavefronts per received row ----
    const uint32_t r = args.rank;
    const uint32_t team_threads = args.team_waves * kWave;
    const uint32_t teams = nthreads / team_threads;
    if (!lay_out_receiver(args.valid_mask, ws, st, r, blockIdx.x == 0, blockIdx.x * teams, args.out_num_tokens,
                          args.dst.out_rows, s_recv, s_order, t))
        return;
    // From here on the workgroup is split into teams that work alone (no barrier): one received row
    // per team at a time.  Every wavefront of a team finds the row's run by itself.
    const PushDst &dst = args.dst;
    const uint32_t num_chunks = args.row_bytes / 16;
    const uint32_t member = tid % team_threads;
    for (uint32_t row = blockIdx.x * teams + tid / team_threads; row < t.rows; row += args.copy_blocks * teams) {
        // the run this arrival belongs to: the one non-empty run with seg[s] <= row < seg[s + 1]
        uint32_t s = 0;
        for (uint32_t s0 = 0; s0 < items; s0 += kWave) {
            const uint32_t cand = s0 + lane;
            const uint64_t hit = __ballot(cand < items && t.seg[cand] <= row && row < t.seg[cand + 1]);
            if (hit != 0) {
                s = s0 + (uint32_t)__builtin_ctzll(hit);
                break;
            }
        }
        const RowMeta m = row_of_run(t, ws, s, row);
        if (row >= st.max_recv) continue;   // flagged by the layout: more rows than the receive region was sized for
        const uint32_t token = st.pos_token[(size_t)m.g * ws.max_tk + m.pos];
        if (member == 0) {
            write_row_tables(t, ws, st, r, row, m, args.max_private);
            st.source_row[(size_t)r * st.max_recv + row] = m.g * st.max_tokens + token;
        }
        if (dst.out_x == nullptr) continue;
        if (m.dst_row >= dst.out_rows) {
            if (member == 0) atomicOr(ws.err, A2A_DEV_RECV_OVERFLOW);
            continue;
        }
        const uint8_t *src = st.send_buf + ((size_t)m.g * st.max_tokens + token) * st.disp_stride;
        copy_received_row(src, st.payload_bytes, num_chunks, args.hidden_dim_scale, dst, m.dst_row, member, team_threads);
    }
}

// The same layout for the steps with few rows (stage_recv_first_few_kernel), where the layout is most of
// what a recv waits for.  In the tables run_row and seg (and pos) a run is w = i * Le + le, i the
// source's place in the order of the layout, as in lay_out_receiver.
//
// The work is spread over all threads, one run (source in the order of the layout, local expert)
// each, and what counts is the number of dependent LDS trips and barriers between the arrival of the
// counts and the first row's load (each about 0.1 us): everything that can be asked for together is,
// reads before writes.  One wavefront doing the layout alone, in loops over the sources with one trip
// per step, was 1.5 us of the 2.2 us a small step's recv waited for its layout.
// After the last barrier inside, a thread's OWN runs (w = tid, tid + blockDim.x, ...) are complete in
// LDS and the first of them is in t.own_*; `all_visible` adds the barrier after which every thread
// may read every run.
__device__ __forceinline__ bool lay_out_receiver_spread(uint32_t valid_mask, const Workspace &ws, const Staging &st, uint32_t r,
                                                 bool publish, uint32_t first_row, int32_t *out_num_tokens,
                                                 uint32_t out_rows, uint32_t *s_recv, uint8_t *s_order,
                                                 ReceiverTables &t, bool all_visible) {
    const uint32_t G = ws.num_groups, E = ws.num_experts, Le = ws.experts_per_rank;
    const uint32_t first = r * Le;
    const uint32_t n_local = first >= E ? 0 : (E - first < Le ? E - first : Le);
    const uint32_t items = G * Le;
    const uint32_t tid = threadIdx.x;
    const uint32_t nthreads = blockDim.x;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = tid / kWave;
    uint32_t *tot = t.tot = s_recv;
    uint32_t *excl = t.excl = tot + items;
    uint32_t *pos_of = t.pos = excl + items;
    uint32_t *run_row = t.run_row = pos_of + items;
    uint32_t *seg = t.seg = run_row + items;
    uint32_t *grp_dst = t.grp_dst = seg + items + 1;
    uint32_t *grp_src = t.grp_src = grp_dst + G;
    uint32_t *grp_cnt = t.grp_cnt = grp_src + G;
    uint32_t *poff = grp_cnt + G;   // [le] rows of a local expert, then its padded first row
    t.order = s_order;

    // The order in which this receiver lays out its sources (one byte per source, from the table the
    // context computed once) is asked for with the counts: every thread takes the first two words (the
    // first eight sources) for its loops over the sources, the first eight threads copy the table's row
    // to LDS for whoever needs the i-th source with an i of its own.  All loads of a thread are asked
    // for before the first is used, none under a condition of its own (a word that does not count is
    // read from a valid place and dropped): waited for one by one they are a trip to memory each.
    const uint32_t *order_row = ws.order + r * (kMaxWorld / 4);
    const uint32_t order_lo = order_row[0], order_hi = order_row[1];
    const uint32_t order_mine = order_row[tid & (kMaxWorld / 4 - 1)];
    uint32_t *order_words = reinterpret_cast<uint32_t *>(s_order);
    for (uint32_t w = tid; w < items; w += nthreads) {
        const uint32_t g = Le > 1 ? __umulhi(w, ws.le_magic) : w;
        const uint32_t le = w - g * Le;
        const uint32_t e = first + le;
        const bool live = le < n_local && (valid_mask >> g & 1);
        const uint32_t at = live ? g * E + e : 0;
        const uint32_t count = ws.num_routed[at];
        const uint32_t upto = ws.expert_offsets[at > 0 ? at - 1 : 0];
        tot[w] = live ? count : 0;
        excl[w] = live && e > 0 ? upto : 0;
    }
    if (tid < (uint32_t)kMaxWorld / 4) order_words[tid] = order_mine;
    __syncthreads();
    const uint32_t o0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)order_lo);
    const uint32_t o1 = (uint32_t)__builtin_amdgcn_readfirstlane((int)order_hi);

    // Rows of local expert `le` from the sources visited before the i-th, and from all of them.
    auto sums_over_sources = [&](uint32_t i, uint32_t le, uint32_t &below, uint32_t &total) {
        below = total = 0;
        for (uint32_t b = 0; b < G; b += 8) {
            // eight sources at a time: their numbers are the same for every thread (scalar), their
            // counts are asked for together
            const uint32_t w0 = b == 0 ? o0 : (uint32_t)__builtin_amdgcn_readfirstlane((int)order_words[b / 4]);
            const uint32_t w1 = b == 0 ? o1 : (uint32_t)__builtin_amdgcn_readfirstlane((int)order_words[b / 4 + 1]);
            uint32_t c[8];
#pragma unroll
            for (uint32_t u = 0; u < 8; ++u) {
                const uint32_t g = ((u < 4 ? w0 : w1) >> (8 * (u & 3))) & 0xFFu;   // (0 past the last source)
                c[u] = tot[g * Le + le];
            }
#pragma unroll
            for (uint32_t u = 0; u < 8; ++u) {
                if (b + u < G) total += c[u];
                if (b + u < i) below += c[u];
            }
        }
    };

    // ---- first trip: everything that needs only the counts.  Run w = tid of this thread first.
    // (A wavefront none of whose threads has a run skips what only runs need: what every wavefront
    // of a workgroup executes costs the SIMDs they share as much time as what one executes alone.)
    const bool has_runs = tid - lane < items;   // the same for a whole wavefront
    const uint32_t w_own = tid < items ? tid : 0;
    const uint32_t i_own = Le > 1 ? __umulhi(w_own, ws.le_magic) : w_own;
    const uint32_t le_own = w_own - i_own * Le;
    const bool source_lane = lane < G && n_local != 0;
    const uint32_t last = source_lane ? lane * Le + n_local - 1 : 0;
    const uint32_t excl_last = excl[last], tot_last = tot[last], excl_first = excl[source_lane ? lane * Le : 0];
    uint32_t visited = 0, g_own = 0, below_own = 0, total_own = 0;
    if (has_runs) {
        visited = s_order[lane < G ? lane : 0];   // lane i: the i-th source in the order of the layout
        g_own = s_order[i_own];
        sums_over_sources(i_own, le_own, below_own, total_own);
    }

    // Rows this receiver gets from source g (lane g; there are at most kMaxWorld <= 64 sources): the
    // sender's scan over its experts gives them without a sum.  Every wavefront adds them up by itself.
    const uint32_t from_source = source_lane ? excl_last + tot_last - excl_first : 0;
    const uint32_t from_lower = wave_inclusive_scan(from_source, lane);   // inclusive over the sources
    const uint32_t rows = t.rows = (uint32_t)__builtin_amdgcn_readlane((int)from_lower, kWave - 1);
    if (!publish && first_row >= rows) return false;   // uniform

    // ---- second trip: the rows of the i-th source visited (lane i), the position and rows of the own run
    uint32_t theirs = 0, pos0_own = 0, pos_own = 0, tot_own = 0;
    if (has_runs) {
        theirs = (uint32_t)__shfl((int)from_source, (int)visited);   // every lane of the wavefront takes part
        pos0_own = excl[g_own * Le];
        pos_own = excl[g_own * Le + le_own];
        tot_own = tot[g_own * Le + le_own];
    }

    // Padded first row of every local expert: a scan over the experts, by the first wavefront, whose
    // thread `le` has the expert's rows already (thread le is run (0, le)).  With more than 64 local
    // experts the counts go through LDS and a barrier.
    const uint32_t pad = ws.expert_padding;
    const bool wide = Le > (uint32_t)kWave;   // uniform
    if (wide) {
        if (tid < Le) poff[tid] = total_own;
        for (uint32_t le = tid + nthreads; le < Le; le += nthreads) {
            uint32_t below, total;
            sums_over_sources(0, le, below, total);
            poff[le] = total;
        }
        __syncthreads();
    }
    if (wave == 0) {
        uint32_t carry = 0;
        for (uint32_t l0 = 0; l0 < Le; l0 += kWave) {
            const uint32_t le = l0 + lane;
            const bool mine = le < n_local;
            const uint32_t tpe = !mine ? 0 : (wide ? poff[le] : total_own);
            const uint32_t padded = pad > 1 ? (tpe + pad - 1) / pad * pad : tpe;
            const uint32_t scan = wave_inclusive_scan(padded, lane);
            const uint32_t mine_off = carry + scan - padded;
            if (le < Le) poff[le] = mine_off;
            if (mine && publish) {
                const uint32_t e = first + le;
                ws.tokens_per_expert[e] = tpe;
                ws.padded_offset[e] = mine_off;
                if (out_num_tokens != nullptr) out_num_tokens[le] = (int32_t)tpe;
                if (mine_off + tpe > out_rows) atomicOr(ws.err, A2A_DEV_RECV_OVERFLOW);
            }
            carry += (uint32_t)__builtin_amdgcn_readlane((int)scan, kWave - 1);
        }
    }

    // Arrival order: sources as the worker visits them, local experts inside a source.  Lane i of every
    // wavefront has the rows of the i-th source visited and those that arrive before them.
    uint32_t arrive = 0, before = 0, seg_own = 0;
    if (has_runs) {
        arrive = lane < G ? theirs : 0;
        before = wave_inclusive_scan(arrive, lane) - arrive;
        // ---- third trip: the own run's source in that order
        const uint32_t base_own = (uint32_t)__shfl((int)before, (int)i_own);    // every lane of the wavefront takes part
        const uint32_t count_own = (uint32_t)__shfl((int)arrive, (int)i_own);
        seg_own = base_own + (le_own < n_local ? pos_own - pos0_own : count_own);
    }
    t.own_g = g_own;
    t.own_pos = pos_own;
    t.own_seg = seg_own;
    t.own_end = seg_own + tot_own;   // (the run after this one begins where this one's rows end)

    // ---- writes
    if (tid < items) {
        seg[tid] = seg_own;
        pos_of[tid] = pos_own;
    }
    if (wave == 0 && lane < G) {
        // Per source: where its rows for this receiver begin in its own send order (dst_group_offset,
        // a2a_worker.rs:571-575) and how many rows the lower-numbered sources send here
        // (src_group_offset, a2a_worker.rs:582-590: numeric order, not the order of arrival).
        grp_dst[lane] = excl_first;
        grp_cnt[lane] = from_source;
        grp_src[lane] = from_lower - from_source;
    }
    if (tid == 0) {
        seg[items] = rows;
        if (publish) {
            if (rows > st.max_recv) atomicOr(ws.err, A2A_DEV_RECV_OVERFLOW);
            st.num_recv[2 * r] = rows;
        }
    }
    // the runs beyond the first of a thread (more runs than threads): the same, one at a time
    for (uint32_t w0 = nthreads; w0 < items; w0 += nthreads) {
        const uint32_t w = w0 + tid;
        const bool real = w < items;
        const uint32_t wc = real ? w : 0;
        const uint32_t i = Le > 1 ? __umulhi(wc, ws.le_magic) : wc;
        const uint32_t le = wc - i * Le;
        uint32_t below, total;
        sums_over_sources(i, le, below, total);
        const uint32_t g = s_order[i];
        const uint32_t p0 = excl[g * Le];
        const uint32_t p = excl[g * Le + le];
        const uint32_t base = (uint32_t)__shfl((int)before, (int)i);    // every lane takes part
        const uint32_t count = (uint32_t)__shfl((int)arrive, (int)i);
        if (real) {
            run_row[w] = below;
            seg[w] = base + (le < n_local ? p - p0 : count);
            pos_of[w] = p;
        }
    }
    __syncthreads();

    // First row of every run: behind the rows of the expert from the sources visited earlier.
    t.own_row = below_own + poff[le_own];
    if (tid < items) {
        run_row[tid] = t.own_row;
        if (publish && le_own < n_local) ws.slot_base[g_own * E + first + le_own] = t.own_row;
    }
    for (uint32_t w = tid + nthreads; w < items; w += nthreads) {
        const uint32_t i = Le > 1 ? __umulhi(w, ws.le_magic) : w;
        const uint32_t le = w - i * Le;
        const uint32_t row = run_row[w] + poff[le];
        run_row[w] = row;
        if (publish && le < n_local) ws.slot_base[(uint32_t)s_order[i] * E + first + le] = row;
    }
    if (publish && tid == 0) {
        // rows that come from other nodes (num_efa_tokens, a2a_worker.rs:681-687)
        const uint32_t remote_segs = (ws.world / ws.node_size - 1) * (ws.node_size / ws.dp_size) * Le;
        st.num_recv[2 * r + 1] = remote_segs < items ? seg[remote_segs] : rows;
    }
    if (all_visible) __syncthreads();
    return true;
}

// What the spread tables say of arrival `row` of run `s` (seg[s] <= row < seg[s + 1]): one LDS trip.
__device__ __forceinline__ RowMeta row_of_run_spread(const ReceiverTables &t, const Workspace &ws, uint32_t s, uint32_t row) {
    const uint32_t Le = ws.experts_per_rank;
    const uint32_t i = Le > 1 ? __umulhi(s, ws.le_magic) : s;
    RowMeta m;
    m.g = t.order[i];
    const uint32_t j = row - t.seg[s];
    m.pos = t.pos[s] + j;
    m.dst_row = t.run_row[s] + j;
    return m;
}

// The step's first recv when the step has few rows (the host gave every row a workgroup as wide as the
// row): the same work as stage_recv_first_kernel with the layout spread over the threads, and the
// whole workgroup serves one row at a time: the thread whose run holds the row says so to the others.
// Dynamic LDS: 5 * G * Le + 1 + 3 * G + Le words.
__global__ __launch_bounds__(1024) void stage_recv_first_few_kernel(const StageRecvArgs args, const Workspace ws,
                                                                    const Staging st) {
    extern __shared__ uint32_t s_recv[];
    __shared__ __align__(16) uint8_t s_order[kMaxWorld];
    __shared__ uint32_t s_meta[3];
    const uint32_t tid = threadIdx.x;
    const uint32_t nthreads = blockDim.x;
    const uint32_t items = ws.num_groups * ws.experts_per_rank;
    ReceiverTables t;

    // The workgroups of the other receivers come first in the grid: their chain (layout, run and token
    // of every row, the row's tables) is as long as the calling rank's (layout, row, copy), and started
    // behind its workgroups they were what the kernel's end waited for (0.15 us).
    const uint32_t other_blocks = gridDim.x - args.copy_blocks;
    if (blockIdx.x < other_blocks) {
        // ---- one of the other receivers: layout, then one thread per received row ----
        const uint32_t w = blockIdx.x;
        uint32_t r = w / args.slices;
        const uint32_t slice = w - r * args.slices;
        if (r >= args.rank) ++r;   // the caller's rank is served by the workgroups behind these
        if (!lay_out_receiver_spread(args.valid_mask, ws, st, r, slice == 0, slice * nthreads, nullptr, 0xFFFFFFFFu,
                                     s_recv, s_order, t, true))
            return;
        const uint32_t total = t.rows < st.max_recv ? t.rows : st.max_recv;   // beyond: flagged and dropped
        for (uint32_t row = slice * nthreads + tid; row < total; row += args.slices * nthreads) {
            // the run this arrival belongs to: the last one with seg[s] <= row (runs without rows share
            // their first arrival with the run after them, so the last such run is the one with rows)
            uint32_t lo = 0, hi = items;   // seg[lo] <= row < seg[hi]
            while (hi - lo > 1) {
                const uint32_t mid = (lo + hi) / 2;
                if (t.seg[mid] <= row) lo = mid; else hi = mid;
            }
            const RowMeta m = row_of_run_spread(t, ws, lo, row);
            // the token behind the position: asked for first, used last
            const uint32_t token = m.pos < ws.max_tk ? st.pos_token[(size_t)m.g * ws.max_tk + m.pos] : 0;
            write_row_tables(t, ws, st, r, row, m, args.max_private);
            st.source_row[(size_t)r * st.max_recv + row] = m.g * st.max_tokens + token;
        }
        return;
    }

    // ---- the caller's rank: layout, then the workgroup's row ----
    const uint32_t r = args.rank;
    const PushDst &dst = args.dst;
    const uint32_t num_chunks = args.row_bytes / 16;
    const uint32_t block = blockIdx.x - other_blocks;
    if (!lay_out_receiver_spread(args.valid_mask, ws, st, r, block == 0, block, args.out_num_tokens,
                                 args.dst.out_rows, s_recv, s_order, t, false))
        return;
    for (uint32_t row = block; row < t.rows; row += args.copy_blocks) {
        if (row != block) __syncthreads();   // the row before this one has been taken from s_meta
        if (tid < items && t.own_seg <= row && row < t.own_end) {   // in the thread's first run: all in registers
            s_meta[0] = t.own_g;
            s_meta[1] = t.own_pos + (row - t.own_seg);
            s_meta[2] = t.own_row + (row - t.own_seg);
        }
        for (uint32_t w = tid + nthreads; w < items; w += nthreads) {
            // (a thread's own runs are complete, and every run's first arrival is there)
            if (t.seg[w] <= row && row < t.seg[w + 1]) {
                const RowMeta mine = row_of_run_spread(t, ws, w, row);
                s_meta[0] = mine.g;
                s_meta[1] = mine.pos;
                s_meta[2] = mine.dst_row;
            }
        }
        __syncthreads();
        RowMeta m;
        m.g = s_meta[0];
        m.pos = s_meta[1];
        m.dst_row = s_meta[2];
        if (row >= st.max_recv) continue;   // flagged by the layout: more rows than the receive region was sized for
        const uint32_t token = st.pos_token[(size_t)m.g * ws.max_tk + m.pos];
        if (tid == 0) {
            write_row_tables(t, ws, st, r, row, m, args.max_private);
            st.source_row[(size_t)r * st.max_recv + row] = m.g * st.max_tokens + token;
        }
        if (dst.out_x != nullptr) {
            if (m.dst_row >= dst.out_rows) {
                if (tid == 0) atomicOr(ws.err, A2A_DEV_RECV_OVERFLOW);
            } else {
                const uint8_t *src = st.send_buf + ((size_t)m.g * st.max_tokens + token) * st.disp_stride;
                copy_received_row(src, st.payload_bytes, num_chunks, args.hidden_dim_scale, dst, m.dst_row, tid, nthreads);
            }
        }
    }
}

__global__ __launch_bounds__(1024) void stage_recv_kernel(const StageRecvArgs args, const Workspace ws,
                                                          const Staging st) {
    // everything a wavefront takes from the argument block, asked for in one go
    A2A_PIN(args.dst.out_x);
    A2A_PIN(args.dst.out_scale);
    A2A_PIN(args.dst.out_stride);
    A2A_PIN(args.dst.os_stride_elem);
    A2A_PIN(args.dst.os_stride_token);
    A2A_PIN(args.dst.out_rows);
    A2A_PIN(args.rank);
    A2A_PIN(args.row_bytes);
    A2A_PIN(args.hidden_dim_scale);
    A2A_PIN(args.team_waves);
    A2A_PIN(st.send_buf);
    A2A_PIN(st.padded_index);
    A2A_PIN(st.source_row);
    A2A_PIN(st.num_recv);
    A2A_PIN(st.disp_stride);
    A2A_PIN(st.payload_bytes);
    A2A_PIN(st.max_recv);
    const uint32_t r = args.rank;
    const uint32_t tid = threadIdx.x;
    const PushDst &dst = args.dst;
    const uint32_t num_chunks = args.row_bytes / 16;
    const uint32_t team = args.team_waves * kWave;   // threads that share a row
    const uint32_t teams = blockDim.x / team;
    const uint32_t member = tid % team;
    const uint32_t *padded_index = st.padded_index + (size_t)r * st.max_recv;
    const uint32_t *source_row = st.source_row + (size_t)r * st.max_recv;
    // The first row's two table words are asked for together with the number of rows received
    // (a row index the tables do not hold reads entry 0 and is dropped by the loop's bound).
    uint32_t row = blockIdx.x * teams + tid / team;
    const uint32_t probe = row < st.max_recv ? row : 0;
    uint32_t dst_row = padded_index[probe];
    uint32_t from = source_row[probe];
    uint32_t total = st.num_recv[2 * r];
    if (total > st.max_recv) total = st.max_recv;   // flagged by the layout: more rows than the region was sized for

    if (blockIdx.x == 0) {
        // the receiver's counts for the caller (a2a_dispatch_recv.cu:220-224)
        const uint32_t E = ws.num_experts, Le = ws.experts_per_rank;
        const uint32_t first = r * Le;
        const uint32_t n_local = first >= E ? 0 : (E - first < Le ? E - first : Le);
        for (uint32_t le = tid; le < n_local; le += blockDim.x) {
            const uint32_t tpe = ws.tokens_per_expert[first + le];
            if (args.out_num_tokens != nullptr) args.out_num_tokens[le] = (int32_t)tpe;
            if (ws.padded_offset[first + le] + tpe > dst.out_rows) atomicOr(ws.err, A2A_DEV_RECV_OVERFLOW);
        }
    }
    if (dst.out_x == nullptr) return;

    const uint32_t stride = gridDim.x * teams;
    while (row < total) {
        // the next row's words travel while this one is copied
        const uint32_t next = row + stride;
        const uint32_t next_probe = next < total ? next : row;
        const uint32_t next_dst = padded_index[next_probe];
        const uint32_t next_from = source_row[next_probe];
        if (dst_row >= dst.out_rows) {
            if (member == 0) atomicOr(ws.err, A2A_DEV_RECV_OVERFLOW);
        } else {
            const uint8_t *src = st.send_buf + (size_t)from * st.disp_stride;
            copy_received_row(src, st.payload_bytes, num_chunks, args.hidden_dim_scale, dst, dst_row, member, team);
        }
        row = next;
        dst_row = next_dst;
        from = next_from;
    }
}

// A later recv of a step with few rows: the host gave every row a workgroup as wide as the row, so a
// workgroup is one team and has one row, seldom two; nothing is divided and no row is asked for ahead.
__global__ __launch_bounds__(1024) void stage_recv_few_kernel(const StageRecvArgs args, const Workspace ws,
                                                              const Staging st) {
    // everything a wavefront takes from the argument block, asked for in one go
    A2A_PIN(args.dst.out_x);
    A2A_PIN(args.dst.out_scale);
    A2A_PIN(args.dst.out_stride);
    A2A_PIN(args.dst.os_stride_elem);
    A2A_PIN(args.dst.os_stride_token);
    A2A_PIN(args.dst.out_rows);
    A2A_PIN(args.rank);
    A2A_PIN(args.row_bytes);
    A2A_PIN(args.hidden_dim_scale);
    A2A_PIN(st.send_buf);
    A2A_PIN(st.padded_index);
    A2A_PIN(st.source_row);
    A2A_PIN(st.num_recv);
    A2A_PIN(st.disp_stride);
    A2A_PIN(st.payload_bytes);
    A2A_PIN(st.max_recv);
    const uint32_t r = args.rank;
    const uint32_t tid = threadIdx.x;
    const PushDst &dst = args.dst;
    const uint32_t num_chunks = args.row_bytes / 16;
    const uint32_t *padded_index = st.padded_index + (size_t)r * st.max_recv;
    const uint32_t *source_row = st.source_row + (size_t)r * st.max_recv;
    // The row's two table words are asked for together with the number of rows received (a row
    // index the tables do not hold reads entry 0 and is dropped by the loop's bound).
    uint32_t row = blockIdx.x;
    const uint32_t probe = row < st.max_recv ? row : 0;
    uint32_t dst_row = padded_index[probe];
    uint32_t from = source_row[probe];
    uint32_t total = st.num_recv[2 * r];
    if (total > st.max_recv) total = st.max_recv;   // flagged by the layout: more rows than the region was sized for

    if (blockIdx.x == 0) {
        // the receiver's counts for the caller (a2a_dispatch_recv.cu:220-224)
        const uint32_t E = ws.num_experts, Le = ws.experts_per_rank;
        const uint32_t first = r * Le;
        const uint32_t n_local = first >= E ? 0 : (E - first < Le ? E - first : Le);
        for (uint32_t le = tid; le < n_local; le += blockDim.x) {
            const uint32_t tpe = ws.tokens_per_expert[first + le];
            if (args.out_num_tokens != nullptr) args.out_num_tokens[le] = (int32_t)tpe;
            if (ws.padded_offset[first + le] + tpe > dst.out_rows) atomicOr(ws.err, A2A_DEV_RECV_OVERFLOW);
        }
    }
    if (dst.out_x == nullptr) return;

    while (row < total) {
        if (dst_row >= dst.out_rows) {
            if (tid == 0) atomicOr(ws.err, A2A_DEV_RECV_OVERFLOW);
        } else {
            const uint8_t *src = st.send_buf + (size_t)from * st.disp_stride;
            copy_received_row(src, st.payload_bytes, num_chunks, args.hidden_dim_scale, dst, dst_row, tid, blockDim.x);
        }
        row += gridDim.x;
        if (row < total) {
            dst_row = padded_index[row];
            from = source_row[row];
        }
    }
}

// ---------------------------------------------------------------------------
// combine send: copy expert_y[padded_index[i]] to the staging row of the copy
// it answers, i.e. row `source_position[i]` of sender `source_rank[i]`
// (a2a_combine_send.cu:124-136,196-205).
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void combine_send_kernel(const CombineSendArgs args,
                                                            const Workspace ws, const Staging st) {
    // everything a wavefront takes from the argument block, asked for in one go
    A2A_PIN(args.y);
    A2A_PIN(args.y_stride);
    A2A_PIN(args.y_rows);
    A2A_PIN(args.row_bytes);
    A2A_PIN(args.team_waves);
    A2A_PIN(ws.dp_size);
    A2A_PIN(ws.max_tk);
    A2A_PIN(st.comb_buf);
    A2A_PIN(st.padded_index);
    A2A_PIN(st.source_rank);
    A2A_PIN(st.source_position);
    A2A_PIN(st.comb_stride);
    A2A_PIN(st.max_recv);
    const uint32_t r = args.rank;
    uint32_t total = st.num_recv[2 * r];
    if (total > st.max_recv) total = st.max_recv;
    const uint32_t num_chunks = args.row_bytes / 16;
    const uint32_t team = args.team_waves * kWave;   // threads that share a row
    const uint32_t teams = blockDim.x / team;
    const uint32_t member = threadIdx.x % team;
    for (uint32_t i = blockIdx.x * teams + threadIdx.x / team; i < total; i += gridDim.x * teams) {
        const uint32_t row = st.padded_index[(size_t)r * st.max_recv + i];
        // every member of the source's dp group reads the same staging rows
        const uint32_t g = st.source_rank[(size_t)r * st.max_recv + i] / ws.dp_size;
        const uint32_t pos = st.source_position[(size_t)r * st.max_recv + i];
        if (row >= args.y_rows || pos >= ws.max_tk) {
            if (member == 0) atomicOr(ws.err, A2A_DEV_BAD_SLOT);
            continue;
        }
        copy_row_by_team(reinterpret_cast<const u32x4 *>(args.y + (size_t)row * args.y_stride),
                         reinterpret_cast<u32x4 *>(st.comb_buf + ((size_t)g * ws.max_tk + pos) * st.comb_stride),
                         num_chunks, member, team);
    }
}

// The combine-send of a step with few rows: the host gave every row a workgroup as wide as the row, so
// a workgroup is one team and has one row, seldom two.  The row's three table words are asked for
// together with the number of rows received (a row index the tables do not hold reads entry 0 and is
// dropped by the loop's bound), and nothing is divided: 128 tokens, 3.3 -> 3.1 us per launch.  (The same
// in the kernel of the large steps made its launches at 4096 tokens 1.5 to 4 % slower.)
__global__ __launch_bounds__(1024) void combine_send_few_kernel(const CombineSendArgs args,
                                                                const Workspace ws, const Staging st) {
    // everything a wavefront takes from the argument block, asked for in one go
    A2A_PIN(args.y);
    A2A_PIN(args.y_stride);
    A2A_PIN(args.y_rows);
    A2A_PIN(args.row_bytes);
    A2A_PIN(ws.dp_size);
    A2A_PIN(ws.max_tk);
    A2A_PIN(st.comb_buf);
    A2A_PIN(st.padded_index);
    A2A_PIN(st.source_rank);
    A2A_PIN(st.source_position);
    A2A_PIN(st.comb_stride);
    A2A_PIN(st.max_recv);
    const uint32_t r = args.rank;
    const uint32_t num_chunks = args.row_bytes / 16;
    const uint32_t *padded_index = st.padded_index + (size_t)r * st.max_recv;
    const uint32_t *source_rank = st.source_rank + (size_t)r * st.max_recv;
    const uint32_t *source_position = st.source_position + (size_t)r * st.max_recv;
    uint32_t i = blockIdx.x;
    const uint32_t probe = i < st.max_recv ? i : 0;
    uint32_t row = padded_index[probe];
    uint32_t peer = source_rank[probe];
    uint32_t pos = source_position[probe];
    uint32_t total = st.num_recv[2 * r];
    if (total > st.max_recv) total = st.max_recv;
    while (i < total) {
        // every member of the source's dp group reads the same staging rows
        const uint32_t g = ws.dp_size > 1 ? peer / ws.dp_size : peer;
        if (row >= args.y_rows || pos >= ws.max_tk) {
            if (threadIdx.x == 0) atomicOr(ws.err, A2A_DEV_BAD_SLOT);
        } else {
            copy_row_by_team(reinterpret_cast<const u32x4 *>(args.y + (size_t)row * args.y_stride),
                             reinterpret_cast<u32x4 *>(st.comb_buf + ((size_t)g * ws.max_tk + pos) * st.comb_stride),
                             num_chunks, threadIdx.x, blockDim.x);
        }
        i += gridDim.x;
        if (i < total) {
            row = padded_index[i];
            peer = source_rank[i];
            pos = source_position[i];
        }
    }
}

uint32_t block_for_chunks(uint32_t chunks) {
    uint32_t threads = (chunks + kWave - 1) / kWave * kWave;
    if (threads < (uint32_t)kWave) threads = kWave;
    if (threads > 1024) threads = 1024;
    return threads;
}

// How the rows of a receiver are shared out: the wider the team of wavefronts that shares a row, the
// shorter the life of a row (what counts when there are few rows), the narrower, the more rows are in
// flight (what counts when there are many).  The host knows an upper bound of the rows (every copy of
// every sender); a receiver typically gets 1/N of it, and the team is sized so that those rows give
// about 4096 wavefronts, as many as the GPU holds at this kernel's occupancy: one wavefront per row from
// about 4096 rows per receiver on, 2 at 2048, 4 at 1024, up to a team as wide as the row below that
// (then one workgroup per row).  Measured per step of 8 receivers, rows of 7 KB in / 14 KB back
// (recv / combine-send, us): 4096 tokens 122 / 198 with one wavefront per row (138 / 210 with two);
// 2048 tokens 83 / 97 with two (93 / 137 with one, 90 / 123 with four); 1024 tokens 59 / 65 with four
// (78 / 105 with one, 65 / 77 with two); 512 tokens 50-53 / 48-53 with four to seven (70 / 97 with one);
// 128 tokens 34 / 31 with the full width (39 / 41 with four).
constexpr uint32_t kMaxRowWorkgroups = 2048;
constexpr uint32_t kFewRowWorkgroups = 512;
constexpr uint32_t kWavefrontsWanted = 4096;

struct RowLaunch {
    uint32_t blocks, threads, team_waves;
};

RowLaunch row_launch(uint32_t max_rows, uint32_t chunks, uint32_t world) {
    RowLaunch l;
    const uint32_t width = block_for_chunks(chunks) / kWave;          // wavefronts that cover a row at one piece a lane
    const uint32_t typical = (max_rows + world - 1) / world;
    uint32_t want = 1;
    while (want < width && want * typical < kWavefrontsWanted) want *= 2;
    if (want >= width) {
        // few rows: one workgroup per row, as wide as the row needs
        l.threads = width * kWave;
        l.team_waves = width;
        l.blocks = max_rows < kFewRowWorkgroups ? max_rows : kFewRowWorkgroups;
        return l;
    }
    l.team_waves = want;
    const uint32_t waves = want < 4 ? 4 : want;                       // wavefronts of a workgroup
    l.threads = waves * kWave;
    const uint32_t teams = waves / want;
    const uint32_t blocks = (max_rows + teams - 1) / teams;
    l.blocks = blocks < kMaxRowWorkgroups ? blocks : kMaxRowWorkgroups;
    return l;
}

}  // namespace

int staging_allocate(Staging &st, const a2a_config &cfg, std::string *error) {
    if (st.allocated) return A2A_OK;
    const size_t N = cfg.world_size;
    const size_t K = cfg.num_experts_per_token;
    const size_t max_tk = (size_t)cfg.max_num_tokens * K;
    // The staged rows keep the reference's format (payload, scales, spare bytes: a2a_dispatch_send.cu:586-588)
    // at a stride rounded up to whole cache lines: the buffer is the library's own, and rows that begin in
    // the middle of a line cost every recv that reads them (4096 tokens: 120.7 -> 115.4 us for the recvs of
    // eight ranks).
    st.disp_stride = align_up_sz(a2a_dispatch_token_stride(&cfg), 256);
    st.comb_stride = a2a_combine_token_stride(&cfg);
    st.payload_bytes = (uint32_t)align_up_sz((size_t)cfg.hidden_dim * cfg.in_elemsize, 16);
    st.max_tokens = cfg.max_num_tokens;
    // Rows of the per-receiver tables: what the caller sized a rank's receive region for
    // (max_recv_tokens), and never more than every copy of every sender.  A receiver that gets
    // more rows than that is flagged (A2A_DEV_RECV_OVERFLOW) and the rows beyond are dropped.
    size_t max_recv = N * max_tk;
    if (cfg.max_recv_tokens != 0 && cfg.max_recv_tokens < max_recv) max_recv = cfg.max_recv_tokens;
    if (max_recv > 0x7FFFFFFFull) {
        if (error) *error = "world_size * max_num_tokens * num_experts_per_token too large";
        return A2A_ERR_UNSUPPORTED;
    }
    st.max_recv = (uint32_t)max_recv;
    if (N * cfg.max_num_tokens > 0xFFFFFFFFull) {   // a staged row is named by sender * max_num_tokens + token
        if (error) *error = "world_size * max_num_tokens too large";
        return A2A_ERR_UNSUPPORTED;
    }

    size_t off = 0;
    auto carve = [&off](size_t bytes) {
        const size_t at = off;
        off = align_up_sz(off + bytes, 256);
        return at;
    };
    const size_t o_send = carve(N * cfg.max_num_tokens * st.disp_stride);
    const size_t o_pos = carve(N * max_tk * sizeof(uint32_t));
    const size_t o_comb = carve(N * max_tk * st.comb_stride);
    const size_t o_pidx = carve(N * max_recv * sizeof(uint32_t));
    const size_t o_srank = carve(N * max_recv * sizeof(uint32_t));
    const size_t o_spos = carve(N * max_recv * sizeof(uint32_t));
    const size_t o_sdo = carve(N * max_recv * sizeof(uint32_t));
    const size_t o_cso = carve(N * max_recv * sizeof(uint32_t));
    const size_t o_srow = carve(N * max_recv * sizeof(uint32_t));
    const size_t o_nrecv = carve(N * 2 * sizeof(uint32_t));
    hipError_t e = hipMalloc(&st.arena, off);
    if (e != hipSuccess) {
        if (error) {
            *error = "hipMalloc(staging, " + std::to_string(off) + " bytes): " + hipGetErrorString(e);
        }
        st.arena = nullptr;
        return A2A_ERR_OUT_OF_MEMORY;
    }
    uint8_t *base = static_cast<uint8_t *>(st.arena);
    st.send_buf = base + o_send;
    st.pos_token = reinterpret_cast<uint32_t *>(base + o_pos);
    st.comb_buf = base + o_comb;
    st.padded_index = reinterpret_cast<uint32_t *>(base + o_pidx);
    st.source_rank = reinterpret_cast<uint32_t *>(base + o_srank);
    st.source_position = reinterpret_cast<uint32_t *>(base + o_spos);
    st.source_dispatch_offset = reinterpret_cast<uint32_t *>(base + o_sdo);
    st.combine_send_offset = reinterpret_cast<uint32_t *>(base + o_cso);
    st.source_row = reinterpret_cast<uint32_t *>(base + o_srow);
    st.num_recv = reinterpret_cast<uint32_t *>(base + o_nrecv);
    // Tables are read before they are written only through misuse; start from zero.
    e = hipMemset(base + o_pos, 0, o_comb - o_pos);
    if (e == hipSuccess) e = hipMemset(base + o_pidx, 0, off - o_pidx);
    if (e == hipSuccess) e = hipDeviceSynchronize();
    if (e != hipSuccess) {
        if (error) *error = std::string("hipMemset(staging): ") + hipGetErrorString(e);
        (void)hipFree(st.arena);
        st.arena = nullptr;
        return (int)e;
    }
    st.allocated = true;
    return A2A_OK;
}

void staging_free(Staging &st) {
    if (st.arena != nullptr) (void)hipFree(st.arena);
    st = Staging();
}

const uint32_t *staging_table(const Staging &st, const a2a_config &cfg, uint32_t rank, uint32_t which,
                              size_t *limit) {
    (void)cfg;
    if (!st.allocated || !(st.recv_mask >> rank & 1)) return nullptr;
    switch (which) {
        case A2A_TABLE_PADDED_INDEX:
            *limit = st.max_recv;
            return st.padded_index + (size_t)rank * st.max_recv;
        case A2A_TABLE_SOURCE_RANK:
            *limit = st.max_recv;
            return st.source_rank + (size_t)rank * st.max_recv;
        case A2A_TABLE_SOURCE_POSITION:
            *limit = st.max_recv;
            return st.source_position + (size_t)rank * st.max_recv;
        case A2A_TABLE_NUM_RECV_TOKENS:
            *limit = 2;
            return st.num_recv + (size_t)rank * 2;
        case A2A_TABLE_SOURCE_DISPATCH_OFFSET:
            *limit = st.max_recv;
            return st.source_dispatch_offset + (size_t)rank * st.max_recv;
        case A2A_TABLE_COMBINE_SEND_OFFSET:
            *limit = st.max_recv;
            return st.combine_send_offset + (size_t)rank * st.max_recv;
        default:
            return nullptr;
    }
}

hipError_t launch_stage_send(const StageSendArgs &args, const Workspace &ws, const Staging &st,
                             bool quantize, hipStream_t stream, KernelTiming timing) {
    if (args.src.num_tokens == 0) return hipSuccess;
    const uint32_t threads = block_for_chunks(quantize ? args.hidden_dim / 16 : args.row_bytes / 16);
    if (quantize) {
        hipExtLaunchKernelGGL(stage_send_kernel<true>, dim3(args.src.num_tokens), dim3(threads), 0, stream,
                              timing.start, timing.stop, 0, args, ws, st);
    } else {
        hipExtLaunchKernelGGL(stage_send_kernel<false>, dim3(args.src.num_tokens), dim3(threads), 0, stream,
                              timing.start, timing.stop, 0, args, ws, st);
    }
    return hipGetLastError();
}

bool stage_send_small_fits(const StageSendArgs &args, const Workspace &ws) {
    const uint64_t T = args.src.num_tokens;
    const uint64_t entries = T * ws.topk;
    return T != 0 && entries <= kSmallMaxEntries && entries * T <= kSmallMaxVisits;
}

hipError_t launch_stage_send_small(const StageSendArgs &args, const Workspace &ws, const Staging &st,
                                   bool quantize, hipStream_t stream, KernelTiming timing) {
    // The quick form: dense index rows, a piece of the row per thread and a wavefront beside them.
    const uint32_t pieces = quantize ? args.hidden_dim / 16 : args.row_bytes / 16;
    if (args.src.indices_stride == ws.topk && pieces + kWave <= 1024) {
        const uint32_t quick_threads = (pieces + kWave - 1) / kWave * kWave + kWave;
        const uint32_t counters = quick_threads - kWave;
        const uint32_t per_thread = (args.src.num_tokens * ws.topk + counters - 1) / counters;
        const size_t quick_lds = (size_t)ws.num_experts * sizeof(uint32_t);
#define A2A_LAUNCH_SEND_QUICK(NB)                                                                                    \
    do {                                                                                                             \
        if (quantize)                                                                                                \
            hipExtLaunchKernelGGL((stage_send_quick_kernel<NB, true>), dim3(args.src.num_tokens),                    \
                                  dim3(quick_threads), quick_lds, stream, timing.start, timing.stop, 0, args, ws,    \
                                  st);                                                                               \
        else                                                                                                         \
            hipExtLaunchKernelGGL((stage_send_quick_kernel<NB, false>), dim3(args.src.num_tokens),                   \
                                  dim3(quick_threads), quick_lds, stream, timing.start, timing.stop, 0, args, ws,    \
                                  st);                                                                               \
    } while (0)
        if (per_thread <= 1) A2A_LAUNCH_SEND_QUICK(1);
        else if (per_thread <= 2) A2A_LAUNCH_SEND_QUICK(2);
        else if (per_thread <= 3) A2A_LAUNCH_SEND_QUICK(3);
        else if (per_thread <= 4) A2A_LAUNCH_SEND_QUICK(4);
        else A2A_LAUNCH_SEND_QUICK(8);
#undef A2A_LAUNCH_SEND_QUICK
        return hipGetLastError();
    }
    const uint32_t threads = block_for_chunks(quantize ? args.hidden_dim / 16 : args.row_bytes / 16);
    const size_t lds = 3 * (size_t)ws.num_experts * sizeof(uint32_t);
    if (quantize) {
        hipExtLaunchKernelGGL(stage_send_small_kernel<true>, dim3(args.src.num_tokens), dim3(threads), lds, stream,
                              timing.start, timing.stop, 0, args, ws, st);
    } else {
        hipExtLaunchKernelGGL(stage_send_small_kernel<false>, dim3(args.src.num_tokens), dim3(threads), lds, stream,
                              timing.start, timing.stop, 0, args, ws, st);
    }
    return hipGetLastError();
}

uint32_t send_single_tokens_per_group(uint32_t tokens) {
    constexpr uint32_t kComputeUnits = 256;
    const uint32_t per_group = (tokens + kComputeUnits - 1) / kComputeUnits;
    return per_group < 1 ? 1 : per_group > kSendTokensPerGroup ? kSendTokensPerGroup : per_group;
}

bool stage_send_single_fits(const StageSendArgs &args, const Workspace &ws, bool quantize) {
    const uint64_t T = args.src.num_tokens;
    const uint32_t team = block_for_chunks(quantize ? args.hidden_dim / 16 : args.row_bytes / 16);
    const uint32_t per_group = send_single_tokens_per_group((uint32_t)T);
    uint32_t teams = 1024 / team;
    if (teams > per_group) teams = per_group;
    // dense index rows (the entries are read as one flat array), one thread per route of a workgroup's tokens
    return T != 0 && T * ws.topk <= kSendSingleMaxEntries && args.src.indices_stride == ws.topk &&
           per_group * ws.topk <= teams * team;
}

hipError_t launch_stage_send_single(const StageSendArgs &args, const Workspace &ws, const Staging &st,
                                    bool quantize, hipStream_t stream, KernelTiming timing) {
    const uint32_t team = block_for_chunks(quantize ? args.hidden_dim / 16 : args.row_bytes / 16);
    const uint32_t per_group = send_single_tokens_per_group(args.src.num_tokens);
    uint32_t teams = 1024 / team;
    if (teams > per_group) teams = per_group;
    const uint32_t blocks = (args.src.num_tokens + per_group - 1) / per_group;
    {
        // With a spare wavefront beside the teams, rows of one piece per thread of a team, a lane of
        // the spare wavefront per route of a workgroup's tokens and at most two rounds: the kernel in
        // which the teams do not wait for the routes.
        const uint32_t pieces = quantize ? args.hidden_dim / 16 : args.row_bytes / 16;
        uint32_t spare_teams = (1024 - kWave) / team;
        if (spare_teams > per_group) spare_teams = per_group;
        const uint32_t rounds = spare_teams != 0 ? (per_group + spare_teams - 1) / spare_teams : 3;
        if (pieces <= team && per_group * ws.topk <= (uint32_t)kWave && rounds <= 2) {
            const uint32_t counters = spare_teams * team;
            const uint32_t per_thread = (args.src.num_tokens * ws.topk + counters - 1) / counters;
            const size_t teams_lds = (size_t)ws.num_experts * sizeof(uint32_t);
#define A2A_LAUNCH_SEND_TEAMS(NB, ROUNDS)                                                                            \
    do {                                                                                                             \
        if (quantize)                                                                                                \
            hipExtLaunchKernelGGL((stage_send_teams_kernel<NB, ROUNDS, true>), dim3(blocks),                         \
                                  dim3(counters + kWave), teams_lds, stream, timing.start, timing.stop, 0, args,     \
                                  ws, st, team, per_group);                                                          \
        else                                                                                                         \
            hipExtLaunchKernelGGL((stage_send_teams_kernel<NB, ROUNDS, false>), dim3(blocks),                        \
                                  dim3(counters + kWave), teams_lds, stream, timing.start, timing.stop, 0, args,     \
                                  ws, st, team, per_group);                                                          \
    } while (0)
#define A2A_LAUNCH_SEND_TEAMS_NB(ROUNDS)                                                                             \
    do {                                                                                                             \
        if (per_thread <= 4) A2A_LAUNCH_SEND_TEAMS(4, ROUNDS);                                                       \
        else if (per_thread <= 8) A2A_LAUNCH_SEND_TEAMS(8, ROUNDS);                                                  \
        else if (per_thread <= 10) A2A_LAUNCH_SEND_TEAMS(10, ROUNDS);                                                \
        else A2A_LAUNCH_SEND_TEAMS(16, ROUNDS);                                                                      \
    } while (0)
            if (rounds <= 1) A2A_LAUNCH_SEND_TEAMS_NB(1);
            else A2A_LAUNCH_SEND_TEAMS_NB(2);
#undef A2A_LAUNCH_SEND_TEAMS_NB
#undef A2A_LAUNCH_SEND_TEAMS
            return hipGetLastError();
        }
    }
    const size_t lds = 2 * (size_t)ws.num_experts * sizeof(uint32_t);
    if (quantize) {
        hipExtLaunchKernelGGL(stage_send_single_kernel<true>, dim3(blocks), dim3(teams * team), lds, stream,
                              timing.start, timing.stop, 0, args, ws, st, team, per_group);
    } else {
        hipExtLaunchKernelGGL(stage_send_single_kernel<false>, dim3(blocks), dim3(teams * team), lds, stream,
                              timing.start, timing.stop, 0, args, ws, st, team, per_group);
    }
    return hipGetLastError();
}

hipError_t launch_stage_send_resolve(const StageSendArgs &args, const Workspace &ws, const Staging &st,
                                     bool quantize, hipStream_t stream, KernelTiming timing) {
    uint32_t threads = block_for_chunks(quantize ? args.hidden_dim / 16 : args.row_bytes / 16);
    const uint32_t blocks = args.src.num_tokens + 1;
    StageSendArgs a = args;
    a.resolver_wave = 0;
    if (threads + kWave <= 1024) {   // a wavefront of its own for the routes (measured: 27.3 against 28.5 us)
        a.resolver_wave = threads / kWave;
        threads += kWave;
    }
    if (quantize) {
        hipExtLaunchKernelGGL(stage_send_resolve_kernel<true>, dim3(blocks), dim3(threads), 0, stream, timing.start,
                              timing.stop, 0, a, ws, st);
    } else {
        hipExtLaunchKernelGGL(stage_send_resolve_kernel<false>, dim3(blocks), dim3(threads), 0, stream, timing.start,
                              timing.stop, 0, a, ws, st);
    }
    return hipGetLastError();
}

hipError_t launch_stage_recv(const StageRecvArgs &args, const Workspace &ws, const Staging &st, bool first_of_step,
                             hipStream_t stream, KernelTiming timing) {
    RowLaunch l = row_launch(args.max_rows, args.row_bytes / 16, ws.world);
    if (l.blocks == 0) l.blocks = 1;    // the counts are handed over even when nothing was sent
    StageRecvArgs a = args;
    a.team_waves = l.team_waves;
    if (!first_of_step) {
        if (l.team_waves * kWave == l.threads) {   // few rows: a workgroup per row
            hipExtLaunchKernelGGL(stage_recv_few_kernel, dim3(l.blocks), dim3(l.threads), 0, stream, timing.start,
                                  timing.stop, 0, a, ws, st);
        } else {
            hipExtLaunchKernelGGL(stage_recv_kernel, dim3(l.blocks), dim3(l.threads), 0, stream, timing.start,
                                  timing.stop, 0, a, ws, st);
        }
        return hipGetLastError();
    }
    // Behind the caller's workgroups: a few per other receiver, enough threads for the rows a receiver
    // typically gets (1/N of the host's upper bound); each repeats that receiver's layout in LDS.
    a.copy_blocks = l.blocks;
    const uint32_t typical = (args.max_rows + ws.world - 1) / ws.world;
    a.slices = (typical + l.threads - 1) / l.threads;
    if (a.slices < 1) a.slices = 1;
    if (a.slices > 16) a.slices = 16;
    const uint32_t blocks = l.blocks + (ws.world - 1) * a.slices;
    const size_t items = (size_t)ws.num_groups * ws.experts_per_rank;
    if (l.team_waves * kWave == l.threads) {   // few rows: a workgroup per row
        const size_t lds = (5 * items + 1 + 3 * (size_t)ws.num_groups + ws.experts_per_rank) * sizeof(uint32_t);
        hipExtLaunchKernelGGL(stage_recv_first_few_kernel, dim3(blocks), dim3(l.threads), lds, stream, timing.start,
                              timing.stop, 0, a, ws, st);
        return hipGetLastError();
    }
    const size_t lds = (4 * items + 1 + 3 * (size_t)ws.num_groups) * sizeof(uint32_t);
    hipExtLaunchKernelGGL(stage_recv_first_kernel, dim3(blocks), dim3(l.threads), lds, stream, timing.start,
                          timing.stop, 0, a, ws, st);
    return hipGetLastError();
}

hipError_t launch_combine_send(const CombineSendArgs &args, const Workspace &ws, const Staging &st,
                               hipStream_t stream, KernelTiming timing) {
    if (args.max_rows == 0) return hipSuccess;
    const RowLaunch l = row_launch(args.max_rows, args.row_bytes / 16, ws.world);
    CombineSendArgs a = args;
    a.team_waves = l.team_waves;
    if (l.team_waves * kWave == l.threads) {   // few rows: a workgroup per row
        hipExtLaunchKernelGGL(combine_send_few_kernel, dim3(l.blocks), dim3(l.threads), 0, stream, timing.start,
                              timing.stop, 0, a, ws, st);
        return hipGetLastError();
    }
    hipExtLaunchKernelGGL(combine_send_kernel, dim3(l.blocks), dim3(l.threads), 0, stream, timing.start, timing.stop,
                          0, a, ws, st);
    return hipGetLastError();
}

hipError_t launch_combine_recv(const CombineRecvArgs &args, const Workspace &ws, const Staging &st,
                               uint32_t in_dtype, uint32_t out_dtype, hipStream_t stream, KernelTiming timing) {
    CombArgs ca;
    std::memset(&ca, 0, sizeof ca);
    ca.dst[args.rank] = args.dst;
    for (uint32_t r = 0; r <= (uint32_t)kMaxWorld; ++r) {
        ca.token_start[r] = r <= args.rank ? 0 : args.dst.num_tokens;
    }
    ca.hidden_dim = args.hidden_dim;
    ca.accumulate = args.accumulate;
    ca.staged_base = st.comb_buf;
    ca.staged_stride = st.comb_stride;
    return launch_combine_gather(ca, ws, in_dtype, out_dtype, args.dst.num_tokens, stream, timing);
}

}  // namespace a2a
