// Shared between the HIP kernels and the host context: argument blocks that
// are passed to kernels BY VALUE (so a launch records everything it needs and
// nothing has to be uploaded first), and the layout of the device workspace.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>

#include "a2a.h"

namespace a2a {

constexpr int kWave = 64;
// Entries ((token, k) pairs) handled by one routing workgroup; one entry per
// thread, so block-local ranks fit in 16 bits.
constexpr int kRouteBlock = 1024;
constexpr uint32_t kInvalidSlot = 0xFFFFFFFFu;
constexpr int kMaxWorld = A2A_MAX_WORLD_SIZE;

// Device workspace, shared by all logical ranks of a context.  Per-rank arrays
// are laid out [world][...] with the strides below.
struct Workspace {
    uint16_t *local_rank;      // [N][max_tk]    rank of an entry among equal experts inside its routing block
    uint32_t *block_hist;      // [N][nb_max][E] per-chunk histogram of a source's entries
    uint32_t *block_prefix;    // [N][nb_max][E] its exclusive prefix over chunks
    uint32_t *num_routed;      // [N][E]         routes per (source, expert)
    uint32_t *expert_offsets;  // [N][E]         inclusive scan of num_routed over experts
    uint32_t *slot_base;       // [N][E]         first receiver row of (source, expert)
    uint32_t *tokens_per_expert;  // [E]         per receiver-local expert, summed over sources
    uint32_t *padded_offset;   // [E]            first row of an expert inside its receiver
    uint32_t *route_slot;      // [N][max_tk]    receiver row of every copy (kInvalidSlot if dropped); after the sends of
                               //                the split calls: the copy's position in its sender's expert-sorted order
    uint32_t *token_offset;    // [N][max_tk]    rank of every copy inside its (source, expert)
    uint32_t *err;             // [1]            A2A_DEV_* bits, sticky
    const uint32_t *order;     // [N][8] words   byte i of receiver r's row: the i-th source it lays out
    const uint32_t *laid_before; // [N][G]       bit s of word [r][g]: receiver r lays out source s before source g
    uint32_t *chunk_counts;    // [N][E][nb_max] block_hist with the chunks of an expert side by side (large group steps)
    uint32_t *totals;          // [2][(G+1)*E]   counts of a step per expert and source ([E][G]), then per expert ([E]),
                               //                accumulated by the routing launch of large group steps; two copies
                               //                used in turn
    uint32_t *turn;            // [2]            [0] copy the next routing launch fills, [1] copy the current step uses
    uint32_t *send_totals;     // [2][E + N]     the same for the send of a split call: counts of ONE source per expert,
                               //                then per owning rank; two copies used in turn
    uint32_t *send_turn;       // [2]            as `turn`, for send_totals
    uint32_t max_tk;           // max_num_tokens * K
    uint32_t nb_max;           // ceil(max_tk / kRouteBlock)
    uint32_t world;            // N logical ranks (receivers)
    uint32_t num_groups;       // G = N / dp_size: groups of ranks that hold the same tokens (sources)
    uint32_t dp_size;          // ranks per group
    uint32_t num_experts;      // E
    uint32_t topk;             // K
    uint32_t experts_per_rank; // Le = ceil(E / N)
    uint32_t node_size;
    uint32_t expert_padding;
    uint32_t le_magic;         // ceil(2^32 / Le) (0 for Le = 1): e / Le = mulhi(e, le_magic) for every expert id
};

struct RouteSrc {
    const int32_t *indices;
    const int32_t *bound_m;
    uint32_t indices_stride;
    uint32_t num_tokens;
};

struct FinalizeArgs {
    int32_t *out_num_tokens[kMaxWorld];   // per receiver, may be null
    uint32_t out_rows[kMaxWorld];         // rows of the receiver's buffer (overflow check)
    uint32_t num_blocks[kMaxWorld];       // routing blocks written per source by the route launch
    uint32_t fold_mask;                   // sources whose block histograms are folded by this launch
    uint32_t valid_mask;                  // sources that count for the layout (others count as empty)
    uint32_t recv_mask;                   // receivers whose layout is computed by this launch
};

struct RouteArgs {
    RouteSrc src[kMaxWorld];
    uint32_t block_start[kMaxWorld + 1];  // first routing block of each source in the grid
};


struct PushSrc {
    const uint8_t *x;
    const float *x_scale;
    const int32_t *indices;
    const int32_t *bound_m;
    uint64_t x_stride;        // bytes
    uint32_t xs_stride_elem;  // elements
    uint32_t xs_stride_token;
    uint32_t indices_stride;
    uint32_t num_tokens;
};

struct PushDst {
    uint8_t *out_x;
    float *out_scale;
    uint64_t out_stride;      // bytes
    uint32_t os_stride_elem;  // elements
    uint32_t os_stride_token;
    uint32_t out_rows;
    uint32_t pad_;
};

struct PushArgs {
    PushSrc src[kMaxWorld];
    PushDst dst[kMaxWorld];
    uint32_t token_start[kMaxWorld + 1];  // first workgroup (token) of each source in the grid
    uint32_t row_bytes;                   // bytes of a dispatched row
    uint32_t hidden_dim;
    uint32_t hidden_dim_scale;
    uint32_t topk_magic;                  // ceil(2^32 / K) (0 for K = 1): n / K = mulhi(n, magic) while n * K < 2^32
    uint32_t single_source;               // set by the launchers.  One-launch dispatches: g + 1 when source g alone has
                                          // tokens and its index rows are dense, else 0.  Resolving pack: g + 1
                                          // when source g alone has tokens.
    PushSrc single;                       // a copy of src[single_source - 1]: at a fixed place in the argument block, so
                                          // that a kernel reaches the token rows and index rows of the one source
                                          // without first loading which source it is (a dependent trip at the head
                                          // of every workgroup: 0.3 us of the 128-token step)
};

struct CombSrc {  // one per receiver rank: the expert outputs it holds
    const uint8_t *y;
    uint64_t y_stride;        // bytes
    uint32_t y_rows;
    uint32_t pad_;
};

struct CombDst {  // one per rank: where its combined tokens go
    uint8_t *out;
    const int32_t *indices;
    const float *weights;
    const int32_t *bound_m;
    uint64_t out_stride;      // bytes
    uint32_t indices_stride;
    uint32_t weights_stride;
    uint32_t num_tokens;
    uint32_t pad_;
};

struct CombArgs {
    CombSrc src[kMaxWorld];
    CombDst dst[kMaxWorld];
    uint32_t token_start[kMaxWorld + 1];
    uint32_t hidden_dim;
    uint32_t accumulate;
    // Split calls: rows are read from a staging buffer at the sender's own
    // positions (exclusive expert offset + token offset) instead of from the
    // receivers' expert_y at route_slot.  Null for the group call.
    const uint8_t *staged_base;
    uint64_t staged_stride;
    // r + 1 when rank r alone has tokens to combine (0 otherwise), and a copy of dst[r] at a fixed place
    // (set by the launcher; see PushArgs::single).
    uint32_t single_rank;
    uint32_t pad_;
    CombDst single;
};

// Events a caller wants recorded when a kernel itself begins and ends (both
// null: an ordinary launch).
struct KernelTiming {
    hipEvent_t start = nullptr;
    hipEvent_t stop = nullptr;
};

// Launchers (defined next to their kernels); all return the hipError_t of the
// launch.
hipError_t launch_route(const RouteArgs &args, const Workspace &ws, uint32_t total_blocks,
                        hipStream_t stream);
// The same, and every chunk adds its counts to the step's totals (large group steps), or to
// the totals of the one source of a split send (`for_send`).
hipError_t launch_route_accumulate(const RouteArgs &args, const Workspace &ws, uint32_t total_blocks,
                                   hipStream_t stream, bool for_send = false,
                                   KernelTiming timing = KernelTiming());
// Pack that resolves its rows from the chunk histograms and the step's totals, with the
// receiver layout and the per-source tables computed by extra workgroups of the same launch.
hipError_t launch_dispatch_resolve(const PushArgs &args, const FinalizeArgs &fin, const Workspace &ws,
                                   bool quantize, uint32_t total_tokens, hipStream_t stream,
                                   KernelTiming timing = KernelTiming());
hipError_t launch_finalize(const FinalizeArgs &args, const Workspace &ws, hipStream_t stream);
hipError_t launch_route_fused(const RouteArgs &args, const FinalizeArgs &fin, const Workspace &ws,
                              hipStream_t stream);
hipError_t launch_dispatch_push(const PushArgs &args, const Workspace &ws, bool quantize,
                                uint32_t total_tokens, hipStream_t stream, KernelTiming timing = KernelTiming());
// One-launch routing + pack for small steps: whether a step qualifies, and the launch.
constexpr uint32_t kSmallMaxEntries = 8192;
constexpr uint32_t kSmallMaxVisits = 3u << 19;   // entries x tokens
bool dispatch_small_fits(const PushArgs &args, const Workspace &ws, bool quantize, uint32_t total_tokens);
hipError_t launch_dispatch_small(const PushArgs &args, const FinalizeArgs &fin, const Workspace &ws,
                                 bool quantize, uint32_t total_tokens, hipStream_t stream,
                                 KernelTiming timing = KernelTiming());
// One-launch routing + pack for steps of one source with dense index rows that are too large for
// the small-step kernel.
constexpr uint32_t kSingleMaxEntries = 8192;
bool dispatch_single_fits(const PushArgs &args, const Workspace &ws, bool quantize, uint32_t total_tokens);
hipError_t launch_dispatch_single(const PushArgs &args, const FinalizeArgs &fin, const Workspace &ws,
                                  bool quantize, uint32_t total_tokens, hipStream_t stream,
                                  KernelTiming timing = KernelTiming());
hipError_t launch_combine_gather(const CombArgs &args, const Workspace &ws, uint32_t in_dtype,
                                 uint32_t out_dtype, uint32_t total_tokens, hipStream_t stream,
                                 KernelTiming timing = KernelTiming());

// Makes a value from the argument block count as used where this stands, so that the scalar loads of
// all such values at the head of a kernel go out together and are waited for once.  Left to itself
// the compiler asks for each value where it is first needed, stage after stage, and a latency-bound
// kernel pays a round trip to the scalar cache per stage (measured on the steps of 128 to 1024
// tokens: 0.1-0.3 us per kernel).
#define A2A_PIN(x) asm volatile("" ::"s"(x))

// Device-side: effective token count of a source (bound_m clamps num_tokens,
// a2a_dispatch_send.cu:172).
__device__ __forceinline__ uint32_t effective_tokens(const int32_t *bound_m, uint32_t num_tokens) {
    if (bound_m == nullptr) return num_tokens;
    int32_t b = *bound_m;
    if (b < 0) b = 0;
    return (uint32_t)b < num_tokens ? (uint32_t)b : num_tokens;
}

// i-th source (dp group) that receiver `rank` lays out (a2a_worker.rs:681-694):
// the groups of the other nodes starting at the next node, then the other
// groups of the own node starting after the own group, then the own group.
__host__ __device__ __forceinline__ uint32_t source_order(uint32_t rank, uint32_t i, uint32_t world,
                                                          uint32_t node_size, uint32_t dp_size) {
    const uint32_t num_nodes = world / node_size;
    const uint32_t groups_per_node = node_size / dp_size;
    const uint32_t rank_node = rank / node_size;
    const uint32_t dp_group = rank / dp_size;
    const uint32_t remote = (num_nodes - 1) * groups_per_node;
    if (i < remote) {
        const uint32_t node = (rank_node + 1 + i / groups_per_node) % num_nodes;
        return node * groups_per_node + i % groups_per_node;
    }
    const uint32_t local = i - remote + 1;  // 1 .. groups_per_node
    if (local < groups_per_node) return rank_node * groups_per_node + (dp_group + local) % groups_per_node;
    return dp_group;
}


// Rank that owns expert `e` (e < num_experts), without a division.
__device__ __forceinline__ uint32_t owner_of_expert(const Workspace &ws, uint32_t e) {
    return ws.experts_per_rank > 1 ? __umulhi(e, ws.le_magic) : e;
}

// The same order from the table the context computes once (kMaxWorld bytes per
// receiver, four to a word).  With a uniform `rank` and `i` the loads are scalar.
__device__ __forceinline__ uint32_t source_order_lookup(const uint32_t *order, uint32_t rank, uint32_t i) {
    return order[rank * (kMaxWorld / 4) + (i >> 2)] >> (8 * (i & 3)) & 0xFFu;
}

}  // namespace a2a
