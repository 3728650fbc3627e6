// Staging buffers and kernels of the split calls (one logical rank per call).
//
// They keep the reference's structure: a send stages the rows of its tokens
// (a2a_dispatch_send.cu:341-367), a recv lays out what it received and copies
// it into the caller's buffers (a2a_worker.rs:526-703 on the CPU there, then
// a2a_dispatch_recv.cu:122-156), combine-send copies expert rows back to the
// staging row of the copy they answer (a2a_combine_send.cu:119-138,182-207)
// and combine-recv gathers them (a2a_combine_recv.cu:94-148).
//
// Differences that follow from every rank living in one HBM: a token is staged
// ONCE (quantised), not once per route, and the receiver finds it through a
// position -> token table; the private / overflow split of the receive buffer
// (max_private_tokens) moves no row here, but the recv still writes the two
// offset tables that encode it (source_dispatch_offset, combine_send_offset),
// bit for bit what the reference's host worker computes.
#pragma once

#include <string>

#include "a2a_internal.h"

namespace a2a {

struct Staging {
    bool allocated = false;
    void *arena = nullptr;
    uint8_t *send_buf = nullptr;         // [N][max_num_tokens][disp_stride]: payload, scales, 16 spare bytes (+ padding to whole lines)
    uint32_t *pos_token = nullptr;       // [N][max_tk]: token behind each row of a sender's expert-sorted order
                                         // (the other way round, copy -> position, is in the workspace's route_slot)
    uint8_t *comb_buf = nullptr;         // [N][max_tk][comb_stride]: combine rows at the sender's positions
    uint32_t *padded_index = nullptr;    // [N][max_recv]
    uint32_t *source_rank = nullptr;     // [N][max_recv]
    uint32_t *source_position = nullptr; // [N][max_recv]
    uint32_t *source_dispatch_offset = nullptr;  // [N][max_recv]  a2a_worker.rs:636-656
    uint32_t *combine_send_offset = nullptr;     // [N][max_recv]  a2a_worker.rs:659-667
    uint32_t *source_row = nullptr;      // [N][max_recv]: staged row a received row is copied from (sender * max_tokens + token)
    uint32_t *num_recv = nullptr;        // [N][2]: received rows, rows from other nodes
    size_t disp_stride = 0;
    size_t comb_stride = 0;
    uint32_t payload_bytes = 0;          // offset of the scales inside a staged dispatch row
    uint32_t max_recv = 0;               // rows per receiver in the tables above
    uint32_t max_tokens = 0;
    uint32_t recv_mask = 0;              // receivers whose tables are valid in this step
    uint32_t combine_sent_mask = 0;
};

struct StageSendArgs {
    PushSrc src;
    uint32_t rank;
    uint32_t row_bytes;
    uint32_t hidden_dim;
    uint32_t hidden_dim_scale;
    uint32_t topk_magic;      // ceil(2^32 / K) (0 for K = 1), for entry -> token without a division
    uint32_t resolver_wave;   // resolving send: wavefront that resolves the routes (set by the launcher)
};

struct StageRecvArgs {
    PushDst dst;
    int32_t *out_num_tokens;  // rows per local expert for the caller, may be null
    uint32_t rank;
    uint32_t row_bytes;
    uint32_t hidden_dim_scale;
    uint32_t max_rows;        // upper bound of received rows known to the host
    uint32_t team_waves;      // wavefronts that share a row (set by the launcher)
    // the first recv of a step only: it lays out every receiver
    uint32_t valid_mask;      // sources that sent tokens in this step (the others count as empty)
    uint32_t max_private;     // rows per source in the private part of a receive region (a2a_worker.rs:646-656)
    uint32_t copy_blocks;     // workgroups that serve the caller's rank; the others lay out the other receivers (launcher)
    uint32_t slices;          // workgroups per other receiver (set by the launcher)
};

struct CombineSendArgs {
    const uint8_t *y;
    uint64_t y_stride;
    uint32_t y_rows;
    uint32_t rank;
    uint32_t row_bytes;
    uint32_t max_rows;
    uint32_t team_waves;      // wavefronts that share a row (set by the launcher)
};

struct CombineRecvArgs {
    CombDst dst;
    uint32_t rank;
    uint32_t hidden_dim;
    uint32_t accumulate;
};

int staging_allocate(Staging &st, const a2a_config &cfg, std::string *error);
void staging_free(Staging &st);
// Device pointer of a receive-side table of `rank`, or null when none exists.
const uint32_t *staging_table(const Staging &st, const a2a_config &cfg, uint32_t rank, uint32_t which,
                              size_t *limit);

hipError_t launch_stage_send(const StageSendArgs &args, const Workspace &ws, const Staging &st,
                             bool quantize, hipStream_t stream, KernelTiming timing = KernelTiming());
// One-launch send (routing counted inside) for small steps: whether a step qualifies, and the launch
// (dense index rows and a wavefront to spare: the kernel in which a spare wavefront resolves the
// positions while the others stage the row; otherwise the one in which every wavefront does both).
bool stage_send_small_fits(const StageSendArgs &args, const Workspace &ws);
hipError_t launch_stage_send_small(const StageSendArgs &args, const Workspace &ws, const Staging &st,
                                   bool quantize, hipStream_t stream, KernelTiming timing = KernelTiming());
// One-launch send for steps of up to 8192 entries that are too large for the small-step kernel
// (a workgroup counts once for several tokens): whether a step qualifies, and the launch (with a
// wavefront to spare, again the kernel in which it resolves the positions beside the teams).
bool stage_send_single_fits(const StageSendArgs &args, const Workspace &ws, bool quantize);
hipError_t launch_stage_send_single(const StageSendArgs &args, const Workspace &ws, const Staging &st,
                                    bool quantize, hipStream_t stream, KernelTiming timing = KernelTiming());
// The send of a large step after launch_route_accumulate(..., for_send = true).
hipError_t launch_stage_send_resolve(const StageSendArgs &args, const Workspace &ws, const Staging &st,
                                     bool quantize, hipStream_t stream, KernelTiming timing = KernelTiming());
// `first_of_step`: no recv has run since the step's sends; this launch also lays out the other receivers.
// Steps with few rows (a workgroup per row) take kernels of their own, here and in the combine-send.
hipError_t launch_stage_recv(const StageRecvArgs &args, const Workspace &ws, const Staging &st, bool first_of_step,
                             hipStream_t stream, KernelTiming timing = KernelTiming());
hipError_t launch_combine_send(const CombineSendArgs &args, const Workspace &ws, const Staging &st,
                               hipStream_t stream, KernelTiming timing = KernelTiming());
hipError_t launch_combine_recv(const CombineRecvArgs &args, const Workspace &ws, const Staging &st,
                               uint32_t in_dtype, uint32_t out_dtype, hipStream_t stream,
                               KernelTiming timing = KernelTiming());

}  // namespace a2a
