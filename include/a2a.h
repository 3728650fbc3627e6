/*
 * C ABI of the MI355X (gfx950) MoE dispatch / combine library.
 *
 * The library replaces the host crate `p2p-all-to-all` of the reference and
 * the four kernel launchers under it.  One `a2a_ctx` stands for a whole
 * expert-parallel group of `world_size` LOGICAL ranks whose buffers all live
 * in the memory of one GPU (loopback): every call names the logical rank it
 * acts as.  Nothing here takes a torch type; pointers are device pointers
 * unless stated, `stream` is a `hipStream_t`.  All calls only enqueue work on
 * `stream` and never synchronise it, except `a2a_ctx_create`,
 * `a2a_ctx_destroy` and `a2a_ctx_status`.
 *
 * A context is not re-entrant (the reference's methods take `&mut self`,
 * a2a_context.rs:275,339,395,437): calls on ONE context, from whatever thread,
 * must not overlap; different contexts are independent.  Calls may be made with
 * any device current: each selects the context's device and restores the
 * caller's.
 *
 * Every function returns 0 on success, a positive `hipError_t` when a HIP call
 * failed, or a negative `a2a_status`; `a2a_last_error` gives the text.  No
 * exception crosses this boundary.
 *
 * Two ways to run a step:
 *   - the four split calls `a2a_dispatch_send / _recv`, `a2a_combine_send /
 *     _recv`, one logical rank at a time, every send of a step before the
 *     first recv of that step (the reference's call order).  Rows travel
 *     through staging buffers the context owns, as in the reference.
 *   - the two group calls `a2a_dispatch` / `a2a_combine`, which take the
 *     arguments of every rank at once (what `world_size` processes would pass
 *     "at the same time") and move every row exactly once.
 */
#ifndef A2A_MI355_H
#define A2A_MI355_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define A2A_MAX_WORLD_SIZE 32
#define A2A_MAX_EXPERTS 1024
#define A2A_MAX_EXPERTS_PER_TOKEN 64

/* Element type tags, same order as the reference's `ScalarType`
 * (rust/torch-lib/src/lib.rs:31-49). */
typedef enum a2a_scalar_type {
    A2A_BOOL = 0, A2A_I8, A2A_U8, A2A_I16, A2A_U16, A2A_I32, A2A_U32, A2A_I64,
    A2A_U64, A2A_F8_E4M3, A2A_F8_E5M2, A2A_F16, A2A_BF16, A2A_F32, A2A_F64
} a2a_scalar_type;

typedef enum a2a_status {
    A2A_OK = 0,
    A2A_ERR_INVALID_ARGUMENT = -1,
    A2A_ERR_TOO_MANY_TOKENS = -2,  /* a2a_context.rs:290-292 */
    A2A_ERR_UNSUPPORTED = -3,      /* the reference asserts: launch_utils.cuh:150-153,189-192 */
    A2A_ERR_OUT_OF_MEMORY = -4,
    A2A_ERR_BAD_ORDER = -5,        /* recv before any send, combine before dispatch */
    A2A_ERR_DEVICE_FLAG = -6       /* a kernel reported bad input, see a2a_ctx_status */
} a2a_status;

/* Bits of the device-side error word read by a2a_ctx_status. */
#define A2A_DEV_BAD_EXPERT_ID   1u  /* an index was >= num_experts; that copy was dropped */
#define A2A_DEV_RECV_OVERFLOW   2u  /* a receive buffer had too few rows; those copies were dropped */
#define A2A_DEV_BAD_SLOT        4u  /* combine met a slot outside expert_y; it contributed 0 */
#define A2A_DEV_INTERNAL        0x80000000u /* a kernel gave up waiting for its own wavefronts: the step's
                                              * results are invalid (a guard against a hang; never observed) */

typedef struct a2a_ctx a2a_ctx;

/*
 * Construction parameters: the scalar arguments of `AllToAllContext::new`
 * (p2p-all-to-all/src/a2a_context.rs:124-160) without the transport handles
 * (RDMA regions, peer pointer lists, worker CPU), which have no counterpart
 * when every rank lives on one GPU.
 */
typedef struct a2a_config {
    uint32_t struct_size;            /* sizeof(a2a_config), for versioning */
    uint32_t hidden_dim;             /* H */
    uint32_t hidden_dim_scale;       /* Hs, 0 = rows carry no scales */
    uint32_t in_elemsize;            /* bytes per element of dispatched rows (1, 2 or 4) */
    uint32_t out_elemsize;           /* bytes per element of combined rows (2 or 4) */
    uint32_t out_dtype;              /* a2a_scalar_type of out_tokens: F16, BF16 or F32 */
    uint32_t scale_elemsize;         /* 0 or 4 */
    uint32_t max_num_tokens;         /* per rank and step */
    uint32_t max_recv_tokens;        /* rows of a rank's staging region */
    uint32_t max_private_tokens;     /* rows per source in the private part of a receive region: moves no row
                                        in loopback, but the offset tables of a2a_dispatch_recv encode it */
    uint32_t num_experts;            /* E <= A2A_MAX_EXPERTS */
    uint32_t expert_padding;         /* each expert's slot range is rounded up to this */
    uint32_t num_experts_per_token;  /* K <= A2A_MAX_EXPERTS_PER_TOKEN */
    uint32_t dp_size;                /* ranks per group that hold the same tokens; divides node_size */
    uint32_t node_size;              /* ranks per node; fixes the order of sources in a receiver */
    uint32_t world_size;             /* N <= A2A_MAX_WORLD_SIZE, divisible by node_size */
    int32_t  device;                 /* HIP device ordinal */
    uint32_t flags;                  /* A2A_FLAG_* */
} a2a_config;

/* Allocate the staging buffers of the split calls in a2a_ctx_create instead of
 * on their first use. */
#define A2A_FLAG_PREALLOC_STAGING 1u
/* Never take the one-launch paths (routing counted inside the dispatch or send
 * kernel: small steps, and group steps of one source up to 8192 copies); always
 * run the routing kernels, then the pack.  Results are identical either way;
 * the flag exists to compare the two. */
#define A2A_FLAG_SEPARATE_ROUTING 2u

/* replaces AllToAllContext::new, a2a_context.rs:124-259 */
int a2a_ctx_create(const a2a_config *config, a2a_ctx **out_ctx);

/* replaces AllToAllContext::destroy / Drop, a2a_context.rs:261-272,490-494 */
int a2a_ctx_destroy(a2a_ctx *ctx);

/* Text of the last error of this context (never NULL).  With ctx == NULL:
 * the last error of a2a_ctx_create or a2a_dispatch_static on this thread. */
const char *a2a_last_error(const a2a_ctx *ctx);

/* Synchronises `stream`, then reads and clears the device-side error word
 * (A2A_DEV_* bits) into *flags.  The counterpart of the reference's sticky
 * transport error (a2a_context.rs:332-334). */
int a2a_ctx_status(a2a_ctx *ctx, void *stream, uint32_t *flags);

/*
 * replaces AllToAllContext::dispatch_send, a2a_context.rs:275-336 (kernel
 * a2a_dispatch_send.cu:112-536).  Counts rank `rank`'s routes per expert,
 * ranks every copy inside its expert (ascending token, then k), scans the
 * offsets, and stages the rows of its tokens.
 *   x_ptr/x_stride        rows of the tokens, stride in BYTES
 *   quantize              0: rows are in_elemsize-wide elements, copied as
 *                            bytes together with x_scale;
 *                         1: rows are bf16; they are quantised to fp8 e4m3 with
 *                            one float scale per 128 elements (needs
 *                            in_elemsize 1, hidden_dim_scale = hidden_dim/128,
 *                            x_scale_ptr NULL).  Per group of 128: amax =
 *                            max(max|x|, 1e-4), scale = amax / 448, code =
 *                            e4m3(x * (448 / amax)), round to nearest even.  A NaN
 *                            in a group makes its scale NaN and its 128 codes
 *                            0x7F; an infinity makes its scale +inf, the code of
 *                            an infinite value 0x7F, of a finite one a signed zero
 *   x_scale_*             optional float scales [T, Hs], strides in ELEMENTS
 *   indices               [T, K] expert ids, row stride in elements
 *   weights               unused by dispatch, as in the reference
 *   bound_m               optional device int32: number of valid tokens
 */
int a2a_dispatch_send(a2a_ctx *ctx, uint32_t rank, size_t num_tokens,
                      const void *x_ptr, size_t x_stride, uint32_t quantize,
                      const float *x_scale_ptr, size_t x_scale_stride_elem,
                      size_t x_scale_stride_token, const int32_t *indices,
                      size_t indices_stride, const float *weights,
                      size_t weights_stride, const int32_t *bound_m,
                      void *stream);

/*
 * replaces AllToAllContext::dispatch_recv, a2a_context.rs:339-388 (kernel
 * a2a_dispatch_recv.cu:16-236) and the receiver half of the host worker's
 * `process_routing_info` (a2a_worker.rs:526-703).  Lays out the rows that the
 * sends of this step routed to `rank` and copies them into out_x / out_x_scale;
 * writes the per-local-expert counts.  `out_x_rows` (rows of out_x) is an
 * addition: copies that would land beyond it are dropped and flagged.
 * The first recv of a step also enqueues, in front of its own copy, the layout
 * of EVERY receiver (once per step, as the reference's worker runs once per
 * rank and step): the recvs of the other ranks must be ordered after it, as
 * they must be ordered after the sends (same stream, or events).
 */
int a2a_dispatch_recv(a2a_ctx *ctx, uint32_t rank, int32_t *out_num_tokens,
                      void *out_x, size_t out_x_stride, size_t out_x_rows,
                      float *out_x_scale, size_t out_x_scale_stride_elem,
                      size_t out_x_scale_stride_token, void *stream);

/*
 * replaces AllToAllContext::combine_send, a2a_context.rs:395-430 (kernel
 * a2a_combine_send.cu:20-235): copies every received row of expert_y back to
 * the staging row of the copy it answers.  `expert_y_rows` is an addition
 * (bounds check).  Stride in BYTES.
 */
int a2a_combine_send(a2a_ctx *ctx, uint32_t rank, const void *expert_y,
                     size_t expert_y_stride, size_t expert_y_rows,
                     void *stream);

/*
 * replaces AllToAllContext::combine_recv, a2a_context.rs:437-487 (kernel
 * a2a_combine_recv.cu:20-167): out[t] = (accumulate ? out[t] : 0) +
 * sum_k weights[t,k] * y(t,k), float accumulation, k ascending.
 * out_tokens_stride is in ELEMENTS, as in the reference.
 */
int a2a_combine_recv(a2a_ctx *ctx, uint32_t rank, size_t num_tokens,
                     size_t num_recv_tokens, uint32_t expert_y_dtype,
                     void *out_tokens, size_t out_tokens_stride,
                     const int32_t *indices, size_t indices_stride,
                     const float *weights, size_t weights_stride,
                     const int32_t *bound_m, uint32_t accumulate, void *stream);

/* Arguments of one rank for the group calls: both halves of its dispatch(). */
typedef struct a2a_dispatch_args {
    /* send half, as a2a_dispatch_send */
    uint64_t num_tokens;
    const void *x_ptr;
    uint64_t x_stride;
    const float *x_scale_ptr;
    uint64_t x_scale_stride_elem;
    uint64_t x_scale_stride_token;
    const int32_t *indices;
    uint64_t indices_stride;
    const float *weights;
    uint64_t weights_stride;
    const int32_t *bound_m;
    /* recv half, as a2a_dispatch_recv */
    int32_t *out_num_tokens;
    void *out_x;
    uint64_t out_x_stride;
    uint64_t out_x_rows;
    float *out_x_scale;
    uint64_t out_x_scale_stride_elem;
    uint64_t out_x_scale_stride_token;
} a2a_dispatch_args;

/* Arguments of one rank for a2a_combine: both halves of its combine(). */
typedef struct a2a_combine_args {
    /* send half, as a2a_combine_send */
    const void *expert_y;
    uint64_t expert_y_stride;
    uint64_t expert_y_rows;
    /* recv half, as a2a_combine_recv */
    uint64_t num_tokens;
    void *out_tokens;
    uint64_t out_tokens_stride;
    const int32_t *indices;
    uint64_t indices_stride;
    const float *weights;
    uint64_t weights_stride;
    const int32_t *bound_m;
} a2a_combine_args;

/*
 * dispatch() of all `world_size` ranks in one call: `args[r]` is what rank r
 * would pass to a2a_dispatch_send followed by a2a_dispatch_recv
 * (python/pplx_garden/kernels/p2p_all_to_all.py:317-440 with do_send and
 * do_recv).  Same results as the split calls; every token row is read once
 * and every copy is written once, straight into the receiver's out_x.
 * A rank that sends nothing passes num_tokens 0.  With dp_size > 1 the ranks of
 * a group pass the same tokens and routing (a2a_dispatch_send.cu:304,508): the
 * send half of the group's first rank is the one that is read.
 */
int a2a_dispatch(a2a_ctx *ctx, const a2a_dispatch_args *args, uint32_t quantize,
                 void *stream);

/*
 * a2a_dispatch without a context and without any allocation.  No counterpart in
 * the reference; it is for callers that cannot allocate device memory where they
 * run a step: code under HIP graph capture, serving loops and harnesses that
 * forbid hipMalloc.  Same arguments and same results as a2a_dispatch on a context
 * created from `config` (its `flags` must be 0), but the routing tables of the
 * step live in a fixed array of A2A_STATIC_SCRATCH_BYTES inside the library
 * (every GPU the library is used on holds one copy until the process ends) and
 * the call neither allocates nor frees nor copies: it enqueues one small kernel
 * that prepares the tables, then the launches of a2a_dispatch.
 *   - The tables are sized for THIS step (largest `num_tokens` among the ranks);
 *     a step whose tables exceed the array is refused with
 *     A2A_ERR_TOO_MANY_TOKENS and a message that names the sizes.  The DeepSeek-V3
 *     prefill step with all 8 ranks sending 4096 tokens needs 3.4 MB.
 *   - All calls on one GPU share the array: calls whose kernels could overlap
 *     (different streams, no ordering between them) race.  Calls on one stream,
 *     or ordered by events, are fine; each call clears what it needs cleared.
 *   - `device_flags`: optional DEVICE pointer to one uint32 that the kernels OR
 *     the A2A_DEV_* bits into (the caller clears it); with NULL bad input is
 *     dropped silently as described at those bits.
 *   - The first call on a GPU also looks up where that GPU holds the array
 *     (hipGetSymbolAddress, once per device): make one call outside any
 *     stream capture before capturing calls into a graph.  A first call on a
 *     stream that is being captured is refused with A2A_ERR_BAD_ORDER.
 *   - A refused call enqueues nothing: every check of the step runs before the
 *     first launch.
 *   - The routing of the step stays inside the library: a2a_combine needs a
 *     context and the a2a_dispatch that goes with it.
 * Error text: a2a_last_error(NULL) on the calling thread.
 */
#define A2A_STATIC_SCRATCH_BYTES (8u << 20)
int a2a_dispatch_static(const a2a_config *config, const a2a_dispatch_args *args,
                        uint32_t quantize, uint32_t *device_flags, void *stream);

/*
 * combine() of all ranks in one call (p2p_all_to_all.py:442-517 with do_send
 * and do_recv); uses the routing of the last a2a_dispatch.  expert_y rows are
 * read in place: no staging copy.
 */
int a2a_combine(a2a_ctx *ctx, const a2a_combine_args *args,
                uint32_t expert_y_dtype, uint32_t accumulate, void *stream);

/*
 * Introspection for parity tests; `which` selects a routing table of the last
 * dispatch of `rank`.  Synchronises `stream` and copies `count` uint32 to the
 * HOST buffer `out`.  No counterpart in the reference, whose tables are private
 * (a2a_context.rs:15-32, a2a_worker.rs:146-151).
 */
typedef enum a2a_table {
    A2A_TABLE_NUM_ROUTED = 0,       /* [E]   count per expert (a2a_dispatch_send.cu:199-204) */
    A2A_TABLE_EXPERT_OFFSETS = 1,   /* [E]   inclusive scan (a2a_dispatch_send.cu:236-242) */
    A2A_TABLE_TOKEN_OFFSET = 2,     /* [T*K] rank of a copy inside its expert (a2a_dispatch_send.cu:189) */
    A2A_TABLE_SLOT = 3,             /* [T*K] receiver row of a copy */
    A2A_TABLE_PADDED_INDEX = 4,     /* [num_recv] a2a_worker.rs:669-671 (split calls only) */
    A2A_TABLE_SOURCE_RANK = 5,      /* [num_recv] a2a_worker.rs:668 (split calls only) */
    A2A_TABLE_SOURCE_POSITION = 6,  /* [num_recv] row in the sender's expert-sorted order (split calls only) */
    A2A_TABLE_NUM_RECV_TOKENS = 7,  /* [2] rows received, rows from other nodes (split calls only) */
    A2A_TABLE_SOURCE_DISPATCH_OFFSET = 8,  /* [num_recv] a2a_worker.rs:636-656: private-region row,
                                              sender's position with bit 31 set (same node), or
                                              overflow-region row (split calls only) */
    A2A_TABLE_COMBINE_SEND_OFFSET = 9      /* [num_recv] a2a_worker.rs:659-667 (split calls only) */
} a2a_table;

int a2a_ctx_read_table(a2a_ctx *ctx, uint32_t rank, uint32_t which,
                       uint32_t *out, size_t count, void *stream);

/* Measuring aid, no counterpart in the reference.  The next call on this context
 * that launches the named kernel launches it so that `start_event` and
 * `stop_event` (hipEvent_t, created by the caller with timing enabled) are
 * recorded when the kernel itself begins and ends; hipEventElapsedTime between
 * them is the kernel's duration, without the queue packets and idle time that
 * events recorded around a call add.
 *   A2A_KERNEL_PACK          the pack of the next a2a_dispatch
 *   A2A_KERNEL_ROUTE         the routing launch that precedes the pack of a large
 *                            step (a2a_dispatch) or the staging of a large send
 *                            (a2a_dispatch_send); a step that counts its routing
 *                            inside the pack or the staging launch (a small one,
 *                            or one source alone with up to 8192 copies) or runs
 *                            several routing kernels (A2A_FLAG_SEPARATE_ROUTING)
 *                            has no such launch and leaves those events alone
 *   A2A_KERNEL_GATHER        the gather of the next a2a_combine or a2a_combine_recv
 *   A2A_KERNEL_STAGE_SEND    the staging launch of the next a2a_dispatch_send
 *   A2A_KERNEL_STAGE_RECV    the copy launch of the next a2a_dispatch_recv
 *   A2A_KERNEL_COMBINE_SEND  the copy launch of the next a2a_combine_send
 * One-shot: the request is consumed by that call (a call that launches nothing,
 * such as a send without tokens, consumes it too).  Pass two nulls to withdraw
 * it.  The stop event must have completed before its time is read (synchronise
 * the stream or the event). */
enum {
    A2A_KERNEL_PACK = 0, A2A_KERNEL_GATHER = 1, A2A_KERNEL_ROUTE = 2,
    A2A_KERNEL_STAGE_SEND = 3, A2A_KERNEL_STAGE_RECV = 4, A2A_KERNEL_COMBINE_SEND = 5
};
int a2a_ctx_time_next_kernel(a2a_ctx *ctx, uint32_t which, void *start_event, void *stop_event);

/* Row strides of the staging buffers (a2a_worker.rs:317-325). */
size_t a2a_dispatch_token_stride(const a2a_config *config);
size_t a2a_combine_token_stride(const a2a_config *config);

/* Library version, "major.minor". */
const char *a2a_version(void);

#ifdef __cplusplus
}
#endif
#endif /* A2A_MI355_H */
