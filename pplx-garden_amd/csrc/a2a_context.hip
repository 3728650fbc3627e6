// Host side of the library: the context object and the C ABI.
//
// Stands in for the reference's Rust crate `p2p-all-to-all`
// (p2p-all-to-all/src/a2a_context.rs): it owns the device workspace
// (DeviceWorkspace, a2a_context.rs:15-97), checks arguments, and turns each
// call into kernel launches on the caller's stream.  The reference's host
// worker thread, its GDRCopy flags and RDMA submissions have no counterpart:
// with every logical rank on one GPU, stream order is the only synchronisation.
#include <hip/hip_runtime.h>

#include <dlfcn.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "a2a_internal.h"
#include "a2a_staged.h"

using namespace a2a;

struct a2a_ctx {
    a2a_config cfg;
    Workspace ws;
    void *arena = nullptr;
    size_t arena_bytes = 0;
    std::string error;
    // A HIP call failed on this context (a launch, a copy): what was enqueued before it may have
    // left the routing tables half updated (the two copies of the step totals are handed over by
    // the launch that consumes them), so every later step would be wrong without saying so.
    // The context refuses further work; destroy it.
    bool poisoned = false;
    std::string first_failure;

    // State of the current step.
    uint32_t sent_mask = 0;        // split calls: ranks whose dispatch_send ran in this step
    uint32_t empty_mask = 0;       // split calls: those of them that sent no tokens (no launch, tables untouched)
    bool step_open = false;        // split calls: a send has run and no recv yet closed the step
    bool recv_seen = false;        // split calls: a recv has run in this step
    bool group_routing = false;    // the last dispatch was a group call (route_slot is valid)
    uint32_t num_tokens[kMaxWorld] = {};  // tokens of each rank in the last dispatch
    uint32_t quantized = 0;        // mode of the last dispatch

    Staging staging;               // buffers and tables of the split calls

    KernelTiming timing[6];        // one-shot events for the next launch of each kernel a2a_ctx_time_next_kernel names
};

// Device memory of a2a_dispatch_static: the routing tables of ONE step, in a
// file-scope array instead of an allocation.  Every GPU the library runs on
// holds its own copy at its own address until the process ends.  In host code
// this name only stands for the symbol: the address kernels get is the one
// hipGetSymbolAddress returns with that GPU current (static_scratch_of).
static __device__ __align__(256) unsigned char scratch[A2A_STATIC_SCRATCH_BYTES];

namespace {

thread_local std::string g_create_error;

int fail(a2a_ctx *ctx, int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    if (ctx != nullptr) {
        ctx->error = buf;
    } else {
        g_create_error = buf;
    }
    return code;
}

int hip_fail(a2a_ctx *ctx, hipError_t e, const char *what) {
    const int rc = fail(ctx, (int)e, "%s: %s", what, hipGetErrorString(e));
    if (ctx != nullptr && !ctx->poisoned) {
        ctx->poisoned = true;
        ctx->first_failure = ctx->error;
    }
    return rc;
}

// Entry check of every call that enqueues work on a context.
int check_usable(a2a_ctx *ctx) {
    if (!ctx->poisoned) return A2A_OK;
    return fail(ctx, A2A_ERR_BAD_ORDER, "this context is unusable after an earlier failure (%s): destroy it",
                ctx->first_failure.c_str());
}

size_t align_up(size_t n, size_t a) { return (n + a - 1) / a * a; }

// Named ranges for profilers around each call (`rocprofv3 --marker-trace`), with the names of the
// reference's NVTX ranges (a2a_dispatch_send.cu:632, a2a_dispatch_recv.cu:316,
// a2a_combine_send.cu:286, a2a_combine_recv.cu:236).  The ROCTX library is looked up at run time,
// once: without it the library has no dependency on it and a range is two null checks.
struct Roctx {
    int (*push)(const char *) = nullptr;
    int (*pop)() = nullptr;
    Roctx() {
        for (const char *name : {"librocprofiler-sdk-roctx.so.1", "librocprofiler-sdk-roctx.so", "libroctx64.so.4",
                                 "libroctx64.so"}) {
            void *lib = dlopen(name, RTLD_NOW | RTLD_LOCAL);
            if (lib == nullptr) continue;
            push = reinterpret_cast<int (*)(const char *)>(dlsym(lib, "roctxRangePushA"));
            pop = reinterpret_cast<int (*)()>(dlsym(lib, "roctxRangePop"));
            if (push != nullptr && pop != nullptr) return;
            push = nullptr;
            pop = nullptr;
            dlclose(lib);
        }
    }
};

const Roctx &roctx() {
    static const Roctx table;
    return table;
}

struct ProfilerRange {
    explicit ProfilerRange(const char *name) {
        if (roctx().push != nullptr) roctx().push(name);
    }
    ~ProfilerRange() {
        if (roctx().pop != nullptr) roctx().pop();
    }
    ProfilerRange(const ProfilerRange &) = delete;
    ProfilerRange &operator=(const ProfilerRange &) = delete;
};

uint32_t ceil_div_u32(uint64_t n, uint64_t m) { return (uint32_t)((n + m - 1) / m); }

bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

struct DeviceGuard {
    int prev = -1;
    bool ok = false;
    explicit DeviceGuard(int dev) {
        if (hipGetDevice(&prev) == hipSuccess) {
            ok = prev == dev || hipSetDevice(dev) == hipSuccess;
        }
    }
    ~DeviceGuard() {
        if (ok && prev >= 0) (void)hipSetDevice(prev);
    }
};

size_t row_bytes_of(const a2a_config &c) { return (size_t)c.hidden_dim * c.in_elemsize; }

int check_config(const a2a_config &c) {
    if (c.struct_size != sizeof(a2a_config))
        return fail(nullptr, A2A_ERR_INVALID_ARGUMENT, "a2a_config.struct_size is %u, expected %zu",
                    c.struct_size, sizeof(a2a_config));
    if (c.world_size == 0 || c.world_size > A2A_MAX_WORLD_SIZE)
        return fail(nullptr, A2A_ERR_UNSUPPORTED, "world_size %u not in [1, %d]", c.world_size,
                    A2A_MAX_WORLD_SIZE);
    if (c.node_size == 0 || c.world_size % c.node_size != 0)
        return fail(nullptr, A2A_ERR_INVALID_ARGUMENT, "node_size %u does not divide world_size %u",
                    c.node_size, c.world_size);
    if (c.dp_size == 0 || c.node_size % c.dp_size != 0)
        return fail(nullptr, A2A_ERR_INVALID_ARGUMENT, "dp_size %u does not divide node_size %u", c.dp_size,
                    c.node_size);
    if (c.num_experts == 0 || c.num_experts > A2A_MAX_EXPERTS)
        return fail(nullptr, A2A_ERR_UNSUPPORTED, "num_experts %u not in [1, %d]", c.num_experts,
                    A2A_MAX_EXPERTS);
    if (c.num_experts_per_token == 0 || c.num_experts_per_token > A2A_MAX_EXPERTS_PER_TOKEN)
        return fail(nullptr, A2A_ERR_UNSUPPORTED, "num_experts_per_token %u not in [1, %d]",
                    c.num_experts_per_token, A2A_MAX_EXPERTS_PER_TOKEN);
    if (c.expert_padding == 0)
        return fail(nullptr, A2A_ERR_INVALID_ARGUMENT, "expert_padding must be at least 1");
    if (c.hidden_dim == 0 || (c.in_elemsize != 1 && c.in_elemsize != 2 && c.in_elemsize != 4))
        return fail(nullptr, A2A_ERR_UNSUPPORTED, "hidden_dim %u / in_elemsize %u", c.hidden_dim,
                    c.in_elemsize);
    if (row_bytes_of(c) % 16 != 0)
        return fail(nullptr, A2A_ERR_UNSUPPORTED,
                    "a dispatched row of %zu bytes is not a multiple of 16 "
                    "(the reference copies 16-byte chunks too, a2a_dispatch_send.cu:341)",
                    row_bytes_of(c));
    const uint32_t od = c.out_dtype;
    if (!((od == A2A_BF16 && c.out_elemsize == 2) || (od == A2A_F16 && c.out_elemsize == 2) ||
          (od == A2A_F32 && c.out_elemsize == 4)))
        return fail(nullptr, A2A_ERR_UNSUPPORTED, "out_dtype %u with out_elemsize %u", od,
                    c.out_elemsize);
    if (c.hidden_dim % (c.out_elemsize == 4 ? 4 : 8) != 0)
        return fail(nullptr, A2A_ERR_UNSUPPORTED,
                    "hidden_dim %u is not a multiple of the combine vector width", c.hidden_dim);
    if (c.hidden_dim_scale != 0 && c.scale_elemsize != 4)
        return fail(nullptr, A2A_ERR_UNSUPPORTED, "scale_elemsize %u: scales must be float",
                    c.scale_elemsize);
    if (c.max_num_tokens == 0)
        return fail(nullptr, A2A_ERR_INVALID_ARGUMENT, "max_num_tokens must be at least 1");
    if (c.flags & ~(uint32_t)(A2A_FLAG_PREALLOC_STAGING | A2A_FLAG_SEPARATE_ROUTING))
        return fail(nullptr, A2A_ERR_INVALID_ARGUMENT, "unknown bits in flags: 0x%x", c.flags);
    if ((uint64_t)c.max_num_tokens * c.num_experts_per_token > 0x7FFFFFFFull)
        return fail(nullptr, A2A_ERR_UNSUPPORTED, "max_num_tokens * num_experts_per_token too large");
    return A2A_OK;
}

int check_rank(a2a_ctx *ctx, uint32_t rank) {
    if (rank >= ctx->cfg.world_size)
        return fail(ctx, A2A_ERR_INVALID_ARGUMENT, "rank %u out of range [0, %u)", rank,
                    ctx->cfg.world_size);
    return A2A_OK;
}

// Arguments of the send half that do not depend on who receives.
int check_send(a2a_ctx *ctx, const a2a_config &c, uint32_t rank, uint64_t num_tokens, const void *x,
               uint64_t x_stride, uint32_t quantize, const float *xs, uint64_t xs_stride_elem,
               uint64_t xs_stride_token, const int32_t *indices, uint64_t indices_stride) {
    if (num_tokens > c.max_num_tokens)
        return fail(ctx, A2A_ERR_TOO_MANY_TOKENS, "Number of tokens exceeds maximum allowed (rank %u: %llu > %u)",
                    rank, (unsigned long long)num_tokens, c.max_num_tokens);
    if (quantize > 1) return fail(ctx, A2A_ERR_INVALID_ARGUMENT, "quantize must be 0 or 1");
    if (quantize) {
        if (c.in_elemsize != 1 || c.hidden_dim % 128 != 0 || c.hidden_dim_scale != c.hidden_dim / 128 ||
            c.scale_elemsize != 4)
            return fail(ctx, A2A_ERR_UNSUPPORTED,
                        "quantise mode needs in_elemsize 1, hidden_dim %% 128 == 0 and "
                        "hidden_dim_scale == hidden_dim / 128 (got %u, %u, %u)",
                        c.in_elemsize, c.hidden_dim, c.hidden_dim_scale);
        if (c.hidden_dim_scale > 1024)
            return fail(ctx, A2A_ERR_UNSUPPORTED, "quantise mode supports hidden_dim up to 131072");
        if (xs != nullptr)
            return fail(ctx, A2A_ERR_INVALID_ARGUMENT, "quantise mode computes the scales: x_scale must be null");
    }
    if (num_tokens == 0) return A2A_OK;
    if (x == nullptr || indices == nullptr)
        return fail(ctx, A2A_ERR_INVALID_ARGUMENT, "rank %u: null x or indices with %llu tokens", rank,
                    (unsigned long long)num_tokens);
    if (!aligned16(x) || x_stride % 16 != 0)
        return fail(ctx, A2A_ERR_UNSUPPORTED, "rank %u: x rows must be 16-byte aligned", rank);
    const uint64_t need = quantize ? (uint64_t)c.hidden_dim * 2 : row_bytes_of(c);
    if (x_stride < need && num_tokens > 1)
        return fail(ctx, A2A_ERR_INVALID_ARGUMENT, "rank %u: x_stride %llu smaller than a row (%llu bytes)",
                    rank, (unsigned long long)x_stride, (unsigned long long)need);
    if (!quantize && c.hidden_dim_scale != 0 && xs == nullptr)
        return fail(ctx, A2A_ERR_INVALID_ARGUMENT, "rank %u: hidden_dim_scale is %u but x_scale is null",
                    rank, c.hidden_dim_scale);
    if (indices_stride < c.num_experts_per_token && num_tokens > 1)
        return fail(ctx, A2A_ERR_INVALID_ARGUMENT, "rank %u: indices_stride %llu smaller than a row of %u ids", rank,
                    (unsigned long long)indices_stride, c.num_experts_per_token);
    // the kernels carry these strides as 32-bit element counts
    if (indices_stride > 0xFFFFFFFFull || xs_stride_elem > 0xFFFFFFFFull || xs_stride_token > 0xFFFFFFFFull)
        return fail(ctx, A2A_ERR_UNSUPPORTED, "rank %u: an index or scale stride does not fit 32 bits", rank);
    return A2A_OK;
}

int check_recv(a2a_ctx *ctx, const a2a_config &c, uint32_t rank, const void *out_x, uint64_t out_stride,
               const float *out_scale, uint64_t os_stride_elem, uint64_t os_stride_token) {
    if (out_x == nullptr) return A2A_OK;  // a rank may decline to receive
    if (!aligned16(out_x) || out_stride % 16 != 0)
        return fail(ctx, A2A_ERR_UNSUPPORTED, "rank %u: out_x rows must be 16-byte aligned", rank);
    if (out_stride < row_bytes_of(c))
        return fail(ctx, A2A_ERR_INVALID_ARGUMENT, "rank %u: out_x_stride %llu smaller than a row", rank,
                    (unsigned long long)out_stride);
    if (c.hidden_dim_scale != 0 && out_scale == nullptr)
        return fail(ctx, A2A_ERR_INVALID_ARGUMENT, "rank %u: hidden_dim_scale is %u but out_x_scale is null",
                    rank, c.hidden_dim_scale);
    if (os_stride_elem > 0xFFFFFFFFull || os_stride_token > 0xFFFFFFFFull)
        return fail(ctx, A2A_ERR_UNSUPPORTED, "rank %u: a stride of out_x_scale does not fit 32 bits", rank);
    return A2A_OK;
}

// The recv half of a combine: the routes it gathers are those the dispatch of the step recorded
// for the rank's group, so it cannot cover more tokens than that dispatch sent.
int check_combine_tokens(a2a_ctx *ctx, uint32_t rank, uint64_t num_tokens, uint64_t indices_stride,
                         uint64_t weights_stride) {
    const uint32_t dispatched = ctx->num_tokens[rank / ctx->cfg.dp_size];
    if (num_tokens > dispatched)
        return fail(ctx, A2A_ERR_INVALID_ARGUMENT,
                    "rank %u combines %llu tokens but the dispatch of this step routed %u of its group", rank,
                    (unsigned long long)num_tokens, dispatched);
    if (indices_stride > 0xFFFFFFFFull || weights_stride > 0xFFFFFFFFull)
        return fail(ctx, A2A_ERR_UNSUPPORTED, "rank %u: an index or weight stride does not fit 32 bits", rank);
    return A2A_OK;
}

uint32_t elem_size_of(uint32_t dtype) {
    switch (dtype) {
        case A2A_F16:
        case A2A_BF16:
            return 2;
        case A2A_F32:
            return 4;
        default:
            return 0;
    }
}

// Upper bound, known to the host, of the rows any receiver got in this step.
uint32_t rows_upper_bound(const a2a_ctx *ctx) {
    uint64_t rows = 0;
    for (uint32_t g = 0; g < ctx->cfg.world_size; ++g) {
        if (ctx->sent_mask >> g & 1) rows += (uint64_t)ctx->num_tokens[g] * ctx->cfg.num_experts_per_token;
    }
    const uint64_t cap = ctx->staging.max_recv;
    return (uint32_t)(rows < cap ? rows : cap);
}

// The one-launch routing pass recounts earlier chunks in every chunk workgroup
// and all entries in every receiver workgroup: quadratic in the chunks of a
// source.  Measured at 8 entries per token: 2 us faster than the two-launch
// pass up to 8 chunks per source, equal at 16, 4 us slower at 32.
constexpr uint32_t kFusedMaxChunks = 12;
bool fused_routing_pays(const FinalizeArgs &fa, uint32_t world, uint32_t total_blocks) {
    for (uint32_t r = 0; r < world; ++r) {
        if (fa.num_blocks[r] > kFusedMaxChunks) return false;
    }
    return total_blocks <= 4 * kFusedMaxChunks;
}

// Dimensions of the device workspace for steps of at most `max_tokens` tokens per
// rank, and its tables carved out of `base` (256-byte aligned each).  With a null
// `base` only the dimensions are filled in.  Returns the bytes the tables take.
size_t carve_workspace(const a2a_config &c, uint32_t max_tokens, uint8_t *base, Workspace &ws) {
    const uint32_t N = c.world_size, E = c.num_experts, K = c.num_experts_per_token;
    ws.max_tk = (max_tokens != 0 ? max_tokens : 1) * K;
    ws.nb_max = ceil_div_u32(ws.max_tk, kRouteBlock);
    ws.world = N;
    ws.num_groups = N / c.dp_size;
    ws.dp_size = c.dp_size;
    ws.num_experts = E;
    ws.topk = K;
    ws.experts_per_rank = ceil_div_u32(E, N);
    ws.node_size = c.node_size;
    ws.expert_padding = c.expert_padding;
    ws.le_magic = ws.experts_per_rank > 1 ? 0xFFFFFFFFu / ws.experts_per_rank + 1 : 0;

    size_t off = 0;
    auto carve = [&off](size_t bytes) {
        const size_t at = off;
        off = align_up(off + bytes, 256);
        return at;
    };
    const size_t o_local = carve((size_t)N * ws.max_tk * sizeof(uint16_t));
    const size_t o_hist = carve((size_t)N * ws.nb_max * E * sizeof(uint32_t));
    const size_t o_block = carve((size_t)N * ws.nb_max * E * sizeof(uint32_t));
    const size_t o_routed = carve((size_t)N * E * sizeof(uint32_t));
    const size_t o_offsets = carve((size_t)N * E * sizeof(uint32_t));
    const size_t o_base = carve((size_t)N * E * sizeof(uint32_t));
    const size_t o_tpe = carve((size_t)E * sizeof(uint32_t));
    const size_t o_poff = carve((size_t)E * sizeof(uint32_t));
    const size_t o_slot = carve((size_t)N * ws.max_tk * sizeof(uint32_t));
    const size_t o_toff = carve((size_t)N * ws.max_tk * sizeof(uint32_t));
    const size_t o_err = carve(sizeof(uint32_t));
    const size_t o_order = carve((size_t)N * kMaxWorld);
    const size_t o_before = carve((size_t)N * ws.num_groups * sizeof(uint32_t));
    const size_t o_chunk_counts = carve((size_t)N * ws.nb_max * E * sizeof(uint32_t));
    const size_t o_totals = carve(2 * ((size_t)ws.num_groups + 1) * E * sizeof(uint32_t));
    const size_t o_turn = carve(2 * sizeof(uint32_t));
    const size_t o_send_totals = carve(2 * ((size_t)E + N) * sizeof(uint32_t));
    const size_t o_send_turn = carve(2 * sizeof(uint32_t));
    if (base != nullptr) {
        ws.local_rank = reinterpret_cast<uint16_t *>(base + o_local);
        ws.block_hist = reinterpret_cast<uint32_t *>(base + o_hist);
        ws.block_prefix = reinterpret_cast<uint32_t *>(base + o_block);
        ws.num_routed = reinterpret_cast<uint32_t *>(base + o_routed);
        ws.expert_offsets = reinterpret_cast<uint32_t *>(base + o_offsets);
        ws.slot_base = reinterpret_cast<uint32_t *>(base + o_base);
        ws.tokens_per_expert = reinterpret_cast<uint32_t *>(base + o_tpe);
        ws.padded_offset = reinterpret_cast<uint32_t *>(base + o_poff);
        ws.route_slot = reinterpret_cast<uint32_t *>(base + o_slot);
        ws.token_offset = reinterpret_cast<uint32_t *>(base + o_toff);
        ws.err = reinterpret_cast<uint32_t *>(base + o_err);
        ws.order = reinterpret_cast<const uint32_t *>(base + o_order);
        ws.laid_before = reinterpret_cast<const uint32_t *>(base + o_before);
        ws.chunk_counts = reinterpret_cast<uint32_t *>(base + o_chunk_counts);
        ws.totals = reinterpret_cast<uint32_t *>(base + o_totals);
        ws.turn = reinterpret_cast<uint32_t *>(base + o_turn);
        ws.send_totals = reinterpret_cast<uint32_t *>(base + o_send_totals);
        ws.send_turn = reinterpret_cast<uint32_t *>(base + o_send_turn);
    }
    return off;
}

// Everything the launches of a group dispatch take, built from the callers' arguments.
struct GroupPlan {
    RouteArgs ra;
    FinalizeArgs fa;
    PushArgs pa;
    uint32_t blocks = 0;                  // routing chunks of all sources
    uint32_t tokens = 0;                  // tokens of all sources
    uint32_t num_tokens[kMaxWorld] = {};  // per source
};

// First half of a group dispatch: every argument check, and the plan.  Enqueues nothing and
// changes nothing: a refused call leaves the stream, the tables and the context as they were.
// `ctx` only receives error texts and may be null (then they go where a2a_last_error(NULL)
// finds them).
int plan_dispatch_group(a2a_ctx *ctx, const a2a_config &c, const a2a_dispatch_args *args, uint32_t quantize,
                        GroupPlan &plan) {
    const uint32_t N = c.world_size, K = c.num_experts_per_token;
    for (uint32_t r = 0; r < N; ++r) {
        const a2a_dispatch_args &a = args[r];
        if (int rc = check_send(ctx, c, r, a.num_tokens, a.x_ptr, a.x_stride, quantize, a.x_scale_ptr,
                                a.x_scale_stride_elem, a.x_scale_stride_token, a.indices, a.indices_stride))
            return rc;
        if (int rc = check_recv(ctx, c, r, a.out_x, a.out_x_stride, a.out_x_scale, a.out_x_scale_stride_elem,
                                a.out_x_scale_stride_token))
            return rc;
    }

    RouteArgs &ra = plan.ra;
    FinalizeArgs &fa = plan.fa;
    PushArgs &pa = plan.pa;
    memset(&ra, 0, sizeof ra);
    memset(&fa, 0, sizeof fa);
    memset(&pa, 0, sizeof pa);
    const uint32_t D = c.dp_size, G = N / D;
    uint32_t blocks = 0, tokens = 0;
    // Sources: one per dp group (its members hold the same tokens; the first member's are read).
    for (uint32_t g = 0; g < G; ++g) {
        const a2a_dispatch_args &a = args[g * D];
        for (uint32_t m = 1; m < D; ++m) {
            if (args[g * D + m].num_tokens != a.num_tokens)
                return fail(ctx, A2A_ERR_INVALID_ARGUMENT, "ranks %u and %u share a dp group but pass %llu and %llu tokens",
                            g * D, g * D + m, (unsigned long long)a.num_tokens,
                            (unsigned long long)args[g * D + m].num_tokens);
        }
        const uint32_t T = (uint32_t)a.num_tokens;
        ra.src[g] = RouteSrc{a.indices, a.bound_m, (uint32_t)a.indices_stride, T};
        ra.block_start[g] = blocks;
        fa.num_blocks[g] = ceil_div_u32((uint64_t)T * K, kRouteBlock);
        blocks += fa.num_blocks[g];
        PushSrc &ps = pa.src[g];
        ps.x = static_cast<const uint8_t *>(a.x_ptr);
        ps.x_scale = a.x_scale_ptr;
        ps.indices = a.indices;
        ps.bound_m = a.bound_m;
        ps.x_stride = a.x_stride;
        ps.xs_stride_elem = (uint32_t)a.x_scale_stride_elem;
        ps.xs_stride_token = (uint32_t)a.x_scale_stride_token;
        ps.indices_stride = (uint32_t)a.indices_stride;
        ps.num_tokens = T;
        pa.token_start[g] = tokens;
        tokens += T;
        plan.num_tokens[g] = T;
    }
    for (uint32_t g = G; g <= (uint32_t)kMaxWorld; ++g) {
        ra.block_start[g] = blocks;
        pa.token_start[g] = tokens;
    }
    // Receivers: every rank.
    for (uint32_t r = 0; r < N; ++r) {
        const a2a_dispatch_args &a = args[r];
        fa.out_num_tokens[r] = a.out_num_tokens;
        fa.out_rows[r] = a.out_x != nullptr ? (uint32_t)(a.out_x_rows > 0xFFFFFFFFull ? 0xFFFFFFFFull : a.out_x_rows)
                                            : 0xFFFFFFFFu;
        PushDst &pd = pa.dst[r];
        pd.out_x = static_cast<uint8_t *>(a.out_x);
        pd.out_scale = a.out_x_scale;
        pd.out_stride = a.out_x_stride;
        pd.os_stride_elem = (uint32_t)a.out_x_scale_stride_elem;
        pd.os_stride_token = (uint32_t)a.out_x_scale_stride_token;
        pd.out_rows = fa.out_rows[r];
    }
    fa.fold_mask = fa.valid_mask = G >= 32 ? 0xFFFFFFFFu : ((1u << G) - 1);
    fa.recv_mask = N >= 32 ? 0xFFFFFFFFu : ((1u << N) - 1);
    pa.row_bytes = (uint32_t)row_bytes_of(c);
    pa.hidden_dim = c.hidden_dim;
    pa.hidden_dim_scale = c.hidden_dim_scale;
    pa.topk_magic = K > 1 ? (uint32_t)((0x100000000ull + K - 1) / K) : 0;
    plan.blocks = blocks;
    plan.tokens = tokens;
    return A2A_OK;
}

// Second half: the launches of an accepted plan on the tables of `ws`.
int launch_dispatch_group(a2a_ctx *ctx, const a2a_config &c, const Workspace &ws, const GroupPlan &plan,
                          uint32_t quantize, hipStream_t s, KernelTiming pack_timing, KernelTiming route_timing) {
    const RouteArgs &ra = plan.ra;
    const FinalizeArgs &fa = plan.fa;
    const PushArgs &pa = plan.pa;
    const uint32_t blocks = plan.blocks, tokens = plan.tokens;
    const uint32_t G = c.world_size / c.dp_size;
    hipError_t e;
    if (!(c.flags & A2A_FLAG_SEPARATE_ROUTING) && dispatch_small_fits(pa, ws, quantize != 0, tokens)) {
        e = launch_dispatch_small(pa, fa, ws, quantize != 0, tokens, s, pack_timing);
        if (e != hipSuccess) return hip_fail(ctx, e, "launch dispatch_small");
    } else if (!(c.flags & A2A_FLAG_SEPARATE_ROUTING) && dispatch_single_fits(pa, ws, quantize != 0, tokens)) {
        e = launch_dispatch_single(pa, fa, ws, quantize != 0, tokens, s, pack_timing);
        if (e != hipSuccess) return hip_fail(ctx, e, "launch dispatch_single");
    } else if (c.flags & A2A_FLAG_SEPARATE_ROUTING) {
        if (fused_routing_pays(fa, G, blocks)) {
            e = launch_route_fused(ra, fa, ws, s);
            if (e != hipSuccess) return hip_fail(ctx, e, "launch route_fused");
        } else {
            e = launch_route(ra, ws, blocks, s);
            if (e != hipSuccess) return hip_fail(ctx, e, "launch route_hist");
            e = launch_finalize(fa, ws, s);
            if (e != hipSuccess) return hip_fail(ctx, e, "launch route_finalize");
        }
        e = launch_dispatch_push(pa, ws, quantize != 0, tokens, s, pack_timing);
        if (e != hipSuccess) return hip_fail(ctx, e, "launch dispatch_push");
    } else {
        // Two launches: chunk histograms that also add up the step's totals, then a pack whose
        // workgroups resolve their own rows from them.
        e = launch_route_accumulate(ra, ws, blocks, s, false, route_timing);
        if (e != hipSuccess) return hip_fail(ctx, e, "launch route_hist (accumulating)");
        e = launch_dispatch_resolve(pa, fa, ws, quantize != 0, tokens, s, pack_timing);
        if (e != hipSuccess) return hip_fail(ctx, e, "launch dispatch_resolve");
    }
    return A2A_OK;
}


// Address of `scratch` on device `dev` (which must be current), looked up once
// per device.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
uint8_t *g_scratch_ptr[kMaxDevices] = {};

int static_scratch_of(int dev, hipStream_t stream, uint8_t **out) {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        // The look-up loads the symbol's module on this device: not a call to make while `stream`
        // is being captured into a graph.
        hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(stream, &capture) == hipSuccess && capture != hipStreamCaptureStatusNone)
            return fail(nullptr, A2A_ERR_BAD_ORDER,
                        "the first a2a_dispatch_static on a GPU looks up where that GPU holds the library's array, "
                        "which a stream capture forbids: make one call on device %d outside the capture first", dev);
        void *ptr = nullptr;
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return hip_fail(nullptr, e, "hipGetSymbolAddress(scratch)");
        g_scratch_ptr[dev] = static_cast<uint8_t *>(ptr);
    }
    *out = g_scratch_ptr[dev];
    return A2A_OK;
}

// What a step on tables that hold another step's leftovers needs before its
// first launch: both copies of the step totals and the word that says whose turn
// it is start at zero, and the two tables that a context uploads once at create
// (the order in which every receiver lays out its sources, and which sources
// come before which) are computed here.  `clear_err`: the error word is the
// library's own (the caller gave none), so nobody reads it; keep it tidy.
__global__ __launch_bounds__(1024) void static_prepare_kernel(const Workspace ws, uint32_t clear_err) {
    const uint32_t N = ws.world, G = ws.num_groups, E = ws.num_experts;
    const uint32_t tid = threadIdx.x;
    const uint32_t words = 2 * (G + 1) * E;
    for (uint32_t i = blockIdx.x * blockDim.x + tid; i < words; i += gridDim.x * blockDim.x) ws.totals[i] = 0;
    if (blockIdx.x != 0) return;
    if (tid < 2) ws.turn[tid] = 0;
    if (clear_err != 0 && tid == 0) *ws.err = 0;
    uint32_t *order = const_cast<uint32_t *>(ws.order);
    for (uint32_t w = tid; w < N * (kMaxWorld / 4); w += blockDim.x) {
        const uint32_t r = w / (kMaxWorld / 4), i0 = (w % (kMaxWorld / 4)) * 4;
        uint32_t word = 0;
        for (uint32_t j = 0; j < 4; ++j) {
            if (i0 + j < G) word |= source_order(r, i0 + j, N, ws.node_size, ws.dp_size) << (8 * j);
        }
        order[w] = word;
    }
    uint32_t *before = const_cast<uint32_t *>(ws.laid_before);
    for (uint32_t w = tid; w < N * G; w += blockDim.x) {
        const uint32_t r = w / G, g = w % G;
        uint32_t seen = 0;
        for (uint32_t i = 0; i < G; ++i) {
            const uint32_t s = source_order(r, i, N, ws.node_size, ws.dp_size);
            if (s == g) break;
            seen |= 1u << s;
        }
        before[w] = seen;
    }
}

}  // namespace

extern "C" {

const char *a2a_version(void) { return "0.1"; }

size_t a2a_dispatch_token_stride(const a2a_config *c) {
    // a2a_worker.rs:317-321
    return align_up((size_t)c->hidden_dim * c->in_elemsize, 16) +
           align_up((size_t)c->hidden_dim_scale * c->scale_elemsize, 16) + 16;
}

size_t a2a_combine_token_stride(const a2a_config *c) {
    // a2a_worker.rs:323-325
    return align_up((size_t)c->hidden_dim * c->out_elemsize, 16);
}

const char *a2a_last_error(const a2a_ctx *ctx) {
    return ctx != nullptr ? ctx->error.c_str() : g_create_error.c_str();
}

int a2a_ctx_create(const a2a_config *config, a2a_ctx **out_ctx) {
    if (config == nullptr || out_ctx == nullptr)
        return fail(nullptr, A2A_ERR_INVALID_ARGUMENT, "null argument");
    *out_ctx = nullptr;
    if (int rc = check_config(*config)) return rc;

    int ndev = 0;
    hipError_t e = hipGetDeviceCount(&ndev);
    if (e != hipSuccess) return hip_fail(nullptr, e, "hipGetDeviceCount");
    if (config->device < 0 || config->device >= ndev)
        return fail(nullptr, A2A_ERR_INVALID_ARGUMENT, "device %d not in [0, %d)", config->device, ndev);
    DeviceGuard guard(config->device);
    if (!guard.ok) return fail(nullptr, A2A_ERR_INVALID_ARGUMENT, "cannot select device %d", config->device);

    a2a_ctx *ctx = new (std::nothrow) a2a_ctx();
    if (ctx == nullptr) return fail(nullptr, A2A_ERR_OUT_OF_MEMORY, "out of host memory");
    ctx->cfg = *config;

    const uint32_t N = config->world_size;
    Workspace &ws = ctx->ws;
    ctx->arena_bytes = carve_workspace(*config, config->max_num_tokens, nullptr, ws);
    e = hipMalloc(&ctx->arena, ctx->arena_bytes);
    if (e != hipSuccess) {
        delete ctx;
        return hip_fail(nullptr, e, "hipMalloc(workspace)");
    }
    e = hipMemset(ctx->arena, 0, ctx->arena_bytes);
    if (e == hipSuccess) e = hipDeviceSynchronize();
    if (e != hipSuccess) {
        (void)hipFree(ctx->arena);
        delete ctx;
        return hip_fail(nullptr, e, "hipMemset(workspace)");
    }
    uint8_t *base = static_cast<uint8_t *>(ctx->arena);
    carve_workspace(*config, config->max_num_tokens, base, ws);
    {
        // i-th source each receiver lays out, and which sources come before which: fixed for the
        // life of the context
        uint8_t table[kMaxWorld * kMaxWorld] = {0};
        uint32_t before[kMaxWorld * kMaxWorld] = {0};
        for (uint32_t r = 0; r < N; ++r) {
            uint32_t seen = 0;
            for (uint32_t i = 0; i < ws.num_groups; ++i) {
                const uint32_t g = source_order(r, i, N, config->node_size, config->dp_size);
                table[r * kMaxWorld + i] = (uint8_t)g;
                before[r * ws.num_groups + g] = seen;
                seen |= 1u << g;
            }
        }
        e = hipMemcpy(const_cast<uint32_t *>(ws.order), table, (size_t)N * kMaxWorld, hipMemcpyHostToDevice);
        if (e == hipSuccess)
            e = hipMemcpy(const_cast<uint32_t *>(ws.laid_before), before, (size_t)N * ws.num_groups * sizeof(uint32_t),
                          hipMemcpyHostToDevice);
        if (e != hipSuccess) {
            (void)hipFree(ctx->arena);
            delete ctx;
            return hip_fail(nullptr, e, "hipMemcpy(source order)");
        }
    }

    if (config->flags & A2A_FLAG_PREALLOC_STAGING) {
        std::string msg;
        const int rc = staging_allocate(ctx->staging, *config, &msg);
        if (rc != 0) {
            (void)hipFree(ctx->arena);
            delete ctx;
            return fail(nullptr, rc, "%s", msg.c_str());
        }
    }
    *out_ctx = ctx;
    return A2A_OK;
}

int a2a_ctx_destroy(a2a_ctx *ctx) {
    if (ctx == nullptr) return A2A_OK;
    DeviceGuard guard(ctx->cfg.device);
    (void)hipDeviceSynchronize();
    staging_free(ctx->staging);
    hipError_t e = hipFree(ctx->arena);
    delete ctx;
    return e == hipSuccess ? A2A_OK : (int)e;
}

int a2a_ctx_status(a2a_ctx *ctx, void *stream, uint32_t *flags) {
    if (ctx == nullptr || flags == nullptr) return A2A_ERR_INVALID_ARGUMENT;
    DeviceGuard guard(ctx->cfg.device);
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipError_t e = hipStreamSynchronize(s);
    if (e != hipSuccess) return hip_fail(ctx, e, "hipStreamSynchronize");
    e = hipMemcpy(flags, ctx->ws.err, sizeof(uint32_t), hipMemcpyDeviceToHost);
    if (e != hipSuccess) return hip_fail(ctx, e, "hipMemcpy(err)");
    if (*flags != 0) {
        e = hipMemset(ctx->ws.err, 0, sizeof(uint32_t));
        if (e != hipSuccess) return hip_fail(ctx, e, "hipMemset(err)");
    }
    return A2A_OK;
}

int a2a_dispatch(a2a_ctx *ctx, const a2a_dispatch_args *args, uint32_t quantize, void *stream) {
    if (ctx == nullptr) return A2A_ERR_INVALID_ARGUMENT;
    ProfilerRange range("dispatch");
    if (int rc = check_usable(ctx)) return rc;
    if (args == nullptr) return fail(ctx, A2A_ERR_INVALID_ARGUMENT, "null args");
    DeviceGuard guard(ctx->cfg.device);
    const KernelTiming pack_timing = ctx->timing[A2A_KERNEL_PACK];
    const KernelTiming route_timing = ctx->timing[A2A_KERNEL_ROUTE];
    ctx->timing[A2A_KERNEL_PACK] = KernelTiming();
    ctx->timing[A2A_KERNEL_ROUTE] = KernelTiming();
    GroupPlan plan;
    if (int rc = plan_dispatch_group(ctx, ctx->cfg, args, quantize, plan)) return rc;
    if (int rc = launch_dispatch_group(ctx, ctx->cfg, ctx->ws, plan, quantize, static_cast<hipStream_t>(stream),
                                       pack_timing, route_timing))
        return rc;
    // only an accepted step replaces what the context knows of the previous one
    memcpy(ctx->num_tokens, plan.num_tokens, sizeof ctx->num_tokens);
    ctx->group_routing = true;
    ctx->step_open = false;
    ctx->sent_mask = 0;
    ctx->empty_mask = 0;
    ctx->quantized = quantize;
    return A2A_OK;
}

int a2a_dispatch_static(const a2a_config *config, const a2a_dispatch_args *args, uint32_t quantize,
                        uint32_t *device_flags, void *stream) {
    if (config == nullptr || args == nullptr) return fail(nullptr, A2A_ERR_INVALID_ARGUMENT, "null argument");
    ProfilerRange range("dispatch_static");
    if (int rc = check_config(*config)) return rc;
    const a2a_config &c = *config;
    if (c.flags != 0)
        return fail(nullptr, A2A_ERR_INVALID_ARGUMENT, "a2a_dispatch_static takes no flags (got 0x%x)", c.flags);
    if (c.device < 0 || c.device >= kMaxDevices)
        return fail(nullptr, A2A_ERR_INVALID_ARGUMENT, "device %d not in [0, %d)", c.device, kMaxDevices);
    // The tables are sized for this step: the largest source decides.
    uint64_t max_tokens = 0;
    for (uint32_t r = 0; r < c.world_size; ++r) {
        if (args[r].num_tokens > max_tokens) max_tokens = args[r].num_tokens;
    }
    if (max_tokens > c.max_num_tokens)
        return fail(nullptr, A2A_ERR_TOO_MANY_TOKENS, "Number of tokens exceeds maximum allowed (%llu > %u)",
                    (unsigned long long)max_tokens, c.max_num_tokens);
    Workspace ws;
    memset(&ws, 0, sizeof ws);
    const size_t need = carve_workspace(c, (uint32_t)max_tokens, nullptr, ws);
    if (need > (size_t)A2A_STATIC_SCRATCH_BYTES)
        return fail(nullptr, A2A_ERR_TOO_MANY_TOKENS,
                    "a step of %u ranks x %llu tokens x %u routes over %u experts needs %zu bytes of routing tables; "
                    "a2a_dispatch_static has %zu (use a2a_ctx_create and a2a_dispatch for larger steps)",
                    c.world_size, (unsigned long long)max_tokens, c.num_experts_per_token, c.num_experts, need,
                    (size_t)A2A_STATIC_SCRATCH_BYTES);
    // Every check of the step before anything is enqueued: a refused call does nothing.
    GroupPlan plan;
    if (int rc = plan_dispatch_group(nullptr, c, args, quantize, plan)) return rc;
    DeviceGuard guard(c.device);
    if (!guard.ok) return fail(nullptr, A2A_ERR_INVALID_ARGUMENT, "cannot select device %d", c.device);
    hipStream_t s = static_cast<hipStream_t>(stream);
    uint8_t *base = nullptr;
    if (int rc = static_scratch_of(c.device, s, &base)) return rc;
    carve_workspace(c, (uint32_t)max_tokens, base, ws);
    if (device_flags != nullptr) ws.err = device_flags;
    const uint32_t words = 2 * (ws.num_groups + 1) * ws.num_experts;
    const uint32_t blocks = words > 8 * 1024 ? 8 : 1;
    hipLaunchKernelGGL(static_prepare_kernel, dim3(blocks), dim3(1024), 0, s, ws, device_flags == nullptr ? 1u : 0u);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return hip_fail(nullptr, e, "launch static_prepare");
    return launch_dispatch_group(nullptr, c, ws, plan, quantize, s, KernelTiming(), KernelTiming());
}

int a2a_combine(a2a_ctx *ctx, const a2a_combine_args *args, uint32_t expert_y_dtype,
                uint32_t accumulate, void *stream) {
    if (ctx == nullptr) return A2A_ERR_INVALID_ARGUMENT;
    ProfilerRange range("combine");
    if (int rc = check_usable(ctx)) return rc;
    if (args == nullptr) return fail(ctx, A2A_ERR_INVALID_ARGUMENT, "null args");
    const a2a_config &c = ctx->cfg;
    const uint32_t N = c.world_size;
    if (!ctx->group_routing)
        return fail(ctx, A2A_ERR_BAD_ORDER, "a2a_combine needs the routing of a preceding a2a_dispatch");
    const uint32_t in_size = elem_size_of(expert_y_dtype);
    if (in_size == 0)
        return fail(ctx, A2A_ERR_UNSUPPORTED, "expert_y dtype %u: only F16, BF16 and F32 are supported",
                    expert_y_dtype);
    const uint32_t vec = 16 / in_size;
    if (c.hidden_dim % vec != 0)
        return fail(ctx, A2A_ERR_UNSUPPORTED, "hidden_dim %u is not a multiple of %u", c.hidden_dim, vec);
    if (accumulate && c.dp_size != 1)   // python/pplx_garden/kernels/p2p_all_to_all.py:457-458
        return fail(ctx, A2A_ERR_UNSUPPORTED, "accumulate needs dp_size 1");
    CombArgs ca;
    memset(&ca, 0, sizeof ca);
    uint32_t tokens = 0;
    for (uint32_t r = 0; r < N; ++r) {
        const a2a_combine_args &a = args[r];
        if (a.num_tokens > c.max_num_tokens)
            return fail(ctx, A2A_ERR_TOO_MANY_TOKENS, "Number of tokens exceeds maximum allowed (rank %u)", r);
        if (int rc = check_combine_tokens(ctx, r, a.num_tokens, a.indices_stride, a.weights_stride)) return rc;
        if (a.expert_y != nullptr && (!aligned16(a.expert_y) || a.expert_y_stride % 16 != 0))
            return fail(ctx, A2A_ERR_UNSUPPORTED, "rank %u: expert_y rows must be 16-byte aligned", r);
        const uint64_t out_stride_bytes = a.out_tokens_stride * c.out_elemsize;
        const uint32_t out_chunk = vec * c.out_elemsize;
        if (a.num_tokens != 0) {
            if (a.out_tokens == nullptr || a.indices == nullptr || a.weights == nullptr)
                return fail(ctx, A2A_ERR_INVALID_ARGUMENT, "rank %u: null out_tokens, indices or weights", r);
            if (((uintptr_t)a.out_tokens % out_chunk) != 0 || out_stride_bytes % out_chunk != 0)
                return fail(ctx, A2A_ERR_UNSUPPORTED, "rank %u: out_tokens rows must be %u-byte aligned", r,
                            out_chunk);
        }
        ca.src[r] = CombSrc{static_cast<const uint8_t *>(a.expert_y), a.expert_y_stride,
                            (uint32_t)(a.expert_y_rows > 0xFFFFFFFFull ? 0xFFFFFFFFull : a.expert_y_rows), 0};
        CombDst &d = ca.dst[r];
        d.out = static_cast<uint8_t *>(a.out_tokens);
        d.indices = a.indices;
        d.weights = a.weights;
        d.bound_m = a.bound_m;
        d.out_stride = out_stride_bytes;
        d.indices_stride = (uint32_t)a.indices_stride;
        d.weights_stride = (uint32_t)a.weights_stride;
        d.num_tokens = (uint32_t)a.num_tokens;
        ca.token_start[r] = tokens;
        tokens += (uint32_t)a.num_tokens;
    }
    for (uint32_t r = N; r <= (uint32_t)kMaxWorld; ++r) ca.token_start[r] = tokens;
    ca.hidden_dim = c.hidden_dim;
    ca.accumulate = accumulate ? 1 : 0;
    DeviceGuard guard(c.device);
    const KernelTiming gather_timing = ctx->timing[A2A_KERNEL_GATHER];
    ctx->timing[A2A_KERNEL_GATHER] = KernelTiming();
    hipError_t e = launch_combine_gather(ca, ctx->ws, expert_y_dtype, c.out_dtype, tokens,
                                         static_cast<hipStream_t>(stream), gather_timing);
    if (e != hipSuccess) return hip_fail(ctx, e, "launch combine_gather");
    return A2A_OK;
}

int a2a_ctx_time_next_kernel(a2a_ctx *ctx, uint32_t which, void *start_event, void *stop_event) {
    if (ctx == nullptr) return A2A_ERR_INVALID_ARGUMENT;
    if (which > A2A_KERNEL_COMBINE_SEND) return fail(ctx, A2A_ERR_INVALID_ARGUMENT, "unknown kernel %u", which);
    if ((start_event == nullptr) != (stop_event == nullptr))
        return fail(ctx, A2A_ERR_INVALID_ARGUMENT, "pass both events or neither");
    ctx->timing[which].start = static_cast<hipEvent_t>(start_event);
    ctx->timing[which].stop = static_cast<hipEvent_t>(stop_event);
    return A2A_OK;
}

int a2a_ctx_read_table(a2a_ctx *ctx, uint32_t rank, uint32_t which, uint32_t *out, size_t count,
                       void *stream) {
    if (ctx == nullptr || out == nullptr) return A2A_ERR_INVALID_ARGUMENT;
    if (int rc = check_rank(ctx, rank)) return rc;
    const Workspace &ws = ctx->ws;
    const uint32_t E = ws.num_experts;
    const uint32_t *src = nullptr;
    size_t limit = 0;
    const uint32_t receiver = rank;
    rank = rank / ws.dp_size;   // sender-side tables belong to the rank's dp group
    switch (which) {
        case A2A_TABLE_NUM_ROUTED:
            src = ws.num_routed + (size_t)rank * E;
            limit = E;
            break;
        case A2A_TABLE_EXPERT_OFFSETS:
            src = ws.expert_offsets + (size_t)rank * E;
            limit = E;
            break;
        case A2A_TABLE_TOKEN_OFFSET:
            src = ws.token_offset + (size_t)rank * ws.max_tk;
            limit = ws.max_tk;
            break;
        case A2A_TABLE_SLOT:
            if (!ctx->group_routing)
                return fail(ctx, A2A_ERR_BAD_ORDER, "slots exist only after a2a_dispatch");
            src = ws.route_slot + (size_t)rank * ws.max_tk;
            limit = ws.max_tk;
            break;
        case A2A_TABLE_PADDED_INDEX:
        case A2A_TABLE_SOURCE_RANK:
        case A2A_TABLE_SOURCE_POSITION:
        case A2A_TABLE_NUM_RECV_TOKENS:
        case A2A_TABLE_SOURCE_DISPATCH_OFFSET:
        case A2A_TABLE_COMBINE_SEND_OFFSET:
            src = staging_table(ctx->staging, ctx->cfg, receiver, which, &limit);
            if (src == nullptr)
                return fail(ctx, A2A_ERR_BAD_ORDER, "receive tables exist only after a2a_dispatch_recv");
            break;
        default:
            return fail(ctx, A2A_ERR_INVALID_ARGUMENT, "unknown table %u", which);
    }
    if (count > limit) return fail(ctx, A2A_ERR_INVALID_ARGUMENT, "count %zu exceeds the table (%zu)", count, limit);
    if (which <= A2A_TABLE_TOKEN_OFFSET && !ctx->group_routing && (ctx->empty_mask >> rank & 1)) {
        // a split send without tokens launches nothing and leaves its tables alone: they read as zeros
        memset(out, 0, count * sizeof(uint32_t));
        return A2A_OK;
    }
    DeviceGuard guard(ctx->cfg.device);
    hipError_t e = hipStreamSynchronize(static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(ctx, e, "hipStreamSynchronize");
    e = hipMemcpy(out, src, count * sizeof(uint32_t), hipMemcpyDeviceToHost);
    if (e != hipSuccess) return hip_fail(ctx, e, "hipMemcpy(table)");
    return A2A_OK;
}

// ---------------------------------------------------------------------------
// Split calls: one logical rank at a time, rows travel through staging.
// ---------------------------------------------------------------------------

int a2a_dispatch_send(a2a_ctx *ctx, uint32_t rank, size_t num_tokens, const void *x_ptr,
                      size_t x_stride, uint32_t quantize, const float *x_scale_ptr,
                      size_t x_scale_stride_elem, size_t x_scale_stride_token,
                      const int32_t *indices, size_t indices_stride, const float *weights,
                      size_t weights_stride, const int32_t *bound_m, void *stream) {
    (void)weights;
    (void)weights_stride;
    if (ctx == nullptr) return A2A_ERR_INVALID_ARGUMENT;
    ProfilerRange range("dispatch_send");
    if (int rc = check_usable(ctx)) return rc;
    if (int rc = check_rank(ctx, rank)) return rc;
    if (int rc = check_send(ctx, ctx->cfg, rank, num_tokens, x_ptr, x_stride, quantize, x_scale_ptr,
                            x_scale_stride_elem, x_scale_stride_token, indices, indices_stride))
        return rc;
    const a2a_config &c = ctx->cfg;
    DeviceGuard guard(c.device);
    if (!ctx->staging.allocated) {
        // the first split call of a context allocates the staging: not while a stream is being captured
        hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(static_cast<hipStream_t>(stream), &capture) == hipSuccess &&
            capture != hipStreamCaptureStatusNone)
            return fail(ctx, A2A_ERR_BAD_ORDER,
                        "the first a2a_dispatch_send of a context allocates its staging buffers, which a stream "
                        "capture forbids: create the context with A2A_FLAG_PREALLOC_STAGING");
        std::string msg;
        if (int rc = staging_allocate(ctx->staging, c, &msg)) return fail(ctx, rc, "%s", msg.c_str());
    }
    // A send after a recv starts a new step.
    if (!ctx->step_open || ctx->recv_seen) {
        ctx->sent_mask = 0;
        ctx->empty_mask = 0;
        ctx->recv_seen = false;
        ctx->step_open = true;
        ctx->staging.recv_mask = 0;
        ctx->staging.combine_sent_mask = 0;
    }
    if (ctx->sent_mask != 0 && ctx->quantized != quantize)
        return fail(ctx, A2A_ERR_INVALID_ARGUMENT, "all sends of a step must use the same mode");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uint32_t K = c.num_experts_per_token;
    const uint32_t T = (uint32_t)num_tokens;
    const KernelTiming send_timing = ctx->timing[A2A_KERNEL_STAGE_SEND];
    const KernelTiming route_timing = ctx->timing[A2A_KERNEL_ROUTE];
    ctx->timing[A2A_KERNEL_STAGE_SEND] = KernelTiming();
    ctx->timing[A2A_KERNEL_ROUTE] = KernelTiming();

    // The sender is the rank's dp group; when several members of a group send, each repeats
    // the same routing and stages the same rows.
    const uint32_t group = rank / c.dp_size;
    if (T == 0) {
        // Nothing to route or stage: no launch.  The receivers of this step count the source as
        // empty (it is left out of their mask of valid sources) and its tables read as zeros.
        ctx->sent_mask |= 1u << group;
        ctx->empty_mask |= 1u << group;
        ctx->num_tokens[group] = 0;
        ctx->quantized = quantize;
        ctx->group_routing = false;
        return A2A_OK;
    }
    ctx->empty_mask &= ~(1u << group);
    StageSendArgs sa;
    memset(&sa, 0, sizeof sa);
    sa.rank = rank;
    sa.src.x = static_cast<const uint8_t *>(x_ptr);
    sa.src.x_scale = x_scale_ptr;
    sa.src.indices = indices;
    sa.src.bound_m = bound_m;
    sa.src.x_stride = x_stride;
    sa.src.xs_stride_elem = (uint32_t)x_scale_stride_elem;
    sa.src.xs_stride_token = (uint32_t)x_scale_stride_token;
    sa.src.indices_stride = (uint32_t)indices_stride;
    sa.src.num_tokens = T;
    sa.row_bytes = (uint32_t)row_bytes_of(c);
    sa.hidden_dim = c.hidden_dim;
    sa.hidden_dim_scale = c.hidden_dim_scale;
    sa.topk_magic = K > 1 ? (uint32_t)((0x100000000ull + K - 1) / K) : 0;

    hipError_t e;
    if (!(c.flags & A2A_FLAG_SEPARATE_ROUTING) && stage_send_small_fits(sa, ctx->ws)) {
        e = launch_stage_send_small(sa, ctx->ws, ctx->staging, quantize != 0, s, send_timing);
        if (e != hipSuccess) return hip_fail(ctx, e, "launch stage_send_small");
    } else if (!(c.flags & A2A_FLAG_SEPARATE_ROUTING) && stage_send_single_fits(sa, ctx->ws, quantize != 0)) {
        e = launch_stage_send_single(sa, ctx->ws, ctx->staging, quantize != 0, s, send_timing);
        if (e != hipSuccess) return hip_fail(ctx, e, "launch stage_send_single");
    } else {
        RouteArgs ra;
        FinalizeArgs fa;
        memset(&ra, 0, sizeof ra);
        memset(&fa, 0, sizeof fa);
        const uint32_t nb = ceil_div_u32((uint64_t)T * K, kRouteBlock);
        ra.src[group] = RouteSrc{indices, bound_m, (uint32_t)indices_stride, T};
        for (uint32_t r = 0; r <= (uint32_t)kMaxWorld; ++r) ra.block_start[r] = r <= group ? 0 : nb;
        fa.num_blocks[group] = nb;
        fa.fold_mask = 1u << group;
        fa.valid_mask = ctx->sent_mask | (1u << group);
        fa.recv_mask = 0;
        if (T != 0 && !(c.flags & A2A_FLAG_SEPARATE_ROUTING)) {
            // two launches: chunk histograms that also add up the sender's totals, then a staging
            // launch whose workgroups resolve their own positions from them
            e = launch_route_accumulate(ra, ctx->ws, nb, s, true, route_timing);
            if (e != hipSuccess) return hip_fail(ctx, e, "launch route_hist (accumulating, send)");
            e = launch_stage_send_resolve(sa, ctx->ws, ctx->staging, quantize != 0, s, send_timing);
            if (e != hipSuccess) return hip_fail(ctx, e, "launch stage_send_resolve");
        } else {
            if (fused_routing_pays(fa, c.world_size / c.dp_size, nb)) {
                e = launch_route_fused(ra, fa, ctx->ws, s);
                if (e != hipSuccess) return hip_fail(ctx, e, "launch route_fused");
            } else {
                e = launch_route(ra, ctx->ws, nb, s);
                if (e != hipSuccess) return hip_fail(ctx, e, "launch route_hist");
                e = launch_finalize(fa, ctx->ws, s);
                if (e != hipSuccess) return hip_fail(ctx, e, "launch route_finalize");
            }
            e = launch_stage_send(sa, ctx->ws, ctx->staging, quantize != 0, s, send_timing);
            if (e != hipSuccess) return hip_fail(ctx, e, "launch stage_send");
        }
    }

    ctx->sent_mask |= 1u << group;
    ctx->num_tokens[group] = T;
    ctx->quantized = quantize;
    ctx->group_routing = false;
    return A2A_OK;
}

int a2a_dispatch_recv(a2a_ctx *ctx, uint32_t rank, int32_t *out_num_tokens, void *out_x,
                      size_t out_x_stride, size_t out_x_rows, float *out_x_scale,
                      size_t out_x_scale_stride_elem, size_t out_x_scale_stride_token,
                      void *stream) {
    if (ctx == nullptr) return A2A_ERR_INVALID_ARGUMENT;
    ProfilerRange range("dispatch_recv");
    if (int rc = check_usable(ctx)) return rc;
    if (int rc = check_rank(ctx, rank)) return rc;
    if (!ctx->step_open || ctx->sent_mask == 0)
        return fail(ctx, A2A_ERR_BAD_ORDER, "a2a_dispatch_recv before any a2a_dispatch_send of the step");
    if (int rc = check_recv(ctx, ctx->cfg, rank, out_x, out_x_stride, out_x_scale, out_x_scale_stride_elem,
                            out_x_scale_stride_token))
        return rc;
    const a2a_config &c = ctx->cfg;
    DeviceGuard guard(c.device);
    hipStream_t s = static_cast<hipStream_t>(stream);

    const uint32_t out_rows = out_x != nullptr ? (uint32_t)(out_x_rows > 0xFFFFFFFFull ? 0xFFFFFFFFull : out_x_rows)
                                               : 0xFFFFFFFFu;
    StageRecvArgs rv;
    memset(&rv, 0, sizeof rv);
    rv.rank = rank;
    rv.dst.out_x = static_cast<uint8_t *>(out_x);
    rv.dst.out_scale = out_x_scale;
    rv.dst.out_stride = out_x_stride;
    rv.dst.os_stride_elem = (uint32_t)out_x_scale_stride_elem;
    rv.dst.os_stride_token = (uint32_t)out_x_scale_stride_token;
    rv.dst.out_rows = out_rows;
    rv.out_num_tokens = out_num_tokens;
    rv.row_bytes = (uint32_t)row_bytes_of(c);
    rv.hidden_dim_scale = c.hidden_dim_scale;
    rv.max_rows = rows_upper_bound(ctx);
    // The first recv of a step lays out every receiver: once per step, as the reference's host
    // worker does (a2a_worker.rs:526-703), not once per recv launch.
    rv.valid_mask = ctx->sent_mask & ~ctx->empty_mask;
    rv.max_private = c.max_private_tokens;
    const KernelTiming recv_timing = ctx->timing[A2A_KERNEL_STAGE_RECV];
    ctx->timing[A2A_KERNEL_STAGE_RECV] = KernelTiming();
    const hipError_t e = launch_stage_recv(rv, ctx->ws, ctx->staging, !ctx->recv_seen, s, recv_timing);
    if (e != hipSuccess) return hip_fail(ctx, e, "launch stage_recv");
    ctx->recv_seen = true;
    ctx->staging.recv_mask |= 1u << rank;
    return A2A_OK;
}

int a2a_combine_send(a2a_ctx *ctx, uint32_t rank, const void *expert_y, size_t expert_y_stride,
                     size_t expert_y_rows, void *stream) {
    if (ctx == nullptr) return A2A_ERR_INVALID_ARGUMENT;
    ProfilerRange range("combine_send");
    if (int rc = check_usable(ctx)) return rc;
    if (int rc = check_rank(ctx, rank)) return rc;
    if (!ctx->staging.allocated || !(ctx->staging.recv_mask >> rank & 1))
        return fail(ctx, A2A_ERR_BAD_ORDER, "a2a_combine_send before a2a_dispatch_recv of rank %u", rank);
    if (expert_y == nullptr || !aligned16(expert_y) || expert_y_stride % 16 != 0)
        return fail(ctx, A2A_ERR_UNSUPPORTED, "rank %u: expert_y rows must be non-null and 16-byte aligned", rank);
    const a2a_config &c = ctx->cfg;
    // The call copies whole staging rows of hidden_dim * out_elemsize bytes and is not told the type
    // of expert_y (neither is the reference's, a2a_combine_send.cu:261): rows that are closer
    // together than that hold narrower elements, and copying them would read past the last row.
    if (expert_y_rows > 1 && expert_y_stride < (size_t)c.hidden_dim * c.out_elemsize)
        return fail(ctx, A2A_ERR_UNSUPPORTED,
                    "rank %u: expert_y rows are %zu bytes apart but a staged combine row holds %zu "
                    "(hidden_dim x %u-byte elements of out_dtype): the split calls need expert_y in a type "
                    "as wide as out_dtype",
                    rank, expert_y_stride, (size_t)c.hidden_dim * c.out_elemsize, c.out_elemsize);
    DeviceGuard guard(c.device);
    CombineSendArgs cs;
    memset(&cs, 0, sizeof cs);
    cs.rank = rank;
    cs.y = static_cast<const uint8_t *>(expert_y);
    cs.y_stride = expert_y_stride;
    cs.y_rows = (uint32_t)(expert_y_rows > 0xFFFFFFFFull ? 0xFFFFFFFFull : expert_y_rows);
    cs.row_bytes = (uint32_t)((size_t)c.hidden_dim * c.out_elemsize);
    cs.max_rows = rows_upper_bound(ctx);
    const KernelTiming timing = ctx->timing[A2A_KERNEL_COMBINE_SEND];
    ctx->timing[A2A_KERNEL_COMBINE_SEND] = KernelTiming();
    hipError_t e = launch_combine_send(cs, ctx->ws, ctx->staging, static_cast<hipStream_t>(stream), timing);
    if (e != hipSuccess) return hip_fail(ctx, e, "launch combine_send");
    ctx->staging.combine_sent_mask |= 1u << rank;
    return A2A_OK;
}

int a2a_combine_recv(a2a_ctx *ctx, uint32_t rank, size_t num_tokens, size_t num_recv_tokens,
                     uint32_t expert_y_dtype, void *out_tokens, size_t out_tokens_stride,
                     const int32_t *indices, size_t indices_stride, const float *weights,
                     size_t weights_stride, const int32_t *bound_m, uint32_t accumulate,
                     void *stream) {
    (void)num_recv_tokens;
    if (ctx == nullptr) return A2A_ERR_INVALID_ARGUMENT;
    ProfilerRange range("combine_recv");
    if (int rc = check_usable(ctx)) return rc;
    if (int rc = check_rank(ctx, rank)) return rc;
    const a2a_config &c = ctx->cfg;
    if (!ctx->staging.allocated || ctx->staging.combine_sent_mask == 0)
        return fail(ctx, A2A_ERR_BAD_ORDER, "a2a_combine_recv before any a2a_combine_send of the step");
    if (num_tokens > c.max_num_tokens)
        return fail(ctx, A2A_ERR_TOO_MANY_TOKENS, "Number of tokens exceeds maximum allowed (rank %u)", rank);
    if (int rc = check_combine_tokens(ctx, rank, num_tokens, indices_stride, weights_stride)) return rc;
    if (accumulate && c.dp_size != 1)   // python/pplx_garden/kernels/p2p_all_to_all.py:457-458
        return fail(ctx, A2A_ERR_UNSUPPORTED, "accumulate needs dp_size 1");
    if (elem_size_of(expert_y_dtype) != c.out_elemsize)
        return fail(ctx, A2A_ERR_UNSUPPORTED,
                    "expert_y dtype %u does not have the %u-byte elements the staging rows were sized for",
                    expert_y_dtype, c.out_elemsize);
    const uint32_t vec = 16 / c.out_elemsize;
    const uint32_t out_chunk = vec * c.out_elemsize;
    if (num_tokens != 0) {
        if (out_tokens == nullptr || indices == nullptr || weights == nullptr)
            return fail(ctx, A2A_ERR_INVALID_ARGUMENT, "rank %u: null out_tokens, indices or weights", rank);
        if (((uintptr_t)out_tokens % out_chunk) != 0 || (out_tokens_stride * c.out_elemsize) % out_chunk != 0)
            return fail(ctx, A2A_ERR_UNSUPPORTED, "rank %u: out_tokens rows must be %u-byte aligned", rank, out_chunk);
    }
    DeviceGuard guard(c.device);
    CombineRecvArgs cr;
    memset(&cr, 0, sizeof cr);
    cr.rank = rank;
    cr.dst.out = static_cast<uint8_t *>(out_tokens);
    cr.dst.indices = indices;
    cr.dst.weights = weights;
    cr.dst.bound_m = bound_m;
    cr.dst.out_stride = out_tokens_stride * c.out_elemsize;
    cr.dst.indices_stride = (uint32_t)indices_stride;
    cr.dst.weights_stride = (uint32_t)weights_stride;
    cr.dst.num_tokens = (uint32_t)num_tokens;
    cr.hidden_dim = c.hidden_dim;
    cr.accumulate = accumulate ? 1 : 0;
    const KernelTiming timing = ctx->timing[A2A_KERNEL_GATHER];
    ctx->timing[A2A_KERNEL_GATHER] = KernelTiming();
    hipError_t e = launch_combine_recv(cr, ctx->ws, ctx->staging, expert_y_dtype, c.out_dtype,
                                       static_cast<hipStream_t>(stream), timing);
    if (e != hipSuccess) return hip_fail(ctx, e, "launch combine_recv");
    return A2A_OK;
}

}  // extern "C"
