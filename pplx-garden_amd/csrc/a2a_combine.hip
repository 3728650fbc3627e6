// Combine: for every token, gather the K expert-output rows of its routes,
// weight them, accumulate in float and write one output row in token order.
//
// What it replaces: the reference's combine-send kernel (copy of every
// expert_y row back to the sender's staging buffer, a2a_combine_send.cu:
// 119-138,182-207) fused with its combine-recv kernel (weighted gather,
// a2a_combine_recv.cu:94-148).  Here the rows are read in place from the
// receivers' expert_y buffers, which live in the same HBM: one read per row,
// no staging write.
//
// Design for CDNA4: one wavefront per (token, slab of 64 sixteen-byte chunks);
// a lane owns 16 bytes of every source row, so K independent 16-byte loads are
// in flight per lane before the first multiply-add.  Row pointers and weights
// are resolved once by the first K lanes and read back as wave-uniform scalars
// (SGPR base + VGPR offset addressing).  Accumulation is an explicit float fused multiply-add
// chain, k ascending, then one round-to-nearest-even to the output type
// (combine_utils.cuh:108-114,14-23).
#include "a2a_internal.h"

namespace a2a {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

struct Bf16 {};
struct F16 {};
struct F32 {};

template <typename T> struct Elem;
template <> struct Elem<Bf16> { static constexpr int kSize = 2; };
template <> struct Elem<F16> { static constexpr int kSize = 2; };
template <> struct Elem<F32> { static constexpr int kSize = 4; };

// Elements per 16-byte source chunk (vector.cuh:14-27: 8 for the 16-bit
// types, 4 for float).
template <typename T> constexpr int vec_elems() { return 16 / Elem<T>::kSize; }

template <typename T, int V>
__device__ __forceinline__ void load_elems(const uint8_t *p, float (&f)[V], bool streaming) {
    if constexpr (Elem<T>::kSize == 4) {
        static_assert(V == 4 || V == 8, "");
#pragma unroll
        for (int h = 0; h < V / 4; ++h) {
            const u32x4 *q = reinterpret_cast<const u32x4 *>(p) + h;
            const u32x4 v = streaming ? __builtin_nontemporal_load(q) : *q;
#pragma unroll
            for (int j = 0; j < 4; ++j) f[4 * h + j] = __uint_as_float(v[j]);
        }
    } else if constexpr (V == 8) {
        const u32x4 *q = reinterpret_cast<const u32x4 *>(p);
        const u32x4 v = streaming ? __builtin_nontemporal_load(q) : *q;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if constexpr (__is_same(T, Bf16)) {
                f[2 * j] = __uint_as_float(v[j] << 16);
                f[2 * j + 1] = __uint_as_float(v[j] & 0xFFFF0000u);
            } else {
                f[2 * j] = (float)__builtin_bit_cast(_Float16, (uint16_t)(v[j] & 0xFFFF));
                f[2 * j + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(v[j] >> 16));
            }
        }
    } else {  // V == 4, 16-bit type: 8 bytes
        const u32x2 *q = reinterpret_cast<const u32x2 *>(p);
        const u32x2 v = streaming ? __builtin_nontemporal_load(q) : *q;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            if constexpr (__is_same(T, Bf16)) {
                f[2 * j] = __uint_as_float(v[j] << 16);
                f[2 * j + 1] = __uint_as_float(v[j] & 0xFFFF0000u);
            } else {
                f[2 * j] = (float)__builtin_bit_cast(_Float16, (uint16_t)(v[j] & 0xFFFF));
                f[2 * j + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(v[j] >> 16));
            }
        }
    }
}

template <typename U>
__device__ __forceinline__ uint32_t pack2(float a, float b) {
    if constexpr (__is_same(U, Bf16)) {
        const uint16_t lo = __builtin_bit_cast(uint16_t, (__bf16)a);
        const uint16_t hi = __builtin_bit_cast(uint16_t, (__bf16)b);
        return (uint32_t)lo | ((uint32_t)hi << 16);
    } else {
        const uint16_t lo = __builtin_bit_cast(uint16_t, (_Float16)a);
        const uint16_t hi = __builtin_bit_cast(uint16_t, (_Float16)b);
        return (uint32_t)lo | ((uint32_t)hi << 16);
    }
}

template <typename U, int V>
__device__ __forceinline__ void store_elems(uint8_t *p, const float (&f)[V]) {
    if constexpr (Elem<U>::kSize == 4) {
#pragma unroll
        for (int h = 0; h < V / 4; ++h) {
            u32x4 v;
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = __float_as_uint(f[4 * h + j]);
            __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(p) + h);
        }
    } else if constexpr (V == 8) {
        u32x4 v;
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = pack2<U>(f[2 * j], f[2 * j + 1]);
        __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(p));
    } else {
        u32x2 v;
#pragma unroll
        for (int j = 0; j < 2; ++j) v[j] = pack2<U>(f[2 * j], f[2 * j + 1]);
        __builtin_nontemporal_store(v, reinterpret_cast<u32x2 *>(p));
    }
}

__device__ __forceinline__ uint64_t read_lane64c(uint64_t v, uint32_t lane) {
    const uint32_t lo = __builtin_amdgcn_readlane((int)(uint32_t)v, (int)lane);
    const uint32_t hi = __builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), (int)lane);
    return ((uint64_t)hi << 32) | lo;
}

// Convert one 16-byte source chunk (raw) and fuse it into the accumulators.
template <typename T, int V>
__device__ __forceinline__ void fma_chunk(const u32x4 raw, float w, float (&acc)[V]) {
    if constexpr (Elem<T>::kSize == 4) {
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] = __builtin_fmaf(w, __uint_as_float(raw[j]), acc[j]);
    } else if constexpr (__is_same(T, Bf16)) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            acc[2 * j] = __builtin_fmaf(w, __uint_as_float(raw[j] << 16), acc[2 * j]);
            acc[2 * j + 1] = __builtin_fmaf(w, __uint_as_float(raw[j] & 0xFFFF0000u), acc[2 * j + 1]);
        }
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            acc[2 * j] = __builtin_fmaf(
                w, (float)__builtin_bit_cast(_Float16, (uint16_t)(raw[j] & 0xFFFF)), acc[2 * j]);
            acc[2 * j + 1] = __builtin_fmaf(
                w, (float)__builtin_bit_cast(_Float16, (uint16_t)(raw[j] >> 16)), acc[2 * j + 1]);
        }
    }
}

constexpr int kCombineWaves = 1;    // wavefronts per workgroup; each works on its own
constexpr int kCombineChunks = 1;   // 16-byte chunks of a row per lane
constexpr int kSlabChunks = kWave * kCombineChunks;
constexpr uint32_t kOneRankMaxTokens = 2048;   // largest step that takes the ONE_RANK variant of the gather

// T: type of the expert_y rows, U: type of out_tokens.  One WAVEFRONT handles
// one slab of 64 sixteen-byte chunks of one token; wavefronts share nothing, so
// a compute unit keeps many of them in flight and the latency of resolving a
// token's routes is hidden by the loads of its neighbours.  KFIX > 0 unrolls
// the route loop (all K loads issued before the first use).  ONE_RANK: one rank
// alone has tokens and the step is small; its descriptor is read from a fixed
// place in the argument block, which takes two dependent scalar loads out of
// the head of every wavefront (0.1-0.4 us of a step of 128 to 1024 tokens; a
// 4096-token step hides them and is 0.3 us faster without the variant).
template <typename T, typename U, int KFIX, bool ONE_RANK>
__global__ __launch_bounds__(kCombineWaves * kWave) void combine_gather_kernel(const CombArgs args,
                                                                              const Workspace ws) {
    constexpr int V = vec_elems<T>();
    if constexpr (ONE_RANK) {
        // everything the head of a wavefront needs from the argument block, asked for in one go
        A2A_PIN(args.token_start[kMaxWorld]);
        A2A_PIN(args.single_rank);
        A2A_PIN(args.hidden_dim);
        A2A_PIN(args.accumulate);
        A2A_PIN(args.staged_base);
        A2A_PIN(args.single.out);
        A2A_PIN(args.single.indices);
        A2A_PIN(args.single.weights);
        A2A_PIN(args.single.bound_m);
        A2A_PIN(args.single.out_stride);
        A2A_PIN(args.single.indices_stride);
        A2A_PIN(args.single.weights_stride);
        A2A_PIN(args.single.num_tokens);
        A2A_PIN(ws.world);
        A2A_PIN(ws.dp_size);
        A2A_PIN(ws.num_experts);
        A2A_PIN(ws.experts_per_rank);
        A2A_PIN(ws.le_magic);
        A2A_PIN(ws.max_tk);
        A2A_PIN(ws.route_slot);
        A2A_PIN(ws.err);
    }
    if constexpr (!ONE_RANK) {
        // (here too; measured on the 4096-token step: 0.7 us a step.  The same in the pack of that step cost
        // 1.2 us and is left out there.)
        A2A_PIN(args.token_start[0]);
        A2A_PIN(args.token_start[1]);
        A2A_PIN(args.hidden_dim);
        A2A_PIN(args.accumulate);
        A2A_PIN(args.staged_base);
        A2A_PIN(ws.world);
        A2A_PIN(ws.dp_size);
        A2A_PIN(ws.num_experts);
        A2A_PIN(ws.experts_per_rank);
        A2A_PIN(ws.le_magic);
        A2A_PIN(ws.max_tk);
        A2A_PIN(ws.route_slot);
        A2A_PIN(ws.err);
    }
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const uint32_t E = ws.num_experts;
    const uint32_t K = KFIX > 0 ? (uint32_t)KFIX : ws.topk;
    const uint32_t num_chunks = args.hidden_dim / V;
    const uint32_t slabs = (num_chunks + kSlabChunks - 1) / kSlabChunks;

    const uint32_t unit = blockIdx.x * kCombineWaves + wave;
    const uint32_t token_global = unit / slabs;
    const uint32_t slab = unit - token_global * slabs;
    uint32_t g = 0, token = token_global;
    if constexpr (ONE_RANK) {
        if (token_global >= args.token_start[kMaxWorld]) return;   // the total, at a fixed place
        g = args.single_rank - 1;
    } else {
        if (token_global >= args.token_start[ws.world]) return;
        while (g + 1 < ws.world && token_global >= args.token_start[g + 1]) ++g;
        token = token_global - args.token_start[g];
    }
    const CombDst &dst = ONE_RANK ? args.single : args.dst[g];
    const uint32_t group = g / ws.dp_size;   // the routing tables belong to the rank's dp group
    if (token >= effective_tokens(dst.bound_m, dst.num_tokens)) return;

    // Lane r holds the descriptor of receiver r; lanes 0..K-1 resolve a route
    // each and pick their receiver's descriptor with a lane shuffle.
    uint64_t y_base = 0, y_stride = 0;
    uint32_t y_rows = 0;
    if (lane < ws.world && args.staged_base == nullptr) {
        y_base = (uint64_t)args.src[lane].y;
        y_stride = args.src[lane].y_stride;
        y_rows = args.src[lane].y_rows;
    }
    uint32_t expert = 0, slot = 0;
    float weight = 0.0f;
    if (lane < K) {
        expert = (uint32_t)dst.indices[(size_t)token * dst.indices_stride + lane];
        weight = dst.weights[(size_t)token * dst.weights_stride + lane];
        // (after a group dispatch: the copy's row in its receiver's buffer; after the sends of the split
        // calls: its position in the sender's expert-sorted order, a2a_combine_recv.cu:67-73 = exclusive
        // offset of the expert + token offset, which the send wrote here so that no second, dependent
        // look-up stands in front of the rows: 0.5 us of a 128-token combine-recv)
        slot = ws.route_slot[(size_t)group * ws.max_tk + token * K + lane];
    }
    const bool expert_ok = expert < E;
    const uint32_t r = expert_ok ? owner_of_expert(ws, expert) : 0;
    const uint64_t r_base = __shfl(y_base, (int)r);
    const uint64_t r_stride = __shfl(y_stride, (int)r);
    const uint32_t r_rows = __shfl(y_rows, (int)r);
    uint64_t row_ptr = 0;
    if (lane < K) {
        bool ok = false;
        if (args.staged_base != nullptr) {
            if (expert_ok && slot < ws.max_tk) {
                row_ptr = (uint64_t)(args.staged_base + ((size_t)group * ws.max_tk + slot) * args.staged_stride);
                ok = true;
            }
        } else if (expert_ok && r_base != 0 && slot < r_rows) {
            row_ptr = r_base + (uint64_t)slot * r_stride;
            ok = true;
        }
        if (!ok && slab == 0) atomicOr(ws.err, A2A_DEV_BAD_SLOT);
    }

    uint32_t c[kCombineChunks];
    bool active[kCombineChunks];
    uint8_t *out_chunk[kCombineChunks];
    float acc[kCombineChunks][V];
#pragma unroll
    for (int u = 0; u < kCombineChunks; ++u) {
        c[u] = slab * kSlabChunks + u * kWave + lane;
        active[u] = c[u] < num_chunks;
        out_chunk[u] = dst.out + (size_t)token * dst.out_stride + (size_t)c[u] * V * Elem<U>::kSize;
#pragma unroll
        for (int j = 0; j < V; ++j) acc[u][j] = 0.0f;
        if (args.accumulate && active[u]) load_elems<U, V>(out_chunk[u], acc[u], false);
    }

    if constexpr (KFIX > 0) {
        u32x4 raw[kCombineChunks][KFIX];
        float w[KFIX];
        bool present[KFIX];
#pragma unroll
        for (int k = 0; k < KFIX; ++k) {
            const uint64_t row = read_lane64c(row_ptr, k);
            w[k] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(weight), k));
            present[k] = row != 0;
#pragma unroll
            for (int u = 0; u < kCombineChunks; ++u) {
                raw[u][k] = u32x4{0, 0, 0, 0};
                if (present[k] && active[u]) {
                    raw[u][k] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(row) + c[u]);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < kCombineChunks; ++u) {
#pragma unroll
            for (int k = 0; k < KFIX; ++k) {
                if (present[k]) fma_chunk<T, V>(raw[u][k], w[k], acc[u]);
            }
        }
    } else {
        for (uint32_t k = 0; k < K; ++k) {
            const uint64_t row = read_lane64c(row_ptr, k);
            const float wk = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(weight), (int)k));
            if (row != 0) {
#pragma unroll
                for (int u = 0; u < kCombineChunks; ++u) {
                    u32x4 raw = {0, 0, 0, 0};
                    if (active[u]) raw = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(row) + c[u]);
                    fma_chunk<T, V>(raw, wk, acc[u]);
                }
            }
        }
    }
#pragma unroll
    for (int u = 0; u < kCombineChunks; ++u) {
        if (active[u]) store_elems<U, V>(out_chunk[u], acc[u]);
    }
}

template <typename T, typename U>
static hipError_t launch_typed(const CombArgs &given, const Workspace &ws, uint32_t total_tokens,
                               hipStream_t stream, KernelTiming timing) {
    constexpr int V = vec_elems<T>();
    CombArgs args = given;
    uint32_t ranks_with_tokens = 0;
    args.single_rank = 0;
    for (uint32_t r = 0; r < ws.world; ++r) {
        if (given.dst[r].num_tokens == 0) continue;
        ++ranks_with_tokens;
        args.single_rank = r + 1;
    }
    if (ranks_with_tokens != 1 || total_tokens > kOneRankMaxTokens) args.single_rank = 0;
    if (args.single_rank != 0) args.single = given.dst[args.single_rank - 1];
    const uint32_t chunks = args.hidden_dim / V;
    const uint32_t slabs = (chunks + kSlabChunks - 1) / kSlabChunks;
    const uint64_t units = (uint64_t)total_tokens * slabs;
    const uint32_t blocks = (uint32_t)((units + kCombineWaves - 1) / kCombineWaves);
#define A2A_LAUNCH_GATHER(KFIX, ONE)                                                                           \
    hipExtLaunchKernelGGL((combine_gather_kernel<T, U, KFIX, ONE>), dim3(blocks), dim3(kCombineWaves * kWave), 0, \
                          stream, timing.start, timing.stop, 0, args, ws)
    if (ws.topk == 8) {
        if (args.single_rank != 0) A2A_LAUNCH_GATHER(8, true); else A2A_LAUNCH_GATHER(8, false);
    } else {
        if (args.single_rank != 0) A2A_LAUNCH_GATHER(0, true); else A2A_LAUNCH_GATHER(0, false);
    }
#undef A2A_LAUNCH_GATHER
    return hipGetLastError();
}

hipError_t launch_combine_gather(const CombArgs &args, const Workspace &ws, uint32_t in_dtype,
                                 uint32_t out_dtype, uint32_t total_tokens, hipStream_t stream, KernelTiming timing) {
    if (total_tokens == 0) return hipSuccess;
#define A2A_COMBINE_CASE(IN_TAG, IN_T, OUT_TAG, OUT_T) \
    if (in_dtype == IN_TAG && out_dtype == OUT_TAG)    \
        return launch_typed<IN_T, OUT_T>(args, ws, total_tokens, stream, timing);
    A2A_COMBINE_CASE(A2A_BF16, Bf16, A2A_BF16, Bf16)
    A2A_COMBINE_CASE(A2A_BF16, Bf16, A2A_F32, F32)
    A2A_COMBINE_CASE(A2A_BF16, Bf16, A2A_F16, F16)
    A2A_COMBINE_CASE(A2A_F16, F16, A2A_F16, F16)
    A2A_COMBINE_CASE(A2A_F16, F16, A2A_F32, F32)
    A2A_COMBINE_CASE(A2A_F16, F16, A2A_BF16, Bf16)
    A2A_COMBINE_CASE(A2A_F32, F32, A2A_F32, F32)
    A2A_COMBINE_CASE(A2A_F32, F32, A2A_BF16, Bf16)
    A2A_COMBINE_CASE(A2A_F32, F32, A2A_F16, F16)
#undef A2A_COMBINE_CASE
    return hipErrorInvalidValue;
}

}  // namespace a2a
